"""ctypes binding of libmoe_hip.so (every symbol include/moe_hip.h declares)."""
from __future__ import annotations

import ctypes as C
import os
import threading

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmoe_hip.so")

_lock = threading.Lock()
_lib = None


class MoeError(RuntimeError):
    """A non-zero return code from the C ABI (message from moe_last_error)."""

    def __init__(self, code, message):
        super().__init__(f"libmoe_hip error {code}: {message}")
        self.code = code


class MoeForwardArgs(C.Structure):
    _fields_ = [
        ("M", C.c_int), ("D", C.c_int), ("E", C.c_int), ("k", C.c_int), ("I", C.c_int), ("SI", C.c_int),
        ("routing", C.c_int), ("n_group", C.c_int), ("topk_group", C.c_int), ("renorm", C.c_int),
        ("routed_scale", C.c_float),
        ("x", C.c_void_p), ("logits", C.c_void_p), ("bias", C.c_void_p),
        ("w_gate", C.c_void_p), ("w_up", C.c_void_p), ("w_down", C.c_void_p),
        ("sw_gate", C.c_void_p), ("sw_up", C.c_void_p), ("sw_down", C.c_void_p),
        ("ws_gate", C.c_void_p), ("ws_up", C.c_void_p), ("ws_down", C.c_void_p),
        ("sws_gate", C.c_void_p), ("sws_up", C.c_void_p), ("sws_down", C.c_void_p),
        ("out", C.c_void_p),
        ("out_idx", C.c_void_p), ("out_w", C.c_void_p), ("out_group_sizes", C.c_void_p),
        ("out_sorted_token_ids", C.c_void_p), ("out_inv_perm", C.c_void_p),
        ("out_hq", C.c_void_p), ("out_sh", C.c_void_p), ("out_hsq", C.c_void_p), ("out_shs", C.c_void_p),
        ("out_y", C.c_void_p), ("out_ys", C.c_void_p),
        ("w_router", C.c_void_p), ("w_shared_gate", C.c_void_p), ("out_logits", C.c_void_p), ("out_shared_gate", C.c_void_p),
        ("norm_weight", C.c_void_p), ("norm_eps", C.c_float), ("add_residual", C.c_int),
    ]


_P, _I, _F, _Z = C.c_void_p, C.c_int, C.c_float, C.c_size_t

# name -> (restype, argtypes); the list mirrors include/moe_hip.h one to one
SIGNATURES = {
    "moe_abi_version": (_I, []),
    "moe_last_error": (C.c_char_p, []),
    "moe_route_softmax_topk": (_I, [_P, _I, _I, _I, _I, _P, _P, _P]),
    "moe_route_sigmoid_grouped": (_I, [_P, _P, _I, _I, _I, _I, _I, _I, _F, _P, _P, _P]),
    "moe_permute_workspace_bytes": (_Z, [_I, _I, _I]),
    "moe_permute": (_I, [_P, _I, _I, _I, _P, _P, _P, _P, _P, _P, _Z, _P]),
    "moe_quant_act": (_I, [_P, _I, _I, _P, _P, _P]),
    "moe_quant_weight_block": (_I, [_P, _I, _I, _I, _I, _P, _P, _P]),
    "moe_gemm_workspace_bytes": (_Z, [_I, _I, _I]),
    "moe_gemm_gateup_swiglu_fp8": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _Z, _P]),
    "moe_gemm_gateup_swiglu_fp8_static": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P]),
    "moe_gemm_down_fp8": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _P, _Z, _P]),
    "moe_gemm_gateup_swiglu_fp8_layout": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _Z, _I, _I, _P]),
    "moe_gemm_down_fp8_layout": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _P, _Z, _I, _P]),
    "moe_gather_scales": (_I, [_P, _P, _I, _I, _P, _P]),
    "moe_combine": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _P, _P]),
    "moe_rmsnorm_quant": (_I, [_P, _P, _F, _I, _I, _P, _P, _P, _P]),
    "moe_router_workspace_bytes": (_Z, [_I, _I, _I]),
    "moe_router_logits": (_I, [_P, _I, _I, _P, _I, _P, _P, _P, _P, _Z, _P]),
    "moe_convert": (_I, [_P, _I, _P, _I, C.c_longlong, _P]),
    "moe_forward_workspace_bytes": (_Z, [_I, _I, _I, _I, _I, _I]),
    "moe_forward": (_I, [C.POINTER(MoeForwardArgs), _P, _Z, _P]),
}


def lib():
    """Load libmoe_hip.so.  Raises if it has not been built: there is no fallback."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build the HIP kernels first "
                "(python -c 'import __graft_entry__ as g; g.build()' at the repository root)")
        dll = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(dll, name)          # AttributeError here = header and library disagree
            fn.restype = res
            fn.argtypes = args
        _lib = dll
        return _lib


def check(code: int):
    if code != 0:
        raise MoeError(code, lib().moe_last_error().decode("utf-8", "replace"))
