"""Host side of the MoE expert forward: the reference's call surface over the C ABI.

Mirrors jax_gpt/models/qwen35/moe.py -- `moe_routing` (:37), `_sort_and_group`
(:58, here `permute`), `expert_forward_single` (:97), `shared_expert_forward`
(:225) and `moe_layer` (:235) -- with torch CUDA tensors as the device buffers
and the current torch stream as the HIP stream.  All arithmetic happens in
libmoe_hip.so; torch only allocates.

Expert weights are block-scaled fp8 dicts ``{'w': (E, out, in) float8_e4m3fn,
'scale_inv': (E, out/128, in/128) float32}`` -- the reference's fp8 layout
(quantize.py:31-42, model.py:89-97) with 128x128 scale blocks instead of
per-row scales; real value = w * scale_inv (moe.py:29).  Plain (E, in, out)
arrays, the reference's unquantised layout, are quantised on the GPU on first
use.  The reference's own fp8 dicts (one scale per output row: experts
``scale_inv (E, out, 1)``, dense layers ``(out, 1)``; quantize.py:18-42,
model.py:79-114 with fp8=True) are accepted too: they are de-quantised once the way
the reference's consumer of each does it (experts: w * scale_inv, moe.py:29; dense
layers and the router: w / scale_inv, fp8.py:87-89) and re-quantised per 128x128
block (a second rounding of the weights), cached for the life of the source tensor.
"""
from __future__ import annotations

import ctypes as C
import weakref

import torch

from ._lib import MoeForwardArgs, check, lib

ROUTING = {"softmax": 0, "sigmoid_grouped": 1}


# ----------------------------------------------------------------------------
# plumbing
# ----------------------------------------------------------------------------

def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return C.c_void_p(0) if t is None else C.c_void_p(t.data_ptr())


def _dev(t, dtype=None, name="tensor"):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name}: expected a torch.Tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise RuntimeError(f"{name}: must live on the GPU (this path has no CPU fallback)")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
    return t.contiguous()


def _codes(t, name):
    """fp8 weights/activations travel as bytes; accept float8_e4m3fn or uint8."""
    if t.dtype == torch.float8_e4m3fn:
        t = t.view(torch.uint8)
    return _dev(t, torch.uint8, name)


def _empty(shape, dtype, like):
    return torch.empty(shape, dtype=dtype, device=like.device)


# ----------------------------------------------------------------------------
# routing (moe.py:37-55) and the DeepSeek-V3 group-limited router
# ----------------------------------------------------------------------------

def route_softmax_topk(logits, k, renorm=True):
    logits = _dev(logits, torch.float32, "logits")
    M, E = logits.shape
    idx = _empty((M, k), torch.int32, logits)
    w = _empty((M, k), torch.float32, logits)
    check(lib().moe_route_softmax_topk(_ptr(logits), M, E, k, int(renorm), _ptr(idx), _ptr(w), _stream()))
    return idx, w


def route_sigmoid_grouped(logits, bias, n_group, topk_group, k, renorm=True, routed_scale=1.0):
    logits = _dev(logits, torch.float32, "logits")
    bias = None if bias is None else _dev(bias, torch.float32, "bias")
    M, E = logits.shape
    if bias is not None and tuple(bias.shape) != (E,):
        raise ValueError(f"bias: expected shape ({E},), got {tuple(bias.shape)}")
    idx = _empty((M, k), torch.int32, logits)
    w = _empty((M, k), torch.float32, logits)
    check(lib().moe_route_sigmoid_grouped(_ptr(logits), _ptr(bias), M, E, n_group, topk_group, k, int(renorm),
                                          float(routed_scale), _ptr(idx), _ptr(w), _stream()))
    return idx, w


# ----------------------------------------------------------------------------
# sort / group (moe.py:58-80)
# ----------------------------------------------------------------------------

def permute(expert_indices, n_experts):
    """Stable sort of the flat (token, slot) list by expert.  Returns a dict with
    group_sizes (E,), group_offsets (E+1,), sorted_token_ids, sort_order, inv_perm (R,)."""
    idx = _dev(expert_indices, torch.int32, "expert_indices")
    M, k = idx.shape
    R = M * k
    out = dict(group_sizes=_empty((n_experts,), torch.int32, idx),
               group_offsets=_empty((n_experts + 1,), torch.int32, idx),
               sorted_token_ids=_empty((R,), torch.int32, idx),
               sort_order=_empty((R,), torch.int32, idx),
               inv_perm=_empty((R,), torch.int32, idx))
    nbytes = lib().moe_permute_workspace_bytes(M, k, n_experts)
    ws = _empty((nbytes,), torch.uint8, idx)
    check(lib().moe_permute(_ptr(idx), M, k, n_experts, _ptr(out["group_sizes"]), _ptr(out["group_offsets"]),
                            _ptr(out["sorted_token_ids"]), _ptr(out["sort_order"]), _ptr(out["inv_perm"]),
                            _ptr(ws), nbytes, _stream()))
    return out


# ----------------------------------------------------------------------------
# quantisers
# ----------------------------------------------------------------------------

def convert(t, dtype):
    """f32 <-> bf16 conversion on the library's own kernel (round-to-nearest-even towards bf16)."""
    if t.dtype == dtype:
        return t
    if {t.dtype, dtype} != {torch.float32, torch.bfloat16}:
        raise TypeError(f"convert: f32 <-> bf16 only, got {t.dtype} -> {dtype}")
    t = _dev(t, None, "t")
    out = _empty(tuple(t.shape), dtype, t)
    check(lib().moe_convert(_ptr(t), int(t.dtype == torch.float32), _ptr(out), int(dtype == torch.float32), t.numel(), _stream()))
    return out


def quant_act(x):
    """(R, K) bf16 -> (codes (R, K) float8_e4m3fn, scale_inv (R, K/128) f32)."""
    x = _dev(x, torch.bfloat16, "x")
    R, K = x.shape
    xq = _empty((R, K), torch.uint8, x)
    sx = _empty((R, K // 128), torch.float32, x)
    check(lib().moe_quant_act(_ptr(x), R, K, _ptr(xq), _ptr(sx), _stream()))
    return xq.view(torch.float8_e4m3fn), sx


def rmsnorm_quant(x, weight, eps=1e-6):
    """primitives.py:16-32 (rms_norm with 1 + weight) fused with the 1x128 activation quantiser.
    x (M, D) bf16, weight (D,) -> (normed (M, D) bf16, codes (M, D) uint8, scale_inv (M, D/128) f32)."""
    x = _dev(x, torch.bfloat16, "x")
    weight = _dev(weight.to(torch.float32), torch.float32, "weight")
    M, D = x.shape
    if tuple(weight.shape) != (D,):
        raise ValueError(f"weight: expected ({D},), got {tuple(weight.shape)}")
    normed = _empty((M, D), torch.bfloat16, x)
    xq = _empty((M, D), torch.uint8, x)
    sx = _empty((M, D // 128), torch.float32, x)
    check(lib().moe_rmsnorm_quant(_ptr(x), _ptr(weight), float(eps), M, D, _ptr(normed), _ptr(xq), _ptr(sx), _stream()))
    return normed, xq, sx


def quantize_weight_block(w):
    """(E, out, in) or (out, in) bf16/f32 -> {'w': float8_e4m3fn, 'scale_inv': f32 (.., out/128, in/128)}.

    The block-scaled counterpart of the reference's `_quantize_weight`
    (quantize.py:18-42); the input is already in (out, in) order."""
    if w.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"weights must be bf16 or f32, got {w.dtype}")
    w = _dev(w, None, "w")
    squeeze = w.dim() == 2
    w3 = w.unsqueeze(0) if squeeze else w
    E, N, K = w3.shape
    wq = _empty((E, N, K), torch.uint8, w)
    sw = _empty((E, N // 128, K // 128), torch.float32, w)
    check(lib().moe_quant_weight_block(_ptr(w3), int(w.dtype == torch.float32), E, N, K, _ptr(wq), _ptr(sw),
                                       _stream()))
    if squeeze:
        wq, sw = wq[0], sw[0]
    return {"w": wq.view(torch.float8_e4m3fn), "scale_inv": sw}


def block_fp8_from_per_row(d, dense=False):
    """The reference's own fp8 dicts carry one scale per output row (`scale_inv` (E, out, 1) or (out, 1),
    quantize.py:18-42).  This path computes with 128x128 blocks: de-quantise (experts: w * scale_inv, moe.py:29;
    `dense` 2-D layers: w / scale_inv, fp8.py:87-89) to f32 and quantise again per block.  A second rounding of
    the weights, so prefer quantising from bf16 where the original weights exist.  (The layer entry points do this
    themselves, once per tensor, when handed such a dict.)"""
    q, s = d["w"], d["scale_inv"]
    if not _per_row_scales(q, s):
        raise ValueError(f"expected per-row scales {tuple(q.shape[:-1]) + (1,)}, got {tuple(s.shape)}")
    wq, sw = _requantise_per_row(q, s, dense)
    if q.dim() == 2:
        wq, sw = wq[0], sw[0]
    return {"w": wq.view(torch.float8_e4m3fn), "scale_inv": sw}


_derived = {}


def _cached(src, tag, build):
    """Derived GPU copies (quantised weights, transposed router weights) are kept per source tensor and version,
    and dropped when the source tensor is garbage-collected or has been modified in place."""
    key = (tag, id(src))
    hit = _derived.get(key)
    if hit is not None and hit[0]() is src and hit[1] == src._version:
        return hit[2]
    val = build()
    if hit is None or hit[0]() is not src:
        weakref.finalize(src, _derived.pop, key, None)
    _derived[key] = (weakref.ref(src), src._version, val)
    return val


def _per_row_scales(q, s):
    """True for the reference's per-row layout: scale_inv (..., out, 1) next to w (..., out, in)."""
    return s.dim() == q.dim() and s.shape[-1] == 1 and tuple(s.shape[:-1]) == tuple(q.shape[:-1])


def _requantise_per_row(q, s, dense):
    """De-quantise a per-row fp8 dict as its consumer in the reference does and quantise per 128x128 block."""
    if q.dtype != torch.float8_e4m3fn:
        q = _codes(q, "w").view(torch.float8_e4m3fn)
    q = _dev(q, None, "w")
    s = _dev(s, None, "scale_inv").to(torch.float32)
    w = q.to(torch.float32) / s if dense else q.to(torch.float32) * s     # fp8.py:87-89 / moe.py:29
    d = quantize_weight_block(w if w.dim() == 3 else w.unsqueeze(0))
    return d["w"].view(torch.uint8), d["scale_inv"]


def _expert_weight(w, name, dense=False):
    """Accept a block-fp8 dict; a per-row fp8 dict of the reference (re-quantised per block once, cached); or a plain
    (E, in, out) array as the reference stores unquantised experts (model.py:98-101), transposed and quantised
    once.  `dense`: a 2-D layer of the shared expert, (in, out) plain or (out, in) fp8 (fp8.py:123-143).
    Returns (codes (E, N, K) uint8, scale_inv (E, N/128, K/128) f32)."""
    if isinstance(w, dict) and "w" in w:
        q, s = w["w"], w["scale_inv"]
        if _per_row_scales(q, s):
            return _cached(q, ("per_row", dense, id(s), s._version), lambda: _requantise_per_row(q, s, dense))
        if q.dim() == 2:
            q, s = q.unsqueeze(0), s.unsqueeze(0)
        E, N, K = q.shape
        if tuple(s.shape) != (E, N // 128, K // 128):
            raise ValueError(
                f"{name}: scale_inv has shape {tuple(s.shape)}; expected 128x128 block scales "
                f"{(E, N // 128, K // 128)} or the reference's per-row scales {(E, N, 1)}")
        return _codes(q, name + "['w']"), _dev(s, torch.float32, name + "['scale_inv']")
    if not isinstance(w, torch.Tensor):
        raise TypeError(f"{name}: expected a tensor or an fp8 dict")

    def build():
        w3 = w.unsqueeze(0) if w.dim() == 2 else w
        if w3.dtype not in (torch.bfloat16, torch.float32):
            w3 = w3.to(torch.float32)
        d = quantize_weight_block(w3.transpose(-1, -2).contiguous())      # (E, in, out) -> (E, out, in)
        return d["w"].view(torch.uint8), d["scale_inv"]
    return _cached(w, "plain", build)


# ----------------------------------------------------------------------------
# grouped GEMMs (moe.py:83-87) and combine (moe.py:90-94)
# ----------------------------------------------------------------------------

def _gemm_ws(R, E, n_out, like):
    nbytes = lib().moe_gemm_workspace_bytes(R, E, n_out)
    return _empty((nbytes,), torch.uint8, like), nbytes


SCALES_ROW_MAJOR, SCALES_BLOCK_MAJOR = 0, 1


def gather_scales(sx, row_ids=None, n_rows=None):
    """Row-major activation scales (rows, KB) -> block-major (KB, R) in row-list order:
    out[kb, p] = sx[row_ids[p], kb] (row_ids None: p).  The layout the grouped GEMMs read fastest."""
    sx = _dev(sx, torch.float32, "sx")
    if row_ids is not None:
        row_ids = _dev(row_ids, torch.int32, "row_ids")
        R = row_ids.numel() if n_rows is None else n_rows
    else:
        R = sx.shape[0] if n_rows is None else n_rows
    KB = sx.shape[1]
    out = _empty((KB, R), torch.float32, sx)
    check(lib().moe_gather_scales(_ptr(sx), _ptr(row_ids), R, KB, _ptr(out), _stream()))
    return out


def gemm_gateup_swiglu(xq, sx, gate, up, group_offsets, row_ids=None, n_rows=None, block_major=False):
    """h = silu(x.Wg^T) * (x.Wu^T) per expert row range, quantised 1x128 -> (hq, sh).
    row_ids maps sorted position -> row of xq (None: rows are already in expert order).
    block_major: sx is a gather_scales() array (KB, R) and sh comes back as (I/128, R)."""
    xq = _codes(xq, "xq")
    sx = _dev(sx, torch.float32, "sx")
    wg, sg = _expert_weight(gate, "gate_proj")
    wu, su = _expert_weight(up, "up_proj")
    E, I, D = wg.shape
    if wu.shape != wg.shape or xq.shape[1] != D:
        raise ValueError(f"shape mismatch: x {tuple(xq.shape)}, gate {tuple(wg.shape)}, up {tuple(wu.shape)}")
    go = _dev(group_offsets, torch.int32, "group_offsets")
    if go.numel() != E + 1:
        raise ValueError(f"group_offsets needs {E + 1} entries, got {go.numel()}")
    if row_ids is not None:
        row_ids = _dev(row_ids, torch.int32, "row_ids")
        R = row_ids.numel() if n_rows is None else n_rows
    else:
        R = xq.shape[0] if n_rows is None else n_rows
    hq = _empty((R, I), torch.uint8, xq)
    ws, nbytes = _gemm_ws(R, E, I, xq)
    if block_major:
        if tuple(sx.shape) != (D // 128, R):
            raise ValueError(f"block-major sx must be {(D // 128, R)}, got {tuple(sx.shape)}")
        sh = _empty((I // 128, R), torch.float32, xq)
        check(lib().moe_gemm_gateup_swiglu_fp8_layout(_ptr(xq), _ptr(sx), _ptr(row_ids), _ptr(wg), _ptr(sg), _ptr(wu),
                                                      _ptr(su), _ptr(go), E, R, D, I, _ptr(hq), _ptr(sh), _ptr(ws), nbytes,
                                                      SCALES_BLOCK_MAJOR, SCALES_BLOCK_MAJOR, _stream()))
        return hq.view(torch.float8_e4m3fn), sh
    sh = _empty((R, I // 128), torch.float32, xq)
    check(lib().moe_gemm_gateup_swiglu_fp8(_ptr(xq), _ptr(sx), _ptr(row_ids), _ptr(wg), _ptr(sg), _ptr(wu), _ptr(su),
                                           _ptr(go), E, R, D, I, _ptr(hq), _ptr(sh), _ptr(ws), nbytes, _stream()))
    return hq.view(torch.float8_e4m3fn), sh


def gemm_down(hq, sh, down, group_offsets, block_major=False):
    """y = h . Wdown[e]^T per expert row range, bf16 (R, D).  block_major: sh is (I/128, R)."""
    hq = _codes(hq, "hq")
    sh = _dev(sh, torch.float32, "sh")
    wd, sd = _expert_weight(down, "down_proj")
    E, D, I = wd.shape
    R = hq.shape[0]
    if hq.shape[1] != I:
        raise ValueError(f"shape mismatch: h {tuple(hq.shape)}, down {tuple(wd.shape)}")
    go = _dev(group_offsets, torch.int32, "group_offsets")
    y = _empty((R, D), torch.bfloat16, hq)
    ws, nbytes = _gemm_ws(R, E, D, hq)
    if block_major:
        if tuple(sh.shape) != (I // 128, R):
            raise ValueError(f"block-major sh must be {(I // 128, R)}, got {tuple(sh.shape)}")
        check(lib().moe_gemm_down_fp8_layout(_ptr(hq), _ptr(sh), _ptr(wd), _ptr(sd), _ptr(go), E, R, I, D, _ptr(y),
                                             _ptr(ws), nbytes, SCALES_BLOCK_MAJOR, _stream()))
        return y
    check(lib().moe_gemm_down_fp8(_ptr(hq), _ptr(sh), _ptr(wd), _ptr(sd), _ptr(go), E, R, I, D, _ptr(y), _ptr(ws),
                                  nbytes, _stream()))
    return y


def combine(y, weights, inv_perm, shared=None, shared_gate=None, residual=None):
    """moe.py:90-94 and the add of :281; `shared_gate` (M,) f32 scales the shared rows (moe.py:278-279);
    `residual` (M, D) bf16 is the layer input added last (block.py:58)."""
    y = _dev(y, torch.bfloat16, "y")
    weights = _dev(weights, torch.float32, "weights")
    inv_perm = _dev(inv_perm, torch.int32, "inv_perm")
    shared = None if shared is None else _dev(shared, torch.bfloat16, "shared")
    shared_gate = None if shared_gate is None else _dev(shared_gate, torch.float32, "shared_gate")
    residual = None if residual is None else _dev(residual, torch.bfloat16, "residual")
    M, k = weights.shape
    D = y.shape[1]
    out = _empty((M, D), torch.bfloat16, y)
    check(lib().moe_combine(_ptr(y), _ptr(weights), _ptr(inv_perm), _ptr(shared), _ptr(shared_gate), _ptr(residual),
                            M, k, D, _ptr(out), _stream()))
    return out


# ----------------------------------------------------------------------------
# the reference's functions
# ----------------------------------------------------------------------------

def expert_forward_single(x, expert_indices, expert_weights, gate_proj, up_proj, down_proj):
    """moe.py:97-114: sort/group, grouped SwiGLU, weighted scatter back.  x (M, D) bf16."""
    x = _dev(x, torch.bfloat16, "x")
    wg, _ = _expert_weight(gate_proj, "gate_proj")
    E = wg.shape[0]
    sg = permute(expert_indices, E)
    xq, sx = quant_act(x)
    hq, sh = gemm_gateup_swiglu(xq, sx, gate_proj, up_proj, sg["group_offsets"], row_ids=sg["sorted_token_ids"])
    y = gemm_down(hq, sh, down_proj, sg["group_offsets"])
    return combine(y, expert_weights, sg["inv_perm"])


def shared_expert_forward(x, gate_proj, up_proj, down_proj):
    """moe.py:225-232: dense SwiGLU MLP on every token (one group holding all rows)."""
    x = _dev(x, torch.bfloat16, "x")
    M = x.shape[0]
    off = torch.tensor([0, M], dtype=torch.int32, device=x.device)
    xq, sx = quant_act(x)
    hq, sh = gemm_gateup_swiglu(xq, sx, gate_proj, up_proj, off)
    return gemm_down(hq, sh, down_proj, off)


def _router_weight(w, name):
    """The reference keeps router weights input-major, (D, E) / (D, 1) (model.py:83-85, used as x @ w at
    moe.py:50 and :278); the kernel wants them K-contiguous, (E, D) bf16: transposed once and cached.  The fp8 form
    of the reference ({'w': (E, D) e4m3, 'scale_inv': (E, 1)}, model.py:107 with fp8=True) is de-quantised once to
    bf16 as fp8.py:87-89 does (w / scale_inv); the matmul then runs in bf16 on f32 accumulators, where the reference
    also quantises the activations per row (fp8.py:30-45)."""
    if isinstance(w, dict) and "w" in w:
        q, sc = w["w"], w["scale_inv"]
        if q.dim() != 2 or not _per_row_scales(q, sc):
            raise ValueError(f"{name}: expected {{'w': (out, in) e4m3, 'scale_inv': (out, 1)}}, got {tuple(q.shape)} / {tuple(sc.shape)}")

        def deq():
            qq = q if q.dtype == torch.float8_e4m3fn else _codes(q, name).view(torch.float8_e4m3fn)
            return (_dev(qq, None, name).to(torch.float32) / _dev(sc, None, name).to(torch.float32)).to(torch.bfloat16).contiguous()
        return _cached(q, ("router_fp8", id(sc), sc._version), deq)
    if not isinstance(w, torch.Tensor):
        raise TypeError(f"{name}: expected a tensor or an fp8 dict")
    if not w.is_cuda:
        raise RuntimeError(f"{name}: must live on the GPU (this path has no CPU fallback)")
    if w.dim() != 2 or w.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"{name}: expected a 2-D bf16/f32 array (D, E), got {tuple(w.shape)} {w.dtype}")
    return _cached(w, "router", lambda: w.t().to(torch.bfloat16).contiguous())


def router_logits(x, gate_weight, shared_expert_gate_weight=None):
    """moe.py:50 (and :278): logits = bf16(x @ gate_weight) as f32 (M, E); with a shared gate weight (D, 1)
    also returns sigmoid(bf16(x @ w)) rounded to bf16, as f32 (M,)."""
    x = _dev(x, torch.bfloat16, "x")
    wr = _router_weight(gate_weight, "gate_weight")
    E, D = wr.shape
    M = x.shape[0]
    if x.shape[1] != D:
        raise ValueError(f"gate_weight: expected ({x.shape[1]}, E), got a weight for hidden size {D}")
    wsg = None
    if shared_expert_gate_weight is not None:
        wsg = _router_weight(shared_expert_gate_weight, "shared_expert_gate_weight")
        if tuple(wsg.shape) != (1, D):
            raise ValueError(f"shared_expert_gate_weight: expected ({D}, 1), got a weight for {tuple(wsg.shape)[::-1]}")
    logits = _empty((M, E), torch.float32, x)
    gate = _empty((M,), torch.float32, x) if wsg is not None else None
    nbytes = lib().moe_router_workspace_bytes(M, D, E)
    ws = _empty((max(nbytes, 16),), torch.uint8, x)
    check(lib().moe_router_logits(_ptr(x), M, D, _ptr(wr), E, _ptr(wsg), _ptr(logits), _ptr(gate), _ptr(ws), nbytes,
                                  _stream()))
    return logits if gate is None else (logits, gate)


def moe_routing(x, gate_weight, n_experts_per_token):
    """moe.py:37-55: router matmul, f32 softmax, top-k, renormalise.  x (M, D) bf16, gate_weight (D, E)."""
    return route_softmax_topk(router_logits(x, gate_weight), n_experts_per_token)


def moe_experts(x, router_logits, *, top_k, experts, routing="softmax", bias=None, n_group=1, topk_group=1,
                renorm=True, routed_scale=1.0, shared=None, return_debug=False, gate_weight=None,
                shared_expert_gate_weight=None, norm_weight=None, norm_eps=1e-6, add_residual=False):
    """Router logits in, combined hidden states out (one C-ABI call, `moe_forward`).

    x (M, D) bf16; router_logits (M, E) f32; experts / shared: dicts with keys
    'gate_proj', 'up_proj', 'down_proj' holding block-fp8 dicts (or plain arrays).
    With `gate_weight` (D, E) the call computes the logits itself (moe.py:50; pass
    router_logits=None); `shared_expert_gate_weight` (D, 1) then scales the shared
    expert's output by its sigmoid gate (moe.py:278-279).  `norm_weight` (D,) puts the
    block's RMSNorm in front (block.py:54) and `add_residual` its `x + moe_out` behind (:58).
    Returns (M, D) bf16, plus, if return_debug, a dict of the integer intermediates and of the quantised
    SwiGLU output the down GEMMs consumed (`hq` (R, I) e4m3 codes as uint8 and `sh` (R, I/128), sorted order;
    `hsq` (M, SI) and `shs` for the shared expert) and of the down GEMMs' rows (`y` (R, D), `ys` (M, D))."""
    x = _dev(x, torch.bfloat16, "x")
    wr = wsg = None
    if gate_weight is not None:
        if router_logits is not None:
            raise ValueError("pass either router_logits or gate_weight, not both")
        wr = _router_weight(gate_weight, "gate_weight")
        if shared_expert_gate_weight is not None:
            wsg = _router_weight(shared_expert_gate_weight, "shared_expert_gate_weight")
        logits = None
    else:
        if shared_expert_gate_weight is not None:
            raise ValueError("shared_expert_gate_weight needs gate_weight (the router runs inside the call)")
        logits = _dev(router_logits, torch.float32, "router_logits")
    if routing not in ROUTING:
        raise ValueError(f"routing must be one of {sorted(ROUTING)}, got {routing!r}")
    M, D = x.shape
    wg, sg = _expert_weight(experts["gate_proj"], "gate_proj")
    wu, su = _expert_weight(experts["up_proj"], "up_proj")
    wd, sd = _expert_weight(experts["down_proj"], "down_proj")
    E, I, _ = wg.shape
    if logits is not None and tuple(logits.shape) != (M, E):
        raise ValueError(f"router_logits: expected {(M, E)}, got {tuple(logits.shape)}")
    if wr is not None and tuple(wr.shape) != (E, D):
        raise ValueError(f"gate_weight: expected {(D, E)} (or its fp8 form ({E}, {D})), got a weight for {tuple(wr.shape)[::-1]}")
    if wsg is not None and tuple(wsg.shape) != (1, D):
        raise ValueError(f"shared_expert_gate_weight: expected {(D, 1)}, got a weight for {tuple(wsg.shape)[::-1]}")
    if wsg is not None and shared is None:
        raise ValueError("shared_expert_gate_weight needs a shared expert")
    if wg.shape != (E, I, D) or wu.shape != (E, I, D) or wd.shape != (E, D, I):
        raise ValueError(f"expert weight shapes {tuple(wg.shape)} {tuple(wu.shape)} {tuple(wd.shape)} do not fit D={D}")
    a = MoeForwardArgs()
    a.M, a.D, a.E, a.k, a.I = M, D, E, top_k, I
    a.routing, a.n_group, a.topk_group, a.renorm, a.routed_scale = ROUTING[routing], n_group, topk_group, int(renorm), routed_scale
    nw = None
    if norm_weight is not None:
        nw = _dev(norm_weight.to(torch.float32), torch.float32, "norm_weight")
        if tuple(nw.shape) != (D,):
            raise ValueError(f"norm_weight: expected ({D},), got {tuple(nw.shape)}")
        a.norm_weight, a.norm_eps = nw.data_ptr(), float(norm_eps)
    a.add_residual = int(bool(add_residual))
    keep = [x, logits, wg, sg, wu, su, wd, sd, wr, wsg, nw]
    a.x = x.data_ptr()
    if logits is not None:
        a.logits = logits.data_ptr()
    if wr is not None:
        a.w_router = wr.data_ptr()
    if wsg is not None:
        a.w_shared_gate = wsg.data_ptr()
    if bias is not None:
        bias = _dev(bias, torch.float32, "bias")
        keep.append(bias)
        a.bias = bias.data_ptr()
    a.w_gate, a.w_up, a.w_down = wg.data_ptr(), wu.data_ptr(), wd.data_ptr()
    a.sw_gate, a.sw_up, a.sw_down = sg.data_ptr(), su.data_ptr(), sd.data_ptr()
    SI = 0
    if shared is not None:
        swg, ssg = _expert_weight(shared["gate_proj"], "shared gate_proj", dense=True)
        swu, ssu = _expert_weight(shared["up_proj"], "shared up_proj", dense=True)
        swd, ssd = _expert_weight(shared["down_proj"], "shared down_proj", dense=True)
        SI = swg.shape[1]
        if swg.shape != (1, SI, D) or swu.shape != (1, SI, D) or swd.shape != (1, D, SI):
            raise ValueError("shared expert weight shapes do not fit")
        keep += [swg, ssg, swu, ssu, swd, ssd]
        a.ws_gate, a.ws_up, a.ws_down = swg.data_ptr(), swu.data_ptr(), swd.data_ptr()
        a.sws_gate, a.sws_up, a.sws_down = ssg.data_ptr(), ssu.data_ptr(), ssd.data_ptr()
    a.SI = SI
    out = _empty((M, D), torch.bfloat16, x)
    a.out = out.data_ptr()
    dbg = None
    if return_debug:
        R = M * top_k
        dbg = dict(indices=_empty((M, top_k), torch.int32, x), weights=_empty((M, top_k), torch.float32, x),
                   group_sizes=_empty((E,), torch.int32, x), sorted_token_ids=_empty((R,), torch.int32, x),
                   inv_perm=_empty((R,), torch.int32, x),
                   hq=_empty((R, I), torch.uint8, x), sh=_empty((R, I // 128), torch.float32, x))
        a.out_hq, a.out_sh = dbg["hq"].data_ptr(), dbg["sh"].data_ptr()
        dbg["y"] = _empty((R, D), torch.bfloat16, x)
        a.out_y = dbg["y"].data_ptr()
        if SI:
            dbg["hsq"], dbg["shs"] = _empty((M, SI), torch.uint8, x), _empty((M, SI // 128), torch.float32, x)
            a.out_hsq, a.out_shs = dbg["hsq"].data_ptr(), dbg["shs"].data_ptr()
            dbg["ys"] = _empty((M, D), torch.bfloat16, x)
            a.out_ys = dbg["ys"].data_ptr()
        if wr is not None:
            dbg["logits"] = _empty((M, E), torch.float32, x)
            a.out_logits = dbg["logits"].data_ptr()
            if wsg is not None:
                dbg["shared_gate"] = _empty((M,), torch.float32, x)
                a.out_shared_gate = dbg["shared_gate"].data_ptr()
        a.out_idx, a.out_w = dbg["indices"].data_ptr(), dbg["weights"].data_ptr()
        a.out_group_sizes = dbg["group_sizes"].data_ptr()
        a.out_sorted_token_ids, a.out_inv_perm = dbg["sorted_token_ids"].data_ptr(), dbg["inv_perm"].data_ptr()
    nbytes = lib().moe_forward_workspace_bytes(M, D, E, top_k, I, SI)
    ws = _empty((max(nbytes, 16),), torch.uint8, x)
    check(lib().moe_forward(C.byref(a), _ptr(ws), nbytes, _stream()))
    del keep
    return (out, dbg) if return_debug else out


def moe_sublayer(x, moe_norm_weight, params, n_experts_per_token, rms_norm_eps=1e-6):
    """The MoE half of a block, block.py:54-58 and :88-91: x + moe_layer(rms_norm(x, moe_norm), params).
    The norm is fused with the activation quantiser and the residual add with the combine."""
    return moe_layer(x, params, n_experts_per_token, _norm_weight=moe_norm_weight, _norm_eps=rms_norm_eps,
                     _add_residual=True)


def moe_layer(x, params, n_experts_per_token, n_devices=1, axis_name="tp", mesh=None, *, _norm_weight=None,
              _norm_eps=1e-6, _add_residual=False):
    """moe.py:235-282: route + routed experts + gated shared expert, (B, T, D) in and out.

    `params` holds the reference's keys (model.py:79-114): gate_weight (D, E); gate_proj, up_proj,
    down_proj (block-fp8 dicts or plain (E, in, out) arrays); shared_gate_proj, shared_up_proj,
    shared_down_proj (dicts or plain (in, out) arrays); shared_expert_gate_weight (D, 1).
    One GPU only: the expert-parallel branch of the reference (moe.py:263-268) is not part of this build."""
    if n_devices != 1 or mesh is not None:
        raise NotImplementedError("moe_layer: this build runs on one GPU (n_devices=1, mesh=None)")
    if x.dim() != 3:
        raise ValueError(f"x: expected (B, T, D), got {tuple(x.shape)}")
    B, T, D = x.shape
    x_flat = x.reshape(B * T, D)
    if x_flat.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"x: expected bf16 or f32 activations, got {x.dtype}")
    if x_flat.dtype == torch.float32:               # the path computes from bf16 activations
        x_flat = convert(_dev(x_flat, torch.float32, "x"), torch.bfloat16)
    shared = None
    if params.get("shared_gate_proj") is not None:
        shared = dict(gate_proj=params["shared_gate_proj"], up_proj=params["shared_up_proj"],
                      down_proj=params["shared_down_proj"])
    out = moe_experts(x_flat, None, top_k=n_experts_per_token,
                      experts=dict(gate_proj=params["gate_proj"], up_proj=params["up_proj"],
                                   down_proj=params["down_proj"]),
                      routing="softmax", shared=shared, gate_weight=params["gate_weight"],
                      shared_expert_gate_weight=params.get("shared_expert_gate_weight") if shared is not None else None,
                      norm_weight=_norm_weight, norm_eps=_norm_eps, add_residual=_add_residual)
    if x.dtype == torch.float32:                    # moe.py:282: back to the caller's dtype
        out = convert(out, torch.float32)
    return out.reshape(B, T, D)
