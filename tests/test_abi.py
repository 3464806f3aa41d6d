"""The C-ABI library loads, exports every symbol include/moe_hip.h declares, and rejects
bad arguments on the host before any launch (no GPU needed: no compute call is made)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def dll():
    import jax_gpt_amd
    from jax_gpt_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    return jax_gpt_amd.lib()


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "moe_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(moe_[a-z0-9_]+)\s*\(", text)))


def test_header_and_library_agree(dll):
    from jax_gpt_amd import _lib
    declared = _declared_functions()
    assert len(declared) >= 14
    for name in declared:
        assert hasattr(dll, name), f"{name} is declared in moe_hip.h but not exported"
    assert sorted(_lib.SIGNATURES) == declared
    assert dll.moe_abi_version() == 6


def test_library_exports_exactly_the_header(dll):
    """Built with hidden visibility: the dynamic symbol table holds the header's functions and no internal ones."""
    import subprocess
    from jax_gpt_amd import _lib
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], check=True, capture_output=True, text=True).stdout
    exported = sorted(ln.split()[-1] for ln in out.splitlines() if ln.split()[-2:-1] == ["T"])
    assert exported == _declared_functions(), set(exported) ^ set(_declared_functions())


def test_router_workspace_covers_both_column_counts(dll):
    """moe_router_workspace_bytes must cover the launch with and without the shared expert's gate column: when E
    is a multiple of 128 the gate-less launch has one column tile fewer and may split K more deeply.  The library
    checks the bytes a launch will write against ws_bytes on the host, before any GPU call: with the advertised
    size no shape may come back as MOE_ERR_WORKSPACE_TOO_SMALL (-3); without a GPU the call then ends with
    MOE_ERR_HIP (-4), with one it would launch, so this runs only where no GPU is present."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("host-side sizing check; runs on the CPU-only host")
    one = C.c_void_p(256)
    for E in (8, 128, 256, 384, 512, 1024):
        for D in (128, 1024, 2048, 4096, 7168):
            for M in (1, 64, 512, 2048, 4096, 8192):
                need = dll.moe_router_workspace_bytes(M, D, E)
                for gate in (None, one):
                    rc = dll.moe_router_logits(one, M, D, one, E, gate, one, gate, one, need, None)
                    assert rc != -3, (E, D, M, gate is not None, dll.moe_last_error())
    # and a buffer sized for the smaller of the two cases is refused for the larger one (E=128, D=2048, M=4096)
    assert dll.moe_router_logits(one, 4096, 2048, one, 128, None, one, None, one, 17_000_000, None) == -3


def test_forward_args_struct_matches_header(dll):
    from jax_gpt_amd._lib import MoeForwardArgs
    text = open(os.path.join(ROOT, "include", "moe_hip.h")).read()
    body = re.search(r"typedef struct MoeForwardArgs \{(.*?)\} MoeForwardArgs;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        for part in decl.split(","):
            names.append(re.findall(r"[A-Za-z_][A-Za-z0-9_]*", part)[-1])
    assert names == [f[0] for f in MoeForwardArgs._fields_]


def test_argument_errors_come_back_as_codes(dll):
    err = lambda: dll.moe_last_error().decode()
    one = C.c_void_p(16)                       # never dereferenced: validation fails first
    assert dll.moe_route_softmax_topk(None, 4, 8, 2, 1, one, one, None) == -5
    assert "null" in err()
    assert dll.moe_route_softmax_topk(one, 4, 2000, 2, 1, one, one, None) == -1
    assert dll.moe_route_softmax_topk(one, 4, 8, 9, 1, one, one, None) == -1
    assert dll.moe_route_sigmoid_grouped(one, None, 4, 30, 4, 2, 2, 1, 1.0, one, one, None) == -1   # 4 does not divide 30
    assert dll.moe_route_sigmoid_grouped(one, None, 4, 32, 4, 1, 9, 1, 1.0, one, one, None) == -1   # k > kept experts
    assert dll.moe_quant_act(one, 4, 100, one, one, None) == -1
    assert "128" in err()
    assert dll.moe_quant_act(C.c_void_p(8), 4, 128, one, one, None) == -2                          # misaligned
    assert dll.moe_permute(one, 4, 2, 8, one, one, one, one, one, one, 0, None) == -3              # workspace too small
    assert dll.moe_gemm_gateup_swiglu_fp8(one, one, None, one, one, one, one, one, 4, 16, 100, 128, one, one, one, 1 << 20, None) == -1
    assert dll.moe_gemm_down_fp8(one, one, one, one, one, 4, 16, 128, 128, one, one, 0, None) == -3
    assert dll.moe_combine(one, one, one, None, None, None, 4, 40, 128, one, None) == -1
    assert dll.moe_combine(one, one, one, None, one, None, 4, 2, 128, one, None) == -5             # gate without shared rows
    assert dll.moe_rmsnorm_quant(one, one, 1e-6, 4, 16384, None, one, one, None) == -1              # D > 8192
    assert dll.moe_router_logits(one, 4, 100, one, 8, None, one, None, one, 1 << 20, None) == -1   # D % 128
    assert dll.moe_router_logits(one, 4, 128, one, 8, one, one, None, one, 1 << 20, None) == -5    # gate weight without output
    assert dll.moe_router_logits(one, 4, 128, one, 8, None, one, None, one, 0, None) == -3
    assert dll.moe_forward(None, one, 0, None) == -5


def test_workspace_sizes_are_monotone(dll):
    a = dll.moe_forward_workspace_bytes(64, 7168, 256, 8, 2048, 2048)
    b = dll.moe_forward_workspace_bytes(8192, 7168, 256, 8, 2048, 2048)
    assert 0 < a < b < 4 << 30
    assert dll.moe_forward_workspace_bytes(0, 7168, 256, 8, 2048, 2048) > 0          # an empty batch sizes a workspace too
    assert dll.moe_router_workspace_bytes(0, 7168, 256) >= 0
    assert dll.moe_router_workspace_bytes(8192, 7168, 256) >= 8192 * 257 * 4
    assert dll.moe_permute_workspace_bytes(8192, 8, 256) >= 32 * 256 * 4
    assert dll.moe_gemm_workspace_bytes(65536, 256, 7168) > dll.moe_gemm_workspace_bytes(512, 256, 7168) > 0


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "jax-gpt_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cc")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src.replace("no CPU fallback", ""), f"{f} mentions the oracle"


def test_host_wrappers_refuse_cpu_tensors(dll):
    import torch
    import jax_gpt_amd as jg
    with pytest.raises(RuntimeError, match="GPU"):
        jg.route_softmax_topk(torch.zeros(4, 8), 2)
    with pytest.raises(RuntimeError, match="GPU"):
        jg.quant_act(torch.zeros(4, 128, dtype=torch.bfloat16))


def test_probe_library_is_separate_and_loads(dll):
    """The K-loop timing probe is a library of its own: it loads, exports its three entry points and nothing of
    the product's, and the product library does not depend on it (no compute call is made here)."""
    import subprocess
    path = os.path.join(ROOT, "jax-gpt_amd", "libmoe_probe.so")
    assert os.path.exists(path), "libmoe_probe.so is not built (python jax-gpt_amd/build.py)"
    probe = C.CDLL(path)
    probe.moe_probe_variant_name.restype = C.c_char_p
    n = probe.moe_probe_variants()
    assert n >= 5 and all(probe.moe_probe_variant_name(v) for v in range(n))
    out = subprocess.run(["nm", "-D", "--defined-only", path], check=True, capture_output=True, text=True).stdout
    exported = sorted(ln.split()[-1] for ln in out.splitlines() if ln.split()[-2:-1] == ["T"])
    assert exported == ["moe_probe_gemm_loop", "moe_probe_variant_name", "moe_probe_variants"]
    from jax_gpt_amd import _lib
    needed = subprocess.run(["readelf", "-d", _lib.LIB_PATH], check=True, capture_output=True, text=True).stdout
    assert "moe_probe" not in needed
