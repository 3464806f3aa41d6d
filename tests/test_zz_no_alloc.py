"""moe_gemm_gateup_swiglu_fp8_static: the gate/up grouped GEMM whose tile list lives in the library's static
device array instead of a caller workspace.  Called through the C ABI twice in a row, the second time on a
smaller problem (the array keeps the first call's tile list), and compared bit for bit with the workspace entry
point, and with the oracle to the stage test's bound."""
import ctypes as C

import numpy as np
import pytest

from oracle import moe_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _case(seed, E, D, I, sizes):
    rng = H.rng_for(seed)
    off = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    R = int(off[-1])
    x = O.bf16_round(rng.standard_normal((R, D), dtype=np.float32))
    xq, sx = O.quant_act_group(x)
    mk = lambda n, kk: O.quant_weight_block(rng.standard_normal((E, n, kk), dtype=np.float32) * np.float32(0.03))
    return off, xq, sx, dict(gate=mk(I, D), up=mk(I, D))


def _run_both(lib, torch, off, xq, sx, ex):
    E, I, D = ex["gate"][0].shape
    R = int(off[-1])
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    d_off, d_xq, d_sx = dev(off), dev(xq), dev(sx)
    wg, sg, wu, su = dev(ex["gate"][0]), dev(ex["gate"][1]), dev(ex["up"][0]), dev(ex["up"][1])
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ptr = lambda t: C.c_void_p(t.data_ptr())
    outs = []
    for static in (False, True):
        hq = torch.full((R, I), 0x7F, dtype=torch.uint8, device="cuda")
        sh = torch.full((R, I // 128), -1.0, dtype=torch.float32, device="cuda")
        if static:
            rc = lib.moe_gemm_gateup_swiglu_fp8_static(ptr(d_xq), ptr(d_sx), None, ptr(wg), ptr(sg), ptr(wu), ptr(su),
                                                       ptr(d_off), E, R, D, I, ptr(hq), ptr(sh), stream)
        else:
            n = lib.moe_gemm_workspace_bytes(R, E, I)
            ws = torch.empty((n,), dtype=torch.uint8, device="cuda")
            rc = lib.moe_gemm_gateup_swiglu_fp8(ptr(d_xq), ptr(d_sx), None, ptr(wg), ptr(sg), ptr(wu), ptr(su),
                                                ptr(d_off), E, R, D, I, ptr(hq), ptr(sh), ptr(ws), n, stream)
        assert rc == 0, lib.moe_last_error().decode()
        torch.cuda.synchronize()
        outs.append((hq.cpu().numpy(), sh.cpu().numpy()))
    return outs


def test_static_scratch_gateup_matches_workspace_entry_point(lib):
    import torch
    assert torch.cuda.is_available()
    torch.cuda.set_device(0)
    # first a larger problem (several tiles per expert, an empty expert), then a smaller one
    for seed, E, D, I, sizes in [(4100, 6, 512, 256, [300, 0, 129, 7, 64, 530]), (4101, 3, 256, 128, [40, 0, 9])]:
        print("static gate/up", E, D, I, sizes, flush=True)
        off, xq, sx, ex = _case(seed, E, D, I, sizes)
        (hq_ws, sh_ws), (hq_st, sh_st) = _run_both(lib, torch, off, xq, sx, ex)
        assert np.array_equal(hq_ws, hq_st), "codes differ between the workspace and the static entry point"
        assert np.array_equal(sh_ws, sh_st), "scales differ between the workspace and the static entry point"
        # and both are the oracle's h to the stage test's bound
        g = O.grouped_gemm(xq, sx, *ex["gate"], off)
        u = O.grouped_gemm(xq, sx, *ex["up"], off)
        rhq, rsh = O.quant_act_group((O.silu(g) * u).astype(np.float32))
        assert np.allclose(sh_st, rsh, rtol=1e-3)
        assert np.mean(hq_st != rhq) < 5e-3
        got, want = O.dequant_act_group(hq_st, sh_st), O.dequant_act_group(rhq, rsh)
        assert np.all(np.abs(got - want) <= 0.13 * np.abs(want) + 0.1 * np.repeat(rsh, 128, axis=1))


def test_static_scratch_rejects_what_does_not_fit(lib):
    one = C.c_void_p(256)
    # 64 Mi rows in 32-row tiles: a tile list far beyond the static array; refused on the host, before any launch
    rc = lib.moe_gemm_gateup_swiglu_fp8_static(one, one, None, one, one, one, one, one, 1024, 1 << 26, 128, 128, one, one, None)
    assert rc == -3, lib.moe_last_error().decode()
    assert "static scratch" in lib.moe_last_error().decode()


def _static_call(lib, torch, bufs, hq, sh):
    d_off, d_xq, d_sx, wg, sg, wu, su, E, R, D, I = bufs
    ptr = lambda t: C.c_void_p(t.data_ptr())
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.moe_gemm_gateup_swiglu_fp8_static(ptr(d_xq), ptr(d_sx), None, ptr(wg), ptr(sg), ptr(wu), ptr(su),
                                               ptr(d_off), E, R, D, I, ptr(hq), ptr(sh), stream)
    assert rc == 0, lib.moe_last_error().decode()


def test_static_scratch_call_allocates_nothing_and_replays_from_a_graph(lib):
    """What the entry point exists for: a call takes no device memory (free memory before = after, read from the
    driver), and it can be captured in a HIP graph and replayed -- every replay, with eager calls in between, gives
    the eager result bit for bit."""
    import torch
    torch.cuda.set_device(0)
    off, xq, sx, ex = _case(4102, 5, 384, 256, [70, 0, 300, 1, 33])
    E, I, D = ex["gate"][0].shape
    R = int(off[-1])
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    bufs = (dev(off), dev(xq), dev(sx), dev(ex["gate"][0]), dev(ex["gate"][1]), dev(ex["up"][0]), dev(ex["up"][1]), E, R, D, I)
    hq = torch.full((R, I), 0x7F, dtype=torch.uint8, device="cuda")
    sh = torch.full((R, I // 128), -1.0, dtype=torch.float32, device="cuda")
    _static_call(lib, torch, bufs, hq, sh)               # (first call on the device: looks up the array's address)
    torch.cuda.synchronize()
    eager = (hq.clone(), sh.clone())
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        _static_call(lib, torch, bufs, hq, sh)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, f"device memory changed across the calls: {free_before} -> {free_after}"
    assert torch.equal(hq, eager[0]) and torch.equal(sh, eager[1])

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _static_call(lib, torch, bufs, hq, sh)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _static_call(lib, torch, bufs, hq, sh)
    for i in range(3):
        print("   static replay", i, flush=True)
        hq.fill_(0x7F)
        sh.fill_(-1.0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(hq, eager[0]) and torch.equal(sh, eager[1]), f"replay {i} differs from the eager call"
        hq2, sh2 = torch.empty_like(hq), torch.empty_like(sh)     # eager work between the replays
        _static_call(lib, torch, bufs, hq2, sh2)
        torch.cuda.synchronize()
        assert torch.equal(hq2, eager[0]) and torch.equal(sh2, eager[1])
