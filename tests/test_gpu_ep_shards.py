"""One GPU's statement of what the reference's expert-parallel forward computes
(jax_gpt/models/qwen35/moe.py:117-222, expert_forward_ep): the experts are cut into contiguous
shards, every shard runs the grouped SwiGLU over ITS slice of the globally sorted rows with ITS
local group sizes (moe.py:184-204), rows outside the shard take no part (moe.py:208-210), and the
shards' weighted rows are summed per token (the psum of moe.py:218).

Here the shards run one after the other on the same GPU through the stage entry points of the C
ABI -- no collective, no second GPU.  A row's arithmetic does not depend on which launch or tile
computes it, so every shard's rows must equal the single-launch rows bit for bit, and the sum over
shards must be the single call's output."""
import numpy as np
import pytest

from oracle import moe_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def jg():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    import jax_gpt_amd as jg_
    jg_.lib()
    return jg_


def _slice_experts(ex, lo, hi):
    return {name: {"w": d["w"][lo:hi], "scale_inv": d["scale_inv"][lo:hi]} for name, d in ex.items()}


@pytest.mark.parametrize("M,D,E,k,I,n_shards,routing,kw", [
    (256, 512, 8, 2, 1024, 4, "softmax", {}),                                        # config 1's layer, 4 shards of 2 experts
    (700, 512, 32, 4, 768, 4, "sigmoid_grouped", dict(n_group=4, topk_group=2)),     # some shards far busier than others
    (64, 256, 16, 2, 512, 8, "softmax", {}),                                         # shards that receive no row at all
])
def test_sum_of_expert_shards_equals_single_device(jg, M, D, E, k, I, n_shards, routing, kw):
    import torch
    prob = H.make_problem(M=M, D=D, E=E, k=k, I=I, seed=70 + n_shards + E, routing=routing)
    if n_shards == 8:
        prob["logits"][:, 4:6] -= np.float32(50)     # nobody routes to the experts of shard 2
    ex = H.experts_to_cuda(prob["experts"])
    bias = None if prob["bias"] is None else H.to_cuda(prob["bias"])
    x = H.to_bf16_cuda(prob["x"])
    out, dbg = jg.moe_experts(x, H.to_cuda(prob["logits"]), top_k=k, experts=ex, routing=routing, bias=bias,
                              return_debug=True, **kw)
    oracle = lambda **h: O.moe_experts(prob["x"], prob["logits"], prob["experts"], top_k=k, bias=prob["bias"],
                                       routing=routing, **kw, **h)
    ref = oracle()
    for name in ("indices", "group_sizes", "sorted_token_ids", "inv_perm"):
        assert np.array_equal(dbg[name].cpu().numpy(), ref[name]), name
    H.check_layer_output(out, dbg, ref, oracle)

    # ---- the shards, one after the other (moe.py:175-219)
    R = M * k
    e_local = E // n_shards
    group_sizes_all = dbg["group_sizes"].cpu().numpy()
    group_offsets = np.concatenate([[0], np.cumsum(group_sizes_all)]).astype(np.int64)       # moe.py:168
    sorted_token_ids = dbg["sorted_token_ids"]
    xq, sx = jg.quant_act(x)
    y_all = torch.zeros((R, D), dtype=torch.bfloat16, device="cuda")
    partial = np.zeros((n_shards, M, D), np.float64)
    w_np = dbg["weights"].cpu().numpy()
    stid_np = ref["sorted_token_ids"]
    inv_np = ref["inv_perm"].reshape(M, k)
    seen_empty = False
    for s in range(n_shards):
        lo, hi = s * e_local, (s + 1) * e_local
        sizes_local = group_sizes_all[lo:hi]                                  # moe.py:184-185
        start = int(group_offsets[lo])                                        # moe.py:194
        n_local = int(sizes_local.sum())                                      # moe.py:201
        seen_empty |= n_local == 0
        if n_local == 0:
            continue                                                          # every row masked (moe.py:208-210)
        # the rolled row list (moe.py:196-198), cut at the local count: rows past it are masked and take no part
        row_ids_local = torch.roll(sorted_token_ids, -start)[:n_local].contiguous()
        off_local = H.to_cuda(np.concatenate([[0], np.cumsum(sizes_local)]).astype(np.int32))
        local = _slice_experts(ex, lo, hi)
        hq_l, sh_l = jg.gemm_gateup_swiglu(xq, sx, local["gate_proj"], local["up_proj"], off_local, row_ids=row_ids_local)
        y_l = jg.gemm_down(hq_l, sh_l, local["down_proj"], off_local)
        # a row's arithmetic is independent of the launch that computes it: bit-equal with the single-device rows
        assert torch.equal(hq_l.view(torch.uint8), dbg["hq"][start:start + n_local]), f"shard {s}: h codes differ"
        assert torch.equal(sh_l, dbg["sh"][start:start + n_local]), f"shard {s}: h scales differ"
        assert torch.equal(y_l, dbg["y"][start:start + n_local]), f"shard {s}: rows differ from the single launch"
        y_all[start:start + n_local] = y_l
        # this shard's share of every token (moe.py:212-215), in float64 on the host
        yl = H.bf16_to_np(y_l).astype(np.float64)
        for t, s_ in zip(*np.nonzero((inv_np >= start) & (inv_np < start + n_local))):
            assert stid_np[inv_np[t, s_]] == t
            partial[s, t] += yl[inv_np[t, s_] - start] * np.float64(w_np[t, s_])
    if n_shards == 8:
        assert seen_empty, "this case is meant to hold a shard without rows"
    torch.cuda.synchronize()
    # the sum over shards (moe.py:218), rounded once, is the single-device output: exactly so through the oracle's
    # combine of the shards' rows (f32 sum in slot order), and to the rounding of the last f32 bit when the shards'
    # own partial sums are added shard by shard instead
    got = H.bf16_to_np(out)
    assert np.array_equal(got, O.combine(H.bf16_to_np(y_all), w_np, ref["inv_perm"]))
    psum = O.bf16_round(partial.sum(axis=0).astype(np.float32))
    differ = got != psum
    assert differ.mean() < 1e-3 and np.all(np.abs(got - psum)[differ] <= 2.0 ** -7 * np.abs(psum)[differ] + 1e-30)
    # and the device's own combine over the shards' rows gives the same bits as the single call
    assert torch.equal(jg.combine(y_all, dbg["weights"], dbg["inv_perm"]), out)
