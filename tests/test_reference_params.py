"""The reference's own fp8 parameter dicts drop into moe_layer: parameters laid out exactly as
jax_gpt/models/qwen35/model.py:79-114 builds them with fp8=True (every weight {'w': (.., out, in) e4m3fn,
'scale_inv': (.., out, 1) f32}, router and shared gate included), at the MoE dimensions of the reference's presets
(config.py:42-47 and :52-135).  The oracle reads the same dicts the way the reference's consumers do (experts:
w * scale_inv, moe.py:29; dense layers and router: w / scale_inv, fp8.py:87-89), quantises per 128x128 block and
runs the path; routing is exact as a function of the kernel's logits."""
import numpy as np
import pytest

from oracle import moe_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


def _fp8(t):
    import torch
    return t.to(torch.float8_e4m3fn)


def _reference_fp8_params(D, E, I, SI, seed, unit_scales=True):
    """model.py:24-35 (_init_linear, fp8=True) and :88-97 (_init_expert_fp8): N(0, 0.02) in bf16, cast to e4m3fn,
    scale_inv = 1.  With unit_scales=False the weights are quantised per row as quantize.py:31-42 does instead
    (scale = amax / 448, scale_inv = 1 / scale)."""
    import torch
    g = torch.Generator().manual_seed(seed)

    def make(*shape):
        w = (torch.randn(*shape, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16)
        if unit_scales:
            return {"w": _fp8(w), "scale_inv": torch.ones(*shape[:-1], 1, dtype=torch.float32)}
        wf = w.float()
        scale = (wf.abs().amax(dim=-1, keepdim=True) / 448.0).clamp_min(torch.finfo(torch.float32).tiny)
        return {"w": _fp8(wf / scale), "scale_inv": (1.0 / scale).float()}

    return {
        "gate_weight": make(E, D),
        "gate_proj": make(E, I, D), "up_proj": make(E, I, D), "down_proj": make(E, D, I),
        "shared_gate_proj": make(SI, D), "shared_up_proj": make(SI, D), "shared_down_proj": make(D, SI),
        "shared_expert_gate_weight": make(1, D),
    }


def _to_cuda(params):
    return {k: {n: t.cuda() for n, t in v.items()} for k, v in params.items()}


def _oracle_view(params):
    """What the reference's consumers make of the dicts, re-quantised per block for the oracle."""
    deq_dense = lambda d: (d["w"].float() / d["scale_inv"]).numpy()          # fp8.py:87-89
    deq_expert = lambda d: (d["w"].float() * d["scale_inv"]).numpy()         # moe.py:29
    experts = {n: O.quant_weight_block(deq_expert(params[n + "_proj"])) for n in ("gate", "up", "down")}
    shared = {n: O.quant_weight_block(deq_dense(params["shared_" + n + "_proj"])[None]) for n in ("gate", "up", "down")}
    wr = O.bf16_round(deq_dense(params["gate_weight"])).T                    # (D, E) as the reference's x @ w
    wg = O.bf16_round(deq_dense(params["shared_expert_gate_weight"])).T      # (D, 1)
    return experts, shared, wr, wg


def _layer_and_debug(jg, x3, dparams, k):
    import torch
    B, T, D = x3.shape
    out = jg.moe_layer(x3, dparams, k)
    assert out.shape == x3.shape and out.dtype == x3.dtype
    out2, dbg = jg.moe_experts(x3.reshape(B * T, D), None, top_k=k,
                               experts={n: dparams[n] for n in ("gate_proj", "up_proj", "down_proj")},
                               shared={n: dparams["shared_" + n] for n in ("gate_proj", "up_proj", "down_proj")},
                               gate_weight=dparams["gate_weight"],
                               shared_expert_gate_weight=dparams["shared_expert_gate_weight"], return_debug=True)
    assert torch.equal(out.reshape(B * T, D), out2)
    return out2, dbg


@pytest.mark.parametrize("unit_scales", [True, False])
def test_mini_preset_reference_fp8_params_in_full(unit_scales):
    """Qwen35Config.mini MoE dimensions (config.py:52-80: hidden 1024, 32 experts top-2, intermediate 512, shared
    512), every row checked against the oracle."""
    import torch
    import jax_gpt_amd as jg
    D, E, k, I, SI, B, T = 1024, 32, 2, 512, 512, 2, 64
    _say("reference fp8 params, mini preset, unit scales:", unit_scales)
    params = _reference_fp8_params(D, E, I, SI, seed=60 + int(unit_scales), unit_scales=unit_scales)
    rng = H.rng_for(61)
    x = O.bf16_round(rng.standard_normal((B * T, D), dtype=np.float32))
    out, dbg = _layer_and_debug(jg, H.to_bf16_cuda(x).reshape(B, T, D), _to_cuda(params), k)
    experts, shared, wr, wg = _oracle_view(params)
    logits = dbg["logits"].cpu().numpy()
    want_l = O.router_logits(x, wr)
    assert float((logits != want_l).mean()) < 0.01 and np.abs(logits - want_l).max() <= 2.0 ** -5
    gate_k = H.kernel_gate(dbg, O.shared_gate(x, wg))
    oracle = lambda **h: O.moe_experts(x, logits, experts, top_k=k, shared=shared, shared_gate_values=gate_k, **h)
    ref = oracle()
    for name in ("indices", "group_sizes", "sorted_token_ids", "inv_perm"):
        assert np.array_equal(dbg[name].cpu().numpy(), ref[name]), name
    assert np.allclose(dbg["weights"].cpu().numpy().sum(-1), 1.0, atol=1e-5)          # tests/qwen35/test_moe.py:52-60
    err, loose, frac = H.check_layer_output(out, dbg, ref, oracle, shared_gate=gate_k)
    _say(f"   max-normalised error {err:.2e} ({frac:.2%} of h codes differ; end to end {loose:.2e})")


def test_derived_weight_copies_are_dropped_with_their_source():
    import gc
    import torch
    import jax_gpt_amd as jg
    from jax_gpt_amd import moe as M_
    w = torch.randn(2, 128, 256, device="cuda") * 0.02                     # plain (E, in, out)
    base = len(M_._derived)
    a = M_._expert_weight(w, "w")
    assert len(M_._derived) == base + 1 and M_._expert_weight(w, "w")[0] is a[0]      # cached
    w.mul_(2.0)                                                            # modified in place: quantised again
    b = M_._expert_weight(w, "w")
    assert b[0] is not a[0] and len(M_._derived) == base + 1
    del w
    gc.collect()
    assert len(M_._derived) == base                                        # the GPU copies went with the source tensor


def test_full_preset_reference_fp8_params_sampled_rows():
    """The full preset's MoE dimensions (config.py:42-47, :133-135: hidden 4096, 512 experts top-10, intermediate
    1024, shared 1024) on 2048 tokens: every integer result exact, 32 sampled token rows against the oracle."""
    import torch
    import jax_gpt_amd as jg
    from tests.test_gpu_full_size import _check_sampled_rows
    D, E, k, I, SI, B, T = 4096, 512, 10, 1024, 1024, 1, 2048
    _say("reference fp8 params, full preset")
    params = _reference_fp8_params(D, E, I, SI, seed=70)
    dparams = _to_cuda(params)
    gen = torch.Generator(device="cuda"); gen.manual_seed(71)
    x = torch.randn((B * T, D), dtype=torch.float32, device="cuda", generator=gen).to(torch.bfloat16)
    out, dbg = _layer_and_debug(jg, x.reshape(B, T, D), dparams, k)
    torch.cuda.synchronize()
    outn = H.bf16_to_np(out)
    assert np.isfinite(outn).all()
    logits = dbg["logits"].cpu().numpy()
    ridx, rw = O.route_softmax_topk(logits, k)
    assert np.array_equal(dbg["indices"].cpu().numpy(), ridx)
    assert np.allclose(dbg["weights"].cpu().numpy(), rw, rtol=2e-6, atol=1e-9)
    sg = O.sort_and_group(ridx, E)
    for name in ("group_sizes", "sorted_token_ids", "inv_perm"):
        assert np.array_equal(dbg[name].cpu().numpy(), sg[name]), name
    rng = H.rng_for(72)
    tokens = sorted(set([0, B * T - 1] + list(rng.integers(0, B * T, 30))))
    tsel = torch.tensor(tokens, device="cuda")
    xs = H.bf16_to_np(x[tsel])
    # logits and gate of the sampled tokens against the oracle's reading of the fp8 router weights
    wr = O.bf16_round((params["gate_weight"]["w"].float() / params["gate_weight"]["scale_inv"]).numpy()).T
    wg = O.bf16_round((params["shared_expert_gate_weight"]["w"].float() / params["shared_expert_gate_weight"]["scale_inv"]).numpy()).T
    want_l = O.router_logits(xs, wr)
    assert float((logits[tokens] != want_l).mean()) < 0.02 and np.abs(logits[tokens] - want_l).max() <= 2.0 ** -5
    og, kg = O.shared_gate(xs, wg), dbg["shared_gate"].cpu().numpy()[tokens]
    assert np.abs(kg - og).max() <= 2.0 ** -7 and int((kg != og).sum()) <= 2
    gate = np.zeros(max(tokens) + 1, np.float32); gate[tokens] = kg
    # the product's block-fp8 copies of the experts are what the kernels computed with: the oracle reads those
    from jax_gpt_amd import moe as M_
    blk = lambda d, dense=False: dict(zip(("w", "scale_inv"), M_._expert_weight(d, "w", dense=dense)))
    experts = {n + "_proj": blk(dparams[n + "_proj"]) for n in ("gate", "up", "down")}
    shared = {n + "_proj": blk(dparams["shared_" + n + "_proj"], True) for n in ("gate", "up", "down")}
    # ... after checking two experts' copies against the oracle's own re-quantisation of the reference dicts
    for e in (0, E - 1):
        for n in ("gate", "up", "down"):
            d = params[n + "_proj"]
            q_ref, s_ref = O.quant_weight_block((d["w"][e].float() * d["scale_inv"][e]).numpy()[None])
            assert np.array_equal(experts[n + "_proj"]["w"][e].cpu().numpy(), q_ref[0])
            assert np.array_equal(experts[n + "_proj"]["scale_inv"][e].cpu().numpy(), s_ref[0])
    _check_sampled_rows(outn, xs, tokens, ridx, rw, experts, shared, dbg, k, shared_gate_values=gate)
