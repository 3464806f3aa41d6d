"""Checkpoint ingest (weight_loader.py:42-63 and the DeepSeek-V3 block-fp8 layout) -> `moe_layer` parameters."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests import helpers as H


def _qwen35_sd(E, D, I, SI, seed, prefix="model.layers.3"):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s, sc=0.05: (torch.randn(*s, generator=g) * sc).to(torch.bfloat16)
    return {
        f"{prefix}.mlp.gate.weight": r(E, D, sc=0.2),
        f"{prefix}.mlp.experts.gate_up_proj": r(E, 2 * I, D),
        f"{prefix}.mlp.experts.down_proj": r(E, D, I),
        f"{prefix}.mlp.shared_expert.gate_proj.weight": r(SI, D),
        f"{prefix}.mlp.shared_expert.up_proj.weight": r(SI, D),
        f"{prefix}.mlp.shared_expert.down_proj.weight": r(D, SI),
        f"{prefix}.mlp.shared_expert_gate.weight": r(1, D, sc=0.2),
    }


def test_qwen35_layouts_on_cpu(tmp_path):
    """Unquantised ingest reproduces the reference loader's layouts (weight_loader.py:42-63): (in, out) arrays,
    gate_up split at I.  Goes through a safetensors file, as a real checkpoint does."""
    from safetensors.torch import load_file, save_file
    import jax_gpt_amd.checkpoint as ck
    E, D, I, SI = 4, 256, 128, 128
    sd0 = _qwen35_sd(E, D, I, SI, 1)
    save_file(sd0, str(tmp_path / "layer.safetensors"))
    sd = load_file(str(tmp_path / "layer.safetensors"))
    p = ck.moe_params_from_qwen35_state_dict(sd, "model.layers.3", I, device="cpu", quantize=False)
    gu = sd0["model.layers.3.mlp.experts.gate_up_proj"]
    assert torch.equal(p["gate_proj"], gu[:, :I, :].transpose(1, 2)) and p["gate_proj"].shape == (E, D, I)
    assert torch.equal(p["up_proj"], gu[:, I:, :].transpose(1, 2))
    assert torch.equal(p["down_proj"], sd0["model.layers.3.mlp.experts.down_proj"].transpose(1, 2))
    assert p["gate_weight"].shape == (D, E) and torch.equal(p["gate_weight"], sd0["model.layers.3.mlp.gate.weight"].t())
    assert p["shared_gate_proj"].shape == (D, SI) and p["shared_down_proj"].shape == (SI, D)
    assert p["shared_expert_gate_weight"].shape == (D, 1)
    with pytest.raises(KeyError, match="down_proj"):
        bad = dict(sd); del bad["model.layers.3.mlp.experts.down_proj"]
        ck.moe_params_from_qwen35_state_dict(bad, "model.layers.3", I, device="cpu", quantize=False)
    with pytest.raises(ValueError, match="gate_up_proj"):
        ck.moe_params_from_qwen35_state_dict(sd, "model.layers.3", I + 128, device="cpu", quantize=False)


def _block_fp8_sd(prob, prefix="model.layers.5"):
    """Oracle-format experts (codes, scale_inv) -> per-expert HF tensors."""
    sd = {}
    E = prob["experts"]["gate"][0].shape[0]
    for name, (q, s) in prob["experts"].items():
        for e in range(E):
            sd[f"{prefix}.mlp.experts.{e}.{name}_proj.weight"] = torch.from_numpy(q[e].copy()).view(torch.float8_e4m3fn)
            sd[f"{prefix}.mlp.experts.{e}.{name}_proj.weight_scale_inv"] = torch.from_numpy(s[e].copy())
    if prob["shared"]:
        for name, (q, s) in prob["shared"].items():
            sd[f"{prefix}.mlp.shared_experts.{name}_proj.weight"] = torch.from_numpy(q[0].copy()).view(torch.float8_e4m3fn)
            sd[f"{prefix}.mlp.shared_experts.{name}_proj.weight_scale_inv"] = torch.from_numpy(s[0].copy())
    return sd, E


def test_block_fp8_stacking_on_cpu():
    import jax_gpt_amd.checkpoint as ck
    prob = H.make_problem(M=8, D=256, E=4, k=2, I=128, SI=128, seed=31, routing="sigmoid_grouped")
    sd, E = _block_fp8_sd(prob)
    sd["model.layers.5.mlp.gate.weight"] = torch.zeros(E, 256, dtype=torch.bfloat16)
    sd["model.layers.5.mlp.gate.e_score_correction_bias"] = torch.arange(E, dtype=torch.float32)
    p = ck.moe_params_from_block_fp8_state_dict(sd, "model.layers.5", E, device="cpu")
    for name in ("gate", "up", "down"):
        q, s = prob["experts"][name]
        assert np.array_equal(p["experts"][name + "_proj"]["w"].view(torch.uint8).numpy(), q)
        assert np.array_equal(p["experts"][name + "_proj"]["scale_inv"].numpy(), s)
        assert p["shared"][name + "_proj"]["w"].shape[0] == 1
    assert p["gate_weight"].shape == (256, E) and torch.equal(p["bias"], torch.arange(E, dtype=torch.float32))
    bad = dict(sd)
    bad["model.layers.5.mlp.experts.0.up_proj.weight_scale_inv"] = torch.zeros(3, 3)
    with pytest.raises(ValueError, match="scales"):
        ck.moe_params_from_block_fp8_state_dict(bad, "model.layers.5", E, device="cpu")


@pytest.mark.gpu
def test_qwen35_ingest_runs_the_layer():
    """Quantised ingest straight from the (out, in) checkpoint layout == quantising the reference-layout arrays."""
    import jax_gpt_amd as jg
    import jax_gpt_amd.checkpoint as ck
    assert torch.cuda.is_available()
    E, D, I, SI, k = 8, 256, 128, 128, 2
    sd = _qwen35_sd(E, D, I, SI, 2)
    pq = ck.moe_params_from_qwen35_state_dict(sd, "model.layers.3", I, device="cuda", quantize=True)
    pp = ck.moe_params_from_qwen35_state_dict(sd, "model.layers.3", I, device="cuda", quantize=False)
    x = (torch.randn(2, 40, D, generator=torch.Generator().manual_seed(3))).to(torch.bfloat16).cuda()
    a, b = jg.moe_layer(x, pq, k), jg.moe_layer(x, pp, k)
    assert torch.equal(a, b) and torch.isfinite(a.float()).all()
    # and against the oracle from the checkpoint tensors themselves
    gu = sd["model.layers.3.mlp.experts.gate_up_proj"].float().numpy()
    experts = dict(gate=O.quant_weight_block(gu[:, :I, :]), up=O.quant_weight_block(gu[:, I:, :]),
                   down=O.quant_weight_block(sd["model.layers.3.mlp.experts.down_proj"].float().numpy()))
    shared = {n: O.quant_weight_block(sd[f"model.layers.3.mlp.shared_expert.{n}_proj.weight"].float().numpy()[None])
              for n in ("gate", "up", "down")}
    xn = x.reshape(-1, D).float().cpu().numpy()
    wr = sd["model.layers.3.mlp.gate.weight"].float().numpy().T
    wg = sd["model.layers.3.mlp.shared_expert_gate.weight"].float().numpy().T
    a2, dbg = jg.moe_experts(x.reshape(-1, D), None, top_k=k,
                             experts={n: pq[n] for n in ("gate_proj", "up_proj", "down_proj")},
                             shared={n: pq["shared_" + n] for n in ("gate_proj", "up_proj", "down_proj")},
                             gate_weight=pq["gate_weight"], shared_expert_gate_weight=pq["shared_expert_gate_weight"],
                             return_debug=True)
    assert torch.equal(a2, a.reshape(-1, D))
    logits = dbg["logits"].cpu().numpy()
    assert float((logits != O.router_logits(xn, wr)).mean()) < 0.01
    gate_k = H.kernel_gate(dbg, O.shared_gate(xn, wg))
    oracle = lambda **h: O.moe_experts(xn, logits, experts, top_k=k, shared=shared, shared_gate_values=gate_k, **h)
    H.check_layer_output(a2, dbg, oracle(), oracle, shared_gate=gate_k)


@pytest.mark.gpu
def test_block_fp8_ingest_runs_the_layer():
    import jax_gpt_amd as jg
    import jax_gpt_amd.checkpoint as ck
    prob = H.make_problem(M=64, D=256, E=8, k=2, I=128, SI=128, seed=32, routing="sigmoid_grouped")
    sd, E = _block_fp8_sd(prob)
    rng = H.rng_for(33)
    wr = O.bf16_round(rng.standard_normal((E, 256), dtype=np.float32) * 0.2)
    sd["model.layers.5.mlp.gate.weight"] = torch.from_numpy(wr).to(torch.bfloat16)
    sd["model.layers.5.mlp.gate.e_score_correction_bias"] = torch.from_numpy(prob["bias"])
    p = ck.moe_params_from_block_fp8_state_dict(sd, "model.layers.5", E, device="cuda")
    x = H.to_bf16_cuda(prob["x"])
    out, dbg = jg.moe_experts(x, None, top_k=2, experts=p["experts"], shared=p["shared"], routing="sigmoid_grouped",
                              bias=p["bias"], n_group=4, topk_group=2, gate_weight=p["gate_weight"], return_debug=True)
    direct = jg.moe_experts(x, dbg["logits"], top_k=2, experts=H.experts_to_cuda(prob["experts"]),
                            shared=H.experts_to_cuda(prob["shared"]), routing="sigmoid_grouped", bias=H.to_cuda(prob["bias"]),
                            n_group=4, topk_group=2)
    assert torch.equal(out, direct)
    oracle = lambda **h: O.moe_experts(prob["x"], dbg["logits"].cpu().numpy(), prob["experts"], top_k=2, shared=prob["shared"],
                                       routing="sigmoid_grouped", bias=prob["bias"], n_group=4, topk_group=2, **h)
    ref = oracle()
    assert np.array_equal(dbg["indices"].cpu().numpy(), ref["indices"])
    H.check_layer_output(out, dbg, ref, oracle)


def _qwen3_moe_sd(E, D, I, seed, prefix="model.layers.1"):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s, sc=0.05: (torch.randn(*s, generator=g) * sc).to(torch.bfloat16)
    sd = {f"{prefix}.mlp.gate.weight": r(E, D, sc=0.2)}
    for e in range(E):
        sd[f"{prefix}.mlp.experts.{e}.gate_proj.weight"] = r(I, D)
        sd[f"{prefix}.mlp.experts.{e}.up_proj.weight"] = r(I, D)
        sd[f"{prefix}.mlp.experts.{e}.down_proj.weight"] = r(D, I)
    return sd


def test_qwen3_moe_layouts_on_cpu():
    """Per-expert (out, in) tensors become the reference's stacked (E, in, out) arrays; a missing expert is named."""
    import jax_gpt_amd.checkpoint as ck
    E, D, I = 4, 256, 128
    sd = _qwen3_moe_sd(E, D, I, 3)
    p = ck.moe_params_from_qwen3_moe_state_dict(sd, "model.layers.1", E, device="cpu", quantize=False)
    assert p["gate_proj"].shape == (E, D, I) and p["down_proj"].shape == (E, I, D)
    for e in range(E):
        assert torch.equal(p["up_proj"][e], sd[f"model.layers.1.mlp.experts.{e}.up_proj.weight"].t())
    assert torch.equal(p["gate_weight"], sd["model.layers.1.mlp.gate.weight"].t())
    assert "shared_gate_proj" not in p
    bad = dict(sd); del bad["model.layers.1.mlp.experts.2.down_proj.weight"]
    with pytest.raises(KeyError, match="experts.2.down_proj"):
        ck.moe_params_from_qwen3_moe_state_dict(bad, "model.layers.1", E, device="cpu", quantize=False)
    bad = dict(sd); bad["model.layers.1.mlp.experts.1.gate_proj.weight"] = torch.zeros(I + 1, D, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="experts.1.gate_proj"):
        ck.moe_params_from_qwen3_moe_state_dict(bad, "model.layers.1", E, device="cpu", quantize=False)


@pytest.mark.gpu
def test_qwen3_moe_checkpoint_runs_the_layer():
    """Quantised at load or on first use, the layer gives the same bits; no shared expert in this family."""
    import jax_gpt_amd as jg
    import jax_gpt_amd.checkpoint as ck
    E, D, I, k = 8, 256, 128, 2
    sd = _qwen3_moe_sd(E, D, I, 4)
    x = (torch.randn(2, 24, D, generator=torch.Generator().manual_seed(5)) * 1.0).to(torch.bfloat16).cuda()
    pq = ck.moe_params_from_qwen3_moe_state_dict(sd, "model.layers.1", E, quantize=True)
    pp = ck.moe_params_from_qwen3_moe_state_dict(sd, "model.layers.1", E, quantize=False)
    out_q = jg.moe_layer(x, pq, k)
    out_p = jg.moe_layer(x, pp, k)
    assert out_q.shape == x.shape and torch.isfinite(out_q.float()).all()
    assert torch.equal(out_q, out_p)
