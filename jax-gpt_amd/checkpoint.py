"""Checkpoint ingest for the MoE layer: HuggingFace state-dict tensors -> the `params` dict of `moe_layer`.

Three on-disk formats feed the kernels:

* Qwen3.5 (what the reference loads, jax_gpt/models/qwen35/weight_loader.py:42-63): bf16/f32 tensors, experts
  fused as `mlp.experts.gate_up_proj` (E, 2I, D) and `mlp.experts.down_proj` (E, D, I).  HF stores Linear
  weights (out, in) -- exactly the K-contiguous layout the kernels read, so nothing is transposed here (the
  reference transposes everything to (in, out) for `x @ w`); the experts are quantised to 128x128-block fp8 on
  the GPU as they are loaded.
* DeepSeek-V3 block fp8: one `experts.{e}.{gate,up,down}_proj.weight` (float8_e4m3fn, (out, in)) and
  `.weight_scale_inv` ((out/128, in/128) f32) pair per expert.  Already the kernels' number format: the tensors
  are stacked along a new expert axis and used as they are.

* Qwen3-MoE (Qwen3-30B-A3B and the like; transformers' Qwen3MoeSparseMoeBlock): bf16 `experts.{e}.{gate,up,down}_proj.weight`
  (out, in) per expert, no shared expert; stacked along a new expert axis, then treated like the Qwen3.5 tensors.

All return plain dicts of torch tensors on `device`; only the bf16 -> fp8 quantisation needs the GPU library.
Inputs are mappings name -> torch.Tensor, e.g. `safetensors.torch.load_file(path)`.
"""
from __future__ import annotations

import torch

from . import moe as _moe


def _get(sd, name):
    try:
        return sd[name]
    except KeyError:
        raise KeyError(f"checkpoint tensor {name!r} is missing") from None


def _router_view(w_ed, device):
    """HF keeps router weights (E, D); `moe_layer` takes the reference's (D, E) array (moe.py:50).  A transposed
    VIEW of the contiguous (E, D) tensor costs nothing, and the kernel-side transpose back is then a plain copy."""
    return w_ed.to(device).contiguous().t()


def moe_params_from_qwen35_state_dict(sd, prefix, moe_intermediate_size, device="cuda", quantize=True):
    """weight_loader.py:42-63 (_load_moe_params_np) for this build's layouts.

    sd: name -> tensor; prefix e.g. 'model.layers.3'.  Returns the dict `moe_layer(x, params, k)` takes.  With
    quantize=False the expert weights stay bf16 in the reference's (E, in, out) layout (moe_layer quantises them
    on first use); with quantize=True (needs the GPU) they become block-fp8 dicts straight from the (out, in)
    checkpoint layout, one expert matrix family at a time so that peak memory stays near the fp8 size."""
    I = int(moe_intermediate_size)
    gate_up = _get(sd, f"{prefix}.mlp.experts.gate_up_proj")          # (E, 2I, D)
    down = _get(sd, f"{prefix}.mlp.experts.down_proj")                # (E, D, I)
    if gate_up.dim() != 3 or gate_up.shape[1] != 2 * I:
        raise ValueError(f"{prefix}.mlp.experts.gate_up_proj: expected (E, {2 * I}, D), got {tuple(gate_up.shape)}")
    E, _, D = gate_up.shape
    if tuple(down.shape) != (E, D, I):
        raise ValueError(f"{prefix}.mlp.experts.down_proj: expected {(E, D, I)}, got {tuple(down.shape)}")

    def expert(w_eoi):                                                # (E, out, in) as stored
        w = w_eoi.to(device)
        if w.dtype not in (torch.bfloat16, torch.float32):
            w = w.to(torch.bfloat16)
        if quantize:
            return _moe.quantize_weight_block(w.contiguous())
        return w.transpose(1, 2).contiguous()                         # reference layout (E, in, out)

    def dense(name):                                                  # shared expert Linear, (out, in) as stored
        w = _get(sd, name).to(device)
        if w.dtype not in (torch.bfloat16, torch.float32):
            w = w.to(torch.bfloat16)
        if quantize:
            return _moe.quantize_weight_block(w.contiguous())
        return w.t().contiguous()                                     # reference layout (in, out)

    return {
        "gate_weight": _router_view(_get(sd, f"{prefix}.mlp.gate.weight"), device),
        "gate_proj": expert(gate_up[:, :I, :]),
        "up_proj": expert(gate_up[:, I:, :]),
        "down_proj": expert(down),
        "shared_gate_proj": dense(f"{prefix}.mlp.shared_expert.gate_proj.weight"),
        "shared_up_proj": dense(f"{prefix}.mlp.shared_expert.up_proj.weight"),
        "shared_down_proj": dense(f"{prefix}.mlp.shared_expert.down_proj.weight"),
        "shared_expert_gate_weight": _router_view(_get(sd, f"{prefix}.mlp.shared_expert_gate.weight"), device),
    }


def moe_params_from_block_fp8_state_dict(sd, prefix, n_experts, device="cuda"):
    """DeepSeek-V3-style layer: per-expert block-fp8 tensors -> stacked (E, out, in) codes and
    (E, out/128, in/128) scales; router weight, selection bias and the shared expert if present.

    Returns dict(experts=..., shared=... or None, gate_weight=(D, E) view, bias=(E,) f32 or None): the keyword
    arguments of `moe_experts` (routing='sigmoid_grouped')."""

    def pair(name):
        w = _get(sd, name + ".weight")
        s = _get(sd, name + ".weight_scale_inv")
        if w.dtype != torch.float8_e4m3fn:
            raise TypeError(f"{name}.weight: expected float8_e4m3fn, got {w.dtype}")
        N, K = w.shape
        if tuple(s.shape) != (N // 128, K // 128) or N % 128 or K % 128:
            raise ValueError(f"{name}: weight {tuple(w.shape)} needs scales {(N // 128, K // 128)}, got {tuple(s.shape)}")
        return w, s.to(torch.float32)

    def stacked(proj):
        ws, ss = zip(*(pair(f"{prefix}.mlp.experts.{e}.{proj}") for e in range(n_experts)))
        return {"w": torch.stack([w.view(torch.uint8) for w in ws]).to(device).view(torch.float8_e4m3fn),
                "scale_inv": torch.stack(ss).to(device)}

    experts = {p: stacked(p) for p in ("gate_proj", "up_proj", "down_proj")}
    shared = None
    if f"{prefix}.mlp.shared_experts.gate_proj.weight" in sd:
        shared = {}
        for p in ("gate_proj", "up_proj", "down_proj"):
            w, s = pair(f"{prefix}.mlp.shared_experts.{p}")
            shared[p] = {"w": w.view(torch.uint8)[None].to(device).view(torch.float8_e4m3fn), "scale_inv": s[None].to(device)}
    bias = sd.get(f"{prefix}.mlp.gate.e_score_correction_bias")
    return {
        "experts": experts,
        "shared": shared,
        "gate_weight": _router_view(_get(sd, f"{prefix}.mlp.gate.weight"), device),
        "bias": None if bias is None else bias.to(device=device, dtype=torch.float32),
    }


def moe_params_from_qwen3_moe_state_dict(sd, prefix, n_experts, device="cuda", quantize=True):
    """Qwen3-MoE layer (transformers' Qwen3MoeSparseMoeBlock): `mlp.gate.weight` (E, D) and per-expert bf16
    `mlp.experts.{e}.{gate,up,down}_proj.weight` in (out, in) layout, no shared expert.

    Returns the dict `moe_layer(x, params, k)` takes (moe.py:235; routing there is softmax top-k with
    renormalisation, which is Qwen3-MoE's norm_topk_prob=True).  quantize as in moe_params_from_qwen35_state_dict;
    the experts of one projection are stacked and quantised before the next projection is touched."""

    def stacked(proj):
        ws = [_get(sd, f"{prefix}.mlp.experts.{e}.{proj}.weight") for e in range(n_experts)]
        shape = tuple(ws[0].shape)
        for e, w in enumerate(ws):
            if w.dim() != 2 or tuple(w.shape) != shape:
                raise ValueError(f"{prefix}.mlp.experts.{e}.{proj}.weight: expected {shape}, got {tuple(w.shape)}")
        w = torch.stack([w.to(device) for w in ws])                  # (E, out, in)
        if w.dtype not in (torch.bfloat16, torch.float32):
            w = w.to(torch.bfloat16)
        if quantize:
            return _moe.quantize_weight_block(w.contiguous())
        return w.transpose(1, 2).contiguous()                         # reference layout (E, in, out)

    return {
        "gate_weight": _router_view(_get(sd, f"{prefix}.mlp.gate.weight"), device),
        "gate_proj": stacked("gate_proj"),
        "up_proj": stacked("up_proj"),
        "down_proj": stacked("down_proj"),
    }
