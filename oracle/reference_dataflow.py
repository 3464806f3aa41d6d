"""CPU port of the reference's literal dataflow.  TEST / BASELINE INFRASTRUCTURE ONLY.

jax_gpt/models/qwen35/moe.py as written: weight-only fp8 (experts de-quantised
to the activation dtype on every call, moe.py:26-34 and :104-106), bf16
activations, three ragged_dot calls (:83-87), bf16 scatter-add (:90-94).  The
reference itself cannot run here (JAX is not installed), so bench.py times this
port on the host cores as the `cpu_baseline` ("kind": "port"), and the tests
use it to report how far the fp8-activation path sits from the reference's
bf16-activation arithmetic.  torch-CPU does the matmuls (f32 on bf16-rounded
values, which is what a CPU backend does with bf16 operands).

Nothing in the product imports this module.
"""
from __future__ import annotations

import time

import numpy as np
import torch

from . import moe_oracle as O


def _dequant_transposed(q, scale_inv, dtype=torch.bfloat16):
    """moe.py:26-34: w.astype(f32) * scale_inv, swap the last two axes, cast.  q (E,N,K) codes."""
    w = torch.from_numpy(q).view(torch.float8_e4m3fn).to(torch.float32)
    s = torch.from_numpy(scale_inv).repeat_interleave(O.BLOCK, dim=-2).repeat_interleave(O.BLOCK, dim=-1)
    return (w * s).transpose(-1, -2).to(dtype)                              # (E, K, N)


def ragged_dot(lhs, rhs, group_sizes):
    """jax.lax.ragged_dot semantics: rows of group e times rhs[e]; bf16 in, bf16 out."""
    out = torch.zeros((lhs.shape[0], rhs.shape[2]), dtype=lhs.dtype)
    start = 0
    for e, n in enumerate(group_sizes.tolist()):
        if n:
            out[start:start + n] = (lhs[start:start + n].float() @ rhs[e].float()).to(lhs.dtype)
        start += n
    return out


def expert_forward_single(x, expert_indices, expert_weights, experts):
    """moe.py:97-114 on torch-CPU tensors.  x (M, D) bf16; experts: gate/up/down -> (codes, scale_inv)."""
    gate_w = _dequant_transposed(*experts["gate"])                          # moe.py:104-106, every call
    up_w = _dequant_transposed(*experts["up"])
    down_w = _dequant_transposed(*experts["down"])
    E = gate_w.shape[0]
    M, D = x.shape
    k = expert_indices.shape[1]
    flat_token_ids = torch.arange(M).repeat_interleave(k)                   # moe.py:68
    flat_expert_ids = expert_indices.reshape(-1).long()
    sort_order = torch.argsort(flat_expert_ids, stable=True)                # moe.py:72
    sorted_token_ids = flat_token_ids[sort_order]
    sorted_weights = expert_weights.reshape(-1)[sort_order]
    group_sizes = torch.bincount(flat_expert_ids, minlength=E)              # moe.py:76-77
    x_sorted = x[sorted_token_ids]                                          # moe.py:79
    gate_out = torch.nn.functional.silu(ragged_dot(x_sorted, gate_w, group_sizes))   # moe.py:85
    up_out = ragged_dot(x_sorted, up_w, group_sizes)
    y = ragged_dot(gate_out * up_out, down_w, group_sizes)                  # moe.py:87
    weighted = (y.float() * sorted_weights[:, None]).to(x.dtype)            # moe.py:92
    out = torch.zeros((M, D), dtype=x.dtype)
    out.index_add_(0, sorted_token_ids, weighted)                           # moe.py:93-94 (bf16 accumulate)
    return out


def moe_layer_reference(x_f32, logits, experts, top_k, shared=None):
    """Softmax routing (moe.py:51-53) + routed experts + un-gated shared expert, all in the
    reference's bf16-activation arithmetic.  Returns f32 numpy (bf16-representable)."""
    x = torch.from_numpy(np.ascontiguousarray(x_f32)).to(torch.bfloat16)
    probs = torch.softmax(torch.from_numpy(logits).float(), dim=-1)
    vals, idx = torch.topk(probs, top_k, dim=-1)
    w = vals / vals.sum(-1, keepdim=True)
    out = expert_forward_single(x, idx, w, experts)
    if shared is not None:
        g = _dequant_transposed(*shared["gate"])[0]
        u = _dequant_transposed(*shared["up"])[0]
        d = _dequant_transposed(*shared["down"])[0]
        h = torch.nn.functional.silu((x.float() @ g.float()).to(x.dtype)) * (x.float() @ u.float()).to(x.dtype)
        out = out + (h.float() @ d.float()).to(x.dtype)
    return out.float().numpy()


def time_expert_sample(D, I, n_experts, rows_per_expert, top_k=8, seed=0, reps=3, threads=None):
    """Times expert_forward_single on a bounded sample of a big config: `n_experts`
    experts of shape (I, D)/(D, I) with `rows_per_expert` routed rows each.
    Returns dict(seconds=median, flops, cores, sample=description)."""
    if threads:
        torch.set_num_threads(threads)
    rng = np.random.Generator(np.random.Philox(seed))
    E = n_experts
    R = E * rows_per_expert
    M = max(R // top_k, 1)
    k = R // M
    R = M * k
    x = torch.from_numpy(rng.standard_normal((M, D), dtype=np.float32)).to(torch.bfloat16)
    # balanced assignment: flat entry f goes to expert f % E (k distinct experts per token when k <= E)
    idx = (torch.arange(R) % E).reshape(M, k)
    w = torch.full((M, k), 1.0 / k)

    def mk(n, kk):
        q = rng.integers(0, 0x7F, size=(E, n, kk), dtype=np.uint8)          # any finite e4m3 code
        q[q == 0x7F] = 0x7E
        s = np.full((E, n // 128, kk // 128), 1e-3, dtype=np.float32)
        return q, s

    experts = dict(gate=mk(I, D), up=mk(I, D), down=mk(D, I))
    expert_forward_single(x, idx, w, experts)                               # warm-up
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        expert_forward_single(x, idx, w, experts)
        times.append(time.perf_counter() - t0)
    return dict(seconds=float(np.median(times)), flops=6.0 * R * D * I, cores=torch.get_num_threads(),
                sample=f"{E} experts x {R // E} rows, D={D}, I={I} (weight de-quantisation included, as moe.py:104-106 does per call)")
