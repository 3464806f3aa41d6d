"""MI355X-native MoE expert forward behind jax-gpt's `moe_layer` call surface.

The compute lives in libmoe_hip.so (hand-written HIP kernels for gfx950, C ABI in
include/moe_hip.h).  This package is the host side: it mirrors the names and
argument meaning of jax_gpt/models/qwen35/moe.py and drives the C ABI through
ctypes with torch tensors as device buffers.  There is no CPU fallback: without
the built library and a GPU every compute call raises.
"""
from ._lib import lib, MoeError  # noqa: F401
from .moe import (  # noqa: F401
    convert,
    gather_scales,
    block_fp8_from_per_row,
    combine,
    expert_forward_single,
    gemm_down,
    gemm_gateup_swiglu,
    moe_experts,
    moe_layer,
    moe_routing,
    moe_sublayer,
    permute,
    quant_act,
    quantize_weight_block,
    rmsnorm_quant,
    route_sigmoid_grouped,
    router_logits,
    route_softmax_topk,
    shared_expert_forward,
)
