// XLA typed-FFI adapter for the MoE expert forward (platform "ROCM").
//
// Wraps moe_forward() of libmoe_hip.so as one custom call so that the JAX host code of
// jax_gpt/models/qwen35/moe.py can replace expert_forward_single (moe.py:97-114) and the
// shared-expert add (moe.py:225-232, :281) with jax.ffi.ffi_call("moe_forward_hip", ...).
// Built only where jaxlib's headers exist (jax.ffi.include_dir()); the image this library
// is developed in has no JAX, so this file is compiled opportunistically and no test depends
// on it.  Buffers: x (M,D) bf16, logits (M,E) f32, bias (E) f32 (may be empty), gate/up/down
// codes (E,I,D)/(E,I,D)/(E,D,I) u8 with f32 block scales, shared-expert codes/scales (may be
// empty) -> out (M,D) bf16 and a u8 workspace result sized by moe_forward_workspace_bytes.
// A second handler, moe_layer_hip, takes hidden states instead of logits: router weight (E,D) bf16
// (params['gate_weight'].T), the shared expert's gate weight (1,D) bf16 and the block's RMSNorm weight (D) f32
// (both may be empty), i.e. moe.py:235-282 with block.py:54-58 around it in one custom call.
#include <cstdint>

#include <hip/hip_runtime_api.h>   // hipStream_t (moe_hip.h itself is plain C and names no HIP type)

#include "moe_hip.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

static ffi::Error MoeForwardImpl(hipStream_t stream, ffi::AnyBuffer x, ffi::AnyBuffer logits, ffi::AnyBuffer bias,
                                 ffi::AnyBuffer w_gate, ffi::AnyBuffer sw_gate, ffi::AnyBuffer w_up,
                                 ffi::AnyBuffer sw_up, ffi::AnyBuffer w_down, ffi::AnyBuffer sw_down,
                                 ffi::AnyBuffer ws_gate, ffi::AnyBuffer sws_gate, ffi::AnyBuffer ws_up,
                                 ffi::AnyBuffer sws_up, ffi::AnyBuffer ws_down, ffi::AnyBuffer sws_down,
                                 ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> workspace,
                                 int32_t top_k, int32_t routing, int32_t n_group, int32_t topk_group, int32_t renorm,
                                 float routed_scale) {
  auto xd = x.dimensions();
  auto wd = w_gate.dimensions();
  if (xd.size() != 2 || wd.size() != 3) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "moe_forward_hip: x must be (M,D), weights (E,I,D)");
  MoeForwardArgs a = {};
  a.M = (int)xd[0]; a.D = (int)xd[1]; a.E = (int)wd[0]; a.I = (int)wd[1]; a.k = top_k;
  a.SI = ws_gate.element_count() ? (int)ws_gate.dimensions()[1] : 0;
  a.routing = routing; a.n_group = n_group; a.topk_group = topk_group; a.renorm = renorm; a.routed_scale = routed_scale;
  a.x = x.untyped_data(); a.logits = (const float*)logits.untyped_data();
  a.bias = bias.element_count() ? (const float*)bias.untyped_data() : nullptr;
  a.w_gate = (const uint8_t*)w_gate.untyped_data(); a.sw_gate = (const float*)sw_gate.untyped_data();
  a.w_up = (const uint8_t*)w_up.untyped_data(); a.sw_up = (const float*)sw_up.untyped_data();
  a.w_down = (const uint8_t*)w_down.untyped_data(); a.sw_down = (const float*)sw_down.untyped_data();
  if (a.SI) {
    a.ws_gate = (const uint8_t*)ws_gate.untyped_data(); a.sws_gate = (const float*)sws_gate.untyped_data();
    a.ws_up = (const uint8_t*)ws_up.untyped_data(); a.sws_up = (const float*)sws_up.untyped_data();
    a.ws_down = (const uint8_t*)ws_down.untyped_data(); a.sws_down = (const float*)sws_down.untyped_data();
  }
  a.out = out->untyped_data();
  int rc = moe_forward(&a, workspace->untyped_data(), workspace->size_bytes(), (moe_stream_t)stream);
  if (rc == MOE_OK) return ffi::Error::Success();
  return ffi::Error(rc == MOE_ERR_HIP ? ffi::ErrorCode::kInternal : ffi::ErrorCode::kInvalidArgument, moe_last_error());
}

static ffi::Error MoeLayerImpl(hipStream_t stream, ffi::AnyBuffer x, ffi::AnyBuffer w_router, ffi::AnyBuffer w_shared_gate,
                               ffi::AnyBuffer norm_weight, ffi::AnyBuffer bias, ffi::AnyBuffer w_gate, ffi::AnyBuffer sw_gate,
                               ffi::AnyBuffer w_up, ffi::AnyBuffer sw_up, ffi::AnyBuffer w_down, ffi::AnyBuffer sw_down,
                               ffi::AnyBuffer ws_gate, ffi::AnyBuffer sws_gate, ffi::AnyBuffer ws_up, ffi::AnyBuffer sws_up,
                               ffi::AnyBuffer ws_down, ffi::AnyBuffer sws_down, ffi::Result<ffi::AnyBuffer> out,
                               ffi::Result<ffi::AnyBuffer> workspace, int32_t top_k, int32_t routing, int32_t n_group,
                               int32_t topk_group, int32_t renorm, float routed_scale, float norm_eps, int32_t add_residual) {
  auto xd = x.dimensions();
  auto wd = w_gate.dimensions();
  if (xd.size() != 2 || wd.size() != 3) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "moe_layer_hip: x must be (M,D), weights (E,I,D)");
  MoeForwardArgs a = {};
  a.M = (int)xd[0]; a.D = (int)xd[1]; a.E = (int)wd[0]; a.I = (int)wd[1]; a.k = top_k;
  a.SI = ws_gate.element_count() ? (int)ws_gate.dimensions()[1] : 0;
  a.routing = routing; a.n_group = n_group; a.topk_group = topk_group; a.renorm = renorm; a.routed_scale = routed_scale;
  a.x = x.untyped_data();
  a.w_router = w_router.untyped_data();
  a.w_shared_gate = w_shared_gate.element_count() ? w_shared_gate.untyped_data() : nullptr;
  a.norm_weight = norm_weight.element_count() ? (const float*)norm_weight.untyped_data() : nullptr;
  a.norm_eps = norm_eps; a.add_residual = add_residual;
  a.bias = bias.element_count() ? (const float*)bias.untyped_data() : nullptr;
  a.w_gate = (const uint8_t*)w_gate.untyped_data(); a.sw_gate = (const float*)sw_gate.untyped_data();
  a.w_up = (const uint8_t*)w_up.untyped_data(); a.sw_up = (const float*)sw_up.untyped_data();
  a.w_down = (const uint8_t*)w_down.untyped_data(); a.sw_down = (const float*)sw_down.untyped_data();
  if (a.SI) {
    a.ws_gate = (const uint8_t*)ws_gate.untyped_data(); a.sws_gate = (const float*)sws_gate.untyped_data();
    a.ws_up = (const uint8_t*)ws_up.untyped_data(); a.sws_up = (const float*)sws_up.untyped_data();
    a.ws_down = (const uint8_t*)ws_down.untyped_data(); a.sws_down = (const float*)sws_down.untyped_data();
  }
  a.out = out->untyped_data();
  int rc = moe_forward(&a, workspace->untyped_data(), workspace->size_bytes(), (moe_stream_t)stream);
  if (rc == MOE_OK) return ffi::Error::Success();
  return ffi::Error(rc == MOE_ERR_HIP ? ffi::ErrorCode::kInternal : ffi::ErrorCode::kInvalidArgument, moe_last_error());
}

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    moe_layer_hip, MoeLayerImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()    // x, router, shared gate, norm
        .Arg<ffi::AnyBuffer>()                                                                      // bias
        .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()    // gate, up
        .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()                                                // down
        .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()    // shared gate, up
        .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()                                                // shared down
        .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()                                                // out, workspace
        .Attr<int32_t>("top_k").Attr<int32_t>("routing").Attr<int32_t>("n_group").Attr<int32_t>("topk_group")
        .Attr<int32_t>("renorm").Attr<float>("routed_scale").Attr<float>("norm_eps").Attr<int32_t>("add_residual"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    moe_forward_hip, MoeForwardImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()                          // x, logits, bias
        .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()    // gate, up
        .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()                                                // down
        .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()    // shared gate, up
        .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()                                                // shared down
        .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()                                                // out, workspace
        .Attr<int32_t>("top_k").Attr<int32_t>("routing").Attr<int32_t>("n_group").Attr<int32_t>("topk_group")
        .Attr<int32_t>("renorm").Attr<float>("routed_scale"));
