// The 1x128 activation quantiser as a device function of one 256-thread block, shared by its own kernel
// (moe_quant.hip) and by the routing kernels (moe_route.hip), whose launch can carry the quantiser's blocks behind
// its own: the two are independent, and on a latency-bound path one launch runs them side by side.
// scale = 448/amax, q = e4m3(clamp(x*scale, +-448)), stored scale = 1/scale (replaces the per-row quantiser of
// jax_gpt/models/qwen35/fp8.py:30-45).
#pragma once
#include "moe_common.h"

struct alignas(16) moe_bf16x8 { bf16_t v[8]; };

// 16 lanes per 128-wide group, 8 bf16 (16 B) per lane; `block` = index of the 256-piece block
__device__ __forceinline__ void moe_quant_act_block(const QuantJob& q, long long block) {
  const long long p = block * 256 + threadIdx.x;
  const bool ok = p < q.n_pieces;
  moe_bf16x8 in = {};
  if (ok) in = ((const moe_bf16x8*)q.x)[p];
  float f[8], amax = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    f[i] = bf16_to_f32(in.v[i]);
    amax = fmaxf(amax, fabsf(f[i]));
  }
#pragma unroll
  for (int off = 1; off < 16; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, MOE_WAVE));
  float scale, scale_inv;
  fp8_scales(amax, scale, scale_inv);
  if (ok) {
    uint2 out;
    out.x = pack4_e4m3(f[0] * scale, f[1] * scale, f[2] * scale, f[3] * scale);
    out.y = pack4_e4m3(f[4] * scale, f[5] * scale, f[6] * scale, f[7] * scale);
    ((uint2*)q.xq)[p] = out;
    if ((threadIdx.x & 15) == 0) {
      const long long g = p >> 4;
      q.sx[g] = scale_inv;
      if (q.sx_blocked) {   // the same scale in the (K/128, R) array
        const int row = (int)(g / q.groups_per_row), kb = (int)(g - (long long)row * q.groups_per_row);
        q.sx_blocked[(size_t)kb * q.R + row] = scale_inv;
      }
    }
  }
}
