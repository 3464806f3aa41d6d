// Weighted unpermute-combine (+ shared-expert add): a deterministic gather.
//
// Replaces jax_gpt/models/qwen35/moe.py:90-94 (_scatter_back: a bf16
// scatter-add) and the final add of moe.py:281.  One workgroup per token; each
// thread owns 8 consecutive columns, reads its k expert rows through the
// inverse permutation, sums in f32 in slot order (the shared expert's row last,
// times its per-token gate of moe.py:278-279 when there is one, then the layer's
// residual input, block.py:58 / :91, when the caller passes it) and rounds once to bf16.
// HBM-bound: reads k+1 rows, writes one, all as 16-byte accesses.
#include "moe_common.h"

namespace {

struct alignas(16) bf16x8 { bf16_t v[8]; };
constexpr int kMaxK = 32;

__global__ __launch_bounds__(256) void combine_kernel(const bf16x8* __restrict__ y, const float* __restrict__ w,
                                                     const int32_t* __restrict__ inv_perm,
                                                     const bf16x8* __restrict__ shared,
                                                     const float* __restrict__ shared_gate,
                                                     const bf16x8* __restrict__ residual, int k, int D8,
                                                     bf16x8* __restrict__ out) {
  __shared__ int pos[kMaxK];
  __shared__ float wt[kMaxK];
  const int t = blockIdx.x;
  if (threadIdx.x < k) {
    pos[threadIdx.x] = inv_perm[(size_t)t * k + threadIdx.x];
    wt[threadIdx.x] = w[(size_t)t * k + threadIdx.x];
  }
  __syncthreads();
  // gridDim.y workgroups share a token's columns (small batches: one workgroup per token would leave the chip idle)
  const int per = (D8 + gridDim.y - 1) / gridDim.y;
  const int c_end = min(D8, (int)(blockIdx.y + 1) * per);
  for (int c = blockIdx.y * per + threadIdx.x; c < c_end; c += 256) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < k; ++s) {
      bf16x8 v;   // (read once, written once: non-temporal accesses leave the caches to the GEMMs' operands, -0.3 to -1 % step time)
      *(v4i*)&v = __builtin_nontemporal_load((const v4i*)&y[(size_t)pos[s] * D8 + c]);
      const float ws = wt[s];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = __fadd_rn(acc[i], __fmul_rn(bf16_to_f32(v.v[i]), ws));
    }
    if (shared) {
      bf16x8 v = shared[(size_t)t * D8 + c];
      if (shared_gate) {
        const float g = shared_gate[t];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __fadd_rn(acc[i], __fmul_rn(bf16_to_f32(v.v[i]), g));
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __fadd_rn(acc[i], bf16_to_f32(v.v[i]));
      }
    }
    if (residual) {
      bf16x8 v = residual[(size_t)t * D8 + c];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = __fadd_rn(acc[i], bf16_to_f32(v.v[i]));
    }
    bf16x8 o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o.v[i] = f32_to_bf16(acc[i]);
    __builtin_nontemporal_store(*(v4i*)&o, (v4i*)&out[(size_t)t * D8 + c]);
  }
}

}  // namespace

extern "C" int moe_combine(const void* y_bf16, const float* w, const int32_t* inv_perm,
                           const void* shared_bf16, const float* shared_gate, const void* residual_bf16, int M,
                           int k, int D, void* out_bf16, moe_stream_t stream) {
  MOE_REQUIRE(M == 0 || (y_bf16 && w && inv_perm && out_bf16), MOE_ERR_NULL, "combine: null pointer");
  MOE_REQUIRE(M >= 0 && k >= 1 && k <= kMaxK && D > 0 && D % 8 == 0, MOE_ERR_BAD_SHAPE,
              "combine: need 1 <= k <= %d and D %% 8 == 0, got M=%d k=%d D=%d", kMaxK, M, k, D);
  MOE_REQUIRE(MOE_ALIGNED16(y_bf16) && MOE_ALIGNED16(out_bf16) && MOE_ALIGNED16(shared_bf16) &&
                  MOE_ALIGNED16(residual_bf16), MOE_ERR_BAD_ALIGN,
              "combine: pointers must be 16-byte aligned");
  MOE_REQUIRE(shared_bf16 || !shared_gate, MOE_ERR_NULL, "combine: a shared gate needs a shared expert output");
  if (M == 0) return MOE_OK;
  // about four workgroups per CU at least: split the columns of a token when there are few tokens
  int split = 1;
  while (split < 8 && (long long)M * split < 1024 && (D / 8) / (split * 2) >= 64) split *= 2;
  hipLaunchKernelGGL(combine_kernel, dim3(M, split), dim3(256), 0, (hipStream_t)stream, (const bf16x8*)y_bf16, w, inv_perm,
                     (const bf16x8*)shared_bf16, shared_gate, (const bf16x8*)residual_bf16, k, D / 8, (bf16x8*)out_bf16);
  return moe_check_hip(hipGetLastError(), "combine launch");
}
