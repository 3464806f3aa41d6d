// Routing kernels: one wavefront per token.
//
// Selection is exact integer work on order-preserving keys, so the indices do
// not depend on any transcendental: softmax routing ranks the logits (softmax
// is monotone), and the group-limited sigmoid router ranks sigmoid(logit)+bias
// where sigmoid is computed by a fixed sequence of individually rounded f32
// operations (no fused multiply-add; this file is compiled with
// -ffp-contract=off) that a CPU can repeat bit for bit.
//
// Replaces jax_gpt/models/qwen35/moe.py:51-53 (softmax, lax.top_k, renormalise).
#include "moe_common.h"
#include "moe_quant_device.h"

namespace {

// value-descending, ties -> lower index: larger key wins.  key 0 = absent.
__device__ __forceinline__ unsigned long long make_key(float v, unsigned idx) {
  unsigned u = __float_as_uint(v + 0.0f);  // -0 -> +0
  u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  return ((unsigned long long)u << 32) | (unsigned long long)(0xffffffffu - idx);
}
__device__ __forceinline__ float key_value(unsigned long long key) {
  unsigned u = (unsigned)(key >> 32);
  u = (u & 0x80000000u) ? (u & 0x7fffffffu) : ~u;
  return __uint_as_float(u);
}
__device__ __forceinline__ unsigned key_index(unsigned long long key) {
  return 0xffffffffu - (unsigned)(key & 0xffffffffu);
}

// Wave-wide maximum of 64-bit keys, result in every lane.  Inside a row of 16 lanes the partners are reached with
// DPP lane permutations (a few cycles each: xor 1, xor 2, mirror of 8, mirror of 16 -- a maximum does not care
// which partner it meets, only that the set closes); the four row maxima are then read as scalars.  The same
// reduction over ds_bpermute takes about 100 cycles per step, and routing is a chain of some thirty reductions.
template <int CTRL> __device__ __forceinline__ unsigned long long dpp_max_u64(unsigned long long k) {
  const int lo = (int)(unsigned)(k & 0xffffffffu), hi = (int)(unsigned)(k >> 32);
  const unsigned olo = (unsigned)__builtin_amdgcn_update_dpp(lo, lo, CTRL, 0xF, 0xF, false);
  const unsigned ohi = (unsigned)__builtin_amdgcn_update_dpp(hi, hi, CTRL, 0xF, 0xF, false);
  const unsigned long long o = ((unsigned long long)ohi << 32) | olo;
  return o > k ? o : k;
}
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long k) {
  k = dpp_max_u64<0xB1>(k);    // quad_perm [1,0,3,2]: lane ^ 1
  k = dpp_max_u64<0x4E>(k);    // quad_perm [2,3,0,1]: lane ^ 2
  k = dpp_max_u64<0x141>(k);   // row_half_mirror: lane i <-> 7 - i within 8
  k = dpp_max_u64<0x140>(k);   // row_mirror: lane i <-> 15 - i within 16
  unsigned long long best = 0ull;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(k & 0xffffffffu), 16 * r);
    const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(k >> 32), 16 * r);
    const unsigned long long o = ((unsigned long long)hi << 32) | lo;
    best = o > best ? o : best;
  }
  return best;
}
__device__ __forceinline__ float wave_max_f32(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, MOE_WAVE));
  return v;
}
__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = __fadd_rn(v, __shfl_xor(v, off, MOE_WAVE));
  return v;
}

constexpr int kWavesPerBlock = 4;

// Logit (t, e).  In partial mode: the slices added in slice order, one bf16 rounding (what the router's own
// finishing pass computes, moe_router.hip), optionally copied out.
__device__ __forceinline__ float fetch_logit(const LogitSource& src, int M, int E, int t, int e) {
  if (!src.partial) return src.logits[(size_t)t * E + e];
  const size_t MN = (size_t)M * src.N, at = (size_t)t * src.N + e;
  float s = src.partial[at];
  for (int z = 1; z < src.splits; ++z) s = __fadd_rn(s, src.partial[(size_t)z * MN + at]);
  const float v = bf16_to_f32(f32_to_bf16(s));
  if (src.out_logits) src.out_logits[(size_t)t * E + e] = v;
  return v;
}
// the shared expert's gate rides in column E of the partial sums: one lane per token finishes it
__device__ __forceinline__ void finish_shared_gate(const LogitSource& src, int M, int E, int t) {
  if (!src.partial || !src.shared_gate || src.N <= E) return;
  const size_t MN = (size_t)M * src.N, at = (size_t)t * src.N + E;
  float s = src.partial[at];
  for (int z = 1; z < src.splits; ++z) s = __fadd_rn(s, src.partial[(size_t)z * MN + at]);
  src.shared_gate[t] = bf16_to_f32(f32_to_bf16(sigmoid_det(bf16_to_f32(f32_to_bf16(s)))));
}

// VPL = values per lane; element e lives in lane e%64, slot e/64.
template <int VPL>
__global__ __launch_bounds__(kWavesPerBlock* MOE_WAVE) void route_softmax_kernel(
    const LogitSource src, int M, int E, int k, int renorm, int32_t* __restrict__ idx,
    float* __restrict__ w, const QuantJob quant) {
  const unsigned route_blocks = gridDim.x - quant.blocks;
  if (blockIdx.x >= route_blocks) {   // the blocks behind the routing blocks quantise the activations (QuantJob)
    moe_quant_act_block(quant, blockIdx.x - route_blocks);
    return;
  }
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (t >= M) return;
  if (lane == 0) finish_shared_gate(src, M, E, t);
  float v[VPL];
  unsigned long long key[VPL];
  float mx = -INFINITY;
#pragma unroll
  for (int s = 0; s < VPL; ++s) {
    int e = lane + 64 * s;
    bool ok = e < E;
    v[s] = ok ? fetch_logit(src, M, E, t, e) : -INFINITY;
    key[s] = ok ? make_key(v[s], (unsigned)e) : 0ull;
    mx = fmaxf(mx, v[s]);
  }
  mx = wave_max_f32(mx);
  float part = 0.f;
#pragma unroll
  for (int s = 0; s < VPL; ++s)
    if (lane + 64 * s < E) part = __fadd_rn(part, exp_det(__fsub_rn(v[s], mx)));
  const float denom = wave_sum_f32(part);

  int my_idx = 0;
  float my_p = 0.f, psum = 0.f;
  for (int sel = 0; sel < k; ++sel) {
    unsigned long long best = 0ull;
#pragma unroll
    for (int s = 0; s < VPL; ++s) best = key[s] > best ? key[s] : best;
    best = wave_max_u64(best);
    const unsigned e = key_index(best);
#pragma unroll
    for (int s = 0; s < VPL; ++s)
      if (key[s] == best) key[s] = 0ull;
    const float p = __fdiv_rn(exp_det(__fsub_rn(key_value(best), mx)), denom);
    psum = __fadd_rn(psum, p);
    if (lane == sel) {
      my_idx = (int)e;
      my_p = p;
    }
  }
  if (lane < k) {
    idx[(size_t)t * k + lane] = my_idx;
    w[(size_t)t * k + lane] = renorm ? __fdiv_rn(my_p, psum) : my_p;
  }
}

template <int VPL>
__global__ __launch_bounds__(kWavesPerBlock* MOE_WAVE) void route_sigmoid_grouped_kernel(
    const LogitSource src, const float* __restrict__ bias, int M, int E, int n_group,
    int topk_group, int k, int renorm, float routed_scale, int32_t* __restrict__ idx,
    float* __restrict__ w, const QuantJob quant) {
  const unsigned route_blocks = gridDim.x - quant.blocks;
  if (blockIdx.x >= route_blocks) {   // the blocks behind the routing blocks quantise the activations (QuantJob)
    moe_quant_act_block(quant, blockIdx.x - route_blocks);
    return;
  }
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (t >= M) return;
  if (lane == 0) finish_shared_gate(src, M, E, t);
  const int per = E / n_group;
  float score[VPL];
  unsigned long long key[VPL];
  int gid[VPL];   // group of each slot's expert (one integer division per slot, not one per group and slot)
#pragma unroll
  for (int s = 0; s < VPL; ++s) {
    int e = lane + 64 * s;
    bool ok = e < E;
    score[s] = ok ? sigmoid_det(fetch_logit(src, M, E, t, e)) : 0.f;
    float choice = __fadd_rn(score[s], (ok && bias) ? bias[e] : 0.f);
    key[s] = ok ? make_key(choice, (unsigned)e) : 0ull;
    gid[s] = ok ? e / per : -1;
  }
  // group score = sum of the two best choice scores of the group (lane g keeps group g's)
  unsigned long long gkey = 0ull;
  for (int g = 0; g < n_group; ++g) {
    unsigned long long b1 = 0ull, b2 = 0ull;
#pragma unroll
    for (int s = 0; s < VPL; ++s) {
      bool in = gid[s] == g;
      b1 = (in && key[s] > b1) ? key[s] : b1;
    }
    b1 = wave_max_u64(b1);
    float gs = key_value(b1);
    if (per >= 2) {
#pragma unroll
      for (int s = 0; s < VPL; ++s) {
        bool in = gid[s] == g && key[s] < b1;
        b2 = (in && key[s] > b2) ? key[s] : b2;
      }
      b2 = wave_max_u64(b2);
      gs = __fadd_rn(gs, key_value(b2));
    }
    if (lane == g) gkey = make_key(gs, (unsigned)g);
  }
  unsigned long long keep = 0ull;  // bit g set = group g kept
  for (int sel = 0; sel < topk_group; ++sel) {
    unsigned long long best = wave_max_u64(gkey);
    if (gkey == best) gkey = 0ull;
    keep |= 1ull << key_index(best);
  }
#pragma unroll
  for (int s = 0; s < VPL; ++s) {
    const int g = gid[s];
    if (g < 0 || g >= n_group || !((keep >> g) & 1ull)) key[s] = 0ull;
  }
  int my_idx = 0;
  float my_w = 0.f, wsum = 0.f;
  for (int sel = 0; sel < k; ++sel) {
    unsigned long long best = 0ull;
#pragma unroll
    for (int s = 0; s < VPL; ++s) best = key[s] > best ? key[s] : best;
    best = wave_max_u64(best);
    const unsigned e = key_index(best);
    float sv = 0.f;
#pragma unroll
    for (int s = 0; s < VPL; ++s) {
      if (key[s] == best) key[s] = 0ull;
      if ((int)(e >> 6) == s) sv = score[s];
    }
    sv = __shfl(sv, (int)(e & 63u), MOE_WAVE);
    wsum = __fadd_rn(wsum, sv);
    if (lane == sel) {
      my_idx = (int)e;
      my_w = sv;
    }
  }
  if (lane < k) {
    float r = my_w;
    if (renorm) r = __fdiv_rn(r, __fadd_rn(wsum, 1e-20f));
    idx[(size_t)t * k + lane] = my_idx;
    w[(size_t)t * k + lane] = __fmul_rn(r, routed_scale);
  }
}

int check_route_args(const LogitSource& src, int M, int E, int k, const int32_t* idx, const float* w) {
  MOE_REQUIRE(M == 0 || ((src.logits || src.partial) && idx && w), MOE_ERR_NULL, "route: null pointer");
  MOE_REQUIRE(!src.partial || (src.splits >= 1 && src.N >= E), MOE_ERR_BAD_SHAPE, "route: bad partial-sum layout");
  MOE_REQUIRE(M >= 0 && E >= 1 && E <= 1024, MOE_ERR_BAD_SHAPE, "route: need 1 <= E <= 1024, got E=%d M=%d", E, M);
  MOE_REQUIRE(k >= 1 && k <= 32 && k <= E, MOE_ERR_BAD_SHAPE, "route: need 1 <= k <= min(32,E), got k=%d E=%d", k, E);
  return MOE_OK;
}

}  // namespace

static_assert(kWavesPerBlock * MOE_WAVE == 256, "a routing block doubles as a quantiser block of 256 pieces");
#define DISPATCH_VPL(E, KERNEL, ...)                                                      \
  do {                                                                                    \
    dim3 grid((M + kWavesPerBlock - 1) / kWavesPerBlock + qj.blocks), block(kWavesPerBlock* MOE_WAVE); \
    int vpl = ((E) + 63) / 64;                                                            \
    if (vpl <= 1) hipLaunchKernelGGL(KERNEL<1>, grid, block, 0, s, __VA_ARGS__);          \
    else if (vpl <= 2) hipLaunchKernelGGL(KERNEL<2>, grid, block, 0, s, __VA_ARGS__);     \
    else if (vpl <= 4) hipLaunchKernelGGL(KERNEL<4>, grid, block, 0, s, __VA_ARGS__);     \
    else if (vpl <= 8) hipLaunchKernelGGL(KERNEL<8>, grid, block, 0, s, __VA_ARGS__);     \
    else hipLaunchKernelGGL(KERNEL<16>, grid, block, 0, s, __VA_ARGS__);                  \
  } while (0)

int moe_route_softmax_impl(const LogitSource& src, int M, int E, int k, int renorm, int32_t* idx, float* w,
                           moe_stream_t stream, const QuantJob* quant) {
  int rc = check_route_args(src, M, E, k, idx, w);
  if (rc) return rc;
  MOE_REQUIRE(!quant || M > 0, MOE_ERR_BAD_SHAPE, "route: nothing to carry a quantisation with");
  if (M == 0) return MOE_OK;
  hipStream_t s = (hipStream_t)stream;
  const QuantJob qj = quant ? *quant : QuantJob{};
  DISPATCH_VPL(E, route_softmax_kernel, src, M, E, k, renorm, idx, w, qj);
  return moe_check_hip(hipGetLastError(), "route_softmax launch");
}

extern "C" int moe_route_softmax_topk(const float* logits, int M, int E, int k, int renorm,
                                      int32_t* idx, float* w, moe_stream_t stream) {
  return moe_route_softmax_impl(LogitSource{logits, nullptr, 0, E, nullptr, nullptr}, M, E, k, renorm, idx, w, stream, nullptr);
}

int moe_route_sigmoid_grouped_impl(const LogitSource& src, const float* bias, int M, int E, int n_group,
                                   int topk_group, int k, int renorm, float routed_scale, int32_t* idx, float* w,
                                   moe_stream_t stream, const QuantJob* quant) {
  int rc = check_route_args(src, M, E, k, idx, w);
  if (rc) return rc;
  MOE_REQUIRE(!quant || M > 0, MOE_ERR_BAD_SHAPE, "route: nothing to carry a quantisation with");
  MOE_REQUIRE(n_group >= 1 && n_group <= 64 && E % n_group == 0, MOE_ERR_BAD_SHAPE,
              "route: n_group=%d must divide E=%d and be <= 64", n_group, E);
  MOE_REQUIRE(topk_group >= 1 && topk_group <= n_group, MOE_ERR_BAD_SHAPE,
              "route: topk_group=%d out of range for n_group=%d", topk_group, n_group);
  MOE_REQUIRE(k <= topk_group * (E / n_group), MOE_ERR_BAD_SHAPE,
              "route: k=%d exceeds the %d experts of the kept groups", k, topk_group * (E / n_group));
  if (M == 0) return MOE_OK;
  hipStream_t s = (hipStream_t)stream;
  const QuantJob qj = quant ? *quant : QuantJob{};
  DISPATCH_VPL(E, route_sigmoid_grouped_kernel, src, bias, M, E, n_group, topk_group, k, renorm,
               routed_scale, idx, w, qj);
  return moe_check_hip(hipGetLastError(), "route_sigmoid_grouped launch");
}

extern "C" int moe_route_sigmoid_grouped(const float* logits, const float* bias, int M, int E,
                                         int n_group, int topk_group, int k, int renorm,
                                         float routed_scale, int32_t* idx, float* w,
                                         moe_stream_t stream) {
  return moe_route_sigmoid_grouped_impl(LogitSource{logits, nullptr, 0, E, nullptr, nullptr}, bias, M, E, n_group,
                                        topk_group, k, renorm, routed_scale, idx, w, stream, nullptr);
}
