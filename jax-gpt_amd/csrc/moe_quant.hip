// Block-scaled e4m3fn quantisers (HBM-bound, 16-byte accesses).
//
// scale = 448/amax, q = e4m3(clamp(x*scale, +-448)), stored scale = 1/scale.
// Activations: 1x128 groups (replaces the per-row quantiser of
// jax_gpt/models/qwen35/fp8.py:30-45).  Weights: 128x128 blocks in the
// (E, out, in) layout of quantize.py:31-42.
#include "moe_common.h"
#include "moe_quant_device.h"

namespace {

typedef moe_bf16x8 bf16x8;

__global__ __launch_bounds__(256) void quant_act_kernel(const QuantJob q) { moe_quant_act_block(q, blockIdx.x); }

// RMSNorm fused with the activation quantiser: one workgroup per row, the row stays in registers between the
// two passes.  normed = bf16((x / sqrt(mean(x^2) + eps)) * (1 + weight)), the Qwen3.5 convention of
// jax_gpt/models/qwen35/primitives.py:16-32 (the step in front of the MoE layer, block.py:54 and :88), then
// the 1x128 quantisation of the bf16 values.  Thread t holds the 16-byte pieces t, t + 256, ... of the row, so
// the 16 lanes of a quantisation group are neighbours as in quant_act_kernel.  Sums are taken in a fixed order
// with individually rounded operations.
constexpr int kNormPieces = 4;   // D <= 256 * 8 * 4 = 8192

__global__ __launch_bounds__(256) void rmsnorm_quant_kernel(const bf16x8* __restrict__ x, const float* __restrict__ weight,
                                                           float eps, int D, bf16x8* __restrict__ normed,
                                                           uint2* __restrict__ xq, float* __restrict__ sx,
                                                           float* __restrict__ sx_blocked) {
  __shared__ float wave_sum[4];
  const int row = blockIdx.x, P = D / 8, t = threadIdx.x;
  const bf16x8* xr = x + (size_t)row * P;
  float f[kNormPieces][8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kNormPieces; ++i) {
    const int p = t + 256 * i;
    bf16x8 in = {};
    if (p < P) in = xr[p];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      f[i][j] = bf16_to_f32(in.v[j]);
      ss = __fadd_rn(ss, __fmul_rn(f[i][j], f[i][j]));
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) ss = __fadd_rn(ss, __shfl_xor(ss, off, MOE_WAVE));
  if ((t & 63) == 0) wave_sum[t >> 6] = ss;
  __syncthreads();
  const float total = __fadd_rn(__fadd_rn(wave_sum[0], wave_sum[1]), __fadd_rn(wave_sum[2], wave_sum[3]));
  const float rms = __fsqrt_rn(__fadd_rn(__fdiv_rn(total, (float)D), eps));
#pragma unroll
  for (int i = 0; i < kNormPieces; ++i) {
    const int p = t + 256 * i;
    const bool ok = p < P;              // uniform over the 16 lanes of a group (P is a multiple of 16)
    float amax = 0.f;
    bf16x8 nb = {};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float wj = ok ? weight[p * 8 + j] : 0.f;
      const float v = __fmul_rn(__fdiv_rn(f[i][j], rms), __fadd_rn(1.0f, wj));
      nb.v[j] = f32_to_bf16(v);
      f[i][j] = bf16_to_f32(nb.v[j]);
      amax = fmaxf(amax, fabsf(f[i][j]));
    }
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, MOE_WAVE));
    float scale, scale_inv;
    fp8_scales(amax, scale, scale_inv);
    if (ok) {
      if (normed) normed[(size_t)row * P + p] = nb;
      uint2 out;
      out.x = pack4_e4m3(f[i][0] * scale, f[i][1] * scale, f[i][2] * scale, f[i][3] * scale);
      out.y = pack4_e4m3(f[i][4] * scale, f[i][5] * scale, f[i][6] * scale, f[i][7] * scale);
      xq[(size_t)row * P + p] = out;
      if ((t & 15) == 0) {
        sx[((size_t)row * P + p) >> 4] = scale_inv;
        if (sx_blocked) sx_blocked[(size_t)(p >> 4) * gridDim.x + row] = scale_inv;   // the (K/128, M) array
      }
    }
  }
}

// one workgroup per 128x128 block; thread t reads row t/2, columns (t%2)*64 .. +64
template <typename T>
__global__ __launch_bounds__(256) void quant_weight_kernel(const T* __restrict__ w, int N, int K,
                                                          uint8_t* __restrict__ wq, float* __restrict__ sw) {
  __shared__ float red[4];
  const int kb = blockIdx.x, nb = blockIdx.y, e = blockIdx.z;
  const int row = nb * 128 + (threadIdx.x >> 1);
  const int col = kb * 128 + (threadIdx.x & 1) * 64;
  const size_t off = ((size_t)e * N + row) * K + col;
  float f[64];
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 64; ++i) {
    if constexpr (sizeof(T) == 2) f[i] = bf16_to_f32(((const bf16_t*)w)[off + i]);
    else f[i] = ((const float*)w)[off + i];
    amax = fmaxf(amax, fabsf(f[i]));
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, MOE_WAVE));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  float scale, scale_inv;
  fp8_scales(amax, scale, scale_inv);
  unsigned* out = (unsigned*)(wq + off);
#pragma unroll
  for (int i = 0; i < 16; ++i)
    out[i] = pack4_e4m3(f[4 * i] * scale, f[4 * i + 1] * scale, f[4 * i + 2] * scale, f[4 * i + 3] * scale);
  if (threadIdx.x == 0) sw[((size_t)e * (N / 128) + nb) * (K / 128) + kb] = scale_inv;
}

}  // namespace

extern "C" int moe_quant_act(const void* x_bf16, int R, int K, uint8_t* xq, float* sx, moe_stream_t stream) {
  return moe_quant_act_impl(x_bf16, R, K, xq, sx, nullptr, stream);
}
// checks the arguments of an activation quantisation and describes it (for its own launch, or a routing launch's)
int moe_quant_act_job(const void* x_bf16, int R, int K, uint8_t* xq, float* sx, float* sx_blocked, QuantJob* job) {
  MOE_REQUIRE(R == 0 || (x_bf16 && xq && sx), MOE_ERR_NULL, "quant_act: null pointer");
  MOE_REQUIRE(R >= 0 && K > 0 && K % MOE_QBLOCK == 0, MOE_ERR_BAD_SHAPE, "quant_act: K=%d must be a positive multiple of 128 (R=%d)", K, R);
  MOE_REQUIRE(MOE_ALIGNED16(x_bf16) && MOE_ALIGNED16(xq), MOE_ERR_BAD_ALIGN, "quant_act: pointers must be 16-byte aligned");
  const long long pieces = (long long)R * K / 8;
  const long long blocks = (pieces + 255) / 256;
  MOE_REQUIRE(blocks < (1ll << 31), MOE_ERR_BAD_SHAPE, "quant_act: too many elements");
  *job = QuantJob{x_bf16, pieces, K / 128, R, xq, sx, sx_blocked, (unsigned)blocks};
  return MOE_OK;
}
int moe_quant_act_impl(const void* x_bf16, int R, int K, uint8_t* xq, float* sx, float* sx_blocked, moe_stream_t stream) {
  QuantJob job;
  if (int rc = moe_quant_act_job(x_bf16, R, K, xq, sx, sx_blocked, &job)) return rc;
  if (R == 0) return MOE_OK;
  hipLaunchKernelGGL(quant_act_kernel, dim3(job.blocks), dim3(256), 0, (hipStream_t)stream, job);
  return moe_check_hip(hipGetLastError(), "quant_act launch");
}

extern "C" int moe_rmsnorm_quant(const void* x_bf16, const float* weight, float eps, int M, int D, void* normed_bf16,
                                 uint8_t* xq, float* sx, moe_stream_t stream) {
  return moe_rmsnorm_quant_impl(x_bf16, weight, eps, M, D, normed_bf16, xq, sx, nullptr, stream);
}
int moe_rmsnorm_quant_impl(const void* x_bf16, const float* weight, float eps, int M, int D, void* normed_bf16,
                           uint8_t* xq, float* sx, float* sx_blocked, moe_stream_t stream) {
  MOE_REQUIRE((M == 0 || (x_bf16 && xq && sx)) && weight, MOE_ERR_NULL, "rmsnorm_quant: null pointer");
  MOE_REQUIRE(M >= 0 && D > 0 && D % MOE_QBLOCK == 0 && D <= 256 * 8 * kNormPieces, MOE_ERR_BAD_SHAPE,
              "rmsnorm_quant: D=%d must be a multiple of 128, at most %d (M=%d)", D, 256 * 8 * kNormPieces, M);
  MOE_REQUIRE(MOE_ALIGNED16(x_bf16) && MOE_ALIGNED16(xq) && MOE_ALIGNED16(normed_bf16), MOE_ERR_BAD_ALIGN,
              "rmsnorm_quant: pointers must be 16-byte aligned");
  if (M == 0) return MOE_OK;
  hipLaunchKernelGGL(rmsnorm_quant_kernel, dim3(M), dim3(256), 0, (hipStream_t)stream, (const bf16x8*)x_bf16, weight, eps,
                     D, (bf16x8*)normed_bf16, (uint2*)xq, sx, sx_blocked);
  return moe_check_hip(hipGetLastError(), "rmsnorm_quant launch");
}

extern "C" int moe_quant_weight_block(const void* w, int src_is_f32, int E, int N, int K, uint8_t* wq,
                                      float* sw, moe_stream_t stream) {
  MOE_REQUIRE(w && wq && sw, MOE_ERR_NULL, "quant_weight_block: null pointer");
  MOE_REQUIRE(E >= 1 && N > 0 && K > 0 && N % 128 == 0 && K % 128 == 0 && E < 65536 && N / 128 < 65536,
              MOE_ERR_BAD_SHAPE, "quant_weight_block: N=%d and K=%d must be multiples of 128 (E=%d)", N, K, E);
  MOE_REQUIRE(MOE_ALIGNED16(w) && MOE_ALIGNED16(wq), MOE_ERR_BAD_ALIGN, "quant_weight_block: pointers must be 16-byte aligned");
  dim3 grid(K / 128, N / 128, E);
  if (src_is_f32)
    hipLaunchKernelGGL(quant_weight_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)w, N, K, wq, sw);
  else
    hipLaunchKernelGGL(quant_weight_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const bf16_t*)w, N, K, wq, sw);
  return moe_check_hip(hipGetLastError(), "quant_weight_block launch");
}

namespace {
// f32 <-> bf16 conversion of a flat array (the layer computes from bf16 activations and returns its caller's
// dtype, moe.py:282): round-to-nearest-even one way, exact the other
__global__ __launch_bounds__(256) void convert_kernel(const void* __restrict__ src, int src_is_f32, void* __restrict__ dst,
                                                     int dst_is_f32, long long n) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float v = src_is_f32 ? ((const float*)src)[i] : bf16_to_f32(((const bf16_t*)src)[i]);
  if (dst_is_f32) ((float*)dst)[i] = v;
  else ((bf16_t*)dst)[i] = f32_to_bf16(v);
}
}  // namespace

extern "C" int moe_convert(const void* src, int src_is_f32, void* dst, int dst_is_f32, long long n, moe_stream_t stream) {
  MOE_REQUIRE(n >= 0 && n < (1ll << 38), MOE_ERR_BAD_SHAPE, "convert: bad element count %lld", n);
  MOE_REQUIRE(n == 0 || (src && dst), MOE_ERR_NULL, "convert: null pointer");
  if (n == 0) return MOE_OK;
  hipLaunchKernelGGL(convert_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, src, src_is_f32,
                     dst, dst_is_f32, n);
  return moe_check_hip(hipGetLastError(), "convert launch");
}

namespace {
// Activation scales, row-major (rows, KB) -> block-major (KB, n) in row-list order: out[kb][p] = sx[ids ? ids[p] : p][kb].
// One thread per list position: it reads its row's KB scales (one or two lines) and writes one float into each of the
// KB output rows, where neighbouring threads write neighbouring floats.
__global__ __launch_bounds__(256) void gather_scales_kernel(const float* __restrict__ sx, const int32_t* __restrict__ ids,
                                                           int n, int KB, float* __restrict__ out) {
  const int p = blockIdx.x * 256 + threadIdx.x;
  if (p >= n) return;
  const float* src = sx + (size_t)(ids ? ids[p] : p) * KB;
  int kb = 0;
  if ((KB & 3) == 0) {
    for (; kb < KB; kb += 4) {
      const float4 v = *(const float4*)(src + kb);
      out[(size_t)kb * n + p] = v.x;
      out[(size_t)(kb + 1) * n + p] = v.y;
      out[(size_t)(kb + 2) * n + p] = v.z;
      out[(size_t)(kb + 3) * n + p] = v.w;
    }
  }
  for (; kb < KB; ++kb) out[(size_t)kb * n + p] = src[kb];
}
}  // namespace

extern "C" int moe_gather_scales(const float* sx, const int32_t* row_ids, int n, int KB, float* out, moe_stream_t stream) {
  MOE_REQUIRE(n >= 0 && KB >= 1, MOE_ERR_BAD_SHAPE, "gather_scales: bad sizes n=%d KB=%d", n, KB);
  MOE_REQUIRE(n == 0 || (sx && out), MOE_ERR_NULL, "gather_scales: null pointer");
  // (rows of a multiple of four scales are read 16 bytes at a time)
  MOE_REQUIRE((KB & 3) || MOE_ALIGNED16(sx), MOE_ERR_BAD_ALIGN, "gather_scales: sx must be 16-byte aligned when KB is a multiple of 4");
  if (n == 0) return MOE_OK;
  hipLaunchKernelGGL(gather_scales_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, sx, row_ids,
                     n, KB, out);
  return moe_check_hip(hipGetLastError(), "gather_scales launch");
}
