// Router logits: logits[t, e] = bf16_round(sum_k x[t, k] * w[e, k]), and the shared expert's sigmoid gate.
//
// Replaces the matmul of jax_gpt/models/qwen35/moe.py:50 (logits = matmul_maybe_fp8(x, gate_weight), a bf16
// result that moe.py:51 widens to f32) and the gate of moe.py:278 (sigmoid(x @ shared_expert_gate_weight)).
// The weights come K-contiguous, (E, D) bf16 -- the checkpoint layout of mlp.gate.weight; the reference's
// in-memory (D, E) array is transposed once by the host mirror.  The shared gate's (1, D) row is one more
// output column of the same product.
//
// Two launches: bf16 MFMA partial sums over K slices (decode-sized batches have too few output tiles to fill
// the chip otherwise), then a finishing pass that adds the slices in slice order, rounds to bf16 as the
// reference's bf16 matmul does and applies the sigmoid.  Floating-point work: the order inside the matrix
// cores is the hardware's, so logits agree with a CPU restatement to rounding, not bit for bit; routing is
// exact as a function of the logits this kernel produces.
#include "moe_common.h"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

constexpr int RT = 64;    // tokens per workgroup
constexpr int RN = 256;   // output columns per workgroup (64 per wave)
constexpr int RK = 32;    // K per MFMA

// Wave tile 64 tokens x 64 columns = 4 x 4 MFMA tiles of 16 x 16.  Lane (fr = lane % 16, fq = lane / 16)
// supplies K elements [8 fq, 8 fq + 8) of row fr for both operands, straight from global memory (16 bytes per
// lane; x and w rows are re-read through L1/L2 by the waves that share them).  Output register r of a tile is
// (token 4 fq + r, column fr).
__global__ __launch_bounds__(256) void router_gemm_kernel(const bf16_t* __restrict__ x, int M, int D,
                                                         const bf16_t* __restrict__ w, int E,
                                                         const bf16_t* __restrict__ w_extra, int N, int k_per_split,
                                                         float* __restrict__ partial) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int fr = lane & 15, fq = lane >> 4;
  const int t0 = blockIdx.x * RT, n0 = blockIdx.y * RN + wave * 64;
  if (n0 >= N) return;   // uniform per wave
  const int k0 = blockIdx.z * k_per_split, k1 = min(D, k0 + k_per_split);
  const bf16_t* xa[4];
  const bf16_t* wb[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    xa[i] = x + (size_t)min(t0 + 16 * i + fr, M - 1) * D + fq * 8;
    const int n = min(n0 + 16 * i + fr, N - 1);
    wb[i] = (n < E ? w + (size_t)n * D : w_extra) + fq * 8;
  }
  v4f acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  for (int k = k0; k < k1; k += RK) {
    bf16x8_t a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a[i] = *(const bf16x8_t*)(xa[i] + k);
      b[i] = *(const bf16x8_t*)(wb[i] + k);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
  }
  float* out = partial + (size_t)blockIdx.z * M * N;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + 16 * j + fr;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int t = t0 + 16 * i + 4 * fq + r;
        if (t < M && n < N) out[(size_t)t * N + n] = acc[i][j][r];
      }
    }
}

__global__ __launch_bounds__(256) void router_finish_kernel(const float* __restrict__ partial, int M, int E, int N,
                                                           int splits, float* __restrict__ logits,
                                                           float* __restrict__ shared_gate) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long long)M * N) return;
  const int t = (int)(i / N), n = (int)(i % N);
  float s = partial[i];
  for (int z = 1; z < splits; ++z) s = __fadd_rn(s, partial[(size_t)z * M * N + i]);
  const float v = bf16_to_f32(f32_to_bf16(s));
  if (n < E) logits[(size_t)t * E + n] = v;
  else shared_gate[t] = bf16_to_f32(f32_to_bf16(sigmoid_det(v)));
}

int choose_splits(int M, int N, int D) {
  long long tiles = (long long)((M + RT - 1) / RT) * ((N + RN - 1) / RN);
  if (tiles < 1) tiles = 1;                  // M = 0
  long long s = (512 + tiles - 1) / tiles;   // aim for about two workgroups per CU
  const int max_s = D / 128;
  if (s > max_s) s = max_s;
  if (s < 1) s = 1;
  return (int)s;
}

}  // namespace

extern "C" size_t moe_router_workspace_bytes(int M, int D, int E) {
  if (M < 0 || D <= 0 || E <= 0) return 0;
  const int N = E + 1;
  return (size_t)choose_splits(M, N, D) * (size_t)M * N * sizeof(float) + 256;
}

extern "C" int moe_router_logits(const void* x_bf16, int M, int D, const void* w_router_bf16, int E,
                                 const void* w_shared_gate_bf16, float* logits, float* shared_gate, void* ws,
                                 size_t ws_bytes, moe_stream_t stream) {
  MOE_REQUIRE((M == 0 || (x_bf16 && logits)) && w_router_bf16 && ws, MOE_ERR_NULL, "router: null pointer");
  MOE_REQUIRE((w_shared_gate_bf16 == nullptr) == (shared_gate == nullptr), MOE_ERR_NULL,
              "router: the shared gate's weight and output come together");
  MOE_REQUIRE(M >= 0 && D > 0 && D % 128 == 0 && E >= 1 && E <= 1024, MOE_ERR_BAD_SHAPE,
              "router: need D %% 128 == 0 and 1 <= E <= 1024, got M=%d D=%d E=%d", M, D, E);
  MOE_REQUIRE(MOE_ALIGNED16(x_bf16) && MOE_ALIGNED16(w_router_bf16) && MOE_ALIGNED16(w_shared_gate_bf16) &&
                  MOE_ALIGNED16(ws),
              MOE_ERR_BAD_ALIGN, "router: pointers must be 16-byte aligned");
  MOE_REQUIRE(ws_bytes >= moe_router_workspace_bytes(M, D, E), MOE_ERR_WORKSPACE_TOO_SMALL,
              "router: workspace %zu < %zu", ws_bytes, moe_router_workspace_bytes(M, D, E));
  if (M == 0) return MOE_OK;
  const int N = E + (w_shared_gate_bf16 ? 1 : 0);
  const int splits = choose_splits(M, N, D);
  const int k_per_split = ((D / RK + splits - 1) / splits) * RK;
  const int used = (D + k_per_split - 1) / k_per_split;   // slices that hold at least one K step
  float* partial = (float*)ws;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(router_gemm_kernel, dim3((M + RT - 1) / RT, (N + RN - 1) / RN, used), dim3(256), 0, s,
                     (const bf16_t*)x_bf16, M, D, (const bf16_t*)w_router_bf16, E, (const bf16_t*)w_shared_gate_bf16, N,
                     k_per_split, partial);
  const long long total = (long long)M * N;
  hipLaunchKernelGGL(router_finish_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, partial, M, E, N,
                     used, logits, shared_gate);
  return moe_check_hip(hipGetLastError(), "router launch");
}
