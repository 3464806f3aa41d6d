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

constexpr int RT = 128;   // tokens per workgroup
constexpr int RN = 128;   // output columns per workgroup
constexpr int RBK = 64;   // K elements per step = one 128-byte LDS row
constexpr int R_TILE = RT * RBK * 2;            // 16 KB per operand tile
constexpr int R_STAGE = 2 * R_TILE;             // activations + weights
constexpr int R_LDS = 2 * R_STAGE;              // two stages: two workgroups fit one CU

// Workgroup = 4 waves in a 2 x 2 grid, wave tile 64 tokens x 64 columns = 4 x 4 MFMA tiles of 16 x 16 (K = 32 per
// v_mfma_f32_16x16x32_bf16, two per step).  Both operand tiles go global -> LDS without registers in between
// (global_load_lds_dwordx4: a wave instruction fills 8 rows of 128 bytes), two stages, copies one step ahead,
// completion counted by hand.  LDS rows are 128 bytes; the 16-byte chunk c of row r sits at position
// c ^ ((r >> 1) & 7), which makes the fragment reads (row = lane % 16, chunk = 4 s + lane / 16) conflict-free.
// Lane (fr = lane % 16, fq = lane / 16) supplies K elements [32 s + 8 fq, +8) of row fr for both operands;
// output register r of a tile is (token 4 fq + r, column fr).  Weight rows take a full address per lane: the
// shared gate's row lives in its own allocation.
__global__ __launch_bounds__(256, 2) void router_gemm_kernel(const bf16_t* __restrict__ x, int M, int D,
                                                            const bf16_t* __restrict__ w, int E,
                                                            const bf16_t* __restrict__ w_extra, int N, int k_per_split,
                                                            float* __restrict__ partial) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;
  const int fr = lane & 15, fq = lane >> 4;
  const int t0 = blockIdx.x * RT, n0 = blockIdx.y * RN;
  const int k0 = blockIdx.z * k_per_split, k1 = min(D, k0 + k_per_split);
  const int steps = (k1 - k0) / RBK;

  // copy sources: wave v fills row groups [4v, 4v + 4) (8 rows each) of both tiles
  const int drow = lane >> 3, dchunk = lane & 7;
  unsigned xoff[4];
  const bf16_t* wsrc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = (wave * 4 + i) * 8 + drow;
    const int piece = dchunk ^ ((r >> 1) & 7);
    xoff[i] = (unsigned)min(t0 + r, M - 1) * (unsigned)D * 2u + piece * 16;   // M * D * 2 < 4 GB (checked by the launcher)
    const int n = min(n0 + r, N - 1);
    wsrc[i] = (n < E ? w + (size_t)n * D : w_extra) + piece * 8 + k0;
  }
  auto issue = [&](int s) {   // 8 operations
    uint8_t* st = lds + (s & 1) * R_STAGE;
    const uint8_t* xk = (const uint8_t*)(x + k0 + (size_t)s * RBK);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma16(xk, xoff[i], st + (wave * 4 + i) * 1024);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma16_addr(wsrc[i] + (size_t)s * RBK, st + R_TILE + (wave * 4 + i) * 1024);
  };
  v4f acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  // column fragments past the last column are never multiplied (uniform per wave)
  const int jmax = min(4, max(0, (N - n0 - wn * 64 + 15) >> 4));

  if (steps > 0) issue(0);
  for (int s = 0; s < steps; ++s) {
    wait_vm<0>();                     // this wave's copies of stage s have landed
    __builtin_amdgcn_s_barrier();     // ... and everyone's; stage s - 1 is free again
    if (s + 1 < steps) issue(s + 1);
    const uint8_t* st = lds + (s & 1) * R_STAGE;
    const uint8_t* xa = st + (wm * 64 + fr) * 128;
    const uint8_t* wb = st + R_TILE + (wn * 64 + fr) * 128;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int pos = ((4 * h + fq) ^ (fr >> 1)) << 4;
      bf16x8_t a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a[i] = __builtin_bit_cast(bf16x8_t, *(const v4i*)(xa + i * 16 * 128 + pos));
        b[i] = __builtin_bit_cast(bf16x8_t, *(const v4i*)(wb + i * 16 * 128 + pos));
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (j < jmax) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
      }
    }
    wait_lgkm0();   // this wave's reads of stage s are done before anyone overwrites it (after the next barrier)
  }
  float* out = partial + (size_t)blockIdx.z * M * N;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + wn * 64 + 16 * j + fr;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int t = t0 + wm * 64 + 16 * i + 4 * fq + r;
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

// K slices that hold at least one K step, and the bytes of their partial sums [slices][M][N]
int slices_used(int M, int N, int D, int* k_per_split) {
  const int splits = choose_splits(M, N, D);
  const int kps = ((D / RBK + splits - 1) / splits) * RBK;
  if (k_per_split) *k_per_split = kps;
  return (D + kps - 1) / kps;
}
size_t partial_bytes(int M, int N, int D) { return (size_t)slices_used(M, N, D, nullptr) * (size_t)M * N * sizeof(float); }

}  // namespace

extern "C" size_t moe_router_workspace_bytes(int M, int D, int E) {
  if (M < 0 || D <= 0 || E <= 0) return 0;
  // With or without the shared expert's gate column: without it N = E can fill one column tile fewer, and the K
  // split chosen for the smaller grid is then deeper, so neither case bounds the other.
  const size_t a = partial_bytes(M, E, D), b = partial_bytes(M, E + 1, D);
  return (a > b ? a : b) + 256;
}

// The matmul alone: split-K partial sums [splits][M][N] at the start of ws (N = E, + 1 with the gate column).
int moe_router_partials(const void* x_bf16, int M, int D, const void* w_router_bf16, int E,
                        const void* w_shared_gate_bf16, void* ws, size_t ws_bytes, int* splits_used, int* n_cols,
                        moe_stream_t stream) {
  MOE_REQUIRE((M == 0 || x_bf16) && w_router_bf16 && ws, MOE_ERR_NULL, "router: null pointer");
  MOE_REQUIRE(M >= 0 && D > 0 && D % 128 == 0 && E >= 1 && E <= 1024, MOE_ERR_BAD_SHAPE,
              "router: need D %% 128 == 0 and 1 <= E <= 1024, got M=%d D=%d E=%d", M, D, E);
  MOE_REQUIRE(MOE_ALIGNED16(x_bf16) && MOE_ALIGNED16(w_router_bf16) && MOE_ALIGNED16(w_shared_gate_bf16) &&
                  MOE_ALIGNED16(ws),
              MOE_ERR_BAD_ALIGN, "router: pointers must be 16-byte aligned");
  MOE_REQUIRE(ws_bytes >= moe_router_workspace_bytes(M, D, E), MOE_ERR_WORKSPACE_TOO_SMALL,
              "router: workspace %zu < %zu", ws_bytes, moe_router_workspace_bytes(M, D, E));
  const int N = E + (w_shared_gate_bf16 ? 1 : 0);
  int k_per_split = 0;
  const int used = slices_used(M, N, D, &k_per_split);
  MOE_REQUIRE(ws_bytes >= (size_t)used * (size_t)M * N * sizeof(float), MOE_ERR_WORKSPACE_TOO_SMALL,
              "router: %d slices of %d x %d partial sums do not fit the workspace (%zu bytes)", used, M, N, ws_bytes);
  *splits_used = used;
  *n_cols = N;
  if (M == 0) return MOE_OK;
  MOE_REQUIRE((long long)M * D * 2 < (1ll << 32), MOE_ERR_BAD_SHAPE, "router: the activations must stay within 4 GB");
  hipStream_t s = (hipStream_t)stream;
  static std::atomic<unsigned long long> lds_raised{0};
  if (int rc = moe_raise_lds_limit((const void*)router_gemm_kernel, R_LDS, lds_raised)) return rc;
  hipLaunchKernelGGL(router_gemm_kernel, dim3((M + RT - 1) / RT, (N + RN - 1) / RN, used), dim3(256), R_LDS, s,
                     (const bf16_t*)x_bf16, M, D, (const bf16_t*)w_router_bf16, E, (const bf16_t*)w_shared_gate_bf16, N,
                     k_per_split, (float*)ws);
  return moe_check_hip(hipGetLastError(), "router launch");
}

extern "C" int moe_router_logits(const void* x_bf16, int M, int D, const void* w_router_bf16, int E,
                                 const void* w_shared_gate_bf16, float* logits, float* shared_gate, void* ws,
                                 size_t ws_bytes, moe_stream_t stream) {
  MOE_REQUIRE(M == 0 || logits, MOE_ERR_NULL, "router: null pointer");
  MOE_REQUIRE((w_shared_gate_bf16 == nullptr) == (shared_gate == nullptr), MOE_ERR_NULL,
              "router: the shared gate's weight and output come together");
  int used = 0, N = 0;
  int rc = moe_router_partials(x_bf16, M, D, w_router_bf16, E, w_shared_gate_bf16, ws, ws_bytes, &used, &N, stream);
  if (rc || M == 0) return rc;
  const long long total = (long long)M * N;
  hipLaunchKernelGGL(router_finish_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const float*)ws, M, E, N, used, logits, shared_gate);
  return moe_check_hip(hipGetLastError(), "router launch");
}
