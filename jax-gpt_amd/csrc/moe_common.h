// Shared device/host helpers for the gfx950 MoE kernels.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <stdint.h>

#include "moe_hip.h"

#define MOE_WAVE 64
#define MOE_QBLOCK 128  // scale granularity along K (and N for weights)
#define MOE_FP8_MAX 448.0f

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned short bf16_t;  // raw bf16 bits

// host side: record an error message for moe_last_error() and return the code
int moe_set_error(int code, const char* fmt, ...);
int moe_check_hip(hipError_t e, const char* what);

// hipFuncSetAttribute applies to the current device: remember, per kernel, on which devices the dynamic LDS limit
// has been raised (bit d of the mask = device d; safe to call from several host threads).
inline int moe_raise_lds_limit(const void* kernel, int bytes, std::atomic<unsigned long long>& done_mask) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return moe_check_hip(e, "hipGetDevice");
  const unsigned long long bit = 1ull << (dev & 63);
  if (done_mask.load(std::memory_order_acquire) & bit) return MOE_OK;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return moe_check_hip(e, "raising the dynamic LDS limit");
  done_mask.fetch_or(bit, std::memory_order_release);
  return MOE_OK;
}

// ---- work list of the grouped GEMMs ----
// One entry per row tile, in [expert][tile] order; every entry carries its EXPERT's row range and the index of the
// expert's first tile, from which a workgroup derives its own tile and column block (moe_gemm.hip).  The list
// depends on the group sizes and the tile height only, so the gate/up and the down GEMM of a layer share it.
struct TileHeader {
  int n_tiles;
  // The first n_static tiles are dealt to the XCDs in fixed shares (xcd_q).  The rest -- the smallest experts, last in
  // the list -- are a pool that the workgroups of every XCD draw from once their share is done, an item at a time
  // through pool_next (one counter per GEMM of the layer: gate/up, down; the list's builder sets them to zero, so a
  // list serves one launch of each).  An XCD that is ahead takes more of the pool: it evens out what the fixed
  // shares cannot know (the XCDs' paces differ by a few per cent, and so does the cost estimate behind the shares).
  int n_static;
  int pool_next[2];
  // Where the work of XCD k begins, as a tile position with 20 fraction bits (xcd_q[0] = 0, xcd_q[8] = n_static << 20);
  // a GEMM with ncb column blocks per row tile gives XCD k the items [xcd_q[k] * ncb >> 20, xcd_q[k + 1] * ncb >> 20).
  long long xcd_q[9];
  long long pad2;
};
constexpr int kTileQBits = 20;
// The pool holds at most max_tiles / 16 tiles, and an XCD may draw up to twice its eighth of it: the grouped GEMM
// launches this many workgroups per XCD beyond its fixed share for a GEMM of ncb column blocks per row tile.
constexpr int kPoolShift = 4;    // (a pool of max_tiles / 8 and up to 4 or 6 tail rounds measured 0.5-1 % slower)
constexpr int kTailRounds = 3;   // rounds of the ranking (8 experts each) that end a bin or go to the pool
__host__ __device__ inline int moe_pool_tile_limit(int max_tiles) { return max_tiles >> kPoolShift; }
__host__ __device__ inline int moe_pool_workgroups(long long pool_items) { return (int)(pool_items >> 2) + 1; }
// The grouped GEMM launches ceil(max_tiles * ncb / 8) + 2 workgroups per XCD: a split whose largest share stays
// within max_tiles / 8 tiles fits whatever ncb is (max_tiles is a worst case over all group sizes, so a real list
// is usually a good deal shorter and its shares fit with room to spare).
__host__ __device__ inline long long moe_xcd_share_cap_q(int max_tiles) {
  return ((long long)max_tiles << kTileQBits) >> 3;
}
struct TileEntry {
  int expert, row_start, rows, first_tile;
};
struct TileList {
  int max_tiles;
  TileHeader* hdr;
  TileEntry* tiles;
};
// An expert with `rows` rows gets ceil(rows / 256) row tiles whose heights, counted in units of 32 rows, differ by
// at most one: no tile computes more than 31 rows of padding, and tiles that share a weight slab take about the same
// time per K step and walk it together, so the later reader finds it in L2.
__host__ __device__ inline int moe_tile_count(int rows) { return rows <= 0 ? 0 : (rows + 255) >> 8; }
// first row (relative to the expert's first) and row count of tile t of nt
__host__ __device__ inline void moe_tile_span(int rows, int nt, int t, int& start, int& count) {
  if (nt == 1) {   // (integer division costs some forty instructions on this hardware: the one-tile case takes none)
    start = 0;
    count = rows;
    return;
  }
  const int units = (rows + 31) >> 5;
  const int base = units / nt, extra = units - base * nt;
  start = (t * base + (t < extra ? t : extra)) << 5;
  const int full = (base + (t < extra ? 1 : 0)) << 5;
  count = full < rows - start ? full : rows - start;
}
#ifdef __HIPCC__
// Where an expert's tiles go in the work list.  The grouped GEMM deals contiguous eighths of the list to the 8 XCDs
// (tiles that share a weight slab then share an L2), so the eighths should cost about the same: with group sizes
// as skewed as a biased router makes them, natural expert order leaves one XCD with up to a tenth more work than the
// average, and the launch ends with its slowest XCD.  The experts are therefore ranked by size (ties: lower index
// first) and dealt to eight bins in snake order (0..7, 7..0, ...); the list holds bin after bin.
// Called by every thread of a workgroup of 2^n >= E threads (at most 1024); thread e owns expert e (rows = 0 for
// e >= E); lds_rows and lds_key are int[blockDim.x] arrays in LDS.  Returns the index of expert e's first tile and, in
// *total_tiles, the length of the list, and writes the list header.
//
// The header's XCD shares are cut by cost, not by count: a row tile of u 32-row units costs about 8 + u (measured:
// 63 us for a 32-row tile of the gate/up GEMM against 112 us for a 256-row one, and the same ratio for the down
// GEMM), and equal counts left the XCD with the tallest tiles some 3 % more work than the average.  All tiles of an
// expert cost alike, so a cut inside an expert sits at the same fraction of its items as of its cost.
__device__ inline int moe_tile_cost(int rows) { return 8 * moe_tile_count(rows) + ((rows + 31) >> 5); }   // (< 2^31 for 2^32 / 128 rows)
__device__ inline void moe_tile_even_shares(TileHeader* hdr, int n_static, int n_tiles) {   // one thread
  hdr->n_tiles = n_tiles;
  hdr->n_static = n_static;
  hdr->pool_next[0] = hdr->pool_next[1] = 0;
  for (int k = 0; k <= 8; ++k) hdr->xcd_q[k] = (((long long)n_static << kTileQBits) * k) >> 3;
}
__device__ inline int moe_tile_first(int e, int E, int rows, int* lds_rows, int* lds_key, int* total_tiles,
                                     TileHeader* hdr, int max_tiles) {
  __shared__ long long cut_q[9];
  __shared__ int tail_tiles[kTailRounds];   // tiles of the last, last but one, ... round of the ranking
  __shared__ int sums[4];                   // non-empty experts; tiles, tiles outside the pool and their cost
  __shared__ int acc_first[1024], acc_cost[1024];
  // The two walks over all experts (the ranking; the tiles and cost in front of an expert) are shared out: with
  // epad = E rounded up to a power of two (at least a wavefront), the workgroup's threads form blockDim / epad parts,
  // thread (part, e2) walks the part's slice of the experts on behalf of expert e2, and the parts' sums meet in LDS
  // (against one thread per expert walking them all: 2 us less of a 17 us launch at 128 experts; most of such a
  // launch is its start -- arguments, first instruction lines, first loads -- and not its arithmetic).
  int epad = 64;
  while (epad < E) epad <<= 1;
  const int parts = (int)blockDim.x / epad;          // >= 1: the caller has at least E threads, a power of two of them
  const int e2 = e & (epad - 1), part = e / epad;
  const int span = (epad + parts - 1) / parts;
  const int o0 = part * span, o1 = o0 + span < E ? o0 + span : E;
  const bool helper = part < parts && e2 < E;
  lds_rows[e] = e < E ? rows : 0;
  lds_key[e] = 0;   // (first the ranks' accumulator)
  acc_first[e] = 0;
  acc_cost[e] = 0;
  if (e < 4) sums[e] = 0;
  if (e < kTailRounds) tail_tiles[e] = 0;
  __syncthreads();
  if (helper) {
    const int mine = lds_rows[e2];
    int ahead = 0;
#pragma unroll 8
    for (int o = o0; o < o1; ++o) {
      const int r = lds_rows[o];
      ahead += (r > mine || (r == mine && o < e2)) ? 1 : 0;
    }
    if (ahead) atomicAdd(&lds_key[e2], ahead);
  }
  {
    const unsigned long long busy = __ballot(e < E && rows > 0);
    if ((e & 63) == 0 && busy) atomicAdd(&sums[0], __popcll(busy));
  }
  __syncthreads();
  int key = e;
  const int rank = lds_key[e], nz = sums[0];
  const int nr = (nz + 7) >> 3;   // rounds that hold a non-empty expert
  const int tail = nr / 4 < kTailRounds ? nr / 4 : kTailRounds;   // (3 rounds = 24 experts over the 8 bins; 6 measured no better)
  const int round = rank >> 3;
  if (e < E && rows > 0 && round >= nr - tail) atomicAdd(&tail_tiles[nr - 1 - round], moe_tile_count(rows));
  __syncthreads();
  // The pool: as many of the tail rounds, from the last one, as fit the launch's spare workgroups.
  int pooled = 0;
  for (int t = 0, sum = 0; e < E && t < tail; ++t) {
    sum += tail_tiles[t];
    if (sum > moe_pool_tile_limit(max_tiles)) break;
    pooled = t + 1;
  }
  if (e < E && rows > 0 && round >= nr - pooled) {
    key = 1024 + rank;   // behind every bin (keys below 1024), the tallest of the pool first
  } else if (e < E) {
    const int posn = rank & 7;
    // Inside a bin the experts alternate between the large and the small end of the ranking (largest, smallest,
    // second largest, ...): tall tiles are matrix work on lines that mostly hit L2, short tiles are weight streams
    // from HBM, and a launch that runs them side by side from start to end keeps both busy and its power draw even
    // (largest first throughout: 1.4 % slower on the heavy-tailed DeepSeek-V3 routing, 4 % on the Qwen3-MoE case).
    // The smallest experts of a bin stay at its end (those that the pool does not take): the launch ends with its
    // shortest items.
    const int mixed = nr - tail;
    const int pos = round >= mixed ? round : (round < (mixed + 1) / 2 ? 2 * round : 2 * (mixed - 1 - round) + 1);
    key = ((round & 1) ? 7 - posn : posn) * 128 + pos;   // E <= 1024: at most 128 rounds
  }
  lds_key[e] = key;
  if (e < E) {   // the whole list's tiles, and the tiles and cost of the fixed shares (outside the pool)
    const int t = moe_tile_count(rows);
    if (t) {
      atomicAdd(&sums[1], t);
      if (key < 1024) {
        atomicAdd(&sums[2], t);
        atomicAdd(&sums[3], moe_tile_cost(rows));
      }
    }
  }
  __syncthreads();
  if (helper) {
    const int key2 = lds_key[e2];
    int tiles_before = 0, cost_before_part = 0;
#pragma unroll 8
    for (int o = o0; o < o1; ++o) {
      const int ko = lds_key[o], ro = lds_rows[o];
      const int t = moe_tile_count(ro);
      const int c = ko < 1024 ? 8 * t + ((ro + 31) >> 5) : 0;   // (not in the pool)
      const bool before = ko < key2;
      tiles_before += before ? t : 0;
      cost_before_part += before ? c : 0;
    }
    if (tiles_before) atomicAdd(&acc_first[e2], tiles_before);
    if (cost_before_part) atomicAdd(&acc_cost[e2], cost_before_part);
  }
  __syncthreads();
  const int first = acc_first[e], cost_before = acc_cost[e];
  const int total = sums[1], n_static = sums[2], cost_all = sums[3];
  *total_tiles = total;
  // cut k sits where the cost of the fixed shares reaches k/8 of their whole: inside exactly one expert, whose
  // thread places it
  if (e < E && rows > 0 && key < 1024) {
    const long long mine = moe_tile_cost(rows);
    const int nt = moe_tile_count(rows);
    for (int k = 1; k < 8; ++k) {
      const long long at = (long long)cost_all * k - (long long)cost_before * 8;   // (cost units x 8)
      if (at >= 0 && at < mine * 8)   // (float: the cut need not be exact, only inside this expert's tiles)
        cut_q[k] = ((long long)first << kTileQBits) +
                   (long long)((float)at / (float)(mine * 8) * (float)nt * (float)(1 << kTileQBits));
    }
  }
  __syncthreads();
  if (e == 0) {
    const int n = total < max_tiles ? total : max_tiles;
    const int ns = n_static < n ? n_static : n;
    cut_q[0] = 0;
    cut_q[8] = (long long)ns << kTileQBits;
    bool fits = ns > 0 && total <= max_tiles;
    for (int k = 0; k < 8 && fits; ++k) fits = cut_q[k + 1] - cut_q[k] <= moe_xcd_share_cap_q(max_tiles);
    moe_tile_even_shares(hdr, ns, n);   // (a share beyond what the launch provides workgroups for: equal counts always fit)
    if (fits)
      for (int k = 0; k <= 8; ++k) hdr->xcd_q[k] = cut_q[k];
  }
  return first;
}
#endif

// Where the routing kernels take a token's logits from: an (M, E) array, or the router matmul's split-K partial
// sums [splits][M][N] (N = E, + 1 when the shared expert's gate is the last column), which they add in slice order
// and round to bf16 themselves -- the logits then never travel through memory unless out_logits asks for them.
struct LogitSource {
  const float* logits;    // (M, E), used when partial is null
  const float* partial;   // [splits][M][N] or null
  int splits, N;
  float* out_logits;      // optional (M, E) copy of what the kernel ranked (partial mode only)
  float* shared_gate;     // (M) sigmoid of column E, written in partial mode when N > E
};
int moe_router_partials(const void* x_bf16, int M, int D, const void* w_router_bf16, int E,
                        const void* w_shared_gate_bf16, void* ws, size_t ws_bytes, int* splits_used, int* n_cols,
                        moe_stream_t stream);
// An activation quantisation that a routing launch carries along (moe_quant_device.h): `blocks` blocks of 256
// 16-byte pieces behind the routing kernel's own blocks.  blocks == 0: none.
struct QuantJob {
  const void* x;        // (R, K) bf16
  long long n_pieces;   // R * K / 8
  int groups_per_row;   // K / 128
  int R;
  uint8_t* xq;
  float* sx;
  float* sx_blocked;    // optional (K/128, R) copy of the scales
  unsigned blocks;
};
int moe_quant_act_job(const void* x_bf16, int R, int K, uint8_t* xq, float* sx, float* sx_blocked, QuantJob* job);
int moe_route_softmax_impl(const LogitSource& src, int M, int E, int k, int renorm, int32_t* idx, float* w,
                           moe_stream_t stream, const QuantJob* quant = nullptr);
int moe_route_sigmoid_grouped_impl(const LogitSource& src, const float* bias, int M, int E, int n_group,
                                   int topk_group, int k, int renorm, float routed_scale, int32_t* idx, float* w,
                                   moe_stream_t stream, const QuantJob* quant = nullptr);
// grouped GEMMs with an optional pre-built tile list in ws (moe_gemm.hip); the extern "C" entry points build their
// own.  moe_gemm_tile_list describes the list the GEMMs of (R rows, E experts) expect in ws, so that the permutation
// kernels, which hold every expert's row range anyway, can write it (moe_permute_impl) and no launch is spent on it.
int moe_gemm_tile_list(int R, int E, void* ws, size_t ws_bytes, TileList* list);
int moe_gemm_build_dense_tile_list(int R, void* ws, size_t ws_bytes, moe_stream_t stream);
// the activation quantisers with an optional second copy of the scales, block-major in row order ((K/128, R): what
// GemmScales{1, R} reads) -- spares the shared expert of a large batch the separate transposition
int moe_quant_act_impl(const void* x_bf16, int R, int K, uint8_t* xq, float* sx, float* sx_blocked, moe_stream_t stream);
int moe_rmsnorm_quant_impl(const void* x_bf16, const float* weight, float eps, int M, int D, void* normed_bf16,
                           uint8_t* xq, float* sx, float* sx_blocked, moe_stream_t stream);
int moe_permute_impl(const int32_t* idx, int M, int k, int E, int32_t* group_sizes, int32_t* group_offsets,
                     int32_t* sorted_token_ids, int32_t* sort_order, int32_t* inv_perm, void* ws, size_t ws_bytes,
                     TileList tiles, moe_stream_t stream);
// Where the grouped GEMMs find an activation scale and put an h scale, in floats: scale of (row, 128-wide K block kb)
// = s[row * in_row + kb * in_kb].  The public entry points use the row-major arrays of the quantisers ({K/128, 1});
// moe_forward hands large batches block-major arrays in row-list order ({1, R}, in_listed = true: indexed by the
// position in the row list, not through row_ids), because a K step then reads its 256 row scales from 8 lines
// instead of 256 (a 4-byte read costs the vector L1 a whole line request: -2 to -3 % GEMM time).
struct GemmScales {
  int in_row, in_kb;
  bool in_listed;
  int out_row, out_cb;   // gate/up only: scale of (row, column block cb) of h = sh[row * out_row + cb * out_cb]
  bool stream_out;       // down only, set by the launch: y is stored with non-temporal stores
};
inline GemmScales moe_row_major_scales(int K, int I) { return GemmScales{K / 128, 1, false, I / 128, 1}; }
int moe_gemm_gateup_impl(const uint8_t* xq, const float* sx, const int32_t* row_ids, const uint8_t* w_gate,
                         const float* sw_gate, const uint8_t* w_up, const float* sw_up, const int32_t* group_offsets,
                         int E, int R, int D, int I, uint8_t* hq, float* sh, void* ws, size_t ws_bytes, bool list_built,
                         GemmScales sc, moe_stream_t stream);
int moe_gemm_down_impl(const uint8_t* hq, const float* sh, const uint8_t* w_down, const float* sw_down,
                       const int32_t* group_offsets, int E, int R, int I, int D, void* y_bf16, void* ws,
                       size_t ws_bytes, bool list_built, GemmScales sc, moe_stream_t stream);

#define MOE_REQUIRE(cond, code, ...) \
  do {                               \
    if (!(cond)) return moe_set_error(code, __VA_ARGS__); \
  } while (0)
#define MOE_ALIGNED16(p) ((((uintptr_t)(p)) & 15u) == 0)

// ---- device helpers -------------------------------------------------------

__device__ __forceinline__ float bf16_to_f32(bf16_t b) { return __uint_as_float(((unsigned)b) << 16); }

__device__ __forceinline__ bf16_t f32_to_bf16(float f) {  // round-to-nearest-even
  unsigned u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (bf16_t)(u >> 16);
}

// two f32 -> two bf16 (RNE) in one dword, low half first: the hardware's packed conversion
__device__ __forceinline__ unsigned pack2_bf16(float lo, float hi) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_hw __attribute__((ext_vector_type(2)));
  const bf16x2_hw b = __builtin_convertvector((f32x2){lo, hi}, bf16x2_hw);
  return __builtin_bit_cast(unsigned, b);
}

// scale = 448/amax (1 when the group is all zero); both quotients are IEEE-rounded
__device__ __forceinline__ void fp8_scales(float amax, float& scale, float& scale_inv) {
  scale = amax > 0.f ? __fdiv_rn(MOE_FP8_MAX, amax) : 1.0f;
  scale_inv = __fdiv_rn(1.0f, scale);
}

// four f32 -> four e4m3fn codes (RNE), clamped to +-448 first
__device__ __forceinline__ unsigned pack4_e4m3(float a, float b, float c, float d) {
  a = fminf(fmaxf(a, -MOE_FP8_MAX), MOE_FP8_MAX);
  b = fminf(fmaxf(b, -MOE_FP8_MAX), MOE_FP8_MAX);
  c = fminf(fmaxf(c, -MOE_FP8_MAX), MOE_FP8_MAX);
  d = fminf(fmaxf(d, -MOE_FP8_MAX), MOE_FP8_MAX);
  int v = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  v = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, v, true);
  return (unsigned)v;
}

// exp and sigmoid as a fixed sequence of individually rounded f32 operations (no fused multiply-add), which a
// CPU can repeat bit for bit; files that use them are compiled with -ffp-contract=off
__device__ __forceinline__ float exp_det(float x) {
#pragma clang fp contract(off)
  x = fminf(fmaxf(x, -87.0f), 88.0f);
  float n = rintf(__fmul_rn(x, 1.44269504088896341f));
  float r = __fsub_rn(x, __fmul_rn(n, 0.693145751953125f));
  r = __fsub_rn(r, __fmul_rn(n, 1.42860682030941723212e-6f));
  float p = 1.9875691500e-4f;
  p = __fadd_rn(__fmul_rn(p, r), 1.3981999507e-3f);
  p = __fadd_rn(__fmul_rn(p, r), 8.3334519073e-3f);
  p = __fadd_rn(__fmul_rn(p, r), 4.1665795894e-2f);
  p = __fadd_rn(__fmul_rn(p, r), 1.6666665459e-1f);
  p = __fadd_rn(__fmul_rn(p, r), 5.0000001201e-1f);
  float r2 = __fmul_rn(r, r);
  float y = __fadd_rn(__fmul_rn(p, r2), r);
  y = __fadd_rn(y, 1.0f);
  float two_n = __uint_as_float((unsigned)((int)n + 127) << 23);
  return __fmul_rn(y, two_n);
}

__device__ __forceinline__ float sigmoid_det(float x) {
  return __fdiv_rn(1.0f, __fadd_rn(1.0f, exp_det(-x)));
}

// ---- global -> LDS copies without registers in between -------------------------------------------------------
// The copies are inline assembly on purpose: when the compiler knows that an instruction writes LDS from
// memory it makes every later LDS read wait for ALL outstanding memory operations, which would empty the
// prefetch queue at every K step.  Completion is tracked by hand instead (wait_vm + barrier); these are the
// only vector-memory operations inside the K loop.  The LDS destination of lane l is m0 + l * size; the
// source address is a uniform 64-bit base (scalar registers) + a per-lane 32-bit byte offset.
__device__ __forceinline__ void dma16(const uint8_t* base, unsigned off, uint8_t* l) {
  const unsigned m0v = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)l);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0v), "v"(off), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void dma4(const uint8_t* base, unsigned off, uint8_t* l) {
  const unsigned m0v = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)l);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(m0v), "v"(off), "s"(base) : "memory", "m0");
}
// the same two copies with the LDS destination given as a 32-bit LDS address (uniform): keeps 64-bit generic
// pointers to LDS, which the compiler holds in vector register pairs, out of the loops that issue the copies
__device__ __forceinline__ void dma16(const uint8_t* base, unsigned off, unsigned lds_addr) {
  const unsigned m0v = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0v), "v"(off), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void dma4(const uint8_t* base, unsigned off, unsigned lds_addr) {
  const unsigned m0v = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(m0v), "v"(off), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void wait_lgkm0() { __builtin_amdgcn_s_waitcnt(0xC07F); }   // lgkmcnt = 0, other counters untouched
template <int N> __device__ __forceinline__ void wait_vm() {
  static_assert(N >= 0 && N < 64, "vmcnt range");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));   // vmcnt = N, other counters untouched
}
// the same copy with a full 64-bit address per lane (rows that live in different allocations)
__device__ __forceinline__ void dma16_addr(const void* lane_addr, uint8_t* l) {
  const unsigned m0v = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)l);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(m0v), "v"(lane_addr) : "memory", "m0");
}
