// Stable counting sort of the flat (token, slot) list by expert id.
//
// Replaces jax_gpt/models/qwen35/moe.py:58-80 (_sort_and_group: argsort of the
// flat expert ids, the scatter-add histogram, and the gathers of token ids).
// Three launches (one fused launch when the whole list fits one chunk), all integer work:
//   1. per-chunk histograms: each wavefront counts its 64 entries with ballot
//      match masks and adds them to an LDS histogram of the chunk;
//   2. one workgroup turns the (chunks x E) counts into group sizes, group
//      offsets and, per chunk, the first output position of every expert;
//   3. each chunk recomputes its entries' rank (earlier entries of the same
//      expert: earlier waves via an LDS prefix, same wave via popcount of the
//      match mask below the lane) and scatters.
#include "moe_common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / MOE_WAVE;
constexpr int kChunk = 2048;  // flat entries per workgroup
constexpr int kRounds = kChunk / kThreads;
constexpr int kMaxE = 1024;

// lanes of this wave whose expert id equals mine (ids < 2^bits); inactive lanes pass id = -1
__device__ __forceinline__ unsigned long long match_any(int id, int bits) {
  unsigned long long m = __ballot(id >= 0);
  for (int b = 0; b < bits; ++b) {
    unsigned long long set = __ballot((id >> b) & 1);
    m &= ((id >> b) & 1) ? set : ~set;
  }
  return id >= 0 ? m : 0ull;
}

__device__ __forceinline__ int ilog2_ceil(int n) {
  int b = 0;
  while ((1 << b) < n) ++b;
  return b;
}

__global__ __launch_bounds__(kThreads) void hist_kernel(const int32_t* __restrict__ ids, int R, int E,
                                                       int32_t* __restrict__ chunk_hist) {
  extern __shared__ int hist[];  // E
  for (int e = threadIdx.x; e < E; e += kThreads) hist[e] = 0;
  __syncthreads();
  const int bits = ilog2_ceil(E);
  const int lane = threadIdx.x & 63;
  const int base = blockIdx.x * kChunk;
  for (int r = 0; r < kRounds; ++r) {
    int f = base + r * kThreads + threadIdx.x;
    int id = f < R ? ids[f] : -1;
    if (id >= E) id = -1;  // out-of-range ids are dropped rather than corrupting LDS
    unsigned long long m = match_any(id, bits);
    // the lowest lane of each match class adds the class size
    if (id >= 0 && (m & ((1ull << lane) - 1ull)) == 0ull) atomicAdd(&hist[id], __popcll(m));
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += kThreads) chunk_hist[(size_t)blockIdx.x * E + e] = hist[e];
}

// one workgroup: thread e owns expert e.  With `cached` the (chunks x E) counts travel through LDS (kScanCacheInts
// says when they fit): every thread of the workgroup loads and stores a share of them, coalesced, in one round of
// independent accesses, and the per-expert walks over the chunks run on LDS.  Otherwise thread e walks its column
// in global memory, in batches of independent loads (one load at a time would pay a memory round trip per chunk).
constexpr int kScanCacheInts = 8192;   // 32 KB of dynamic LDS beside the static arrays (this kernel's and the tile helper's)
__global__ __launch_bounds__(kMaxE) void scan_kernel(int32_t* __restrict__ chunk_hist, int n_chunks, int E,
                                                    int32_t* __restrict__ group_sizes,
                                                    int32_t* __restrict__ group_offsets, TileList tl, int cached) {
  extern __shared__ int cache[];   // [n_chunks][E] when cached
  __shared__ int tot[kMaxE];
  __shared__ int wave_tot[kMaxE / MOE_WAVE];
  __shared__ int tile_key[kMaxE];
  const int e = threadIdx.x;
  constexpr int kBatch = 8;
  const int n_counts = n_chunks * E;
  int total = 0;
  if (cached) {
    for (int i = threadIdx.x; i < n_counts; i += kMaxE) cache[i] = chunk_hist[i];
    __syncthreads();
    if (e < E)
      for (int c = 0; c < n_chunks; ++c) total += cache[c * E + e];
  } else if (e < E) {
    for (int c0 = 0; c0 < n_chunks; c0 += kBatch) {
      int v[kBatch];
#pragma unroll
      for (int i = 0; i < kBatch; ++i) v[i] = c0 + i < n_chunks ? chunk_hist[(size_t)(c0 + i) * E + e] : 0;
#pragma unroll
      for (int i = 0; i < kBatch; ++i) total += v[i];
    }
  }
  if (e < E) group_sizes[e] = total;
  // exclusive scan of totals over experts: wave scan + scan of wave totals
  const int lane = e & 63, wv = e >> 6;
  int incl = e < E ? total : 0;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    int o = __shfl_up(incl, off, MOE_WAVE);
    if (lane >= off) incl += o;
  }
  if (lane == 63) wave_tot[wv] = incl;
  __syncthreads();
  int wbase = 0;
  for (int i = 0; i < wv; ++i) wbase += wave_tot[i];
  const int excl = wbase + incl - (e < E ? total : 0);
  tot[e] = excl;
  if (e < E) {
    group_offsets[e] = excl;
    if (e == E - 1) group_offsets[E] = excl + total;
  }
  // counts -> absolute first position of the expert's rows within each chunk, in place
  if (cached) {
    if (e < E) {
      int run = excl;
      for (int c = 0; c < n_chunks; ++c) {
        const int v = cache[c * E + e];
        cache[c * E + e] = run;
        run += v;
      }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n_counts; i += kMaxE) chunk_hist[i] = cache[i];
  } else if (e < E) {
    int run = excl;
    for (int c0 = 0; c0 < n_chunks; c0 += kBatch) {
      int v[kBatch];
#pragma unroll
      for (int i = 0; i < kBatch; ++i) v[i] = c0 + i < n_chunks ? chunk_hist[(size_t)(c0 + i) * E + e] : 0;
#pragma unroll
      for (int i = 0; i < kBatch; ++i)
        if (c0 + i < n_chunks) {
          chunk_hist[(size_t)(c0 + i) * E + e] = run;
          run += v[i];
        }
    }
  }
  if (tl.tiles) {   // the grouped GEMMs' row tiles, an expert's tiles side by side (uniform branch)
    __syncthreads();   // (tot is read above by nobody else: it doubles as the helper's scratch from here on)
    int all = 0;
    const int nt = e < E ? moe_tile_count(total) : 0;
    const int first = moe_tile_first(e, E, e < E ? total : 0, tot, tile_key, &all, tl.hdr, tl.max_tiles);
    for (int t = 0; t < nt; ++t)
      if (first + t < tl.max_tiles) tl.tiles[first + t] = TileEntry{e, excl, total, first};
  }
}

// Each wave places a contiguous quarter of the chunk, in flat order, from counters of its own: the waves first count
// their quarters, a prefix over the waves turns the counts into each wave's first position per expert, and from there
// on no wave waits for another (taking turns round by round cost two workgroup barriers per wave and round).
constexpr int kWaveSpan = kChunk / kWaves;        // flat entries per wave
constexpr int kWaveRounds = kWaveSpan / MOE_WAVE;
__global__ __launch_bounds__(kThreads) void scatter_kernel(const int32_t* __restrict__ ids, int R, int E, int k,
                                                          const int32_t* __restrict__ chunk_base,
                                                          int32_t* __restrict__ sorted_token_ids,
                                                          int32_t* __restrict__ sort_order,
                                                          int32_t* __restrict__ inv_perm) {
  extern __shared__ int smem[];  // [kWaves][E]: a wave's counts, then its next free output position per expert
  const int bits = ilog2_ceil(E);
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  int* next = smem + wv * E;
  for (int e = lane; e < E; e += MOE_WAVE) next[e] = 0;   // (a wave's LDS accesses complete in program order)
  const int base = blockIdx.x * kChunk + wv * kWaveSpan;
  int my_id[kWaveRounds];
#pragma unroll
  for (int r = 0; r < kWaveRounds; ++r) {
    const int f = base + r * MOE_WAVE + lane;
    int id = f < R ? ids[f] : -1;
    if (id >= E) id = -1;  // out-of-range ids are dropped rather than corrupting LDS
    my_id[r] = id;
    const unsigned long long m = match_any(id, bits);
    // the lowest lane of each match class adds the class size (one writer per counter and instruction)
    if (id >= 0 && (m & ((1ull << lane) - 1ull)) == 0ull) next[id] += __popcll(m);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += kThreads) {
    int run = chunk_base[(size_t)blockIdx.x * E + e];
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const int c = smem[w * E + e];
      smem[w * E + e] = run;
      run += c;
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < kWaveRounds; ++r) {
    const int f = base + r * MOE_WAVE + lane;
    const int id = my_id[r];
    const unsigned long long m = match_any(id, bits);
    const int rank = __popcll(m & ((1ull << lane) - 1ull));
    if (id >= 0) {
      const int pos = next[id] + rank;   // every lane of a class reads before its leader bumps the counter
      if (rank == 0) next[id] += __popcll(m);
      if (sort_order) sort_order[pos] = f;
      if (sorted_token_ids) sorted_token_ids[pos] = f / k;
      if (inv_perm) inv_perm[f] = pos;
    }
  }
}

// R <= kChunk: the three steps in one workgroup, one launch (decode-sized batches are launch-bound).
__global__ __launch_bounds__(kThreads) void permute_small_kernel(const int32_t* __restrict__ ids, int R, int E, int k,
                                                                int32_t* __restrict__ group_sizes,
                                                                int32_t* __restrict__ group_offsets,
                                                                int32_t* __restrict__ sorted_token_ids,
                                                                int32_t* __restrict__ sort_order,
                                                                int32_t* __restrict__ inv_perm, TileList tl) {
  __shared__ int hist[kMaxE];   // counts, then next free output position per expert
  __shared__ int wave_tot[kWaves];
  __shared__ int wave_tiles[kWaves];
  for (int e = threadIdx.x; e < kMaxE; e += kThreads) hist[e] = 0;
  __syncthreads();
  const int bits = ilog2_ceil(E);
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int rounds = (R + kThreads - 1) / kThreads;   // uniform; the rounds past the end have nothing to place
  int my_id[kRounds];
#pragma unroll
  for (int r = 0; r < kRounds; ++r) {
    my_id[r] = -1;
    if (r >= rounds) continue;
    const int f = r * kThreads + threadIdx.x;
    int id = f < R ? ids[f] : -1;
    if (id >= E) id = -1;
    my_id[r] = id;
    const unsigned long long m = match_any(id, bits);
    if (id >= 0 && (m & ((1ull << lane) - 1ull)) == 0ull) atomicAdd(&hist[id], __popcll(m));
  }
  __syncthreads();
  // exclusive scan over experts: thread t owns experts [4t, 4t + 4)
  constexpr int kPer = kMaxE / kThreads;
  int c[kPer], sum = 0;
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    c[i] = hist[threadIdx.x * kPer + i];
    sum += c[i];
  }
  int incl = sum;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int o = __shfl_up(incl, off, MOE_WAVE);
    if (lane >= off) incl += o;
  }
  if (lane == 63) wave_tot[wv] = incl;
  int nt = 0, tincl = 0;
  if (tl.tiles) {   // the grouped GEMMs' row tiles, [expert][tile] (uniform branch)
#pragma unroll
    for (int i = 0; i < kPer; ++i) nt += moe_tile_count(c[i]);   // (experts >= E count nothing)
    tincl = nt;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int o = __shfl_up(tincl, off, MOE_WAVE);
      if (lane >= off) tincl += o;
    }
    if (lane == 63) wave_tiles[wv] = tincl;
  }
  __syncthreads();
  int run = incl - sum;
  for (int i = 0; i < wv; ++i) run += wave_tot[i];
  int first = tincl - nt, all = 0;
  if (tl.tiles) {
    for (int i = 0; i < kWaves; ++i) {
      if (i < wv) first += wave_tiles[i];
      all += wave_tiles[i];
    }
    if (threadIdx.x == 0) {   // (at most 2048 rows in all: the tiles are few and short, equal shares by count, no pool)
      const int n = all < tl.max_tiles ? all : tl.max_tiles;
      moe_tile_even_shares(tl.hdr, n, n);
    }
  }
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int e = threadIdx.x * kPer + i;
    if (e < E) {
      group_sizes[e] = c[i];
      group_offsets[e] = run;
      if (e == E - 1) group_offsets[E] = run + c[i];
    }
    if (tl.tiles) {
      const int n = moe_tile_count(c[i]);
      for (int t = 0; t < n; ++t)
        if (first + t < tl.max_tiles) tl.tiles[first + t] = TileEntry{e, run, c[i], first};
      first += n;
    }
    hist[e] = run;
    run += c[i];
  }
  __syncthreads();
  if (!sorted_token_ids && !sort_order && !inv_perm) return;
#pragma unroll
  for (int r = 0; r < kRounds; ++r) {
    if (r >= rounds) break;
    const int f = r * kThreads + threadIdx.x;
    const int id = my_id[r];
    const unsigned long long m = match_any(id, bits);
    const int rank = __popcll(m & ((1ull << lane) - 1ull));
    const int cnt = __popcll(m);
    int pos = 0;
    for (int turn = 0; turn < kWaves; ++turn) {   // waves take their turn in flat-index order so ranks stay stable
      if (wv == turn && id >= 0) pos = hist[id] + rank;
      __syncthreads();
      if (wv == turn && id >= 0 && rank == 0) hist[id] += cnt;
      __syncthreads();
    }
    if (id >= 0) {
      if (sort_order) sort_order[pos] = f;
      if (sorted_token_ids) sorted_token_ids[pos] = f / k;
      if (inv_perm) inv_perm[f] = pos;
    }
  }
}

}  // namespace

extern "C" size_t moe_permute_workspace_bytes(int M, int k, int E) {
  long long R = (long long)M * k;
  long long chunks = (R + kChunk - 1) / kChunk;
  if (chunks < 1) chunks = 1;
  return (size_t)(chunks * E * sizeof(int32_t) + 256);
}

int moe_permute_impl(const int32_t* idx, int M, int k, int E, int32_t* group_sizes, int32_t* group_offsets,
                     int32_t* sorted_token_ids, int32_t* sort_order, int32_t* inv_perm, void* ws, size_t ws_bytes,
                     TileList tiles, moe_stream_t stream) {
  MOE_REQUIRE((idx || M == 0) && group_sizes && group_offsets && ws, MOE_ERR_NULL, "permute: null pointer");
  MOE_REQUIRE(M >= 0 && k >= 1 && E >= 1 && E <= kMaxE, MOE_ERR_BAD_SHAPE,
              "permute: need k >= 1 and 1 <= E <= %d, got M=%d k=%d E=%d", kMaxE, M, k, E);
  MOE_REQUIRE((long long)M * k < (1ll << 31), MOE_ERR_BAD_SHAPE, "permute: M*k overflows int32");
  MOE_REQUIRE(ws_bytes >= moe_permute_workspace_bytes(M, k, E), MOE_ERR_WORKSPACE_TOO_SMALL,
              "permute: workspace %zu < %zu", ws_bytes, moe_permute_workspace_bytes(M, k, E));
  hipStream_t s = (hipStream_t)stream;
  const int R = M * k;
  int n_chunks = (R + kChunk - 1) / kChunk;
  if (n_chunks < 1) n_chunks = 1;
  if (R <= kChunk) {
    hipLaunchKernelGGL(permute_small_kernel, dim3(1), dim3(kThreads), 0, s, idx, R, E, k, group_sizes, group_offsets,
                       sorted_token_ids, sort_order, inv_perm, tiles);
    return moe_check_hip(hipGetLastError(), "permute launch");
  }
  int32_t* chunk_hist = (int32_t*)ws;
  hipLaunchKernelGGL(hist_kernel, dim3(n_chunks), dim3(kThreads), E * sizeof(int), s, idx, R, E, chunk_hist);
  const int cached = (long long)n_chunks * E <= kScanCacheInts;
  hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(kMaxE), cached ? (size_t)n_chunks * E * sizeof(int) : 0, s, chunk_hist,
                     n_chunks, E, group_sizes, group_offsets, tiles, cached);
  if (R > 0 && (sorted_token_ids || sort_order || inv_perm))
    hipLaunchKernelGGL(scatter_kernel, dim3(n_chunks), dim3(kThreads), kWaves * E * sizeof(int), s, idx, R, E, k,
                       chunk_hist, sorted_token_ids, sort_order, inv_perm);
  return moe_check_hip(hipGetLastError(), "permute launch");
}

extern "C" int moe_permute(const int32_t* idx, int M, int k, int E, int32_t* group_sizes,
                           int32_t* group_offsets, int32_t* sorted_token_ids, int32_t* sort_order,
                           int32_t* inv_perm, void* ws, size_t ws_bytes, moe_stream_t stream) {
  return moe_permute_impl(idx, M, k, E, group_sizes, group_offsets, sorted_token_ids, sort_order, inv_perm, ws,
                          ws_bytes, TileList{0, nullptr, nullptr}, stream);
}
