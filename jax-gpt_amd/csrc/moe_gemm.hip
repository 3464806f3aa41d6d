// Grouped fp8 GEMMs over ragged expert row ranges on the CDNA4 fp8 matrix cores.
//
// Replaces the three jax.lax.ragged_dot calls of
// jax_gpt/models/qwen35/moe.py:83-87 (_expert_swiglu):
//   MODE_GATEUP: h = silu(x . Wgate[e]^T) * (x . Wup[e]^T), then 1x128 e4m3 quantisation of h
//   MODE_DOWN:   y = h . Wdown[e]^T, bf16
// for the rows [group_offsets[e], group_offsets[e+1]) of every expert e.
//
// Shape of the computation.  Both operands are K-contiguous e4m3 with one f32
// scale per 128 K-elements (activations: per row; weights: per 128 rows), so
// one v_mfma_f32_16x16x128_f8f6f4 consumes exactly one scale block: its 16x16
// f32 result is a partial sum that is multiplied by sx[row,kb]*sw[nblk,kb] and
// added to the f32 accumulator on the vector ALU.  The weight fragment is the
// MFMA's row operand and the activation fragment its column operand, so a lane
// holds four weight rows of ONE activation row: one activation scale per lane
// per fragment instead of four.
//
// Tiling.  A workgroup (4 waves) owns a work item = (expert, <=128 activation
// rows, 256 weight rows) and walks K in steps of 128 with two LDS buffers.
// In MODE_GATEUP the 256 weight rows are 128 gate rows + the 128 up rows of
// the same output columns, so silu(g)*u and the 1x128 amax stay inside the
// workgroup.  Wave w owns weight rows {32w..32w+31} of each half (GATEUP) or
// {64w..64w+63} (DOWN) against all 128 activation rows: 4x8 MFMA tiles.
// LDS rows are 128 B; 16-byte chunks are XOR-swizzled with (row & 7) so that
// both the cooperative tile stores and the per-lane fragment reads are
// conflict-free.  Work items are listed on the device by build_items_kernel
// (no host read-back of group sizes) in [expert][column block][row tile] order
// and dealt to the 8 XCDs in contiguous ranges, so the row tiles that share a
// weight slab run together under one L2.
#include "moe_common.h"

namespace {

constexpr int BM = 128;       // activation rows per work item
constexpr int BW = 256;       // weight rows per work item
constexpr int BK = 128;       // K step = scale block
constexpr int NT = 256;       // threads
constexpr int MODE_GATEUP = 0;
constexpr int MODE_DOWN = 1;

constexpr int W_TILE_BYTES = BW * BK;   // 32 KB
constexpr int X_TILE_BYTES = BM * BK;   // 16 KB
constexpr int BUF_BYTES = W_TILE_BYTES + X_TILE_BYTES + BM * 4;  // + activation scales
constexpr int LDS_BYTES = 2 * BUF_BYTES;

struct WorkHeader {
  int n_items;
  int pad[3];
};
struct WorkItem {
  int expert, row_start, row_count, col_block;
};

// ---- work list -----------------------------------------------------------

// One workgroup.  tiles[e] = ceil(rows_e / BM); item order [expert][col_block][row tile].
__global__ __launch_bounds__(1024) void build_items_kernel(const int32_t* __restrict__ group_offsets, int E,
                                                          int n_col_blocks, int max_items,
                                                          WorkHeader* __restrict__ hdr, WorkItem* __restrict__ items) {
  __shared__ int tile_prefix[1025];
  __shared__ int wave_tot[16];
  const int e = threadIdx.x;
  const int lane = e & 63, wv = e >> 6;
  int rows = 0;
  if (e < E) rows = group_offsets[e + 1] - group_offsets[e];
  int tiles = rows > 0 ? (rows + BM - 1) / BM : 0;
  int incl = tiles;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    int o = __shfl_up(incl, off, MOE_WAVE);
    if (lane >= off) incl += o;
  }
  if (lane == 63) wave_tot[wv] = incl;
  __syncthreads();
  int wbase = 0;
  for (int i = 0; i < wv; ++i) wbase += wave_tot[i];
  if (e < E) tile_prefix[e + 1] = wbase + incl;
  if (e == 0) tile_prefix[0] = 0;
  __syncthreads();
  int total = tile_prefix[E] * n_col_blocks;
  if (total > max_items) total = max_items;  // cannot happen for consistent offsets; keeps writes in bounds
  if (e == 0) hdr->n_items = total;
  for (int it = threadIdx.x; it < total; it += blockDim.x) {
    const int tile_major = it / n_col_blocks;  // which expert: search on tile_prefix * n_col_blocks
    // find expert x with tile_prefix[x]*ncb <= it < tile_prefix[x+1]*ncb
    int lo = 0, hi = E;  // invariant: tile_prefix[lo]*ncb <= it < tile_prefix[hi]*ncb
    while (hi - lo > 1) {
      int mid = (lo + hi) >> 1;
      if (tile_prefix[mid] * n_col_blocks <= it) lo = mid; else hi = mid;
    }
    (void)tile_major;
    const int x = lo;
    const int tiles_x = tile_prefix[x + 1] - tile_prefix[x];
    const int local = it - tile_prefix[x] * n_col_blocks;
    const int cb = local / tiles_x, rt = local % tiles_x;
    const int start = group_offsets[x], rows_x = group_offsets[x + 1] - start;
    WorkItem w;
    w.expert = x;
    w.row_start = start + rt * BM;
    w.row_count = min(BM, rows_x - rt * BM);
    w.col_block = cb;
    items[it] = w;
  }
}

// ---- main kernel ---------------------------------------------------------

__device__ __forceinline__ int swz(int row, int chunk) { return row * BK + ((chunk ^ (row & 7)) << 4); }

template <int MODE>
__global__ __launch_bounds__(NT) void grouped_gemm_kernel(
    const uint8_t* __restrict__ xq, const float* __restrict__ sx, const int32_t* __restrict__ row_ids,
    const uint8_t* __restrict__ w0, const float* __restrict__ sw0,   // gate (GATEUP) or down (DOWN)
    const uint8_t* __restrict__ w1, const float* __restrict__ sw1,   // up (GATEUP only)
    const WorkHeader* __restrict__ hdr, const WorkItem* __restrict__ items,
    int K, int N,                                                    // contraction length; weight rows per matrix
    void* __restrict__ out, float* __restrict__ out_scale) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  // deal contiguous item ranges to the 8 XCDs (workgroup ids are issued round-robin over XCDs)
  const int n_items = hdr->n_items;
  const int per_xcd = (n_items + 7) >> 3;
  const int slot = blockIdx.x >> 3;
  const int item_id = (blockIdx.x & 7) * per_xcd + slot;
  if (slot >= per_xcd || item_id >= n_items) return;
  const WorkItem item = items[item_id];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int KB = K / BK;
  const int nkb_scale = KB;  // scale columns per weight row block
  const int e = item.expert;

  // weight rows of this item: GATEUP -> rows [cb*128, +128) of gate and of up; DOWN -> rows [cb*256, +256) of down
  const int wrow0 = MODE == MODE_GATEUP ? item.col_block * 128 : item.col_block * 256;
  const uint8_t* wbase0 = w0 + ((size_t)e * N) * K;
  const uint8_t* wbase1 = MODE == MODE_GATEUP ? w1 + ((size_t)e * N) * K : nullptr;

  // ---- per-thread global sources for the cooperative tile loads (16 B each)
  const int ld_chunk = tid & 7, ld_row = tid >> 3;  // rows ld_row + 32*i
  const uint8_t* wsrc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    int r = ld_row + 32 * i;  // 0..255 within the weight tile
    const uint8_t* base;
    int grow;
    if (MODE == MODE_GATEUP) {
      base = r < 128 ? wbase0 : wbase1;
      grow = wrow0 + (r & 127);
    } else {
      base = wbase0;
      grow = min(wrow0 + r, N - 1);
    }
    wsrc[i] = base + (size_t)grow * K + ld_chunk * 16;
  }
  const uint8_t* xsrc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int r = min(ld_row + 32 * i, item.row_count - 1);
    int g = item.row_start + r;
    if (row_ids) g = row_ids[g];
    xsrc[i] = xq + (size_t)g * K + ld_chunk * 16;
  }
  const float* sxsrc = nullptr;
  if (tid < BM) {
    int g = item.row_start + min(tid, item.row_count - 1);
    if (row_ids) g = row_ids[g];
    sxsrc = sx + (size_t)g * KB;
  }
  // weight scale rows for this wave
  const float* swp0;
  const float* swp1 = nullptr;
  if (MODE == MODE_GATEUP) {
    swp0 = sw0 + ((size_t)e * (N / 128) + item.col_block) * nkb_scale;
    swp1 = sw1 + ((size_t)e * (N / 128) + item.col_block) * nkb_scale;
  } else {
    int nb = min(item.col_block * 2 + (wave >> 1), N / 128 - 1);
    swp0 = sw0 + ((size_t)e * (N / 128) + nb) * nkb_scale;
  }

  v4i wreg[8], xreg[4];
  float sxreg = 0.f;
  auto load_tile = [&](int kb) {
#pragma unroll
    for (int i = 0; i < 8; ++i) wreg[i] = *(const v4i*)(wsrc[i] + (size_t)kb * BK);
#pragma unroll
    for (int i = 0; i < 4; ++i) xreg[i] = *(const v4i*)(xsrc[i] + (size_t)kb * BK);
    if (tid < BM) sxreg = sxsrc[kb];
  };
  auto store_tile = [&](int buf) {
    uint8_t* wl = lds + buf * BUF_BYTES;
    uint8_t* xl = wl + W_TILE_BYTES;
    float* sl = (float*)(xl + X_TILE_BYTES);
#pragma unroll
    for (int i = 0; i < 8; ++i) *(v4i*)(wl + swz(ld_row + 32 * i, ld_chunk)) = wreg[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) *(v4i*)(xl + swz(ld_row + 32 * i, ld_chunk)) = xreg[i];
    if (tid < BM) sl[tid] = sxreg;
  };

  // ---- fragment geometry
  const int fr = lane & 15;        // row of the fragment this lane feeds
  const int fq = lane >> 4;        // K quarter (32 B) this lane feeds
  int wfrag_row[4];
#pragma unroll
  for (int f = 0; f < 4; ++f)
    wfrag_row[f] = MODE == MODE_GATEUP ? ((f >> 1) * 128 + wave * 32 + (f & 1) * 16 + fr) : (wave * 64 + f * 16 + fr);

  v4f acc[4][8];
#pragma unroll
  for (int f = 0; f < 4; ++f)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[f][j] = (v4f){0.f, 0.f, 0.f, 0.f};

  load_tile(0);
  store_tile(0);
  __syncthreads();

  for (int kb = 0; kb < KB; ++kb) {
    const int buf = kb & 1;
    if (kb + 1 < KB) load_tile(kb + 1);

    const uint8_t* wl = lds + buf * BUF_BYTES;
    const uint8_t* xl = wl + W_TILE_BYTES;
    const float* sl = (const float*)(xl + X_TILE_BYTES);
    const float s0 = swp0[kb];
    const float s1 = MODE == MODE_GATEUP ? swp1[kb] : s0;

    v8i wf[4];
#pragma unroll
    for (int f = 0; f < 4; ++f) {
      v4i lo = *(const v4i*)(wl + swz(wfrag_row[f], 2 * fq));
      v4i hi = *(const v4i*)(wl + swz(wfrag_row[f], 2 * fq + 1));
      wf[f] = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int xr = j * 16 + fr;
      v4i lo = *(const v4i*)(xl + swz(xr, 2 * fq));
      v4i hi = *(const v4i*)(xl + swz(xr, 2 * fq + 1));
      v8i xf = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      const float sxv = sl[xr];
      const float sc0 = sxv * s0, sc1 = sxv * s1;
#pragma unroll
      for (int f = 0; f < 4; ++f) {
        v4f p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[f], xf, (v4f){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
        const float sc = (MODE == MODE_GATEUP && f >= 2) ? sc1 : sc0;
        acc[f][j] += p * sc;
      }
    }
    if (kb + 1 < KB) store_tile(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue.  Lane holds, for fragment (f, j): activation row j*16+fr, weight rows (fragment base)+4*fq+{0..3}.
  if (MODE == MODE_GATEUP) {
    float* amax_s = (float*)lds;                       // [4 waves][128 rows]
    uint8_t* tile = lds + 4 * BM * sizeof(float);      // [128 rows][128 B], swizzled
    float amax[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float m = 0.f;
#pragma unroll
      for (int f = 0; f < 2; ++f)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float g = acc[f][j][r], u = acc[f + 2][j][r];
          float h = g / (1.0f + __expf(-g)) * u;
          acc[f][j][r] = h;
          m = fmaxf(m, fabsf(h));
        }
      m = fmaxf(m, __shfl_xor(m, 16, MOE_WAVE));
      m = fmaxf(m, __shfl_xor(m, 32, MOE_WAVE));
      amax[j] = m;
      if (fq == 0) amax_s[wave * BM + j * 16 + fr] = m;
    }
    __syncthreads();
    const int I = N;
    uint8_t* hq = (uint8_t*)out;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int xr = j * 16 + fr;
      float m = fmaxf(fmaxf(amax_s[xr], amax_s[BM + xr]), fmaxf(amax_s[2 * BM + xr], amax_s[3 * BM + xr]));
      float scale, scale_inv;
      fp8_scales(m, scale, scale_inv);
#pragma unroll
      for (int f = 0; f < 2; ++f) {
        unsigned q = pack4_e4m3(acc[f][j][0] * scale, acc[f][j][1] * scale, acc[f][j][2] * scale, acc[f][j][3] * scale);
        const int col = wave * 32 + f * 16 + fq * 4;  // byte column within the 128-wide slab
        *(unsigned*)(tile + swz(xr, col >> 4) + (col & 15)) = q;
      }
      if (wave == 0 && fq == 0 && xr < item.row_count)
        out_scale[(size_t)(item.row_start + xr) * (I / 128) + item.col_block] = scale_inv;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = ld_row + 32 * i;
      if (r < item.row_count) {
        v4i v = *(const v4i*)(tile + swz(r, ld_chunk));
        *(v4i*)(hq + (size_t)(item.row_start + r) * I + item.col_block * 128 + ld_chunk * 16) = v;
      }
    }
  } else {
    // bf16 tile [128 rows][256 cols] = 512 B per row, 32 chunks of 16 B, swizzled with (row & 7)
    uint8_t* tile = lds;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int xr = j * 16 + fr;
#pragma unroll
      for (int f = 0; f < 4; ++f) {
        const int col = wave * 64 + f * 16 + fq * 4;  // output column within the 256-wide slab
        uint2 v;
        v.x = (unsigned)f32_to_bf16(acc[f][j][0]) | ((unsigned)f32_to_bf16(acc[f][j][1]) << 16);
        v.y = (unsigned)f32_to_bf16(acc[f][j][2]) | ((unsigned)f32_to_bf16(acc[f][j][3]) << 16);
        const int chunk = col >> 3;  // 8 bf16 per 16-byte chunk
        *(uint2*)(tile + xr * 512 + ((chunk ^ (xr & 7)) << 4) + (col & 7) * 2) = v;
      }
    }
    __syncthreads();
    bf16_t* y = (bf16_t*)out;
    const int c32 = tid & 31, r8 = tid >> 5;
    const int ncols = min(256, N - wrow0);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int r = r8 + 8 * i;
      if (r < item.row_count && c32 * 8 < ncols) {
        v4i v = *(const v4i*)(tile + r * 512 + ((c32 ^ (r & 7)) << 4));
        *(v4i*)(y + (size_t)(item.row_start + r) * N + wrow0 + c32 * 8) = v;
      }
    }
  }
}

int max_items_for(int R, int E, int n_col_blocks) {
  long long tiles = (long long)(R + BM - 1) / BM + (E < R ? E : R);
  return (int)(tiles * n_col_blocks);
}

template <int MODE>
int launch(const uint8_t* xq, const float* sx, const int32_t* row_ids, const uint8_t* w0, const float* sw0,
           const uint8_t* w1, const float* sw1, const int32_t* group_offsets, int E, int R, int K, int N,
           void* out, float* out_scale, void* ws, size_t ws_bytes, hipStream_t s) {
  const int ncb = MODE == MODE_GATEUP ? N / 128 : (N + 255) / 256;
  const size_t need = moe_gemm_workspace_bytes(R, E, N);
  MOE_REQUIRE(ws_bytes >= need, MOE_ERR_WORKSPACE_TOO_SMALL, "gemm: workspace %zu < %zu", ws_bytes, need);
  if (R == 0) return MOE_OK;
  const int max_items = max_items_for(R, E, ncb);
  WorkHeader* hdr = (WorkHeader*)ws;
  WorkItem* items = (WorkItem*)((char*)ws + sizeof(WorkHeader));
  hipLaunchKernelGGL(build_items_kernel, dim3(1), dim3(1024), 0, s, group_offsets, E, ncb, max_items, hdr, items);
  static bool attr_set[2] = {false, false};
  if (!attr_set[MODE]) {
    hipError_t err = hipFuncSetAttribute((const void*)grouped_gemm_kernel<MODE>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    if (err != hipSuccess) return moe_check_hip(err, "gemm: raising the dynamic LDS limit");
    attr_set[MODE] = true;
  }
  const int grid = ((max_items + 7) / 8) * 8;
  hipLaunchKernelGGL(grouped_gemm_kernel<MODE>, dim3(grid), dim3(NT), LDS_BYTES, s, xq, sx, row_ids, w0, sw0, w1,
                     sw1, hdr, items, K, N, out, out_scale);
  return moe_check_hip(hipGetLastError(), "gemm launch");
}

}  // namespace

extern "C" size_t moe_gemm_workspace_bytes(int R, int E, int N_out) {
  // enough for either GEMM: column blocks of 128 bound both cases
  int ncb = (N_out + 127) / 128;
  return sizeof(WorkHeader) + (size_t)max_items_for(R, E, ncb) * sizeof(WorkItem) + 256;
}

extern "C" int moe_gemm_gateup_swiglu_fp8(const uint8_t* xq, const float* sx, const int32_t* row_ids,
                                          const uint8_t* w_gate, const float* sw_gate, const uint8_t* w_up,
                                          const float* sw_up, const int32_t* group_offsets, int E, int R, int D,
                                          int I, uint8_t* hq, float* sh, void* ws, size_t ws_bytes,
                                          moe_stream_t stream) {
  MOE_REQUIRE(xq && sx && w_gate && sw_gate && w_up && sw_up && group_offsets && hq && sh && ws, MOE_ERR_NULL,
              "gemm_gateup: null pointer");
  MOE_REQUIRE(E >= 1 && E <= 1024 && R >= 0 && D > 0 && I > 0 && D % 128 == 0 && I % 128 == 0, MOE_ERR_BAD_SHAPE,
              "gemm_gateup: need D %% 128 == 0 and I %% 128 == 0 and 1 <= E <= 1024, got E=%d R=%d D=%d I=%d", E, R, D, I);
  MOE_REQUIRE(MOE_ALIGNED16(xq) && MOE_ALIGNED16(w_gate) && MOE_ALIGNED16(w_up) && MOE_ALIGNED16(hq) && MOE_ALIGNED16(ws),
              MOE_ERR_BAD_ALIGN, "gemm_gateup: pointers must be 16-byte aligned");
  return launch<MODE_GATEUP>(xq, sx, row_ids, w_gate, sw_gate, w_up, sw_up, group_offsets, E, R, D, I, hq, sh, ws,
                             ws_bytes, (hipStream_t)stream);
}

extern "C" int moe_gemm_down_fp8(const uint8_t* hq, const float* sh, const uint8_t* w_down, const float* sw_down,
                                 const int32_t* group_offsets, int E, int R, int I, int D, void* y_bf16, void* ws,
                                 size_t ws_bytes, moe_stream_t stream) {
  MOE_REQUIRE(hq && sh && w_down && sw_down && group_offsets && y_bf16 && ws, MOE_ERR_NULL, "gemm_down: null pointer");
  MOE_REQUIRE(E >= 1 && E <= 1024 && R >= 0 && D > 0 && I > 0 && D % 128 == 0 && I % 128 == 0, MOE_ERR_BAD_SHAPE,
              "gemm_down: need D %% 128 == 0 and I %% 128 == 0 and 1 <= E <= 1024, got E=%d R=%d I=%d D=%d", E, R, I, D);
  MOE_REQUIRE(MOE_ALIGNED16(hq) && MOE_ALIGNED16(w_down) && MOE_ALIGNED16(y_bf16) && MOE_ALIGNED16(ws), MOE_ERR_BAD_ALIGN,
              "gemm_down: pointers must be 16-byte aligned");
  return launch<MODE_DOWN>(hq, sh, nullptr, w_down, sw_down, nullptr, nullptr, group_offsets, E, R, I, D, y_bf16,
                           nullptr, ws, ws_bytes, (hipStream_t)stream);
}
