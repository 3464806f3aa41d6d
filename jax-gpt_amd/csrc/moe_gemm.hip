// Grouped fp8 GEMMs over ragged expert row ranges on the CDNA4 fp8 matrix cores.
//
// Replaces the three jax.lax.ragged_dot calls of
// jax_gpt/models/qwen35/moe.py:83-87 (_expert_swiglu):
//   MODE_GATEUP: h = silu(x . Wgate[e]^T) * (x . Wup[e]^T), then 1x128 e4m3 quantisation of h
//   MODE_DOWN:   y = h . Wdown[e]^T, bf16
// for the rows [group_offsets[e], group_offsets[e+1]) of every expert e.
//
// Arithmetic.  Both operands are K-contiguous e4m3 with one f32 scale per 128
// K-elements (activations: per row; weights: per 128 rows), so one
// v_mfma_f32_16x16x128_f8f6f4 consumes exactly one scale block: its 16x16 f32
// result is a partial sum that is multiplied by sx[row,kb]*sw[nblk,kb] and
// added to the f32 accumulator on the vector ALU (the matrix unit has no f32
// scale input).  The weight fragment is the MFMA's row operand and the
// activation fragment its column operand, so a lane holds four weight rows of
// ONE activation row: one activation scale per lane per fragment, not four.
//
// Data movement.  A workgroup (8 waves, two per SIMD, one workgroup per CU) owns a
// work item = (expert, <= 256 activation rows, 256 weight rows) and walks K in
// steps of 128 through a ring of LDS stages.  Tiles are copied global -> LDS by
// global_load_lds (no registers in between) ahead of their use, by one wave of
// each SIMD (wave set 0); the other (set 1) only computes.  In
// MODE_GATEUP the 256 weight rows are 128 gate rows + the 128 up rows of the
// same output columns, so silu(g)*u is lane-local and the 1x128 amax stays
// inside the workgroup.  Waves form a 4 x 2 grid: wave (wi, xj) owns weight rows
// {32wi..32wi+31} of each half (GATEUP) or {64wi..64wi+63} (DOWN) against the
// 16-row activation fragments 2j + xj (alternating between the two wave sets, so
// a short tile still splits evenly).
//
// What bounds a work item.  A K step of a full tile moves 64 KB into LDS (72 copy instructions per CU) and holds
// 2048 matrix-core cycles per SIMD.  The L2 can fill one CU's LDS at about 125 GB/s with this copy pattern (all CUs
// at once); a CU streaming alone from HBM gets about 22 GB/s whatever its queue depth, and all 256 together reach
// the memory's rate.  The activation tile is shared by the item's 16 column blocks and comes from L2, the weight
// tile comes from L2 when a neighbouring row tile of the same expert has just fetched it and from HBM or the
// memory-side cache otherwise (always, for an expert of one row tile).  An expert of few rows is therefore a
// weight stream at the per-CU HBM rate whatever the kernel does with its rows; the kernel's part is to keep that
// stream and the large experts' matrix work going side by side on different CUs, and to waste neither.  Measured
// on full tiles, the copies cost the loop a quarter of its speed even from an L2-hot source: it is their issue
// (address generation, back-pressure from the L1) in the instruction stream of the waves that feed the matrix core.
//
// Row tiles are listed on the device (build_tiles_kernel here, or the permutation
// kernels inside moe_forward: no host read-back of group sizes); a workgroup's
// work item is a (row tile, column block) pair derived from its index, in
// [expert][column block][row tile] order, and the items are dealt to the 8 XCDs in
// contiguous ranges, so the row tiles and column blocks that share a weight slab
// or an activation tile run together under one L2.  The items of the smallest
// experts (weight streams, nothing to share) are not dealt out: they sit behind
// the eight ranges as a pool from which the workgroups that follow an XCD's range
// draw one item each through a counter (TileHeader), so an XCD that is ahead
// takes more of them.
#include <stdlib.h>

#include <mutex>
#include <type_traits>

#include "moe_common.h"

// Tile list of moe_gemm_gateup_swiglu_fp8_static: one copy per GPU, held until the process ends.  In host code this
// name is only a handle for hipGetSymbolAddress; kernels get the address that call returns.
static __device__ __align__(256) unsigned char scratch[MOE_STATIC_SCRATCH_BYTES];

namespace {

constexpr int BW = 256;       // weight rows per work item
constexpr int BK = 128;       // K step = scale block
constexpr int NWAVES = 8;
constexpr int NT = 64 * NWAVES;
constexpr int MODE_GATEUP = 0;
constexpr int MODE_DOWN = 1;
constexpr int MAX_KB = 256;   // K <= 32768
constexpr int W_TILE_BYTES = BW * BK;   // 32 KB
constexpr int ROTC = 2;       // MFMA groups by which wave set 1 trails wave set 0 (measured: 1 to 3 within 2 %)

// ---- work list -----------------------------------------------------------

// One workgroup lists the row tiles of every expert (an expert's tiles side by side; which expert where: see
// moe_tile_first); thread e owns expert e.
// (dense_rows >= 0: one group of that many rows, whatever group_offsets holds -- the shared expert)
__global__ __launch_bounds__(1024) void build_tiles_kernel(const int32_t* __restrict__ group_offsets, int E,
                                                          TileList l, int dense_rows) {
  __shared__ int s_rows[1024];
  __shared__ int s_key[1024];
  const int e = threadIdx.x;
  int start = 0, rows = 0;
  if (dense_rows >= 0) {
    rows = e == 0 ? dense_rows : 0;
  } else if (e < E) {
    start = group_offsets[e];
    rows = group_offsets[e + 1] - start;
  }
  const int tiles = moe_tile_count(rows);
  int total = 0;
  const int first = moe_tile_first(e, E, rows, s_rows, s_key, &total, l.hdr, l.max_tiles);
  for (int t = 0; t < tiles; ++t)
    if (first + t < l.max_tiles) l.tiles[first + t] = TileEntry{e, start, rows, first};   // (cannot overflow for consistent offsets)
}

// ---- the kernel ------------------------------------------------------------------------------------------------
//
// LDS = [ring of weight tiles 256 x 128 B][ring of (activation tile 32 XF x 128 B, its 32 XF activation scales)].
// Tiles are row-major with 128-byte rows; the 16-byte chunk c of row r sits at chunk position
// c ^ ((r >> 1) & 7).  A fragment lane (row fr = lane % 16, quarter fq = lane / 16) feeds the
// MFMA with K bytes [16 fq, +16) and [64 + 16 fq, +16) of its row -- the same choice for both
// operands, so the contraction is unchanged -- which makes every ds_read_b128 of a fragment
// conflict-free (measured ~240 B/clk/CU against ~125 B/clk for 32 contiguous bytes per lane).
// global_load_lds_dwordx4 writes LDS base + lane * 16, i.e. one wave instruction fills 8
// consecutive tile rows; the swizzle is applied by choosing which 16-byte piece of the row
// each lane fetches.  No asynchronous load ever targets a register.

// epilogue staging tile: 128-byte rows, chunk c of row r at position c ^ (r & 7)
__device__ __forceinline__ int swz(int row, int chunk) { return row * BK + ((chunk ^ (row & 7)) << 4); }

// One launch, row tiles of every height.  A work item's row tile (at most 256 rows, near-equal cuts of its
// expert) is served by the smallest of eight compiled tile classes that holds it -- 32 XF rows, XF = 1 .. 8 MFMA
// groups per wave and K step -- each a branch-free, fully unrolled K loop of its own with its own LDS ring: the
// short classes have short activation tiles and use the room for more stages (256 rows: two stages; 160 to 224
// rows: three weight stages, two activation stages; 64 to 128 rows: three stages, copies two steps ahead; 32 rows:
// four stages, three steps ahead), because an item of a few rows only streams its 256 weight rows and lives on the
// bytes it keeps in flight.  Rows past the end of a tile are multiplied like the others (their copies re-read the tile's last
// row) and never stored.
//
// K step of a wave: XF groups; group j = its four weight fragments against activation fragment j (4 MFMAs, results
// in p[0..3]).  The 16 FMAs that scale group j's results into the accumulators are issued between the MFMAs of
// group j + 1 -- FMA quadruple f just before MFMA f, which overwrites p[f] -- so the matrix core works on the next
// group while the vector ALU finishes the last one, with one set of result registers.  The last group of a step is
// finished behind the next step's barrier, while that step's first fragments travel from LDS.
template <int XF, int MODE = MODE_GATEUP> struct Cls {
  static constexpr int BM = 32 * XF, HALF = BM / 2;
  // Two rings: weight tiles (32 KB each) and activation tiles with their scales.  Where 160 KB allow it the weight
  // ring is one stage deeper than the activation ring (160 to 224 rows: three weight stages, two activation
  // stages): the weight tile is the one that may come from HBM, the activation tile is shared by the item's column
  // blocks and comes from L2.  Measured on the loop's skeleton, weights two steps ahead instead of one: 5-7 % on a
  // weight slab that four workgroups share or that a workgroup streams alone, nothing when every line is an L2 hit.
  static constexpr int X_NST = XF >= 5 ? 2 : XF >= 2 ? 3 : 4;
  static constexpr int W_NST = XF == 8 ? 2 : XF >= 2 ? 3 : 4;
  // A weight stage is read once per step: every wave loads its four weight fragments into registers when it enters
  // the step, and from then on the stage is free.  With W_EARLY the next tenant's copies are issued right there, in
  // the middle of the step, and not behind the next barrier: the weights of step kb + 2 are then in flight while step
  // kb still computes, as if the ring were a stage deeper, in the same LDS.  The weight rows that wave (wi, 0) copies
  // are read by itself and by wave (wi, 1) alone, so the release is a word in LDS between those two (early_flag)
  // and no barrier.  Only the 256-row class of the gate/up GEMM, which has no room for a third stage: -4.5 % where
  // every workgroup streams its own weight slab, -3 % where 8 row tiles share one, -1 % on the mixed tile
  // heights of skewed routing; the down GEMM (16 K steps at the DeepSeek-V3 shape) gained 2 % in the first case and
  // lost 1 % in the second, and the classes with three weight stages cannot gain: their copies complete in issue
  // order behind the activation copies of the step before, which must have landed a step earlier.
  static constexpr bool W_EARLY = XF == 8 && MODE == MODE_GATEUP;
  static constexpr int EARLY_G = 3;   // the group behind which the weight copies of a W_EARLY step begin (2 and 4: within 1 %)
  static constexpr int X_PRE = X_NST - 1, W_PRE = W_NST - 1 + (W_EARLY ? 1 : 0);   // steps that a copy runs ahead of its use
  static constexpr int X_STAGE_S_OFF = BM * BK;                // the scales behind the tile
  // + 256: every copying wave copies 64 scale slots from its first one on (no lane mask, which would cut the
  // unrolled K step into blocks); the surplus lanes rewrite other waves' slots with the same values or land in this pad
  static constexpr int X_STAGE_BYTES = BM * BK + BM * 4 + 256;
  static constexpr int X_RING_OFF = W_NST * W_TILE_BYTES;
  static constexpr int RING_BYTES = X_RING_OFF + X_NST * X_STAGE_BYTES;
  // Only wave set 0 (waves 0-3) issues copies: a copy instruction can hold its wave at the memory pipeline's door
  // while the L1's queue is full, and with one wave of each SIMD never there the matrix core always has a wave that
  // can feed it (2-3 % over all eight waves copying).  Wave v copies 8 weight row groups (the rows that it reads
  // itself), activation row groups v, v + 4, ... and 64 scale slots.
  static constexpr int X_OPS = XF;                     // activation copies per copying wave and step
  static constexpr int XS_OPS = X_OPS + 1;             // + 1 scale copy
  static constexpr int OPS = 8 + XS_OPS;               // + 8 weight row groups
  // Copies complete in the order of their issue, so within a step those with the earlier deadline go first: with
  // the deeper weight ring the activation copies (and scales), then the weights; with rings of one depth the
  // weights first (they are the ones that may miss).
  static constexpr bool X_FIRST = W_PRE > X_PRE;
  static constexpr bool is_w(int i) { return X_FIRST ? i >= XS_OPS : i < 8; }
  static constexpr int w_index(int i) { return X_FIRST ? i - XS_OPS : i; }
  static constexpr bool is_s(int i) { return X_FIRST ? i == X_OPS : i == OPS - 1; }
  static constexpr int x_index(int i) { return X_FIRST ? i : i - 8; }
  // what may still be in flight when a step starts that found every later copy issued: the activation stages and
  // weight stages of the steps after it
  static constexpr int IN_FLIGHT = (X_PRE - 1) * XS_OPS + (W_PRE - 1) * 8;
  // The same count for a step rem = KB - 1 - kb steps from the item's end: the copies issued behind the last one that
  // the step needs (its activation tile and scales, from X_PRE steps back), where a step that is r steps from the
  // end issued activation copies if r >= X_PRE and weight copies if r >= W_PRE.
  static constexpr int allowed(int rem) {
    int n = 0;
    if (X_FIRST && rem + X_PRE >= W_PRE) n += 8;   // the weight copies behind the needed ones in their own step
    for (int r = rem + X_PRE - 1; r > rem; --r) n += (r >= X_PRE ? XS_OPS : 0) + (r >= W_PRE ? 8 : 0);
    return n;
  }
  static_assert(allowed(W_PRE + X_PRE) == IN_FLIGHT, "the steady state of the rule is the count above");
  // copy operations issued after group g: spread over the first SPREAD groups of the step.  Rings of one depth must
  // have the step's copies out early (they land before the next barrier or hold it up); with the deeper weight ring
  // the weight copies have a step more, and an even spread over the whole step is best (all groups against the
  // first three: gate/up -2 to -4 %, down -1 to -3 % on tiles of 160-224 rows; all at once: +2 %)
  static constexpr int SPREAD = X_FIRST ? XF : XF >= 6 ? XF / 2 : XF >= 3 ? 3 : XF;
  // (W_EARLY: the activation copies and scales behind groups 0 .. EARLY_G - 1, the weight copies behind the rest)
  static constexpr int first(int g) {
    if (W_EARLY)
      return g <= 0 ? 0 : g < EARLY_G ? (XS_OPS * g) / EARLY_G : g >= XF ? OPS : XS_OPS + (8 * (g - EARLY_G)) / (XF - EARLY_G);
    return g <= 0 ? 0 : g >= SPREAD ? OPS : (OPS * g) / SPREAD;
  }
};
constexpr int cmax(int a, int b) { return a > b ? a : b; }
constexpr int CLS_RING = cmax(cmax(cmax(Cls<8>::RING_BYTES, Cls<7>::RING_BYTES), cmax(Cls<6>::RING_BYTES, Cls<5>::RING_BYTES)),
                              cmax(cmax(Cls<4>::RING_BYTES, Cls<3>::RING_BYTES), cmax(Cls<2>::RING_BYTES, Cls<1>::RING_BYTES)));
constexpr int CLS_WSCALE_OFF = CLS_RING;                       // [2][MAX_KB] weight block scales of the work item
constexpr int CLS_FLAG_OFF = CLS_WSCALE_OFF + 2 * MAX_KB * 4;  // [4] early_flag: the step whose weight fragments wave (wi, 1) holds, + 1
constexpr int CLS_LDS_BYTES = CLS_FLAG_OFF + 16;              // 160016; the epilogues stage through the ring (<= 128 KB)
static_assert(CLS_LDS_BYTES <= 160 * 1024, "LDS");

struct Item { int expert, row_start, row_count, col_block; };

template <int MODE, int XF>
__device__ __forceinline__ void item_body(const Item& item, uint8_t* lds, const uint8_t* __restrict__ xq,
                                          const float* __restrict__ sx, const int32_t* __restrict__ row_ids,
                                          const uint8_t* __restrict__ w0, const float* __restrict__ sw0,
                                          const uint8_t* __restrict__ w1, const float* __restrict__ sw1, int K, int N,
                                          void* __restrict__ out, float* __restrict__ out_scale, const GemmScales sc) {
  using C = Cls<XF, MODE>;
  constexpr int BM = C::BM, HALF = C::HALF;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wi = wave & 3, xj = wave >> 2;
  const int fr = lane & 15, fq = lane >> 4;
  const int KB = K / BK;
  const int e = item.expert;
  const int wrow0 = MODE == MODE_GATEUP ? item.col_block * 128 : item.col_block * 256;

  // ---- copy sources: copying wave cv (waves 0-3; 4-7 compute the same values and never use them) fills the weight
  // rows that the waves wi = cv read (down: tile rows [64 cv, +64); gate/up: [32 cv, +32) of the gate half and of
  // the up half), activation row groups cv, cv + 4, ... and 64 scale slots
  const int drow = lane >> 3, dchunk = lane & 7;
  const int cv = wave & 3;
  const uint8_t* wmat = w0 + (size_t)e * N * K;   // uniform
  const uint8_t* wmat1 = MODE == MODE_GATEUP ? w1 + (size_t)e * N * K : wmat;
  unsigned woff[2];
  {
    int grow = MODE == MODE_GATEUP ? wrow0 + cv * 32 : wrow0 + cv * 64;
    if (MODE == MODE_DOWN && grow >= N) grow = N - 64;   // (a half-full last column block: re-read valid rows)
    const int piece = dchunk ^ (drow >> 1);
    woff[0] = (unsigned)(grow + drow) * (unsigned)K + piece * 16;
    woff[1] = (unsigned)(grow + drow) * (unsigned)K + (piece ^ 4) * 16;
  }
  unsigned xoff[C::X_OPS];
#pragma unroll
  for (int i = 0; i < C::X_OPS; ++i) {
    const int grp = i * 4 + cv;
    const int r = grp * 8 + drow;                              // row within the activation tile
    const int piece = dchunk ^ ((r >> 1) & 7);
    int g = item.row_start + min(r, item.row_count - 1);
    if (row_ids) g = row_ids[g];
    xoff[i] = (unsigned)g * (unsigned)K + piece * 16;
  }
  const int sbase = BM >= 64 ? min(cv * 64, BM - 64) : 0;   // first of the 64 scale slots this wave copies
  unsigned soff;
  {
    const int p = min(sbase + lane, BM - 1);   // slots past the tile land in the pad
    const int q = p % HALF;
    const int r = 16 * (2 * (q % XF) + p / HALF) + q / XF;
    int g = item.row_start + min(r, item.row_count - 1);
    if (row_ids && !sc.in_listed) g = row_ids[g];
    soff = (unsigned)g * (unsigned)sc.in_row * 4u;
  }
  const unsigned lds0 = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)lds);
  // copies of step t's operands: weight row group w of this wave, activation row group x, the scales
  auto copy_w = [&](int t, int w) {
    if (MODE == MODE_GATEUP)   // row groups 0-3 of the wave's gate rows, then of its up rows (tile rows 128 ..)
      dma16((w < 4 ? wmat : wmat1) + (size_t)t * BK + (size_t)(w & 3) * 8 * K, woff[w & 1],
            lds0 + (unsigned)(t % C::W_NST) * W_TILE_BYTES + ((w < 4 ? 0 : 16) + cv * 4 + (w & 3)) * 1024u);
    else
      dma16(wmat + (size_t)t * BK + (size_t)w * 8 * K, woff[w & 1], lds0 + (unsigned)(t % C::W_NST) * W_TILE_BYTES + (cv * 8 + w) * 1024u);
  };
  auto copy_x = [&](int t, int x) {
    dma16(xq + (size_t)t * BK, xoff[x], lds0 + C::X_RING_OFF + (unsigned)(t % C::X_NST) * C::X_STAGE_BYTES + (x * 4 + cv) * 1024u);
  };
  auto copy_s = [&](int t) {
    dma4((const uint8_t*)(sx + (size_t)t * sc.in_kb), soff,
         lds0 + C::X_RING_OFF + (unsigned)(t % C::X_NST) * C::X_STAGE_BYTES + C::X_STAGE_S_OFF + sbase * 4u);
  };
  // operation i of the copies that step kb issues: each kind runs its ring's depth ahead of its use
  auto issue_op = [&](int kb, int i) {
    if (C::is_w(i)) copy_w(kb + C::W_PRE, C::w_index(i));
    else if (C::is_s(i)) copy_s(kb + C::X_PRE);
    else copy_x(kb + C::X_PRE, C::x_index(i));
  };
  if (xj == 0) {
    // what the steps before the first would have issued, in their order (completion is counted in issue order)
#pragma unroll
    for (int j = -C::W_PRE; j < 0; ++j) {
#pragma unroll
      for (int i = 0; i < C::OPS; ++i) {
        const int t = j + (C::is_w(i) ? C::W_PRE : C::X_PRE);
        if (t >= 0 && t < KB) issue_op(j, i);
      }
    }
  }

  volatile int* early_flag = (volatile int*)(lds + CLS_FLAG_OFF);
  if (C::W_EARLY && tid < 4) early_flag[tid] = 0;
  const unsigned my_flag = lds0 + CLS_FLAG_OFF + wi * 4;
  float* wscale = (float*)(lds + CLS_WSCALE_OFF);
  for (int i = tid; i < 2 * KB; i += NT) {
    const int h = i >= KB, kk = h ? i - KB : i;
    float v;
    if (MODE == MODE_GATEUP) v = (h ? sw1 : sw0)[((size_t)e * (N / 128) + item.col_block) * KB + kk];
    else v = sw0[((size_t)e * (N / 128) + min(item.col_block * 2 + h, N / 128 - 1)) * KB + kk];
    wscale[h * MAX_KB + kk] = v;
  }
  const float* ws0 = wscale + (MODE == MODE_GATEUP ? 0 : (wi >> 1) * MAX_KB);
  const float* ws1 = wscale + MAX_KB;   // GATEUP only
  __syncthreads();   // (the compiler waits here for the scale loads, and with them for the copies issued above)

  const int lane_off0 = fr * BK + ((fq ^ (fr >> 1)) << 4);         // K bytes [16 fq, +16)
  const int lane_off1 = fr * BK + (((fq + 4) ^ (fr >> 1)) << 4);   // K bytes [64 + 16 fq, +16)
  int wfrag_off[4];
#pragma unroll
  for (int f = 0; f < 4; ++f)
    wfrag_off[f] = (MODE == MODE_GATEUP ? ((f >> 1) * 128 + wi * 32 + (f & 1) * 16) : (wi * 64 + f * 16)) * BK;
  auto read_frag = [&](const uint8_t* base) {
    const v4i lo = *(const v4i*)(base + lane_off0);
    const v4i hi = *(const v4i*)(base + lane_off1);
    return (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };

  v4f acc[4][XF];
#pragma unroll
  for (int f = 0; f < 4; ++f)
#pragma unroll
    for (int j = 0; j < XF; ++j) acc[f][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  v8i wf[4];
  v4f p[4];
  float pc0 = 0.f, pc1 = 0.f;   // scales of the group whose FMAs are pending
  auto fm = [&](int f, int jj, float c0, float c1) {
    acc[f][jj] += p[f] * ((MODE == MODE_GATEUP && f >= 2) ? c1 : c0);
  };
  auto mm = [&](int f, const v8i& x) {
    p[f] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[f], x, (v4f){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
  };
  auto fence = [&]() {
    __builtin_amdgcn_sched_barrier(0);
  };
  // The two waves of a SIMD belong to different wave sets (xj = 0 / 1).  Set 1 runs ROT groups behind set 0: it
  // carries the last ROT activation fragments of a step (and their scales) in registers across the barrier and
  // multiplies them, against the previous step's weights, first thing behind it -- so one wave of each SIMD has
  // matrix work in registers while the other waits for its first fragments from LDS.
  auto run = [&](auto rot_c, auto issue_c) {
    constexpr int ROT = decltype(rot_c)::value;
    constexpr bool ISSUE = decltype(issue_c)::value;   // this wave set issues the copies (and waits for them)
    constexpr int NG = XF - ROT;   // groups of the current step done before the next barrier
    constexpr int NH = ROT > 0 ? ROT : 1;
    v8i held[NH];
    float hc0[NH], hc1[NH];
    // copy_c: what the step issues -- 2: every copy; 1: the activation tile and scales only (the deeper weight
    // ring has reached the item's last K block); 0: nothing
    auto step = [&](int kb, auto first_c, auto copy_c) {
      constexpr bool FIRST = decltype(first_c)::value;
      constexpr int KIND = decltype(copy_c)::value;
      constexpr bool COPY = KIND > 0 && ISSUE;
      constexpr int NOPS = KIND == 2 ? C::OPS : C::XS_OPS;   // (KIND 1 exists only where the activation copies come first)
      // stage kb of both rings has landed once only the copies of later steps are outstanding
      if (!ISSUE) {
        // (the copying waves wait for their copies before the barrier; this set has none in flight)
      } else if (KIND == 2) {
        wait_vm<C::IN_FLIGHT>();
      } else {
        const int rem = KB - 1 - kb;        // the last steps: fewer and fewer copies are in flight
        static_assert(C::W_PRE <= 3, "steps that issue no weight copies are less than W_PRE from the end");
        if (rem >= 2) wait_vm<C::allowed(2)>();
        else if (rem == 1) wait_vm<C::allowed(1)>();
        else wait_vm<0>();
      }
      if (ROT > 0) wait_lgkm0();      // this wave's reads of stage kb - 1 are done before anyone overwrites it
      __builtin_amdgcn_s_barrier();   // stage kb is complete for every wave; every wave is done with stage kb - 1
      if constexpr (ROT > 0) {        // groups NG .. XF-1 of the previous step: held fragments, the previous weights
        if (!FIRST) {
#pragma unroll
          for (int i = 0; i < ROT; ++i) {
#pragma unroll
            for (int f = 0; f < 4; ++f) {
              fm(f, NG + i - 1, pc0, pc1);
              mm(f, held[i]);
            }
            pc0 = hc0[i];
            pc1 = hc1[i];
            if (COPY) {
#pragma unroll
              for (int o = C::first(i); o < C::first(i + 1); ++o)
                if (o < NOPS) issue_op(kb, o);
            }
            fence();
          }
        } else if (COPY) {
#pragma unroll
          for (int o = 0; o < C::first(ROT); ++o)
            if (o < NOPS) issue_op(kb, o);
        }
      }
      const uint8_t* wt = lds + (kb % C::W_NST) * W_TILE_BYTES;
      const uint8_t* xs = lds + C::X_RING_OFF + (kb % C::X_NST) * C::X_STAGE_BYTES;
      const float s0 = ws0[kb], s1 = MODE == MODE_GATEUP ? ws1[kb] : s0;
      const uint8_t* xt = xs + xj * 16 * BK;
      // Every wave of a wave set asks LDS for its first fragments at this moment: the reads come back in issue
      // order, so the first MFMA's operands (activation fragment 0, weight fragment 0) are asked for first and the
      // scales last; the FMAs that finish the previous step's last group run while the reads travel.
      v8i xf[2];
      xf[0] = read_frag(xt);
#pragma unroll
      for (int f = 0; f < 4; ++f) wf[f] = read_frag(wt + wfrag_off[f]);
      float sxv[XF];
      {
        const uint8_t* sp = xs + C::X_STAGE_S_OFF + xj * HALF * 4 + fr * XF * 4;
        if constexpr (XF % 4 == 0) {
#pragma unroll
          for (int j = 0; j < XF; j += 4) {
            const v4f a = *(const v4f*)(sp + j * 4);
            sxv[j] = a[0]; sxv[j + 1] = a[1]; sxv[j + 2] = a[2]; sxv[j + 3] = a[3];
          }
        } else if constexpr (XF % 2 == 0) {
#pragma unroll
          for (int j = 0; j < XF; j += 2) {
            const float2 a = *(const float2*)(sp + j * 4);
            sxv[j] = a.x; sxv[j + 1] = a.y;
          }
        } else {
#pragma unroll
          for (int j = 0; j < XF; ++j) sxv[j] = *(const float*)(sp + j * 4);
        }
      }
      if (!FIRST) {
#pragma unroll
        for (int f = 0; f < 4; ++f) fm(f, XF - 1, pc0, pc1);
      }
      fence();
#pragma unroll
      for (int j = 0; j < NG; ++j) {
        if (j + 1 < NG) xf[(j + 1) & 1] = read_frag(xt + (j + 1) * 32 * BK);
        if (ROT > 0 && j == 0) {
#pragma unroll
          for (int i = 0; i < ROT; ++i) {
            held[i] = read_frag(xt + (NG + i) * 32 * BK);
            hc0[i] = sxv[NG + i] * s0;
            hc1[i] = sxv[NG + i] * s1;
          }
        }
#pragma unroll
        for (int f = 0; f < 4; ++f) {
          if (j > 0) fm(f, j - 1, pc0, pc1);
          mm(f, xf[j & 1]);
        }
        // pinned order: the next group's fragment reads first (a whole group of latency cover), then FMA quadruple f
        // just before MFMA f (left alone the compiler puts all 16 FMAs before the 4 MFMAs: down GEMM 3-6 % slower)
        if (j + 1 < NG) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        if (ROT > 0 && j == 0) {
#pragma unroll
          for (int i = 0; i < ROT; ++i) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
#pragma unroll
        for (int f = 0; f < 4; ++f) {
          if (j > 0) __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        pc0 = sxv[j] * s0;
        pc1 = sxv[j] * s1;
        if (C::W_EARLY && COPY && KIND == 2 && ROT + j == C::EARLY_G) {
          // The weight copies from here on overwrite the stage that this step reads: this wave is past its own
          // fragment loads; the other reader of its rows, wave (wi, 1), says so through early_flag.  (It entered the
          // step through the same barrier and signals without waiting for anyone: the loop ends.  Inline assembly
          // so that the unrolled step stays one block for the scheduler.)
          fence();
          int seen;
          asm volatile("1:\n\tds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)\n\tv_cmp_ge_i32 vcc, %2, %0\n\ts_cbranch_vccnz 1b"
                       : "=&v"(seen) : "v"(my_flag), "s"(kb) : "vcc", "memory");
          fence();
        }
        if (COPY) {
#pragma unroll
          for (int o = C::first(ROT + j); o < C::first(ROT + j + 1); ++o)
            if (o < NOPS) issue_op(kb, o);
        }
        fence();
        if (C::W_EARLY && !ISSUE && j == 0) {
          // behind the MFMAs of the first group with this step's weights: all four weight fragments are in registers
          early_flag[wi] = kb + 1;   // (every lane, one value: no branch)
          fence();
        }
      }
    };
    constexpr std::true_type yes{};
    constexpr std::false_type no{};
    constexpr std::integral_constant<int, 2> all{};
    constexpr std::integral_constant<int, 1> x_only{};
    constexpr std::integral_constant<int, 0> none{};
    const int n_all = KB - C::W_PRE;   // steps 0 .. n_all-1 issue every copy
    const int n_x = KB - C::X_PRE;     // steps up to n_x-1 still issue the activation tile of a later step
    if (n_all > 0) {
      step(0, yes, all);
    } else {
      bool done = false;
      if constexpr (C::X_FIRST) {
        if (n_x > 0) {
          step(0, yes, x_only);
          done = true;
        }
      }
      if (!done) step(0, yes, none);
    }
    int kb = 1;
    for (; kb < n_all; ++kb) step(kb, no, all);
    if constexpr (C::X_FIRST) {
      for (; kb < n_x; ++kb) step(kb, no, x_only);
    }
    for (; kb < KB; ++kb) step(kb, no, none);
    if constexpr (ROT > 0) {   // the groups carried out of the last step
#pragma unroll
      for (int i = 0; i < ROT; ++i) {
#pragma unroll
        for (int f = 0; f < 4; ++f) {
          fm(f, NG + i - 1, pc0, pc1);
          mm(f, held[i]);
        }
        pc0 = hc0[i];
        pc1 = hc1[i];
      }
    }
#pragma unroll
    for (int f = 0; f < 4; ++f) fm(f, XF - 1, pc0, pc1);
  };
  constexpr int ROT1 = XF > ROTC ? ROTC : XF - 1;   // (fewer groups than that: what there is)
  if (xj == 0) run(std::integral_constant<int, 0>{}, std::true_type{});
  else run(std::integral_constant<int, ROT1>{}, std::false_type{});
  __syncthreads();   // every wave is done reading the ring before the epilogue reuses LDS

  // ---- epilogue.  Lane holds, for fragment (f, j): tile row (2j + xj)*16 + fr, weight rows (fragment base) + 4*fq + {0..3}.
  if (MODE == MODE_GATEUP) {
    float* amax_s = (float*)lds;                       // [4 weight-wave groups][BM rows]
    uint8_t* tile = lds + 4 * BM * sizeof(float);      // [BM rows][128 B], swizzled
#pragma unroll
    for (int j = 0; j < XF; ++j) {
      float m = 0.f;
#pragma unroll
      for (int f = 0; f < 2; ++f)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float g = acc[f][j][r], u = acc[f + 2][j][r];
          float h = g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u;   // (reciprocal to 1 ulp: far inside the fp8 step)
          acc[f][j][r] = h;
          m = fmaxf(m, fabsf(h));
        }
      m = fmaxf(m, __shfl_xor(m, 16, MOE_WAVE));
      m = fmaxf(m, __shfl_xor(m, 32, MOE_WAVE));
      if (fq == 0) amax_s[wi * BM + (2 * j + xj) * 16 + fr] = m;
    }
    __syncthreads();
    const int I = N;
    uint8_t* hq = (uint8_t*)out;
#pragma unroll
    for (int j = 0; j < XF; ++j) {
      const int xr = (2 * j + xj) * 16 + fr;
      float m = fmaxf(fmaxf(amax_s[xr], amax_s[BM + xr]), fmaxf(amax_s[2 * BM + xr], amax_s[3 * BM + xr]));
      float scale, scale_inv;
      fp8_scales(m, scale, scale_inv);
#pragma unroll
      for (int f = 0; f < 2; ++f) {
        int q = 0;   // (|h| <= amax, so the products stay within a rounding of +-448: one median clamps them)
        q = __builtin_amdgcn_cvt_pk_fp8_f32(__builtin_amdgcn_fmed3f(acc[f][j][0] * scale, -MOE_FP8_MAX, MOE_FP8_MAX),
                                            __builtin_amdgcn_fmed3f(acc[f][j][1] * scale, -MOE_FP8_MAX, MOE_FP8_MAX), q, false);
        q = __builtin_amdgcn_cvt_pk_fp8_f32(__builtin_amdgcn_fmed3f(acc[f][j][2] * scale, -MOE_FP8_MAX, MOE_FP8_MAX),
                                            __builtin_amdgcn_fmed3f(acc[f][j][3] * scale, -MOE_FP8_MAX, MOE_FP8_MAX), q, true);
        const int col = wi * 32 + f * 16 + fq * 4;  // byte column within the 128-wide slab
        *(unsigned*)(tile + swz(xr, col >> 4) + (col & 15)) = q;
      }
      if (wi == 0 && fq == 0 && xr < item.row_count)
        out_scale[(size_t)(item.row_start + xr) * sc.out_row + (size_t)item.col_block * sc.out_cb] = scale_inv;
    }
    __syncthreads();
    const int ld_chunk = tid & 7, ld_row = tid >> 3;   // 64 rows per pass
#pragma unroll
    for (int i = 0; i < (BM + 63) / 64; ++i) {
      const int r = ld_row + 64 * i;
      if (r < item.row_count) {
        v4i v = *(const v4i*)(tile + swz(r, ld_chunk));
        *(v4i*)(hq + (size_t)(item.row_start + r) * I + item.col_block * 128 + ld_chunk * 16) = v;
      }
    }
  } else {
    // bf16 tile [BM rows][256 cols] = 512 B per row, 32 chunks of 16 B, swizzled with (row & 7)
    uint8_t* tile = lds;
#pragma unroll
    for (int j = 0; j < XF; ++j) {
      const int xr = (2 * j + xj) * 16 + fr;
#pragma unroll
      for (int f = 0; f < 4; ++f) {
        const int col = wi * 64 + f * 16 + fq * 4;  // output column within the 256-wide slab
        uint2 v;
        v.x = pack2_bf16(acc[f][j][0], acc[f][j][1]);
        v.y = pack2_bf16(acc[f][j][2], acc[f][j][3]);
        const int chunk = col >> 3;  // 8 bf16 per 16-byte chunk
        *(uint2*)(tile + xr * 512 + ((chunk ^ (xr & 7)) << 4) + (col & 7) * 2) = v;
      }
    }
    __syncthreads();
    bf16_t* y = (bf16_t*)out;
    const int c32 = tid & 31, r16 = tid >> 5;          // 16 rows per pass
    const int ncols = min(256, N - wrow0);
#pragma unroll
    for (int i = 0; i < BM / 16; ++i) {
      const int r = r16 + 16 * i;
      if (r < item.row_count && c32 * 8 < ncols) {
        v4i v = *(const v4i*)(tile + r * 512 + ((c32 ^ (r & 7)) << 4));
        v4i* dst = (v4i*)(y + (size_t)(item.row_start + r) * N + wrow0 + c32 * 8);
        if (sc.stream_out) __builtin_nontemporal_store(v, dst);
        else *dst = v;
      }
    }
  }
}

template <int MODE>
__global__ __launch_bounds__(NT, 1) void grouped_gemm_kernel(
    const uint8_t* __restrict__ xq, const float* __restrict__ sx, const int32_t* __restrict__ row_ids,
    const uint8_t* __restrict__ w0, const float* __restrict__ sw0, const uint8_t* __restrict__ w1,
    const float* __restrict__ sw1, TileHeader* hdr, const TileEntry* __restrict__ tiles, int K,
    int N, void* __restrict__ out, float* __restrict__ out_scale, const GemmScales sc) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  // work items = (row tile, column block) pairs in [expert][column block][row tile] order, dealt to the 8 XCDs in
  // contiguous ranges of about equal cost (workgroup ids are issued round-robin over XCDs)
  const int ncb = MODE == MODE_GATEUP ? N / 128 : (N + 255) / 256;
  const int xcd = blockIdx.x & 7;
  int item_id = (int)((hdr->xcd_q[xcd] * ncb) >> kTileQBits) + (int)(blockIdx.x >> 3);
  const int share_end = (int)((hdr->xcd_q[xcd + 1] * ncb) >> kTileQBits);
  if (item_id >= share_end) {
    // behind the XCD's fixed share: the pool of the smallest experts' items, drawn one at a time by whoever gets
    // there (TileHeader); an XCD may draw up to twice its eighth of it
    const int pool_first = hdr->n_static * ncb;
    const int pool_items = (hdr->n_tiles - hdr->n_static) * ncb;
    if (pool_items == 0 || item_id - share_end >= moe_pool_workgroups(pool_items)) return;   // (uniform: the whole workgroup leaves)
    int* slot = (int*)lds;
    if (threadIdx.x == 0) *slot = atomicAdd(&hdr->pool_next[MODE], 1);   // (the one field of the list a GEMM writes)
    __syncthreads();
    const int drawn = *slot;
    __syncthreads();   // (the work item's first copies overwrite the slot)
    if (drawn >= pool_items) return;
    item_id = pool_first + drawn;
  }
  Item item;
  {
    const TileEntry te = tiles[item_id / ncb];   // entries [first_tile, first_tile + tiles) all describe this expert
    const int nt = moe_tile_count(te.rows);
    const int local = item_id - te.first_tile * ncb;
    int rt;
    if (nt < 16) {
      item.col_block = nt == 1 ? local : local / nt;
      rt = local - item.col_block * nt;
    } else {
      // An expert of many row tiles goes through its column blocks once per group of 8 to 11 row tiles: the 32 CUs
      // of an XCD then work on about 8 row tiles x 4 column blocks at a time (12 distinct operand tiles per K step)
      // instead of 32 row tiles of one column block (33 distinct tiles, every CU pulling the same weight lines at
      // once): 32 row tiles per expert ran 19 % slower than 8.  Below 16 tiles a split does not pay (11 tiles as
      // 6 + 5 measured 1 % slower than unsplit).
      const int ng = nt >> 3;
      const int base = nt / ng, extra = nt - base * ng;   // the first `extra` groups hold base + 1 tiles
      const int big = (base + 1) * ncb * extra;
      int sz, l2, t0;
      if (local < big) {
        sz = base + 1;
        const int g = local / (sz * ncb);
        l2 = local - g * sz * ncb;
        t0 = g * sz;
      } else {
        sz = base;
        const int l = local - big, g = l / (sz * ncb);
        l2 = l - g * sz * ncb;
        t0 = extra * (base + 1) + g * sz;
      }
      item.col_block = l2 / sz;
      rt = t0 + (l2 - item.col_block * sz);
    }
    item.expert = te.expert;
    int t0, tn;
    moe_tile_span(te.rows, nt, rt, t0, tn);
    item.row_start = te.row_start + t0;
    item.row_count = tn;
  }
  const int rows = __builtin_amdgcn_readfirstlane(item.row_count);
#define MOE_ITEM(XF) item_body<MODE, XF>(item, lds, xq, sx, row_ids, w0, sw0, w1, sw1, K, N, out, out_scale, sc)
  switch ((rows + 31) >> 5) {
    case 8: MOE_ITEM(8); break;
    case 7: MOE_ITEM(7); break;
    case 6: MOE_ITEM(6); break;
    case 5: MOE_ITEM(5); break;
    case 4: MOE_ITEM(4); break;
    case 3: MOE_ITEM(3); break;
    case 2: MOE_ITEM(2); break;
    default: MOE_ITEM(1); break;
  }
#undef MOE_ITEM
}
int col_blocks(int mode, int N) { return mode == MODE_GATEUP ? N / 128 : (N + 255) / 256; }

int max_tiles_for(int R, int E) { return (int)((long long)(R + 255) / 256 + (E < R ? E : R)); }

TileList tile_list(void* ws, int R, int E) {
  return TileList{max_tiles_for(R, E), (TileHeader*)ws, (TileEntry*)((char*)ws + sizeof(TileHeader))};
}

template <int MODE>
int launch(const uint8_t* xq, const float* sx, const int32_t* row_ids, const uint8_t* w0, const float* sw0,
           const uint8_t* w1, const float* sw1, const int32_t* group_offsets, int E, int R, int K, int N,
           void* out, float* out_scale, void* ws, size_t ws_bytes, bool list_built, GemmScales sc, hipStream_t s) {
  const size_t need = moe_gemm_workspace_bytes(R, E, N);
  MOE_REQUIRE(ws_bytes >= need, MOE_ERR_WORKSPACE_TOO_SMALL, "gemm: workspace %zu < %zu", ws_bytes, need);
  MOE_REQUIRE(K <= MAX_KB * BK, MOE_ERR_BAD_SHAPE, "gemm: contraction length %d exceeds %d", K, MAX_KB * BK);
  MOE_REQUIRE((long long)N * K <= (1ll << 32) && (long long)R * K <= (1ll << 32), MOE_ERR_BAD_SHAPE,
              "gemm: one expert matrix and the activation array must each stay within 4 GB (N=%d K=%d R=%d)", N, K, R);
  if (R == 0) return MOE_OK;
  const TileList l = tile_list(ws, R, E);
  if (!list_built) hipLaunchKernelGGL(build_tiles_kernel, dim3(1), dim3(1024), 0, s, group_offsets, E, l, -1);
  static std::atomic<unsigned long long> lds_raised{0};
  if (int rc = moe_raise_lds_limit((const void*)grouped_gemm_kernel<MODE>, CLS_LDS_BYTES, lds_raised)) return rc;
  // An output that the memory-side cache (256 MB) cannot hold until the combine reads it goes past the caches
  // (config 3: 0.94 GB, step -0.6 %); a smaller one stays cached (config 5: 235 MB, 0.4 % slower when streamed).
  sc.stream_out = MODE == MODE_DOWN && (size_t)R * N * 2 > ((size_t)192 << 20);
  const long long max_items = (long long)l.max_tiles * col_blocks(MODE, N);
  MOE_REQUIRE(max_items < (1ll << 30), MOE_ERR_BAD_SHAPE, "gemm: %lld work items exceed the grid limit", max_items);
  // sized by the worst case of the largest XCD share (moe_xcd_share_cap_q) and of an XCD's draws from the pool;
  // surplus workgroups exit at once
  const long long pool_max = (long long)moe_pool_tile_limit(l.max_tiles) * col_blocks(MODE, N);
  const int grid = 8 * (int)((max_items + 7) / 8 + 2 + moe_pool_workgroups(pool_max));
  hipLaunchKernelGGL((grouped_gemm_kernel<MODE>), dim3(grid), dim3(NT), CLS_LDS_BYTES, s, xq, sx, row_ids, w0, sw0, w1,
                     sw1, l.hdr, l.tiles, K, N, out, out_scale, sc);
  return moe_check_hip(hipGetLastError(), "gemm launch");
}

}  // namespace

extern "C" size_t moe_gemm_workspace_bytes(int R, int E, int N_out) {
  (void)N_out;   // the tile list does not depend on the number of output columns
  return sizeof(TileHeader) + (size_t)max_tiles_for(R, E) * sizeof(TileEntry) + 256;
}

int moe_gemm_gateup_impl(const uint8_t* xq, const float* sx, const int32_t* row_ids, const uint8_t* w_gate,
                         const float* sw_gate, const uint8_t* w_up, const float* sw_up, const int32_t* group_offsets,
                         int E, int R, int D, int I, uint8_t* hq, float* sh, void* ws, size_t ws_bytes, bool list_built,
                         GemmScales sc, moe_stream_t stream) {
  MOE_REQUIRE((R == 0 || (xq && sx && hq && sh)) && w_gate && sw_gate && w_up && sw_up && group_offsets && ws, MOE_ERR_NULL,
              "gemm_gateup: null pointer");
  MOE_REQUIRE(E >= 1 && E <= 1024 && R >= 0 && D > 0 && I > 0 && D % 128 == 0 && I % 128 == 0, MOE_ERR_BAD_SHAPE,
              "gemm_gateup: need D %% 128 == 0 and I %% 128 == 0 and 1 <= E <= 1024, got E=%d R=%d D=%d I=%d", E, R, D, I);
  MOE_REQUIRE(MOE_ALIGNED16(xq) && MOE_ALIGNED16(w_gate) && MOE_ALIGNED16(w_up) && MOE_ALIGNED16(hq) && MOE_ALIGNED16(ws),
              MOE_ERR_BAD_ALIGN, "gemm_gateup: pointers must be 16-byte aligned");
  MOE_REQUIRE((long long)R * sc.in_row * 4 <= (1ll << 32) && (long long)R * sc.out_row + (long long)(I / 128) * sc.out_cb <= (1ll << 40),
              MOE_ERR_BAD_SHAPE, "gemm_gateup: scale array out of the addressable range");
  return launch<MODE_GATEUP>(xq, sx, row_ids, w_gate, sw_gate, w_up, sw_up, group_offsets, E, R, D, I, hq, sh, ws,
                             ws_bytes, list_built, sc, (hipStream_t)stream);
}

extern "C" int moe_gemm_gateup_swiglu_fp8(const uint8_t* xq, const float* sx, const int32_t* row_ids,
                                          const uint8_t* w_gate, const float* sw_gate, const uint8_t* w_up,
                                          const float* sw_up, const int32_t* group_offsets, int E, int R, int D,
                                          int I, uint8_t* hq, float* sh, void* ws, size_t ws_bytes,
                                          moe_stream_t stream) {
  return moe_gemm_gateup_impl(xq, sx, row_ids, w_gate, sw_gate, w_up, sw_up, group_offsets, E, R, D, I, hq, sh, ws,
                              ws_bytes, false, moe_row_major_scales(D, I), stream);
}

namespace {
int check_layout(int layout, const char* what) {
  MOE_REQUIRE(layout == MOE_SCALES_ROW_MAJOR || layout == MOE_SCALES_BLOCK_MAJOR, MOE_ERR_BAD_SHAPE,
              "%s: unknown scale layout %d", what, layout);
  return MOE_OK;
}
}  // namespace

extern "C" int moe_gemm_gateup_swiglu_fp8_layout(const uint8_t* xq, const float* sx, const int32_t* row_ids,
                                                 const uint8_t* w_gate, const float* sw_gate, const uint8_t* w_up,
                                                 const float* sw_up, const int32_t* group_offsets, int E, int R, int D,
                                                 int I, uint8_t* hq, float* sh, void* ws, size_t ws_bytes, int sx_layout,
                                                 int sh_layout, moe_stream_t stream) {
  if (int rc = check_layout(sx_layout, "gemm_gateup: sx")) return rc;
  if (int rc = check_layout(sh_layout, "gemm_gateup: sh")) return rc;
  GemmScales sc = moe_row_major_scales(D, I);
  if (sx_layout == MOE_SCALES_BLOCK_MAJOR) sc.in_row = 1, sc.in_kb = R, sc.in_listed = true;
  if (sh_layout == MOE_SCALES_BLOCK_MAJOR) sc.out_row = 1, sc.out_cb = R;
  return moe_gemm_gateup_impl(xq, sx, row_ids, w_gate, sw_gate, w_up, sw_up, group_offsets, E, R, D, I, hq, sh, ws,
                              ws_bytes, false, sc, stream);
}

namespace {
// The device address of `scratch` on the current device, looked up once per device.
int static_scratch(void** out) {
  static std::mutex mu;
  static void* ptrs[64] = {};
  int dev = 0;
  if (int rc = moe_check_hip(hipGetDevice(&dev), "static scratch: hipGetDevice")) return rc;
  MOE_REQUIRE(dev >= 0 && dev < 64, MOE_ERR_HIP, "static scratch: device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void* p = nullptr;
    if (int rc = moe_check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "static scratch: hipGetSymbolAddress")) return rc;
    MOE_REQUIRE(p != nullptr, MOE_ERR_HIP, "static scratch: no device address");
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  return MOE_OK;
}
}  // namespace

extern "C" int moe_gemm_gateup_swiglu_fp8_static(const uint8_t* xq, const float* sx, const int32_t* row_ids,
                                                 const uint8_t* w_gate, const float* sw_gate, const uint8_t* w_up,
                                                 const float* sw_up, const int32_t* group_offsets, int E, int R,
                                                 int D, int I, uint8_t* hq, float* sh, moe_stream_t stream) {
  MOE_REQUIRE(E >= 1 && E <= 1024 && R >= 0, MOE_ERR_BAD_SHAPE, "gemm_gateup_static: need 1 <= E <= 1024, got E=%d R=%d", E, R);
  const size_t need = moe_gemm_workspace_bytes(R, E, I);
  MOE_REQUIRE(need <= (size_t)MOE_STATIC_SCRATCH_BYTES, MOE_ERR_WORKSPACE_TOO_SMALL,
              "gemm_gateup_static: the tile list of R=%d rows, E=%d experts needs %zu bytes, the static scratch holds %u",
              R, E, need, (unsigned)MOE_STATIC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  // the tile list (header and every entry the GEMM reads) is rewritten by this call's first kernel: nothing of
  // an earlier call's contents is read
  return moe_gemm_gateup_impl(xq, sx, row_ids, w_gate, sw_gate, w_up, sw_up, group_offsets, E, R, D, I, hq, sh, ws,
                              MOE_STATIC_SCRATCH_BYTES, false, moe_row_major_scales(D, I), stream);
}

int moe_gemm_down_impl(const uint8_t* hq, const float* sh, const uint8_t* w_down, const float* sw_down,
                       const int32_t* group_offsets, int E, int R, int I, int D, void* y_bf16, void* ws,
                       size_t ws_bytes, bool list_built, GemmScales sc, moe_stream_t stream) {
  MOE_REQUIRE((R == 0 || (hq && sh && y_bf16)) && w_down && sw_down && group_offsets && ws, MOE_ERR_NULL,
              "gemm_down: null pointer");
  MOE_REQUIRE(E >= 1 && E <= 1024 && R >= 0 && D > 0 && I > 0 && D % 128 == 0 && I % 128 == 0, MOE_ERR_BAD_SHAPE,
              "gemm_down: need D %% 128 == 0 and I %% 128 == 0 and 1 <= E <= 1024, got E=%d R=%d I=%d D=%d", E, R, I, D);
  MOE_REQUIRE(MOE_ALIGNED16(hq) && MOE_ALIGNED16(w_down) && MOE_ALIGNED16(y_bf16) && MOE_ALIGNED16(ws), MOE_ERR_BAD_ALIGN,
              "gemm_down: pointers must be 16-byte aligned");
  MOE_REQUIRE((long long)R * sc.in_row * 4 <= (1ll << 32), MOE_ERR_BAD_SHAPE, "gemm_down: scale array out of the addressable range");
  return launch<MODE_DOWN>(hq, sh, nullptr, w_down, sw_down, nullptr, nullptr, group_offsets, E, R, I, D, y_bf16,
                           nullptr, ws, ws_bytes, list_built, sc, (hipStream_t)stream);
}

extern "C" int moe_gemm_down_fp8(const uint8_t* hq, const float* sh, const uint8_t* w_down, const float* sw_down,
                                 const int32_t* group_offsets, int E, int R, int I, int D, void* y_bf16, void* ws,
                                 size_t ws_bytes, moe_stream_t stream) {
  return moe_gemm_down_impl(hq, sh, w_down, sw_down, group_offsets, E, R, I, D, y_bf16, ws, ws_bytes, false,
                            moe_row_major_scales(I, D), stream);
}

extern "C" int moe_gemm_down_fp8_layout(const uint8_t* hq, const float* sh, const uint8_t* w_down, const float* sw_down,
                                        const int32_t* group_offsets, int E, int R, int I, int D, void* y_bf16,
                                        void* ws, size_t ws_bytes, int sh_layout, moe_stream_t stream) {
  if (int rc = check_layout(sh_layout, "gemm_down: sh")) return rc;
  GemmScales sc = moe_row_major_scales(I, D);
  if (sh_layout == MOE_SCALES_BLOCK_MAJOR) sc.in_row = 1, sc.in_kb = R, sc.in_listed = true;
  return moe_gemm_down_impl(hq, sh, w_down, sw_down, group_offsets, E, R, I, D, y_bf16, ws, ws_bytes, false, sc, stream);
}

// Builds, ahead of the GEMM launches, the list that they read from ws when they are told list_built = true:
// one group of R rows (the shared expert).
int moe_gemm_build_dense_tile_list(int R, void* ws, size_t ws_bytes, moe_stream_t stream) {
  TileList l;
  if (int rc = moe_gemm_tile_list(R, 1, ws, ws_bytes, &l)) return rc;
  hipLaunchKernelGGL(build_tiles_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, (const int32_t*)nullptr, 1, l, R);
  return moe_check_hip(hipGetLastError(), "gemm tiles launch");
}

// The tile list that the GEMM launches of (R rows, E experts) read from ws when they are told list_built = true.
int moe_gemm_tile_list(int R, int E, void* ws, size_t ws_bytes, TileList* list) {
  MOE_REQUIRE(ws && list, MOE_ERR_NULL, "gemm tiles: null pointer");
  MOE_REQUIRE(E >= 1 && E <= 1024 && R >= 0, MOE_ERR_BAD_SHAPE, "gemm tiles: need 1 <= E <= 1024, got E=%d R=%d", E, R);
  MOE_REQUIRE(ws_bytes >= moe_gemm_workspace_bytes(R, E, 0), MOE_ERR_WORKSPACE_TOO_SMALL, "gemm tiles: workspace too small");
  *list = tile_list(ws, R, E);
  return MOE_OK;
}
