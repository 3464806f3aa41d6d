// Timing probe for the K loop of the grouped fp8 GEMM (moe_gemm.hip): skeletons of the loop -- the same
// instruction mix, LDS traffic and copy traffic, no epilogue, results meaningless -- run on all 256 CUs, so
// that the ceilings the design argues from can be measured again on any box:
//   * what the compute pattern alone reaches (MFMAs + block-scale FMAs + fragment reads from LDS + barrier);
//   * what the copies cost when every line is an L2 hit, when 4 workgroups of an XCD share each weight slab
//     streamed from HBM (an expert of 4 row tiles), and when every workgroup streams its own (an expert of one);
//   * what the copy pattern alone moves, without any arithmetic;
//   * three alternative structures that were measured and not adopted (B, C, A with W2).
// Operand data are random fp8 codes by default: the matrix cores' power draw, and through it the clock, depends
// on the data -- constant bytes read 25-30 % faster than anything a real layer can reach.
//
// Built into libmoe_probe.so (jax-gpt_amd/build.py), driven by `python bench.py --probe`; not part of the product
// library and not on any product path.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <type_traits>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
#define KROW 7168   // bytes per operand row (K of the DeepSeek-V3 gate/up GEMM)
#define KB 56       // K steps per work item

namespace {

__device__ __forceinline__ const uint8_t* uniform_ptr(const uint8_t* p) {   // (readfirstlane returns int: no sign extension of the low half)
  return (const uint8_t*)(((uintptr_t)(unsigned)__builtin_amdgcn_readfirstlane((unsigned)((uintptr_t)p >> 32)) << 32) |
                          (uintptr_t)(unsigned)__builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)p));
}
__device__ __forceinline__ void dma16(const uint8_t* base, unsigned off, unsigned lds_addr) {
  const unsigned m0v = __builtin_amdgcn_readfirstlane(lds_addr);
  base = uniform_ptr(base);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0v), "v"(off), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void dma4(const uint8_t* base, unsigned off, unsigned lds_addr) {
  const unsigned m0v = __builtin_amdgcn_readfirstlane(lds_addr);
  base = uniform_ptr(base);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(m0v), "v"(off), "s"(base) : "memory", "m0");
}
template <int N> __device__ __forceinline__ void wait_vm() { __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14)); }

// The weight slab (256 rows x KROW bytes) of a workgroup's item: `share` workgroups of one XCD read the same
// slab at the same time, every item takes a new one, slabs walk through wspan bytes.
__device__ __forceinline__ size_t slab_of(int share, size_t wspan, int it) {
  const int x = blockIdx.x & 7, i = blockIdx.x >> 3;
  return ((size_t)(((it * 32 + i) / share) * 8 + x) * (size_t)(256 * KROW)) % wspan;
}

// ---------------- A: the structure of grouped_gemm_kernel's 256-row class
// COPY 0: no copies at all.  NGRP: MFMA groups per step (8 = the full tile's work, 0 = copies only).
// W2 1: the weight tile two steps ahead inside the two stages (issued once its fragments are in registers), the
// activation tile one step ahead and issued first.
template <int COPY, int NGRP = 8, int W2 = 0>
__global__ __launch_bounds__(512, 1) void kA(float* out, int items, const float* scp, const uint8_t* wsrc, size_t wspan,
                                             const uint8_t* xsrc, int share) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int XF = 8;
  constexpr int STAGE = 65536 + 1024 + 256;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wi = wave & 3, xj = wave >> 2;
  for (int i = threadIdx.x; i < 2 * STAGE / 4; i += 512) ((int*)lds)[i] = ((const int*)xsrc)[i + (blockIdx.x & 15) * 1000];
  __syncthreads();
  const int fr = lane & 15, fq = lane >> 4;
  const int off0 = fr * 128 + ((fq ^ (fr >> 1)) << 4), off1 = fr * 128 + (((fq + 4) ^ (fr >> 1)) << 4);
  auto rd = [&](const uint8_t* base) {
    const v4i lo = *(const v4i*)(base + off0);
    const v4i hi = *(const v4i*)(base + off1);
    return (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  const uint8_t* xb = xsrc + (size_t)((blockIdx.x >> 7) & 7) * (256 * KROW);
  const int drow = lane >> 3, dch = lane & 7;
  unsigned woff[8], xoff[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    woff[u] = (unsigned)((wi * 64 + u * 8 + drow) * KROW + ((dch ^ (drow >> 1)) << 4));
    xoff[u] = (unsigned)(((u * 4 + wi) * 8 + drow) * KROW + ((dch ^ (drow >> 1)) << 4));
  }
  const unsigned soff = (unsigned)(wi * 64 + lane) * 4u;
  const unsigned lds0 = (unsigned)(uintptr_t)lds;
  v4f acc[4][XF];
  for (int f = 0; f < 4; ++f) for (int j = 0; j < XF; ++j) acc[f][j] = (v4f){0, 0, 0, 0};
  const v4f z = {0, 0, 0, 0};
  for (int it = 0; it < items; ++it) {
    const uint8_t* wb = wsrc + slab_of(share, wspan, it);
    auto issueW = [&](int kb) {
      const unsigned st = lds0 + (kb & 1) * STAGE;
#pragma unroll
      for (int u = 0; u < 8; ++u) dma16(wb + (size_t)kb * 128, woff[u], st + (wi * 8 + u) * 1024);
    };
    auto issueX = [&](int kb) {
      const unsigned st = lds0 + (kb & 1) * STAGE;
#pragma unroll
      for (int u = 0; u < 8; ++u) dma16(xb + (size_t)kb * 128, xoff[u], st + 32768 + (u * 4 + wi) * 1024);
      dma4((const uint8_t*)scp, soff, st + 65536 + wi * 256);
    };
    auto issue = [&](int kb) { issueW(kb); issueX(kb); };
    if (COPY && xj == 0) { issue(0); if (W2) issueW(1); }
    for (int kb = 0; kb < KB; ++kb) {
      if (xj == 0) { if (W2) wait_vm<8>(); else wait_vm<0>(); }
      __builtin_amdgcn_s_barrier();
      if (COPY && xj == 0 && kb + 1 < KB) { if (W2) issueX(kb + 1); else issue(kb + 1); }
      const uint8_t* st = lds + (kb & 1) * STAGE;
      v8i wf[4], xf[2];
      const v4f s0 = *(const v4f*)(st + 65536 + xj * 512 + fr * 32), s1 = *(const v4f*)(st + 65536 + xj * 512 + fr * 32 + 16);
      const float sc[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
#pragma unroll
      for (int f = 0; f < 4; ++f) wf[f] = rd(st + (wi * 64 + f * 16) * 128);
      xf[0] = rd(st + 32768 + xj * 2048);
      v4f p[2][4];
#pragma unroll
      for (int j = 0; j <= NGRP; ++j) {
        if (NGRP == 0) break;
        if (j + 1 < NGRP) xf[(j + 1) & 1] = rd(st + 32768 + (2 * (j + 1) + xj) * 2048);
#pragma unroll
        for (int f = 0; f < 4; ++f) {
          if (j < NGRP) p[j & 1][f] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[f], xf[j & 1], z, 0, 0, 0, 0, 0, 0);
          if (j > 0) acc[f][j - 1] += p[(j - 1) & 1][f] * sc[j - 1];
        }
#pragma unroll
        for (int f = 0; f < 4; ++f) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
          if (f < 2) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (W2 && COPY && j == 1 && xj == 0) { issueW(kb + 2 < KB ? kb + 2 : KB - 1); __builtin_amdgcn_sched_barrier(0); }
      }
    }
    wait_vm<0>();
    __syncthreads();
  }
  float s = 0;
  for (int f = 0; f < 4; ++f) for (int j = 0; j < XF; ++j) s += acc[f][j][0] + acc[f][j][1] + acc[f][j][2] + acc[f][j][3];
  if (s == 12345.f) out[0] = s;
}



// ---------------- C: structure A with the 32x32x64 form of the MFMA (half the instructions and operand-register reads)
typedef float v16f __attribute__((ext_vector_type(16)));
template <int DUMMY>
__global__ __launch_bounds__(512, 1) void kC(float* out, int items, const float* scp, const uint8_t* wsrc, size_t wspan,
                                             const uint8_t* xsrc, int share) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int XB = 4;   // 32-row activation blocks per wave
  constexpr int STAGE = 65536 + 1024 + 256;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wi = wave & 3, xj = wave >> 2;
  for (int i = threadIdx.x; i < 2 * STAGE / 4; i += 512) ((int*)lds)[i] = i * 0x01010101;
  __syncthreads();
  const int r = lane & 31, g = lane >> 5;
  int offc[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int chunk = (c >> 1) * 4 + 2 * g + (c & 1);
    offc[c] = r * 128 + ((chunk ^ ((r >> 1) & 7)) << 4);
  }
  auto rd = [&](const uint8_t* base, int h) {
    const v4i lo = *(const v4i*)(base + offc[2 * h]);
    const v4i hi = *(const v4i*)(base + offc[2 * h + 1]);
    return (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  const uint8_t* xb = xsrc + (size_t)((blockIdx.x >> 7) & 7) * (256 * KROW);
  const int drow = lane >> 3, dch = lane & 7;
  unsigned woff[8], xoff[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    woff[u] = (unsigned)((wi * 64 + u * 8 + drow) * KROW + ((dch ^ (drow >> 1)) << 4));
    xoff[u] = (unsigned)(((u * 4 + wi) * 8 + drow) * KROW + ((dch ^ (drow >> 1)) << 4));
  }
  const unsigned soff = (unsigned)(wi * 64 + lane) * 4u;
  const unsigned lds0 = (unsigned)(uintptr_t)lds;
  v16f acc[2][XB];
  for (int b = 0; b < 2; ++b) for (int j = 0; j < XB; ++j) for (int i = 0; i < 16; ++i) acc[b][j][i] = 0.f;
  v16f z; for (int i = 0; i < 16; ++i) z[i] = 0.f;
  for (int it = 0; it < items; ++it) {
    const uint8_t* wb = wsrc + slab_of(share, wspan, it);
    auto issue = [&](int kb) {
      const unsigned st = lds0 + (kb & 1) * STAGE;
#pragma unroll
      for (int u = 0; u < 8; ++u) dma16(wb + (size_t)kb * 128, woff[u], st + (wi * 8 + u) * 1024);
#pragma unroll
      for (int u = 0; u < 8; ++u) dma16(xb + (size_t)kb * 128, xoff[u], st + 32768 + (u * 4 + wi) * 1024);
      dma4((const uint8_t*)scp, soff, st + 65536 + wi * 256);
    };
    if (xj == 0) issue(0);
    for (int kb = 0; kb < KB; ++kb) {
      if (xj == 0) wait_vm<0>();
      __builtin_amdgcn_s_barrier();
      if (xj == 0 && kb + 1 < KB) issue(kb + 1);
      const uint8_t* st = lds + (kb & 1) * STAGE;
      v8i wf[2][2], xf[2][2];
      const v4f sc = *(const v4f*)(st + 65536 + xj * 512 + r * 16);
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int h = 0; h < 2; ++h) wf[b][h] = rd(st + (wi * 64 + b * 32) * 128, h);
      xf[0][0] = rd(st + 32768 + xj * 4096, 0);
      xf[0][1] = rd(st + 32768 + xj * 4096, 1);
      v16f p[2];
#pragma unroll
      for (int j = 0; j < XB; ++j) {
        if (j + 1 < XB) {
          xf[(j + 1) & 1][0] = rd(st + 32768 + (2 * (j + 1) + xj) * 4096, 0);
          xf[(j + 1) & 1][1] = rd(st + 32768 + (2 * (j + 1) + xj) * 4096, 1);
        }
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          if (j > 0) acc[b][j - 1] += p[b] * sc[j - 1];
          p[b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[b][0], xf[j & 1][0], z, 0, 0, 0, 0, 0, 0);
        }
#pragma unroll
        for (int b = 0; b < 2; ++b)
          p[b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[b][1], xf[j & 1][1], p[b], 0, 0, 0, 0, 0, 0);
        if (j + 1 < XB) __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          if (j > 0) __builtin_amdgcn_sched_group_barrier(0x002, 16, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int b = 0; b < 2; ++b) acc[b][XB - 1] += p[b] * sc[XB - 1];
    }
    __syncthreads();
  }
  float s = 0;
  for (int b = 0; b < 2; ++b) for (int j = 0; j < XB; ++j) for (int i = 0; i < 16; ++i) s += acc[b][j][i];
  if (s == 12345.f) out[0] = s;
}


// ---------------- B: 8x1, W straight to registers, X ring of 4 stages, a barrier every BSTEP steps
// XDMA = 1: X by lds-dma (asm); XDMA = 0: no X copies at all (upper bound); WLOAD = 0: no W loads (registers reused)
template <int XDMA, int WLOAD, int BSTEP>
__global__ __launch_bounds__(512, 1) void kB(float* out, int items, const float* scp, const uint8_t* wsrc, size_t wspan,
                                             const uint8_t* xsrc, int share) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int NF = 16;
  constexpr int STAGE = 32768 + 1024 + 256;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  for (int i = threadIdx.x; i < 4 * STAGE / 4; i += 512) ((int*)lds)[i] = ((const int*)xsrc)[i + (blockIdx.x & 15) * 1000];
  __syncthreads();
  const int fr = lane & 15, fq = lane >> 4;
  const int off0 = fr * 128 + ((fq ^ (fr >> 1)) << 4), off1 = fr * 128 + (((fq + 4) ^ (fr >> 1)) << 4);
  auto rd = [&](const uint8_t* base) {
    const v4i lo = *(const v4i*)(base + off0);
    const v4i hi = *(const v4i*)(base + off1);
    return (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  const uint8_t* xb = xsrc + (size_t)((blockIdx.x >> 7) & 7) * (256 * KROW);
  const int drow = lane >> 3, dch = lane & 7;
  unsigned xoff[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) xoff[u] = (unsigned)(((wave * 4 + u) * 8 + drow) * KROW + ((dch ^ (drow >> 1)) << 4));
  const unsigned soff = (unsigned)(min(wave * 32, 192) + lane) * 4u;
  const unsigned lds0 = (unsigned)(uintptr_t)lds;
  // W fragment f of this wave: rows wave*32 + f*16 + fr, K bytes [16 fq, +16) and [64 + 16 fq, +16)
  const uint8_t* wlane = wsrc + (size_t)(wave * 32 + fr) * KROW + fq * 16;
  v8i wbuf[3][2];
  auto loadW = [&](auto bc, int kb) {
    constexpr int B = decltype(bc)::value;
    if (WLOAD) {
#pragma unroll
      for (int f = 0; f < 2; ++f) {
        const v4i lo = *(const v4i*)(wlane + (size_t)f * 16 * KROW + (size_t)kb * 128);
        const v4i hi = *(const v4i*)(wlane + (size_t)f * 16 * KROW + (size_t)kb * 128 + 64);
        wbuf[B][f] = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      }
    }
  };
  auto issueX = [&](int kb) {
    if (XDMA) {
      const unsigned st = lds0 + (kb & 3) * STAGE;
#pragma unroll
      for (int u = 0; u < 4; ++u) dma16(xb + (size_t)kb * 128, xoff[u], st + (wave * 4 + u) * 1024);
      dma4((const uint8_t*)scp, soff, st + 32768 + min(wave * 32, 192) * 4);
    }
  };
  v4f acc[2][NF];
  for (int f = 0; f < 2; ++f) for (int j = 0; j < NF; ++j) acc[f][j] = (v4f){0, 0, 0, 0};
  for (int f = 0; f < 2; ++f) for (int b = 0; b < 3; ++b) for (int i = 0; i < 8; ++i) wbuf[b][f][i] = ((const int*)xsrc)[threadIdx.x * 8 + i + 4096 * (f + 2 * b)];
  const v4f z = {0, 0, 0, 0};
  v4f p[2];
  float pc = 0.f;
  auto step = [&](auto bc, auto parc, auto copyc, int kb) {
    constexpr int B = decltype(bc)::value;
    constexpr int PAR = decltype(parc)::value;
    constexpr bool COPY = decltype(copyc)::value;
    wait_vm<4>();   // every copy of this wave except the youngest W loads has landed (before anything new is issued)
    if (PAR % BSTEP == 0) __builtin_amdgcn_s_barrier();
    if (COPY) {
      issueX(kb + 2);
      loadW(std::integral_constant<int, (B + 2) % 3>{}, kb + 2);
    }
    const uint8_t* st = lds + (kb & 3) * STAGE;
    v8i xf[3];
    xf[0] = rd(st);
    xf[1] = rd(st + 2048);
    v4f sxa;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < NF; ++j) {
      if (j + 2 < NF) xf[(j + 2) % 3] = rd(st + (j + 2) * 2048);
      if ((j & 3) == 0) sxa = *(const v4f*)(st + 32768 + fr * 64 + (j >> 2) * 16);
#pragma unroll
      for (int f = 0; f < 2; ++f) {
        acc[f][(j + NF - 1) % NF] += p[f] * pc;   // the previous group's results (group -1 of the first step: garbage x 0)
        p[f] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wbuf[B][f], xf[j % 3], z, 0, 0, 0, 0, 0, 0);
      }
      pc = sxa[j & 3];
      if (j + 2 < NF) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      if ((j & 3) == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
#pragma unroll
      for (int f = 0; f < 2; ++f) {
        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  p[0] = z; p[1] = z;
  for (int it = 0; it < items; ++it) {
    wlane = wsrc + slab_of(share, wspan, it) + (size_t)(wave * 32 + fr) * KROW + fq * 16;
    issueX(0);
    loadW(std::integral_constant<int, 0>{}, 0);
    issueX(1);
    loadW(std::integral_constant<int, 1>{}, 1);
#define ST(B, P, C, k) step(std::integral_constant<int, B>{}, std::integral_constant<int, P>{}, std::integral_constant<bool, C>{}, k)
    int kb = 0;
    for (; kb + 6 <= KB - 2; kb += 6) {   // (KB = 56: nine rounds of six, then two steps that issue nothing)
      ST(0, 0, true, kb); ST(1, 1, true, kb + 1); ST(2, 0, true, kb + 2);
      ST(0, 1, true, kb + 3); ST(1, 0, true, kb + 4); ST(2, 1, true, kb + 5);
    }
    ST(0, 0, false, kb); ST(1, 1, false, kb + 1);
    __syncthreads();
  }
  float s = 0;
  for (int f = 0; f < 2; ++f) for (int j = 0; j < NF; ++j) s += acc[f][j][0] + acc[f][j][1] + acc[f][j][2] + acc[f][j][3];
  if (s == 12345.f) out[0] = s;
}


struct Buffers {
  float* out = nullptr;
  float* scales = nullptr;
  uint8_t* w = nullptr;
  uint8_t* x = nullptr;
  int filled = -1;   // 0 / 1: constant / random data in place
};
constexpr size_t kWBytes = (size_t)6 << 30;
constexpr size_t kWSlack = (size_t)64 << 20;
constexpr size_t kXBytes = (size_t)16 << 20;

int fill(Buffers& b, int random_data) {
  if (!b.w) {
    if (hipMalloc(&b.out, 1024) != hipSuccess || hipMalloc(&b.scales, 4096) != hipSuccess ||
        hipMalloc(&b.w, kWBytes + kWSlack) != hipSuccess || hipMalloc(&b.x, kXBytes) != hipSuccess)
      return -1;
  }
  if (b.filled == random_data) return 0;
  if (hipMemset(b.w, 1, kWBytes + kWSlack) != hipSuccess || hipMemset(b.x, 2, kXBytes) != hipSuccess ||
      hipMemset(b.scales, 0, 4096) != hipSuccess)
    return -1;
  if (random_data) {   // fp8 codes with a Gaussian-like spread of exponents, no NaN codes; no two slabs alike
    const size_t blk = (size_t)32 << 20;
    uint8_t* h = (uint8_t*)malloc(blk);
    if (!h) return -1;
    uint64_t rs = 88172645463325252ull;
    for (size_t i = 0; i < blk; ++i) {
      for (;;) {
        rs ^= rs << 13; rs ^= rs >> 7; rs ^= rs << 17;
        const uint8_t c = (uint8_t)(rs >> 24);
        const int e = (c >> 3) & 15;
        if ((c & 0x7f) == 0x7f) continue;
        if ((e < 4 || e > 13) && ((rs >> 40) & 3)) continue;
        h[i] = c;
        break;
      }
    }
    hipError_t err = hipMemcpy(b.w, h, blk, hipMemcpyHostToDevice);
    for (size_t o = blk; err == hipSuccess && o < kWBytes + kWSlack; o += blk - 4096) {
      size_t n = blk - 4096;
      if (o + n > kWBytes + kWSlack) n = kWBytes + kWSlack - o;
      err = hipMemcpy(b.w + o, b.w + ((o / 7) % 4096), n, hipMemcpyDeviceToDevice);
    }
    if (err == hipSuccess) err = hipMemcpy(b.x, h + 12345, kXBytes, hipMemcpyHostToDevice);
    float hs[1024];
    for (int i = 0; i < 1024; ++i) hs[i] = 0.5f + (float)(((unsigned)i * 2654435761u) >> 8 & 0xffff) / 65536.f;
    if (err == hipSuccess) err = hipMemcpy(b.scales, hs, 4096, hipMemcpyHostToDevice);
    free(h);
    if (err != hipSuccess) return -1;
  }
  b.filled = random_data;
  return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
}

typedef void (*kernel_t)(float*, int, const float*, const uint8_t*, size_t, const uint8_t*, int);
struct Variant {
  const char* name;
  kernel_t kernel;
  int lds_bytes;
  double work;   // fraction of a full tile's MFMA work that the skeleton does (0: copies only)
};
const Variant kVariants[] = {
    {"A  structure of the 256-row class: both tiles by lds-dma one step ahead, barrier per step", kA<1>, 2 * 66816, 1.0},
    {"A  compute only: no copies (operands stay in LDS)", kA<0>, 2 * 66816, 1.0},
    {"A  copies only: no MFMA work", kA<1, 0>, 2 * 66816, 0.0},
    {"A  half the MFMA work per step (4 groups: a 128-row tile's)", kA<1, 4>, 2 * 66816, 0.5},
    {"A2 weight tile two steps ahead inside the two stages, activation tile issued first", kA<1, 8, 1>, 2 * 66816, 1.0},
    {"B  8x1 wave grid: weights global->VGPR two steps ahead, activations lds-dma (4 stages), barrier per 2 steps", kB<1, 1, 2>, 4 * 34048, 1.0},
    {"B  the same with a barrier per step", kB<1, 1, 1>, 4 * 34048, 1.0},
    {"B  compute only", kB<0, 0, 2>, 4 * 34048, 1.0},
    {"C  structure A with the 32x32x64 form of the MFMA", kC<0>, 2 * 66816, 1.0},
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

}  // namespace

#define PROBE_API extern "C" __attribute__((visibility("default")))

PROBE_API int moe_probe_variants(void) { return kNumVariants; }
PROBE_API const char* moe_probe_variant_name(int v) { return v >= 0 && v < kNumVariants ? kVariants[v].name : ""; }

// Runs variant v `reps` times on 256 workgroups of 16 work items (56 K steps each) and reports the average launch
// time and the fp8 FLOP rate of the MFMA work done.  w_source: 0 = every weight line an L2 hit, 1 = slabs streamed
// from HBM, four workgroups of an XCD sharing each, 2 = every workgroup streams its own.  Returns 0, or -1 on a HIP error.
PROBE_API int moe_probe_gemm_loop(int v, int w_source, int random_data, int reps, double* ms_per_launch, double* tflops,
                                  double* weight_gbs) {
  static Buffers b;
  if (v < 0 || v >= kNumVariants || w_source < 0 || w_source > 2 || reps < 1) return -1;
  if (fill(b, random_data ? 1 : 0)) return -1;
  const Variant& var = kVariants[v];
  if (hipFuncSetAttribute((const void*)var.kernel, hipFuncAttributeMaxDynamicSharedMemorySize, var.lds_bytes) != hipSuccess) return -1;
  const int workgroups = 256, items = 16;
  const size_t span = w_source == 0 ? (size_t)256 * KROW * 8 : kWBytes;
  const int share = w_source == 1 ? 4 : 1;
  auto launch = [&]() {
    hipLaunchKernelGGL(var.kernel, dim3(workgroups), dim3(512), var.lds_bytes, 0, b.out, items, b.scales, b.w, span, b.x, share);
  };
  hipEvent_t t0, t1;
  if (hipEventCreate(&t0) != hipSuccess || hipEventCreate(&t1) != hipSuccess) return -1;
  launch();
  if (hipDeviceSynchronize() != hipSuccess) return -1;
  (void)hipEventRecord(t0, 0);
  for (int i = 0; i < reps; ++i) launch();
  (void)hipEventRecord(t1, 0);
  if (hipEventSynchronize(t1) != hipSuccess || hipGetLastError() != hipSuccess) return -1;
  float ms = 0.f;
  (void)hipEventElapsedTime(&ms, t0, t1);
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  ms /= reps;
  const double flops = (double)workgroups * items * KB * 256 * 65536.0 * var.work;
  if (ms_per_launch) *ms_per_launch = ms;
  if (tflops) *tflops = flops / ms / 1e9;
  if (weight_gbs) *weight_gbs = (double)workgroups * items * KB * 32768.0 / ms / 1e6;   // weight-tile bytes copied per second
  return 0;
}
