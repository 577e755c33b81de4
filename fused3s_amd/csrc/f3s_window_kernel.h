// The attention kernel with one workgroup per 16-row window, and its launchers, as templates:
// f3s_attention.hip builds them with 32-bit row offsets in the K / V gathers (arrays below
// 4 GiB), f3s_attention_wide.hip with 64-bit offsets (the reference indexes rows with int64_t,
// src/F3S_kernel.cu:1422-1423); two translation units, because keeping both address forms in one
// kernel costs the common one 17 vector registers.
//
// Replaces the reference kernels f3sKernel1tb1rw / ...Scheduled / ...ScheduledPermutedQKV
// [ScaleQK], f2sKernel1tb1rw and f3sKernel1tb1tcb (src/F3S_kernel.cu:997-1175, 1371-1800,
// 1999-2182, 2186-2327, 677-877) and their launchers (src/F3S_kernel.cu:325-458, 581-671).
//
// A workgroup of four waves owns one window. The window's TC blocks are cut into four contiguous
// runs, one per wave; a wave walks its run with the shared pair pipeline (f3s_pair_pipeline.h:
// K/V rows gathered straight into the wave's LDS ring, scores and outputs in MFMA accumulators,
// running (m, l, O) in registers), and one LDS merge per window combines the four partial
// results (log-sum-exp) instead of the reference's three block barriers per iteration.
#pragma once
#include <stdlib.h>
#include <string.h>

#include "f3s_common.h"
#include "f3s_pair_pipeline.h"

namespace f3s {
namespace window {

using pipe::float4v;
using pipe::kLog2e;

// Waves per SIMD the register allocator is held to: the LDS rings allow four workgroups per CU at
// D = 32, two up to D = 128 and one above.
constexpr int waves_per_simd(int d) { return d <= 32 ? 4 : d <= 128 ? 2 : 1; }

// Constant-rate (100 MHz) timestamp shared by all CUs, and an id of the CU this wave runs on:
// XCC id in bits 8.., {SE, SH, CU} of HW_ID in bits 0..7. Used only by the timed variant, which
// replaces the reference's %globaltimer / %smid reads (src/F3S_kernel.cu:30-40).
__device__ __forceinline__ unsigned long long realtime_ticks() {
  return __builtin_amdgcn_s_memrealtime();
}
__device__ __forceinline__ unsigned cu_key() {
  unsigned hw, xcc;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw));
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
  return ((xcc & 0xFu) << 8) | ((hw >> 8) & 0xFFu);
}

// HEADS = false: Q/K/V are [N, D] contiguous, one workgroup per window (blockIdx.x = position in
// the window order). HEADS = true: Q/K/V are [N, nHeads, D] with a row pitch of ldIn elements,
// out is [N, nHeads * D] with a row pitch of ldOut floats, and blockIdx.x = position * nHeads +
// head, so that the workgroups of one window's heads are dispatched together and share the
// window's column ids and bitmaps (and the neighbouring pieces of its K/V rows) in L2.
// W8 = true: the structure comes from preprocessing with 8-column blocks (the reference's
// 1tb1tcb path, src/F3S_kernel.cu:677-877). Column ids and bitmap words of two consecutive 16x8
// blocks are laid out exactly like one 16x16 block, so the same pipeline runs over four 16x8
// blocks per step; rowWindowOffset then counts 16x8 blocks, a window may end in the middle of a
// step, and sddmm (if not null) receives the masked, unscaled scores, row-major 16x8 per block
// (saveSddmmResult, src/F3S_kernel.cu:99-115).
// PERSIST = true (single head, 16x16 blocks, not timed): the grid is as many workgroups as fit the
// GPU at once; a workgroup starts at position blockIdx.x of the window order and draws every
// further position from a device-wide cursor (the draw for the next window is in flight while the
// current one is computed), so the order is served first come, first served without relying on
// the order in which the hardware starts workgroups. The cursor is put back to zero by a
// one-thread kernel in front of every launch of this form (a launch that was cut short must not
// leave it behind); launches of this form must not overlap on one device.
static __device__ int g_windowCursor = 0;

template <int UNUSED = 0>
__global__ void reset_window_cursor_kernel() {
  g_windowCursor = 0;
}

// WIDE: 64-bit row offsets in the K / V gathers.
template <typename ET, int D, int NWAVES, bool SOFTMAX, bool CLOCKED, bool HEADS, bool W8,
          bool WIDE, bool PERSIST = false>
__global__ __launch_bounds__(NWAVES * 64)
__attribute__((amdgpu_waves_per_eu(waves_per_simd(D), waves_per_simd(D)))) void f3s_fwd_kernel(
    const int32_t* __restrict__ rowWindowOffset, const int32_t* __restrict__ windowOrder,
    const int32_t* __restrict__ sparseAToXidx, const uint8_t* __restrict__ bitmapBytes, int N,
    int nRW, int64_t nTcb, const ET* __restrict__ Q, const ET* __restrict__ K,
    const ET* __restrict__ V, float scaleLog2, float* __restrict__ out,
    unsigned long long* __restrict__ cuTimer, int nHeads, int ldIn, int ldOut,
    float* __restrict__ sddmm, int minBlocks, int nPositions) {
  typedef pipe::PairPipeline<ET, D, SOFTMAX, HEADS, W8, WIDE> Pipe;
  constexpr int T = D / 16;
  constexpr int OSTRIDE = D + 4;
  constexpr int BPS = W8 ? 4 : 2;  // blocks of the structure per pipeline step
  extern __shared__ __align__(1024) unsigned char smem[];
  unsigned long long tBegin = 0;
  if constexpr (CLOCKED) tBegin = realtime_ticks();

  static_assert(!PERSIST || (!CLOCKED && !HEADS && !W8), "the persistent form is single-head");
  __shared__ int sNextPos[2];
  __shared__ int sUnitCount;
  __shared__ int sUnitList[NWAVES * 64];
  int pos = HEADS ? (int)(blockIdx.x / (unsigned)nHeads) : (int)blockIdx.x;
  int head = HEADS ? (int)(blockIdx.x - (unsigned)pos * (unsigned)nHeads) : 0;
  // A launch that shares the windows with the wave-per-window kernel (minBlocks >= 0) covers the
  // (position, head) units of the order's first nPositions positions with a grid of its own
  // size: thread t of workgroup b looks at unit b + t * gridDim.x, and the workgroup computes
  // the units it finds long, one after the other. When no window is long, which is the usual
  // case on a graph of short windows, the launch is a thousand workgroups that read a count each
  // and leave, instead of one workgroup per unit; in a heavy-first order the long units are the
  // first ones and are dealt out round-robin.
  const bool scan = !PERSIST && minBlocks >= 0;
  int nMine = 1;
  if (scan) {
    if (threadIdx.x == 0) sUnitCount = 0;
    __syncthreads();
    const int heads = HEADS ? nHeads : 1;
    const int64_t nUnits = (int64_t)nPositions * heads;
    const int64_t u = (int64_t)blockIdx.x + (int64_t)threadIdx.x * (int64_t)gridDim.x;
    if (u < nUnits) {
      const int p = (int)(u / heads);
      const int w = windowOrder ? windowOrder[p] : p;
      if ((unsigned)w < (unsigned)nRW) {
        const int t0 = rowWindowOffset[w];
        const int t1 = rowWindowOffset[w + 1];
        if (t0 >= 0 && (int64_t)t1 <= nTcb && t1 - t0 > minBlocks)
          sUnitList[atomicAdd(&sUnitCount, 1)] = (int)u;
      }
    }
    __syncthreads();
    nMine = sUnitCount;
  }
  const int pitchOut = HEADS ? ldOut : D;
  const int lane = threadIdx.x & 63;
  const int wave = pipe::uniform(threadIdx.x >> 6);
  const int g = lane >> 4;
  const int c = lane & 15;
  for (int iter = 0;; iter++) {
  if (scan) {
    if (iter >= nMine) break;
    const int u = sUnitList[iter];
    pos = HEADS ? u / nHeads : u;
    head = HEADS ? u - pos * nHeads : 0;
  }
  if constexpr (PERSIST) {
    if (pos >= nPositions) break;
    // position of the window after this one; read at the end of this iteration
    if (threadIdx.x == 0) sNextPos[iter & 1] = atomicAdd(&g_windowCursor, 1) + (int)gridDim.x;
  }
  do {
  const int w = windowOrder ? windowOrder[pos] : pos;
  if ((unsigned)w >= (unsigned)nRW) break;  // a corrupt order entry must not index out of range

  int t0 = rowWindowOffset[w];
  int t1 = rowWindowOffset[w + 1];
  // block ranges that do not fit the structure (a mismatched rowWindowOffset) are not followed:
  // the window is treated as empty
  if (t0 < 0 || (int64_t)t1 > nTcb || t1 < t0) t1 = t0;
  // windows of at most minBlocks blocks belong to the wave-per-window kernel of the same call
  // (f3s_fwd_unit_kernel); -1 when this kernel computes every window
  if (t1 - t0 <= minBlocks) break;
  const int nSteps = (t1 - t0 + BPS - 1) / BPS;

  pipe::Problem<ET> pb;
  pb.sparseAToXidx = sparseAToXidx;
  pb.bitmapBytes = bitmapBytes;
  pb.Q = Q;
  pb.K = K;
  pb.V = V;
  pb.N = N;
  pb.scaleLog2 = scaleLog2;
  pb.pitchIn = HEADS ? ldIn : D;
  pb.pitchQ = pb.pitchIn;
  pb.nTcb = nTcb;
  pb.sddmm = sddmm;
  const unsigned ringAddr =
      (unsigned)(uintptr_t)(F3S_LDS unsigned char*)smem + (unsigned)wave * pipe::Geo<D>::WAVE_BYTES;
  Pipe pp;
  pp.init(pb, w, ringAddr, head);
  {
    // wave v takes steps [v * nSteps / NWAVES, (v + 1) * nSteps / NWAVES)
    const int sb = (int)((int64_t)wave * nSteps / NWAVES);
    const int se = (int)((int64_t)(wave + 1) * nSteps / NWAVES);
    const int rb = t0 + sb * BPS;
    const int re = (t0 + se * BPS) < t1 ? (t0 + se * BPS) : t1;
    if (re > rb) pp.run(pb, rb, re);
  }

  // ---- merge the waves' partial (m, l, O) and write the window's rows. The merge buffers reuse
  // the rings' memory once every wave has left its loop.
  __syncthreads();
  float* sM = reinterpret_cast<float*>(smem);                    // [NWAVES][16]
  float* sL = sM + NWAVES * 16;                                  // [NWAVES][16]
  float* sO = sL + NWAVES * 16;                                  // [NWAVES][16][OSTRIDE]
  float l = pp.l;
  if constexpr (SOFTMAX) l = pipe::row_sum4(l);
  if (g == 0) {
    sM[wave * 16 + c] = pp.m;
    sL[wave * 16 + c] = l;
  }
#pragma unroll
  for (int j = 0; j < T; j++)
    *reinterpret_cast<float4v*>(&sO[(wave * 16 + c) * OSTRIDE + 16 * j + 4 * g]) = pp.o[j];
  __syncthreads();

  constexpr int VEC_PER_ROW = D / 4;
  for (int idx = threadIdx.x; idx < 16 * VEC_PER_ROW; idx += NWAVES * 64) {
    const int q = idx / VEC_PER_ROW;
    const int cv = idx % VEC_PER_ROW;
    const int64_t row = (int64_t)w * 16 + q;
    if (row >= N) continue;
    float4 acc = {0.f, 0.f, 0.f, 0.f};
    if constexpr (SOFTMAX) {
      float mAll = sM[q];
#pragma unroll
      for (int v = 1; v < NWAVES; v++) mAll = fmaxf(mAll, sM[v * 16 + q]);
      float lAll = 0.0f;
#pragma unroll
      for (int v = 0; v < NWAVES; v++) {
        const float f = pipe::fast_exp2(sM[v * 16 + q] - mAll);
        lAll = fmaf(f, sL[v * 16 + q], lAll);
        const float4 ov = *reinterpret_cast<const float4*>(&sO[(v * 16 + q) * OSTRIDE + cv * 4]);
        acc.x = fmaf(f, ov.x, acc.x);
        acc.y = fmaf(f, ov.y, acc.y);
        acc.z = fmaf(f, ov.z, acc.z);
        acc.w = fmaf(f, ov.w, acc.w);
      }
      const float inv = (lAll == 0.0f) ? 0.0f : 1.0f / lAll;
      acc.x *= inv;
      acc.y *= inv;
      acc.z *= inv;
      acc.w *= inv;
    } else {
#pragma unroll
      for (int v = 0; v < NWAVES; v++) {
        const float4 ov = *reinterpret_cast<const float4*>(&sO[(v * 16 + q) * OSTRIDE + cv * 4]);
        acc.x += ov.x;
        acc.y += ov.y;
        acc.z += ov.z;
        acc.w += ov.w;
      }
    }
    *reinterpret_cast<float4*>(out + row * pitchOut + head * D + cv * 4) = acc;
  }
  } while (false);
  if constexpr (!PERSIST) {
    if (!scan) break;
  }
  __syncthreads();  // the merge buffers are free again, the next position has arrived
  if constexpr (PERSIST) pos = sNextPos[iter & 1];
  }
  if constexpr (CLOCKED) {
    // {first tick, last tick, CU} of this workgroup, as the reference's timed kernels record
    // {begin, end, smid} per block (src/F3S_kernel.cu:1363-1367)
    __syncthreads();
    if (threadIdx.x == 0) {
      cuTimer[3 * (size_t)blockIdx.x + 0] = tBegin;
      cuTimer[3 * (size_t)blockIdx.x + 1] = realtime_ticks();
      cuTimer[3 * (size_t)blockIdx.x + 2] = cu_key();
    }
  }
}

// LDS of a workgroup: its waves' rings; above 64 KiB the kernel has to be told
template <typename KernelT>
int allow_lds(KernelT kernel, size_t bytes) {
  if (bytes > 64 * 1024)
    F3S_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
  return 0;
}

// F3S_WINDOW_PERSISTENT=1 in the environment (read per call): the workgroup-per-window kernel in
// its cursor form
inline bool window_cursor_requested() {
  const char* e = getenv("F3S_WINDOW_PERSISTENT");
  return e && strcmp(e, "1") == 0;
}

struct HeadLayout {
  int nHeads;       // 0: contiguous [N, d] single head
  int ldIn;         // row pitch of Q/K/V in elements
  int ldOut;        // row pitch of out in floats
  int minBlocks;    // this kernel skips windows of at most minBlocks blocks (-1: none)
  int gridWindows;  // positions of the window order this launch covers (<= nRW)
  int64_t nTcb;     // TC blocks of the structure (bounds every window's block range)
};

template <typename ET, int D, bool SOFTMAX, bool WIDE>
int launch_d(const int32_t* rwo, const int32_t* order, const int32_t* atox, const uint64_t* bitmap,
             int N, const void* Q, const void* K, const void* V, float scaleLog2, float* out,
             unsigned long long* cuTimer, HeadLayout hl, hipStream_t stream) {
  constexpr int NWAVES = 4;
  const int nRW = (N + kWinRows - 1) / kWinRows;
  if (nRW == 0) return 0;
  const auto* bm = reinterpret_cast<const uint8_t*>(bitmap);
  const auto* q = static_cast<const ET*>(Q);
  const auto* k = static_cast<const ET*>(K);
  const auto* v = static_cast<const ET*>(V);
  const dim3 block(NWAVES * 64);
  const unsigned gw = (unsigned)(hl.gridWindows < nRW ? hl.gridWindows : nRW);
  if (gw == 0) return 0;
  constexpr size_t lds = (size_t)NWAVES * pipe::Geo<D>::WAVE_BYTES;
#define F3S_LAUNCH(CLOCKED_, HEADS_, GRID)                                                      \
  {                                                                                             \
    auto kernel = f3s_fwd_kernel<ET, D, NWAVES, SOFTMAX, CLOCKED_, HEADS_, false, WIDE>;        \
    if (int rc = allow_lds(kernel, lds)) return rc;                                             \
    hipLaunchKernelGGL(kernel, dim3(GRID), block, lds, stream, rwo, order, atox, bm, N, nRW,    \
                       hl.nTcb, q, k, v, scaleLog2, out, cuTimer, hl.nHeads > 0 ? hl.nHeads : 1,\
                       hl.nHeads > 0 ? hl.ldIn : D, hl.nHeads > 0 ? hl.ldOut : D,               \
                       (float*)nullptr, hl.minBlocks, (int)gw);                                 \
  }
  // a launch next to the wave-per-window kernel looks for its units itself (see the kernel):
  // 256 units per workgroup at most, 1024 workgroups when that is enough
  const unsigned units = gw * (unsigned)(hl.nHeads > 0 ? hl.nHeads : 1);
  unsigned scanGrid = (units + NWAVES * 64 - 1) / (NWAVES * 64);
  if (scanGrid < 1024u) scanGrid = units < 1024u ? units : 1024u;
  const bool scan = hl.minBlocks >= 0;
  bool launched = false;
  if constexpr (!WIDE) {
    if (hl.nHeads == 0 && !cuTimer && hl.minBlocks < 0 && window_cursor_requested()) {
      // F3S_WINDOW_PERSISTENT=1: as many workgroups as the GPU holds at once, windows drawn from
      // a cursor (measured slower than launch order, which therefore stays the default)
      auto kernel = f3s_fwd_kernel<ET, D, NWAVES, SOFTMAX, false, false, false, false, true>;
      if (int rc = allow_lds(kernel, lds)) return rc;
      int dev = 0, nCu = 0, perCu = 0;
      F3S_HIP_CHECK(hipGetDevice(&dev));
      F3S_HIP_CHECK(hipDeviceGetAttribute(&nCu, hipDeviceAttributeMultiprocessorCount, dev));
      F3S_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(
          &perCu, reinterpret_cast<const void*>(kernel), NWAVES * 64, lds));
      unsigned grid = (unsigned)(nCu * (perCu > 0 ? perCu : 1));
      if (grid > gw) grid = gw;
      hipLaunchKernelGGL(reset_window_cursor_kernel<0>, dim3(1), dim3(1), 0, stream);
      hipLaunchKernelGGL(kernel, dim3(grid), block, lds, stream, rwo, order, atox, bm, N, nRW,
                         hl.nTcb, q, k, v, scaleLog2, out, cuTimer, 1, D, D, (float*)nullptr,
                         hl.minBlocks, (int)gw);
      launched = true;
    }
  }
  if (launched) {
  } else if (hl.nHeads > 0) {
    F3S_LAUNCH(false, true, scan ? scanGrid : units)
  } else if (cuTimer) {
    F3S_LAUNCH(true, false, scan ? scanGrid : gw)
  } else {
    F3S_LAUNCH(false, false, scan ? scanGrid : gw)
  }
#undef F3S_LAUNCH
  F3S_HIP_CHECK(hipGetLastError());
  return 0;
}

template <int D, bool SOFTMAX, bool WIDE>
int launch_tcb8(const int32_t* rwo, const int32_t* order, const int32_t* atox,
                const uint64_t* bitmap, int N, const void* Q, const void* K, const void* V,
                float scaleLog2, float* out, float* sddmm, int64_t nTcb8, hipStream_t stream) {
  constexpr int NWAVES = 4;
  const int nRW = (N + kWinRows - 1) / kWinRows;
  if (nRW == 0) return 0;
  constexpr size_t lds = (size_t)NWAVES * pipe::Geo<D>::WAVE_BYTES;
  auto kernel = f3s_fwd_kernel<_Float16, D, NWAVES, SOFTMAX, false, false, true, WIDE>;
  if (int rc = allow_lds(kernel, lds)) return rc;
  hipLaunchKernelGGL(kernel, dim3(nRW), dim3(NWAVES * 64), lds, stream, rwo, order, atox,
                     reinterpret_cast<const uint8_t*>(bitmap), N, nRW, nTcb8,
                     static_cast<const _Float16*>(Q), static_cast<const _Float16*>(K),
                     static_cast<const _Float16*>(V), scaleLog2, out, nullptr, 1, D, D, sddmm, -1,
                     nRW);
  F3S_HIP_CHECK(hipGetLastError());
  return 0;
}

template <typename ET, bool WIDE>
int dispatch_d(const int32_t* rwo, const int32_t* order, const int32_t* atox,
               const uint64_t* bitmap, int N, int d, const void* Q, const void* K, const void* V,
               float scaleLog2, int applySoftmax, float* out, unsigned long long* cuTimer,
               HeadLayout hl, hipStream_t stream) {
#define F3S_DISPATCH(DD)                                                                        \
  if (d == DD)                                                                                  \
    return applySoftmax ? launch_d<ET, DD, true, WIDE>(rwo, order, atox, bitmap, N, Q, K, V,    \
                                                       scaleLog2, out, cuTimer, hl, stream)     \
                        : launch_d<ET, DD, false, WIDE>(rwo, order, atox, bitmap, N, Q, K, V,   \
                                                        scaleLog2, out, cuTimer, hl, stream);
  F3S_FOR_EACH_HEAD_DIM(F3S_DISPATCH)
#undef F3S_DISPATCH
  return fail(-2, "f3s_attention_fwd: head dim %d unsupported (a multiple of 32 up to 256)", d);
}


}  // namespace window
}  // namespace f3s
