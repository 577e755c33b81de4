// Fused 3S attention with one wave per unit of work (gfx950). The step over a TC-block pair is
// the one every attention kernel here runs (f3s_pair_pipeline.h documents its data flow and its
// numerics); what differs from the workgroup-per-window kernel of f3s_attention.hip is the
// decomposition. Two uses of the one kernel, f3s_fwd_unit_kernel:
//
// Column-sliced schedule, for graphs with long windows:
//   * the column range is cut into S = 8 * P slices. Workgroup b runs on XCD b % 8 (the hardware
//     deals workgroups round-robin over the eight XCDs), and the grid is laid out so that XCD x
//     only ever works on slices x, x + 8, x + 16, ..., one after the other. The K/V rows of a
//     slice mostly stay in the XCD's 4 MiB L2, so a row is fetched from the memory side about
//     once per XCD instead of once per window that names it;
//   * a wave computes one (window, slice) unit: the window's TC blocks whose first column falls
//     into the slice, with (m, l, O) in registers, and writes the unit's partial result to
//     scratch. A second kernel merges a window's partials (log-sum-exp) and writes its rows.
//
// Wave per window, for graphs of short windows: a unit is a whole window (of one head); the rows
// are written straight from the registers.
//
// The reference has no counterpart: its kernels (src/F3S_kernel.cu:1371-1583) walk one window
// per thread block from its first TC block to its last. Its window order (src/utils.cu:400-436)
// is kept: units are issued heavy windows first.
#include <stdlib.h>

#include <mutex>

#include "f3s_common.h"
#include "f3s_pair_pipeline.h"

namespace f3s {
namespace {

using pipe::float4v;
using pipe::uniform;

constexpr int kXcds = 8;
constexpr int kMaxPhases = 16;
constexpr int kUnitWaves = 4;  // waves (= units) per workgroup; they do not cooperate
// the same for the wave-per-window launches of graphs with short windows (measured on the 100k-node
// 8-head layers: 0.093 / 0.171 ms with two, 0.099 / 0.175 ms with four, 0.121 / 0.197 ms with one)
constexpr int kShortUnitWaves = 2;
constexpr int kQueueBatch = 8;  // units a persistent wave takes per visit to a queue

// sliceStart[w * (S + 1) + s] = first TC block of window w whose first (smallest) column id is
// >= s * sliceWidth; entry S is the window's end. One thread per entry, binary search over the
// window's blocks (their first columns ascend).
__global__ void slice_index_kernel(const int32_t* __restrict__ rowWindowOffset,
                                   const int32_t* __restrict__ sparseAToXidx, int nRW, int S,
                                   int sliceWidth, int32_t* __restrict__ sliceStart,
                                   int32_t* __restrict__ cursors) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < kXcds) cursors[idx] = 0;  // work queues of f3s_fwd_sliced_kernel
  const int per = S + 1;
  if (idx >= (int64_t)nRW * per) return;
  const int w = (int)(idx / per), b = (int)(idx % per);
  int lo = rowWindowOffset[w], hi = rowWindowOffset[w + 1];
  if (b == S) {
    sliceStart[idx] = hi;
    return;
  }
  const int64_t limit = (int64_t)b * sliceWidth;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (sparseAToXidx[(int64_t)mid * 16] < limit)
      lo = mid + 1;
    else
      hi = mid;
  }
  sliceStart[idx] = lo;
}

// Partial result of a unit: D/4 + 2 dwords per lane, stored register by register so that every
// store and load is one coalesced 256-byte row: [o[0][0..3], ..., o[T-1][0..3], m, l][64 lanes].
// Lane (g, c) holds O[q = c][16j + 4g + i] in o[j][i].
template <int D>
constexpr int partial_dwords() {
  return (D / 4 + 2) * 64;
}

// waves per SIMD the register allocator is held to; the LDS rings allow two workgroups per CU at
// D >= 64 and four at D = 32
constexpr int unit_waves_per_simd(int d) { return d <= 32 ? 4 : 2; }

// One wave per unit, four independent units per workgroup. A unit is
//   SLICED:  the TC blocks of one (window, column slice); the result is a partial (m, l, O);
//   !SLICED: one whole window (of one head, if HEADS); the result is the window's output rows.
//            Windows of more than maxBlocks TC blocks among the first longPrefix positions of
//            the order are left to f3s_fwd_kernel, whose four waves share a window and whose
//            grid covers exactly those positions (with a heavy-first order no long window lies
//            beyond them; with any other order such a window is simply computed here). Unit u =
//            position * nHeads + head, so the waves of a workgroup mostly work on the heads of
//            one window and share its column ids and bitmaps.
template <typename ET, int D, bool SOFTMAX, bool SLICED, bool HEADS>
__global__ __launch_bounds__(kUnitWaves * 64)
__attribute__((amdgpu_waves_per_eu(unit_waves_per_simd(D), unit_waves_per_simd(D)))) void
f3s_fwd_unit_kernel(const int32_t* __restrict__ windowOrder,
                    const int32_t* __restrict__ rowWindowOffset,
                    const int32_t* __restrict__ sparseAToXidx,
                    const uint8_t* __restrict__ bitmapBytes,
                    const int32_t* __restrict__ sliceStart, int S, int nGroups, int N, int nRW,
                    int64_t nTcb, const ET* __restrict__ Q, const ET* __restrict__ K,
                    const ET* __restrict__ V, float scaleLog2, float* __restrict__ partial,
                    float* __restrict__ out, int nHeads, int ldIn, int ldOut, int maxBlocks,
                    int longPrefix) {
  typedef pipe::PairPipeline<ET, D, SOFTMAX, HEADS, false> Pipe;
  constexpr int T = D / 16;
  extern __shared__ __align__(1024) unsigned char smem[];

  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int g = lane >> 4;
  const int c = lane & 15;

  int w, t0, t1, slice = 0, head = 0;
  if constexpr (SLICED) {
    // workgroup -> (phase, group of four consecutive windows of the order, XCD)
    const int xcd = blockIdx.x % kXcds;
    const int j = blockIdx.x / kXcds;
    const int phase = j / nGroups;
    const int pos = (j - phase * nGroups) * (int)(blockDim.x >> 6) + wave;
    if (pos >= nRW) return;
    slice = phase * kXcds + xcd;
    w = uniform(windowOrder ? windowOrder[pos] : pos);
    if ((unsigned)w >= (unsigned)nRW) return;  // a corrupt order entry must not index out of range
    t0 = uniform(sliceStart[(int64_t)w * (S + 1) + slice]);
    t1 = uniform(sliceStart[(int64_t)w * (S + 1) + slice + 1]);
    if (t1 <= t0) return;  // empty unit: nothing is written, the merge skips it
  } else {
    const int64_t u = (int64_t)blockIdx.x * (int)(blockDim.x >> 6) + wave;
    const int pos = HEADS ? (int)(u / nHeads) : (int)u;
    head = HEADS ? (int)(u - (int64_t)pos * nHeads) : 0;
    if (pos >= nRW) return;
    w = uniform(windowOrder ? windowOrder[pos] : pos);
    if ((unsigned)w >= (unsigned)nRW) return;
    t0 = uniform(rowWindowOffset[w]);
    t1 = uniform(rowWindowOffset[w + 1]);
    if (t1 - t0 > maxBlocks && pos < longPrefix) return;  // f3s_fwd_kernel's
  }
  // block ranges that do not fit the structure (a mismatched rowWindowOffset) are not followed
  if (t0 < 0 || (int64_t)t1 > nTcb) return;

  pipe::Problem<ET> pb;
  pb.sparseAToXidx = sparseAToXidx;
  pb.bitmapBytes = bitmapBytes;
  pb.Q = Q;
  pb.K = K;
  pb.V = V;
  pb.N = N;
  pb.scaleLog2 = scaleLog2;
  pb.pitchIn = HEADS ? ldIn : D;
  pb.nTcb = nTcb;
  pb.sddmm = nullptr;
  const unsigned ringAddr =
      (unsigned)(uintptr_t)(F3S_LDS unsigned char*)smem + (unsigned)wave * pipe::Geo<D>::WAVE_BYTES;
  Pipe pp;
  pp.init(pb, w, ringAddr, head);
  pp.run(pb, t0, t1);

  if constexpr (SLICED) {
    float* dst = partial + ((int64_t)w * S + slice) * partial_dwords<D>() + lane;
#pragma unroll
    for (int jj = 0; jj < T; jj++)
#pragma unroll
      for (int i = 0; i < 4; i++)
        __builtin_nontemporal_store(pp.o[jj][i], dst + (jj * 4 + i) * 64);
    __builtin_nontemporal_store(pp.m, dst + (D / 4) * 64);
    __builtin_nontemporal_store(pp.l, dst + (D / 4 + 1) * 64);
  } else {
    float inv = 1.0f;
    if constexpr (SOFTMAX) {
      const float lAll = pipe::row_sum4(pp.l);
      inv = (lAll == 0.0f) ? 0.0f : 1.0f / lAll;
    }
    const int64_t row = (int64_t)w * 16 + c;
    if (row < N) {
      float* dst = out + row * (HEADS ? ldOut : D) + head * D + 4 * g;
#pragma unroll
      for (int jj = 0; jj < T; jj++) {
        const float4v v = pp.o[jj] * inv;
        *reinterpret_cast<float4v*>(dst + 16 * jj) = v;
      }
    }
  }
}

// The column-sliced schedule with persistent waves and work queues, the form that does not lean
// on how the hardware deals workgroups to XCDs or on the order in which it starts them. The grid
// is a fixed number of workgroups (as many as fit the CUs); every wave pulls (window, slice) units
// from a queue per XCD until all are done: queue x holds the units of slices x, x + 8, ... in
// heavy-first window order, phase by phase, and a wave serves the queue of the XCD it runs on
// (read from the hardware, XCC_ID) before it helps out on the others.
// Measured on the 233k-node benchmark graph (d = 64): 1.72 ms with eight units per queue visit,
// 2.0 ms with one (a device-wide atomic is served on the memory side and one address takes about
// ten million of them per second), against 1.54 ms for f3s_fwd_unit_kernel, where the launch order
// is the schedule. It is therefore the fallback, used when workgroups turn out not to be dealt
// round-robin to the XCDs (xcd_round_robin, below), or on request (F3S_SLICED_PERSISTENT=1).
template <typename ET, int D, bool SOFTMAX>
__global__ __launch_bounds__(kUnitWaves * 64)
__attribute__((amdgpu_waves_per_eu(unit_waves_per_simd(D), unit_waves_per_simd(D)))) void
f3s_fwd_sliced_kernel(const int32_t* __restrict__ windowOrder,
                      const int32_t* __restrict__ sparseAToXidx,
                      const uint8_t* __restrict__ bitmapBytes,
                      const int32_t* __restrict__ sliceStart, int32_t* __restrict__ cursors, int S,
                      int P, int N, int nRW, int64_t nTcb, const ET* __restrict__ Q,
                      const ET* __restrict__ K, const ET* __restrict__ V, float scaleLog2,
                      float* __restrict__ partial) {
  typedef pipe::PairPipeline<ET, D, SOFTMAX, false, false> Pipe;
  constexpr int T = D / 16;
  extern __shared__ __align__(1024) unsigned char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  unsigned xcc;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
  const int home = (int)(xcc & (kXcds - 1));

  pipe::Problem<ET> pb;
  pb.sparseAToXidx = sparseAToXidx;
  pb.bitmapBytes = bitmapBytes;
  pb.Q = Q;
  pb.K = K;
  pb.V = V;
  pb.N = N;
  pb.scaleLog2 = scaleLog2;
  pb.pitchIn = D;
  pb.nTcb = nTcb;
  pb.sddmm = nullptr;
  const unsigned ringAddr =
      (unsigned)(uintptr_t)(F3S_LDS unsigned char*)smem + (unsigned)wave * pipe::Geo<D>::WAVE_BYTES;
  const int total = P * nRW;  // units per queue (empty ones included)
  int batchNext = 0, batchLeft = 0;
  for (int k = 0; k < kXcds; k++) {
    const int x = (home + k) & (kXcds - 1);
    while (true) {
      int u = 0;
      // a device-wide atomic is served on the memory side (the XCDs' L2s are not coherent
      // with each other): a wave takes kQueueBatch units per visit to keep the queue's address
      // from becoming the bottleneck
      if (batchLeft == 0) {
        if (lane == 0) batchNext = atomicAdd(&cursors[x], kQueueBatch);
        batchNext = uniform(batchNext);
        batchLeft = kQueueBatch;
      }
      u = batchNext++;
      batchLeft--;
      if (u >= total) {
        batchLeft = 0;
        break;
      }
      const int phase = u / nRW;
      const int pos = u - phase * nRW;
      const int slice = phase * kXcds + x;
      const int w = uniform(windowOrder ? windowOrder[pos] : pos);
      if ((unsigned)w >= (unsigned)nRW) continue;  // a corrupt order entry is not followed
      const int t0 = uniform(sliceStart[(int64_t)w * (S + 1) + slice]);
      const int t1 = uniform(sliceStart[(int64_t)w * (S + 1) + slice + 1]);
      if (t1 <= t0) continue;  // empty unit: nothing is written, the merge skips it
      if (t0 < 0 || (int64_t)t1 > nTcb) continue;
      Pipe pp;
      pp.init(pb, w, ringAddr, 0);
      pp.run(pb, t0, t1);
      float* dst = partial + ((int64_t)w * S + slice) * partial_dwords<D>() + lane;
#pragma unroll
      for (int jj = 0; jj < T; jj++)
#pragma unroll
        for (int i = 0; i < 4; i++)
          __builtin_nontemporal_store(pp.o[jj][i], dst + (jj * 4 + i) * 64);
      __builtin_nontemporal_store(pp.m, dst + (D / 4) * 64);
      __builtin_nontemporal_store(pp.l, dst + (D / 4 + 1) * 64);
    }
  }
}

// One wave per window: log-sum-exp merge of the window's unit partials, then the window's rows.
// Lane (g, c) holds O[q = c][16j + 4g + i] in O[j * 4 + i], as in the unit kernel.
template <int D, bool SOFTMAX>
__global__ __launch_bounds__(256) void f3s_merge_slices_kernel(
    const int32_t* __restrict__ sliceStart, int S, int N, int nRW,
    const float* __restrict__ partial, float* __restrict__ out) {
  constexpr int T = D / 16;
  constexpr int R = D / 4;  // O registers per lane
  const int lane = threadIdx.x & 63;
  const int w = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= nRW) return;
  const int g = lane >> 4;
  const int c = lane & 15;
  float M = 0.0f, L = 0.0f;
  float O[R];
#pragma unroll
  for (int r = 0; r < R; r++) O[r] = 0.0f;
  const int32_t* ss = sliceStart + (int64_t)w * (S + 1);
  int prev = ss[0];
  for (int s = 0; s < S; s++) {
    const int next = ss[s + 1];
    const bool live = next > prev;
    prev = next;
    if (!live) continue;
    const float* src = partial + ((int64_t)w * S + s) * partial_dwords<D>() + lane;
    float v[R];
#pragma unroll
    for (int r = 0; r < R; r++) v[r] = __builtin_nontemporal_load(src + r * 64);
    if constexpr (SOFTMAX) {
      const float ms = __builtin_nontemporal_load(src + R * 64);
      const float ls = __builtin_nontemporal_load(src + (R + 1) * 64);
      const float mx = fmaxf(M, ms);
      const float a = pipe::fast_exp2(M - mx), b = pipe::fast_exp2(ms - mx);
      M = mx;
      L = fmaf(a, L, b * ls);
#pragma unroll
      for (int r = 0; r < R; r++) O[r] = fmaf(a, O[r], b * v[r]);
    } else {
#pragma unroll
      for (int r = 0; r < R; r++) O[r] += v[r];
    }
  }
  float inv = 1.0f;
  if constexpr (SOFTMAX) {
    const float lAll = pipe::row_sum4(L);
    inv = (lAll == 0.0f) ? 0.0f : 1.0f / lAll;
  }
  const int64_t row = (int64_t)w * 16 + c;
  if (row < N) {
    float* dst = out + row * D + 4 * g;
#pragma unroll
    for (int jj = 0; jj < T; jj++) {
      const float4v v = {O[jj * 4] * inv, O[jj * 4 + 1] * inv, O[jj * 4 + 2] * inv,
                         O[jj * 4 + 3] * inv};
      *reinterpret_cast<float4v*>(dst + 16 * jj) = v;
    }
  }
}

// LDS of a workgroup of kUnitWaves rings; above 64 KiB the kernel has to be told once
template <typename KernelT>
int allow_lds(KernelT kernel, size_t bytes) {
  if (bytes > 64 * 1024)
    F3S_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
  return 0;
}

// Phases P (S = 8 P slices). One slice's K + V rows are held to about 8 MiB: twice an XCD's L2,
// which already catches 4 of 5 accesses on the 233k-node benchmark graph (P = 1), while more and
// shorter units cost more than their higher hit rate returns (measured 1.99 / 2.23 / 2.48 ms at
// P = 1 / 2 / 3). F3S_SLICE_PHASES in the environment overrides the choice.
int choose_phases(int N, int d) {
  const char* e = getenv("F3S_SLICE_PHASES");  // read per call: tests walk through the phases
  const int forced = e ? atoi(e) : 0;
  if (forced > 0) return forced > kMaxPhases ? kMaxPhases : forced;
  const int64_t bytes = (int64_t)N * d * 4;  // K + V
  const int64_t perPhase = (int64_t)kXcds * 8 * 1024 * 1024;
  int P = (int)((bytes + perPhase - 1) / perPhase);
  if (P < 1) P = 1;
  if (P > kMaxPhases) P = kMaxPhases;
  return P;
}

// f3s_fwd_unit_kernel's slice-to-XCD mapping assumes that workgroup b of a launch runs on XCD
// b % 8. That is how the hardware deals workgroups in the partition mode with all eight XCDs
// behind one device; it is checked once per process and device with a 64-workgroup launch that
// records XCC_ID (into `scratch64`, 64 ints of the caller's workspace). Returns 0 in *ok when the
// assumption does not hold; the queue-based kernel is then used.
__global__ void xcd_probe_kernel(int32_t* __restrict__ out) {
  unsigned xcc;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
  if (threadIdx.x == 0) out[blockIdx.x] = (int32_t)(xcc & 0xFu);
}

int xcd_round_robin(int32_t* scratch64, hipStream_t stream, int* ok) {
  constexpr int kMaxDev = 64;
  static std::mutex mu;
  static int known[kMaxDev] = {};  // 0 unknown, 1 round-robin, 2 not
  int dev = 0;
  F3S_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDev) {
    *ok = 0;
    return 0;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (known[dev] == 0) {
    int32_t host[64];
    hipLaunchKernelGGL(xcd_probe_kernel, dim3(64), dim3(64), 0, stream, scratch64);
    F3S_HIP_CHECK(hipGetLastError());
    F3S_HIP_CHECK(hipMemcpyAsync(host, scratch64, sizeof(host), hipMemcpyDeviceToHost, stream));
    F3S_HIP_CHECK(hipStreamSynchronize(stream));
    bool rr = true;
    for (int b = 0; b < 64; b++) rr = rr && host[b] == b % kXcds;
    known[dev] = rr ? 1 : 2;
  }
  *ok = known[dev] == 1;
  return 0;
}

template <typename ET, int D, bool SOFTMAX>
int launch_sliced_d(const int32_t* rwo, const int32_t* order, const int32_t* atox,
                    const uint64_t* bitmap, int N, const void* Q, const void* K, const void* V,
                    float scaleLog2, float* out, int32_t* sliceStart, int32_t* cursors,
                    float* partial, int P, int64_t nTcb, hipStream_t stream) {
  const int nRW = (N + kWinRows - 1) / kWinRows;
  const int S = P * kXcds;
  const int sliceWidth = (N + S - 1) / S;
  const int64_t entries = (int64_t)nRW * (S + 1);
  const char* env = getenv("F3S_SLICED_PERSISTENT");
  const int forced = env ? (env[0] == '0' ? -1 : 1) : 0;
  bool persistent = forced > 0;
  if (forced == 0) {  // before the index kernel: the check borrows the cursors' memory
    int rr = 0;
    if (int rc = xcd_round_robin(cursors, stream, &rr)) return rc;
    persistent = rr == 0;
  }
  hipLaunchKernelGGL(slice_index_kernel, dim3((unsigned)((entries + 255) / 256)), dim3(256), 0,
                     stream, rwo, atox, nRW, S, sliceWidth, sliceStart, cursors);
  F3S_HIP_CHECK(hipGetLastError());
  if (persistent) {
    constexpr size_t ldsP = (size_t)kUnitWaves * pipe::Geo<D>::WAVE_BYTES;
    auto kernel = f3s_fwd_sliced_kernel<ET, D, SOFTMAX>;
    if (int rc = allow_lds(kernel, ldsP)) return rc;
    int dev = 0, cus = 0;
    F3S_HIP_CHECK(hipGetDevice(&dev));
    F3S_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int perCu = (int)((160 * 1024) / ldsP) > 0 ? (int)((160 * 1024) / ldsP) : 1;
    hipLaunchKernelGGL(kernel, dim3((unsigned)(cus * perCu)), dim3(kUnitWaves * 64), ldsP, stream,
                       order, atox, reinterpret_cast<const uint8_t*>(bitmap), sliceStart, cursors,
                       S, P, N, nRW, nTcb, static_cast<const ET*>(Q), static_cast<const ET*>(K),
                       static_cast<const ET*>(V), scaleLog2, partial);
    F3S_HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL((f3s_merge_slices_kernel<D, SOFTMAX>), dim3((unsigned)((nRW + 3) / 4)),
                       dim3(256), 0, stream, sliceStart, S, N, nRW, partial, out);
    F3S_HIP_CHECK(hipGetLastError());
    return 0;
  }
  const int nGroups = (nRW + kUnitWaves - 1) / kUnitWaves;
#ifdef F3S_PROBE_LDS_PAD
  constexpr size_t lds = (size_t)kUnitWaves * pipe::Geo<D>::WAVE_BYTES + F3S_PROBE_LDS_PAD;
#else
  constexpr size_t lds = (size_t)kUnitWaves * pipe::Geo<D>::WAVE_BYTES;
#endif
  if (int rc = allow_lds(f3s_fwd_unit_kernel<ET, D, SOFTMAX, true, false>, lds)) return rc;
  hipLaunchKernelGGL((f3s_fwd_unit_kernel<ET, D, SOFTMAX, true, false>),
                     dim3((unsigned)(P * nGroups * kXcds)), dim3(kUnitWaves * 64), lds, stream,
                     order, rwo, atox, reinterpret_cast<const uint8_t*>(bitmap), sliceStart, S,
                     nGroups, N, nRW, nTcb, static_cast<const ET*>(Q), static_cast<const ET*>(K),
                     static_cast<const ET*>(V), scaleLog2, partial, out, 1, D, D, 0, 0);
  F3S_HIP_CHECK(hipGetLastError());
  hipLaunchKernelGGL((f3s_merge_slices_kernel<D, SOFTMAX>), dim3((unsigned)((nRW + 3) / 4)),
                     dim3(256), 0, stream, sliceStart, S, N, nRW, partial, out);
  F3S_HIP_CHECK(hipGetLastError());
  return 0;
}

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

}  // namespace

size_t attention_sliced_workspace_bytes(int N, int d) {
  const int P = choose_phases(N, d);
  const size_t nRW = (size_t)(N + kWinRows - 1) / kWinRows;
  const size_t S = (size_t)P * kXcds;
  return align256(nRW * (S + 1) * sizeof(int32_t)) + 256 + nRW * S * (size_t)(d / 4 + 2) * 64 * 4;
}

int launch_attention_sliced(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                            const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int d,
                            int dtype, const void* Q, const void* K, const void* V,
                            float scaleLog2, int applySoftmax, float* out, void* workspace,
                            size_t wsBytes, int64_t nTcb, hipStream_t stream) {
  if (wsBytes < attention_sliced_workspace_bytes(N, d))
    return fail(-2, "f3s_attention_fwd: workspace %zu B < required %zu B", wsBytes,
                attention_sliced_workspace_bytes(N, d));
  const int P = choose_phases(N, d);
  const size_t nRW = (size_t)(N + kWinRows - 1) / kWinRows;
  // layout: slice boundaries | the eight queue cursors (256 bytes) | partial results
  int32_t* sliceStart = static_cast<int32_t*>(workspace);
  const size_t indexBytes = align256(nRW * ((size_t)P * kXcds + 1) * 4);
  int32_t* cursors = reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + indexBytes);
  float* partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + indexBytes + 256);
#define F3S_SLICED(ET, DD)                                                                     \
  case DD:                                                                                     \
    return applySoftmax ? launch_sliced_d<ET, DD, true>(rowWindowOffset, windowOrder,          \
                                                        sparseAToXidx, bitmap, N, Q, K, V,     \
                                                        scaleLog2, out, sliceStart, cursors,   \
                                                        partial, P, nTcb, stream)              \
                        : launch_sliced_d<ET, DD, false>(rowWindowOffset, windowOrder,         \
                                                         sparseAToXidx, bitmap, N, Q, K, V,    \
                                                         scaleLog2, out, sliceStart, cursors,  \
                                                         partial, P, nTcb, stream);
  if (dtype == 0) {
    switch (d) {
      F3S_SLICED(_Float16, 32)
      F3S_SLICED(_Float16, 64)
      F3S_SLICED(_Float16, 128)
    }
  } else {
    switch (d) {
      F3S_SLICED(__bf16, 32)
      F3S_SLICED(__bf16, 64)
      F3S_SLICED(__bf16, 128)
    }
  }
#undef F3S_SLICED
  return fail(-2, "f3s_attention_fwd: head dim %d unsupported (32, 64, 128)", d);
}

namespace {

template <typename ET, int D, bool SOFTMAX>
int launch_short_d(const int32_t* rwo, const int32_t* order, const int32_t* atox,
                   const uint64_t* bitmap, int N, const void* Q, const void* K, const void* V,
                   float scaleLog2, float* out, int nHeads, int ldIn, int ldOut, int maxBlocks,
                   int longPrefix, int64_t nTcb, hipStream_t stream) {
  const int64_t nRW = ((int64_t)N + kWinRows - 1) / kWinRows;
  const int64_t units = nRW * (nHeads > 0 ? nHeads : 1);
  const dim3 grid((unsigned)((units + kShortUnitWaves - 1) / kShortUnitWaves)),
      block(kShortUnitWaves * 64);
  const auto* bm = reinterpret_cast<const uint8_t*>(bitmap);
  const auto* q = static_cast<const ET*>(Q);
  const auto* k = static_cast<const ET*>(K);
  const auto* v = static_cast<const ET*>(V);
  constexpr size_t lds = (size_t)kShortUnitWaves * pipe::Geo<D>::WAVE_BYTES;
  if (nHeads > 0) {
    if (int rc = allow_lds(f3s_fwd_unit_kernel<ET, D, SOFTMAX, false, true>, lds)) return rc;
    hipLaunchKernelGGL((f3s_fwd_unit_kernel<ET, D, SOFTMAX, false, true>), grid, block, lds,
                       stream, order, rwo, atox, bm, nullptr, 0, 0, N, (int)nRW, nTcb, q, k, v,
                       scaleLog2, nullptr, out, nHeads, ldIn, ldOut, maxBlocks, longPrefix);
  } else {
    if (int rc = allow_lds(f3s_fwd_unit_kernel<ET, D, SOFTMAX, false, false>, lds)) return rc;
    hipLaunchKernelGGL((f3s_fwd_unit_kernel<ET, D, SOFTMAX, false, false>), grid, block, lds,
                       stream, order, rwo, atox, bm, nullptr, 0, 0, N, (int)nRW, nTcb, q, k, v,
                       scaleLog2, nullptr, out, 1, D, D, maxBlocks, longPrefix);
  }
  F3S_HIP_CHECK(hipGetLastError());
  return 0;
}

template <typename ET>
int launch_short_et(const int32_t* rwo, const int32_t* order, const int32_t* atox,
                    const uint64_t* bitmap, int N, int d, const void* Q, const void* K,
                    const void* V, float scaleLog2, int applySoftmax, float* out, int nHeads,
                    int ldIn, int ldOut, int maxBlocks, int longPrefix, int64_t nTcb,
                    hipStream_t stream) {
#define F3S_SHORT(DD)                                                                          \
  case DD:                                                                                     \
    return applySoftmax ? launch_short_d<ET, DD, true>(rwo, order, atox, bitmap, N, Q, K, V,   \
                                                       scaleLog2, out, nHeads, ldIn, ldOut,    \
                                                       maxBlocks, longPrefix, nTcb, stream)    \
                        : launch_short_d<ET, DD, false>(rwo, order, atox, bitmap, N, Q, K, V,  \
                                                        scaleLog2, out, nHeads, ldIn, ldOut,   \
                                                        maxBlocks, longPrefix, nTcb, stream);
  switch (d) {
    F3S_SHORT(32)
    F3S_SHORT(64)
    F3S_SHORT(128)
    default:
      return fail(-2, "f3s_attention_fwd: head dim %d unsupported (32, 64, 128)", d);
  }
#undef F3S_SHORT
}

}  // namespace

// One wave per window, for every window except those of more than maxBlocks TC blocks among the
// first longPrefix positions of the order (nHeads = 0: contiguous single head).
int launch_attention_short_windows(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                                   const int32_t* sparseAToXidx, const uint64_t* bitmap, int N,
                                   int d, int dtype, const void* Q, const void* K, const void* V,
                                   float scaleLog2, int applySoftmax, float* out, int nHeads,
                                   int ldIn, int ldOut, int maxBlocks, int longPrefix,
                                   int64_t nTcb, hipStream_t stream) {
  return dtype == 0
             ? launch_short_et<_Float16>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, d,
                                         Q, K, V, scaleLog2, applySoftmax, out, nHeads, ldIn,
                                         ldOut, maxBlocks, longPrefix, nTcb, stream)
             : launch_short_et<__bf16>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, d, Q,
                                       K, V, scaleLog2, applySoftmax, out, nHeads, ldIn, ldOut,
                                       maxBlocks, longPrefix, nTcb, stream);
}

}  // namespace f3s
