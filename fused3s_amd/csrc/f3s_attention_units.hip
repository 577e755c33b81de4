// Fused 3S attention with one wave per unit of work (gfx950). The step over a TC-block pair is
// the one every attention kernel here runs (f3s_pair_pipeline.h documents its data flow and its
// numerics); what differs from the workgroup-per-window kernel of f3s_attention.hip is the
// decomposition.
//
// Column-sliced schedule, for graphs with long windows:
//   * the column range is cut into S = 8 * P slices and XCD x only ever works on slices x, x + 8,
//     x + 16, ..., one after the other. The K/V rows of a slice mostly stay in the XCD's 4 MiB L2,
//     so a row is fetched from the memory side about once per XCD instead of once per window
//     that names it;
//   * a wave computes one (window, slice[, head]) unit: the window's TC blocks whose first column
//     falls into the slice, with (m, l, O) in registers, and writes the unit's partial result to
//     scratch. A second kernel merges a window's partials (log-sum-exp) and writes its rows;
//   * two forms of the unit kernel. f3s_fwd_unit_kernel: the launch order is the schedule
//     (workgroup b of a launch runs on XCD b % 8: that is how the hardware deals workgroups when
//     all eight XCDs sit behind one device; elsewhere the results are the same and only the
//     locality is lost). f3s_fwd_resident_kernel: a grid that fits the GPU at once, every
//     workgroup asks the hardware which XCD it runs on and works through that XCD's units.
//
// Wave per window, for graphs of short windows (f3s_fwd_unit_kernel, SLICED = false): a unit is a
// whole window (of one head); the rows are written straight from the registers.
//
// The reference has no counterpart: its kernels (src/F3S_kernel.cu:1371-1583) walk one window
// per thread block from its first TC block to its last. Its window order (src/utils.cu:400-436)
// is kept: units are issued heavy windows first.
#include <stdlib.h>

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

// Partial result of a unit: D/4 + 2 dwords per lane, stored register by register so that every
// store and load is one coalesced 256-byte row: [o[0][0..3], ..., o[T-1][0..3], m, l][64 lanes].
// Lane (g, c) holds O[q = c][16j + 4g + i] in o[j][i].
template <int D>
constexpr int partial_dwords() {
  return (D / 4 + 2) * 64;
}

// waves per SIMD the register allocator is held to; the LDS rings allow four workgroups of four
// waves per CU at D = 32, two up to D = 128 and one above
constexpr int unit_waves_per_simd(int d) { return d <= 32 ? 4 : d <= 128 ? 2 : 1; }

template <typename ET, int D, bool HEADS>
__device__ __forceinline__ pipe::Problem<ET> make_problem(const int32_t* sparseAToXidx,
                                                          const uint8_t* bitmapBytes, const ET* Q,
                                                          const ET* K, const ET* V, int N,
                                                          float scaleLog2, int ldIn,
                                                          int64_t nTcb, int ldQ = 0) {
  pipe::Problem<ET> pb;
  pb.sparseAToXidx = sparseAToXidx;
  pb.bitmapBytes = bitmapBytes;
  pb.Q = Q;
  pb.K = K;
  pb.V = V;
  pb.N = N;
  pb.scaleLog2 = scaleLog2;
  pb.pitchIn = HEADS ? ldIn : D;
  pb.pitchQ = (HEADS && ldQ > 0) ? ldQ : pb.pitchIn;  // Q may lie apart from K / V
  pb.nTcb = nTcb;
  pb.sddmm = nullptr;
  return pb;
}

// probe builds: the partials through the caches instead of past them
#ifdef F3S_PROBE_PARTIAL_CACHED_STORE
#define F3S_PARTIAL_STORE(v, p) (*(p) = (v))
#else
#define F3S_PARTIAL_STORE(v, p) __builtin_nontemporal_store((v), (p))
#endif
#ifdef F3S_PROBE_PARTIAL_CACHED_LOAD
#define F3S_PARTIAL_LOAD(p) (*(p))
#else
#define F3S_PARTIAL_LOAD(p) __builtin_nontemporal_load(p)
#endif

template <int D, typename PipeT>
__device__ __forceinline__ void store_partial(const PipeT& pp, float* __restrict__ dst) {
#pragma unroll
  for (int jj = 0; jj < D / 16; jj++)
#pragma unroll
    for (int i = 0; i < 4; i++) F3S_PARTIAL_STORE(pp.o[jj][i], dst + (jj * 4 + i) * 64);
  F3S_PARTIAL_STORE(pp.m, dst + (D / 4) * 64);
  F3S_PARTIAL_STORE(pp.l, dst + (D / 4 + 1) * 64);
}

// One wave per unit, kUnitWaves independent units per workgroup. A unit is
//   SLICED:  the TC blocks of one (window, column slice[, head]); the result is a partial
//            (m, l, O). Workgroup b: XCD b % 8, then (phase, group of kUnitWaves consecutive
//            units of the order); unit = position * nHeads + head; slice = phase * 8 + XCD.
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
                    int longPrefix, int ldQ) {
  typedef pipe::PairPipeline<ET, D, SOFTMAX, HEADS, false> Pipe;
  constexpr int T = D / 16;
  extern __shared__ __align__(1024) unsigned char smem[];

  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int g = lane >> 4;
  const int c = lane & 15;

  int w, t0, t1, slice = 0, head = 0;
  if constexpr (SLICED) {
    const int xcd = blockIdx.x % kXcds;
    const int j = blockIdx.x / kXcds;
    const int phase = j / nGroups;
#ifdef F3S_PROBE_SAME_UNIT
    // probe: the four waves of a workgroup all compute its first unit, at the same time
    const int64_t u = (int64_t)(j - phase * nGroups) * (int)(blockDim.x >> 6);
#else
    const int64_t u = (int64_t)(j - phase * nGroups) * (int)(blockDim.x >> 6) + wave;
#endif
    const int pos = HEADS ? (int)(u / nHeads) : (int)u;
    head = HEADS ? (int)(u - (int64_t)pos * nHeads) : 0;
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
  // block ranges that do not fit the structure (a mismatched rowWindowOffset) are not followed;
  // the slice index never holds one (sliced_setup_kernel makes such a window empty)
  if (t0 < 0 || (int64_t)t1 > nTcb) return;

  const pipe::Problem<ET> pb = make_problem<ET, D, HEADS>(sparseAToXidx, bitmapBytes, Q, K, V, N,
                                                          scaleLog2, ldIn, nTcb, ldQ);
  const unsigned ringAddr =
      (unsigned)(uintptr_t)(F3S_LDS unsigned char*)smem + (unsigned)wave * pipe::Geo<D>::WAVE_BYTES;
  Pipe pp;
  pp.init(pb, w, ringAddr, head);
  pp.run(pb, t0, t1);

  if constexpr (SLICED) {
    const int64_t wh = (int64_t)w * (HEADS ? nHeads : 1) + head;
    store_partial<D>(pp, partial + (wh * S + slice) * partial_dwords<D>() + lane);
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

// ---- workspace of the column-sliced schedule (f3s_attention_workspace_bytes) ------------------
//   header (256 B) | tickets of the resident grid (256 B) | sliceStart [nRW * (S + 1)] |
//   partial results [nRW * nHeads * S]
// The slice boundaries depend on the TC-block structure only. sliced_setup_kernel builds them at
// the start of every call unless the header says that f3s_attention_prepare built them for
// exactly these arrays.
struct SlicedHeader {
  uint32_t magic;
  int32_t N, S, prepared;
  int64_t nTcb;
  const void* rwo;
  const void* atox;
};
constexpr uint32_t kSlicedMagic = 0xF35C0DE5u;

// sliceStart[w * (S + 1) + s] = first TC block of window w whose first (smallest) column id is
// >= s * sliceWidth; entry S is the window's end. One thread per entry, binary search over the
// window's blocks (their first columns ascend). A block range that does not fit the structure
// (a mismatched rowWindowOffset) makes the window empty: every entry 0.
// mode 0: part of an attention call, index rebuilt; mode 1: f3s_attention_prepare (index built,
// header written); mode 2: part of an attention call whose caller says the workspace is prepared:
// the index is kept if the header confirms it and rebuilt otherwise.
__global__ __launch_bounds__(256) void sliced_setup_kernel(
    const int32_t* __restrict__ rowWindowOffset, const int32_t* __restrict__ sparseAToXidx, int N,
    int nRW, int S, int sliceWidth, int64_t nTcb, SlicedHeader* __restrict__ hdr, int mode,
    int32_t* __restrict__ tickets, int32_t* __restrict__ sliceStart) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < kXcds) tickets[idx] = 0;
  if (mode == 2) {
    const bool cached = hdr->magic == kSlicedMagic && hdr->prepared == 1 && hdr->N == N &&
                        hdr->S == S && hdr->nTcb == nTcb && hdr->rwo == rowWindowOffset &&
                        hdr->atox == sparseAToXidx;
    if (cached) return;
  }
  if (idx == 0) {
    if (mode == 1) {
      hdr->magic = kSlicedMagic;
      hdr->N = N;
      hdr->S = S;
      hdr->nTcb = nTcb;
      hdr->rwo = rowWindowOffset;
      hdr->atox = sparseAToXidx;
      hdr->prepared = 1;
    } else {
      hdr->prepared = 0;  // the index no longer belongs to an earlier f3s_attention_prepare
    }
  }
  const int per = S + 1;
  if (idx >= (int64_t)nRW * per) return;
  const int w = (int)(idx / per), b = (int)(idx % per);
  int lo = rowWindowOffset[w], hi = rowWindowOffset[w + 1];
  if (lo < 0 || (int64_t)hi > nTcb || hi < lo) lo = hi = 0;
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

// The resident form: as many workgroups as the GPU holds at once, NW independent waves each.
//   * A workgroup takes a ticket of the XCD it runs on (XCC_ID from the hardware) and with it a
//     slot (xcd, rank); if that XCD's slots are gone (the hardware did not deal the workgroups
//     evenly) it takes a slot of the next XCD. Every slot is taken exactly once, so the result
//     does not depend on where workgroups run; only the L2 locality does.
//   * Slot (x, r) owns groups of NW consecutive units of XCD x's list (phase by phase, heavy
//     windows first), dealt to the ranks in boustrophedon order (r, 2R-1-r, 2R+r, ...: every rank
//     gets an equal share of heavy and light units); the workgroup's waves draw their next unit
//     from a counter in LDS. No device-wide atomic is on the path of a unit.
//   * The window of the unit after next and the block range of the next unit are requested before
//     the current unit runs, so they have arrived when it ends.
// Measured on the 233k-node benchmark graph at d = 64: 1.51 ms against 1.45 ms for the launch-order
// kernel (static shares leave a tail that the hardware's dispatch of fresh workgroups does not),
// so this form is the one to ask for (F3S_SLICED_PERSISTENT=1) where workgroups are not dealt
// round-robin to the XCDs. A variant in which the wave that finishes a window's last unit merges
// its partials (an arrival counter per window, partials written through) took 1.92 ms: the wait
// for the stores and the returning atomic sit on every unit's path.
template <typename ET, int D, bool SOFTMAX, bool HEADS, int NW>
__global__ __launch_bounds__(NW * 64)
__attribute__((amdgpu_waves_per_eu(unit_waves_per_simd(D), unit_waves_per_simd(D)))) void
f3s_fwd_resident_kernel(const int32_t* __restrict__ windowOrder,
                        const int32_t* __restrict__ sliceStart, int P, int nRW, int S, int N,
                        int64_t nTcb, int32_t* __restrict__ tickets,
                        const int32_t* __restrict__ sparseAToXidx,
                        const uint8_t* __restrict__ bitmapBytes, const ET* __restrict__ Q,
                        const ET* __restrict__ K, const ET* __restrict__ V, float scaleLog2,
                        float* __restrict__ partial, int nHeads, int ldIn) {
  typedef pipe::PairPipeline<ET, D, SOFTMAX, HEADS, false> Pipe;
  extern __shared__ __align__(1024) unsigned char smem[];
  __shared__ int sCtl[2];  // slot of this workgroup; next unit of its sequence

  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int per = (int)(gridDim.x / kXcds);  // slots per XCD
  if (threadIdx.x == 0) {
    unsigned xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    int slot = -1;
    for (int k = 0; k < kXcds && slot < 0; k++) {
      const int x = (int)((xcc + k) & (kXcds - 1));
      const int r = __hip_atomic_fetch_add(&tickets[x], 1, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
      if (r < per) slot = x * per + r;
    }
    sCtl[0] = slot;
    sCtl[1] = 0;
  }
  __syncthreads();
  const int slot = sCtl[0];
  if (slot < 0) return;  // cannot happen: the grid is a multiple of 8, every workgroup finds a slot
  const int x = slot / per;
  const int r = slot - x * per;
  const int heads = HEADS ? nHeads : 1;
  const int64_t units = (int64_t)P * nRW * heads;  // units of one XCD

  const pipe::Problem<ET> pb = make_problem<ET, D, HEADS>(sparseAToXidx, bitmapBytes, Q, K, V, N,
                                                          scaleLog2, ldIn, nTcb);
  const unsigned ringAddr =
      (unsigned)(uintptr_t)(F3S_LDS unsigned char*)smem + (unsigned)wave * pipe::Geo<D>::WAVE_BYTES;

  // k-th unit of this workgroup's sequence -> index in the XCD's unit space, -1 past its end,
  // -2 when the sequence is over
  auto unit_index = [&](int k) -> int64_t {
    const int j = k / NW;
    if ((int64_t)j * per * NW >= units) return -2;
    const int grp = (j & 1) ? j * per + (per - 1 - r) : j * per + r;
    const int64_t u = (int64_t)grp * NW + (k - j * NW);
    return u < units ? u : -1;
  };
  auto claim = [&]() -> int64_t {
    int k = 0;
    if (lane == 0)
      k = __hip_atomic_fetch_add(&sCtl[1], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    return unit_index(uniform(k));
  };
  // unit -> (phase, position of the order, head)
  auto window_of = [&](int64_t u) -> int {
    if (u < 0) return -1;
    const int pos = (int)((u / heads) % nRW);
    const int w = windowOrder ? windowOrder[pos] : pos;
    return (unsigned)w < (unsigned)nRW ? w : -1;
  };
  auto slice_of = [&](int64_t u) -> int { return (int)((u / heads) / nRW) * kXcds + x; };

  // three units in flight: `u` runs, u1 has its window and is fetching its block range, u2 is
  // fetching its window
  int64_t u = claim();
  int w = window_of(u);
  int t0 = 0, t1 = 0;
  if (w >= 0) {
    t0 = sliceStart[(int64_t)w * (S + 1) + slice_of(u)];
    t1 = sliceStart[(int64_t)w * (S + 1) + slice_of(u) + 1];
  }
  int64_t u1 = u == -2 ? -2 : claim();
  int w1 = window_of(u1);
  while (u != -2) {
    int t0n = 0, t1n = 0;
    if (w1 >= 0) {
      t0n = sliceStart[(int64_t)w1 * (S + 1) + slice_of(u1)];
      t1n = sliceStart[(int64_t)w1 * (S + 1) + slice_of(u1) + 1];
    }
    const int64_t u2 = u1 == -2 ? -2 : claim();
    const int w2 = window_of(u2);
    const int wu = uniform(w), t0u = uniform(t0), t1u = uniform(t1);
    if (wu >= 0 && t1u > t0u && t0u >= 0 && (int64_t)t1u <= nTcb) {
      const int head = HEADS ? (int)(u % heads) : 0;
      Pipe pp;
      pp.init(pb, wu, ringAddr, head);
      pp.run(pb, t0u, t1u);
      const int64_t wh = (int64_t)wu * heads + head;
      store_partial<D>(pp, partial + (wh * S + slice_of(u)) * partial_dwords<D>() + lane);
    }
    u = u1;
    w = w1;
    t0 = t0n;
    t1 = t1n;
    u1 = u2;
    w1 = w2;
  }
}

// One wave per (window, head): log-sum-exp merge of the unit partials in slice order, then the
// window's rows. Lane (g, c) holds O[q = c][16j + 4g + i] in O[j * 4 + i], as in the unit
// kernels. The partials of up to B live slices are requested together.
template <int D, bool SOFTMAX>
__global__ __launch_bounds__(256) void f3s_merge_slices_kernel(
    const int32_t* __restrict__ sliceStart, int S, int N, int nRW, int nHeads,
    const float* __restrict__ partial, float* __restrict__ out, int ldOut) {
  constexpr int T = D / 16;
  constexpr int R = D / 4;  // O registers per lane
  constexpr int B = D <= 64 ? 4 : D <= 128 ? 2 : 1;
  const int lane = threadIdx.x & 63;
  const int64_t wh = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (wh >= (int64_t)nRW * nHeads) return;
  const int w = (int)(wh / nHeads);
  const int head = (int)(wh - (int64_t)w * nHeads);
  const int g = lane >> 4;
  const int c = lane & 15;
  float M = 0.0f, L = 0.0f;
  float O[R];
#pragma unroll
  for (int r = 0; r < R; r++) O[r] = 0.0f;
  const int32_t* ss = sliceStart + (int64_t)w * (S + 1);
  const float* base = partial + wh * S * partial_dwords<D>() + lane;
  for (int s0 = 0; s0 < S; s0 += 64) {
    const int s = s0 + lane;
    unsigned long long live = __builtin_amdgcn_ballot_w64(s < S && ss[s + 1] > ss[s]);
    while (live) {
      int sel[B];
      float v[B][R + 2];
#pragma unroll
      for (int k = 0; k < B; k++) {
        sel[k] = -1;
        if (live) {
          sel[k] = s0 + __builtin_ctzll(live);
          live &= live - 1;
          const float* src = base + (int64_t)sel[k] * partial_dwords<D>();
#pragma unroll
          for (int r = 0; r < R + (SOFTMAX ? 2 : 0); r++)
            v[k][r] = F3S_PARTIAL_LOAD(src + r * 64);
        }
      }
#pragma unroll
      for (int k = 0; k < B; k++) {
        if (sel[k] < 0) continue;
        if constexpr (SOFTMAX) {
          const float ms = v[k][R], ls = v[k][R + 1];
          const float mx = fmaxf(M, ms);
          const float a = pipe::fast_exp2(M - mx), b = pipe::fast_exp2(ms - mx);
          M = mx;
          L = fmaf(a, L, b * ls);
#pragma unroll
          for (int r = 0; r < R; r++) O[r] = fmaf(a, O[r], b * v[k][r]);
        } else {
#pragma unroll
          for (int r = 0; r < R; r++) O[r] += v[k][r];
        }
      }
    }
  }
  float inv = 1.0f;
  if constexpr (SOFTMAX) {
    const float lAll = pipe::row_sum4(L);
    inv = (lAll == 0.0f) ? 0.0f : 1.0f / lAll;
  }
  const int64_t row = (int64_t)w * 16 + c;
  if (row < N) {
    float* dst = out + row * ldOut + head * D + 4 * g;
#pragma unroll
    for (int jj = 0; jj < T; jj++) {
      const float4v v4 = {O[jj * 4] * inv, O[jj * 4 + 1] * inv, O[jj * 4 + 2] * inv,
                          O[jj * 4 + 3] * inv};
      *reinterpret_cast<float4v*>(dst + 16 * jj) = v4;
    }
  }
}

// LDS of a workgroup of rings; above 64 KiB the kernel has to be told once
template <typename KernelT>
int allow_lds(KernelT kernel, size_t bytes) {
  if (bytes > 64 * 1024)
    F3S_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
  return 0;
}

// Phases P (S = 8 P slices). One slice's K + V rows are held to about 8 MiB: twice an XCD's L2,
// which already catches 4 of 5 accesses on the 233k-node benchmark graph (P = 1), while more and
// shorter units cost more than their higher hit rate returns (measured 1.54 / 1.69 / 1.86 ms at
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

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// byte offsets of the parts of the workspace
struct SlicedLayout {
  int P, S;
  size_t tickets, sliceStart, partial, total;
  size_t padded;  // 0, or where the copies of K and V with 256-byte rows start (single head, d = 64)
};
// Rows of 128 bytes gathered from addresses that are multiples of 256 are served faster than rows
// from the odd 128-byte lines in between (233k-node graph, d = 64: 1.42 ms with every row on an
// even line, 1.55 ms with every row on an odd line, 1.48 ms for contiguous rows, which alternate;
// the L2 hit and miss counts are the same in all three). The single-head call at d = 64 therefore
// gathers from copies of K and V with a row pitch of 256 bytes, made at the start of the call.
constexpr int kPaddedRowBytes = 256;
// nHeads = 0: the single-head layout
SlicedLayout sliced_layout(int N, int d, int nHeads) {
  const int heads = nHeads > 0 ? nHeads : 1;
  SlicedLayout L;
  L.P = choose_phases(N, d * heads);
  L.S = L.P * kXcds;
  const size_t nRW = (size_t)(N + kWinRows - 1) / kWinRows;
  L.tickets = 256;
  L.sliceStart = L.tickets + 256;
  L.partial = L.sliceStart + align256(nRW * (L.S + 1) * sizeof(int32_t));
  L.total = align256(L.partial + nRW * heads * L.S * (size_t)(d / 4 + 2) * 64 * sizeof(float));
  L.padded = 0;
  if (nHeads == 0 && d == 64) {
    L.padded = L.total;
    L.total += 2 * (size_t)N * kPaddedRowBytes;
  }
  return L;
}

// K and V rows of 128 bytes copied to a pitch of 256 bytes (one thread per 16 bytes of each)
typedef int pad_chunk __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void pad_rows_kernel(const pad_chunk* __restrict__ K,
                                                       const pad_chunk* __restrict__ V,
                                                       int64_t chunks, pad_chunk* __restrict__ Kp,
                                                       pad_chunk* __restrict__ Vp) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= chunks) return;
  const int64_t row = i >> 3;
  const int c = (int)(i & 7);
  const pad_chunk k = __builtin_nontemporal_load(K + i);  // read once, by nobody else
  const pad_chunk v = __builtin_nontemporal_load(V + i);
  Kp[row * (kPaddedRowBytes / 16) + c] = k;
  Vp[row * (kPaddedRowBytes / 16) + c] = v;
}

bool padded_rows_requested() {
  const char* e = getenv("F3S_PAD_ROWS");  // read per call; 0 switches the copies off
  return !(e && e[0] == '0');
}

// workgroups of NW waves the GPU holds at once (LDS rings, waves per SIMD), a multiple of 8
template <int D, int NW>
int resident_grid(int* grid) {
  constexpr int kMaxDev = 64;
  static int cusOf[kMaxDev] = {};
  int dev = 0;
  F3S_HIP_CHECK(hipGetDevice(&dev));
  int cus = (dev >= 0 && dev < kMaxDev) ? cusOf[dev] : 0;
  if (cus == 0) {
    F3S_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    if (dev >= 0 && dev < kMaxDev) cusOf[dev] = cus;
  }
  // the rings plus the 1 KiB the two control words cost in front of the 1 KiB-aligned rings
  constexpr size_t lds = (size_t)NW * pipe::Geo<D>::WAVE_BYTES + 1024;
  int perCu = (int)((160 * 1024) / lds);
  const int byWaves = unit_waves_per_simd(D) * 4 / NW;
  if (perCu > byWaves) perCu = byWaves;
  if (perCu < 1) perCu = 1;
  int gsz = cus * perCu / kXcds * kXcds;
  if (gsz < kXcds) gsz = kXcds;
  *grid = gsz;
  return 0;
}

bool resident_requested() {
  const char* e = getenv("F3S_SLICED_PERSISTENT");  // read per call
  return e && e[0] == '1';
}

template <typename ET, int D, bool SOFTMAX, bool HEADS>
int launch_sliced_units(const int32_t* rwo, const int32_t* order, const int32_t* atox,
                        const uint8_t* bm, int N, int nRW, const ET* Q, const ET* K, const ET* V,
                        float scaleLog2, float* out, int32_t* tickets, int32_t* sliceStart,
                        float* partial, const SlicedLayout& L, int heads, int ldIn, int ldOut,
                        int64_t nTcb, hipStream_t stream, int ldQ = 0) {
  constexpr size_t lds = (size_t)kUnitWaves * pipe::Geo<D>::WAVE_BYTES;
  if (resident_requested()) {
    auto kernel = f3s_fwd_resident_kernel<ET, D, SOFTMAX, HEADS, kUnitWaves>;
    if (int rc = allow_lds(kernel, lds)) return rc;
    int grid = 0;
    if (int rc = resident_grid<D, kUnitWaves>(&grid)) return rc;
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kUnitWaves * 64), lds, stream, order,
                       sliceStart, L.P, nRW, L.S, N, nTcb, tickets, atox, bm, Q, K, V, scaleLog2,
                       partial, heads, ldIn);
  } else {
    auto kernel = f3s_fwd_unit_kernel<ET, D, SOFTMAX, true, HEADS>;
    if (int rc = allow_lds(kernel, lds)) return rc;
    const int64_t nGroups = ((int64_t)nRW * heads + kUnitWaves - 1) / kUnitWaves;
    const int64_t grid = (int64_t)L.P * nGroups * kXcds;
    if (grid >= ((int64_t)1 << 31))
      return fail(-2, "f3s_attention: too many (window, slice, head) units for one launch");
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kUnitWaves * 64), lds, stream, order, rwo,
                       atox, bm, sliceStart, L.S, (int)nGroups, N, nRW, nTcb, Q, K, V, scaleLog2,
                       partial, out, heads, ldIn, ldOut, 0, 0, ldQ);
  }
  F3S_HIP_CHECK(hipGetLastError());
  return 0;
}

template <typename ET, int D, bool SOFTMAX>
int launch_sliced_d(const int32_t* rwo, const int32_t* order, const int32_t* atox,
                    const uint64_t* bitmap, int N, const void* Q, const void* K, const void* V,
                    float scaleLog2, float* out, char* ws, const SlicedLayout& L, int nHeads,
                    int ldIn, int ldOut, int mode, int64_t nTcb, hipStream_t stream) {
  const int nRW = (N + kWinRows - 1) / kWinRows;
  const int S = L.S;
  const int sliceWidth = (N + S - 1) / S;
  const int heads = nHeads > 0 ? nHeads : 1;
  auto* hdr = reinterpret_cast<SlicedHeader*>(ws);
  auto* tickets = reinterpret_cast<int32_t*>(ws + L.tickets);
  auto* sliceStart = reinterpret_cast<int32_t*>(ws + L.sliceStart);
  auto* partial = reinterpret_cast<float*>(ws + L.partial);
  const int64_t entries = (int64_t)nRW * (S + 1);
  hipLaunchKernelGGL(sliced_setup_kernel, dim3((unsigned)((entries + 255) / 256)), dim3(256), 0,
                     stream, rwo, atox, N, nRW, S, sliceWidth, nTcb, hdr, mode, tickets,
                     sliceStart);
  F3S_HIP_CHECK(hipGetLastError());
  if (mode == 1) return 0;
  const auto* bm = reinterpret_cast<const uint8_t*>(bitmap);
  const auto* q = static_cast<const ET*>(Q);
  const auto* k = static_cast<const ET*>(K);
  const auto* v = static_cast<const ET*>(V);
  int rc;
  if (nHeads > 0) {
    rc = launch_sliced_units<ET, D, SOFTMAX, true>(rwo, order, atox, bm, N, nRW, q, k, v,
                                                   scaleLog2, out, tickets, sliceStart, partial, L,
                                                   heads, ldIn, ldOut, nTcb, stream);
  } else if (L.padded != 0 && padded_rows_requested() && !resident_requested() &&
             !gather_needs_wide_offsets(N, kPaddedRowBytes, true)) {
    // copies of K and V with 256-byte rows, gathered through the pitched (multi-head) form of the
    // unit kernel with one head; Q stays where it is
    auto* kp = reinterpret_cast<ET*>(ws + L.padded);
    auto* vp = kp + (size_t)N * (kPaddedRowBytes / sizeof(ET));
    const int64_t chunks = (int64_t)N * (D * (int)sizeof(ET) / 16);
    hipLaunchKernelGGL(pad_rows_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0,
                       stream, reinterpret_cast<const pad_chunk*>(k),
                       reinterpret_cast<const pad_chunk*>(v), chunks,
                       reinterpret_cast<pad_chunk*>(kp), reinterpret_cast<pad_chunk*>(vp));
    F3S_HIP_CHECK(hipGetLastError());
    rc = launch_sliced_units<ET, D, SOFTMAX, true>(
        rwo, order, atox, bm, N, nRW, q, kp, vp, scaleLog2, out, tickets, sliceStart, partial, L, 1,
        kPaddedRowBytes / (int)sizeof(ET), D, nTcb, stream, D);
  } else {
    rc = launch_sliced_units<ET, D, SOFTMAX, false>(rwo, order, atox, bm, N, nRW, q, k, v,
                                                    scaleLog2, out, tickets, sliceStart, partial,
                                                    L, 1, D, D, nTcb, stream);
  }
  if (rc != 0) return rc;
  const int64_t merges = (int64_t)nRW * heads;
  hipLaunchKernelGGL((f3s_merge_slices_kernel<D, SOFTMAX>), dim3((unsigned)((merges + 3) / 4)),
                     dim3(256), 0, stream, sliceStart, S, N, nRW, heads, partial, out,
                     nHeads > 0 ? ldOut : D);
  F3S_HIP_CHECK(hipGetLastError());
  return 0;
}

}  // namespace

size_t attention_sliced_workspace_bytes(int N, int d, int nHeads) {
  return sliced_layout(N, d, nHeads).total;
}

// mode 0 / 2: an attention call (2: on a prepared workspace); mode 1: f3s_attention_prepare
// (index only, Q/K/V/out unused)
int launch_attention_sliced(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                            const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int d,
                            int dtype, const void* Q, const void* K, const void* V,
                            float scaleLog2, int applySoftmax, float* out, void* workspace,
                            size_t wsBytes, int64_t nTcb, int nHeads, int ldIn, int ldOut,
                            int mode, hipStream_t stream) {
  if (!head_dim_supported(d))
    return fail(-2, "f3s_attention: head dim %d unsupported (a multiple of 32 up to 256)", d);
  const SlicedLayout L = sliced_layout(N, d, nHeads);
  if (wsBytes < L.total)
    return fail(-2, "f3s_attention: workspace %zu B < required %zu B", wsBytes, L.total);
  char* ws = static_cast<char*>(workspace);
#define F3S_SLICED(DD)                                                                         \
  if (d == DD) {                                                                               \
    if (dtype == 0)                                                                            \
      return applySoftmax ? launch_sliced_d<_Float16, DD, true>(                               \
                                rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, Q, K,  \
                                V, scaleLog2, out, ws, L, nHeads, ldIn, ldOut, mode,     \
                                nTcb, stream)                                                  \
                          : launch_sliced_d<_Float16, DD, false>(                              \
                                rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, Q, K,  \
                                V, scaleLog2, out, ws, L, nHeads, ldIn, ldOut, mode,     \
                                nTcb, stream);                                                 \
    return applySoftmax ? launch_sliced_d<__bf16, DD, true>(                                   \
                              rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, Q, K, V, \
                              scaleLog2, out, ws, L, nHeads, ldIn, ldOut, mode, nTcb,    \
                              stream)                                                          \
                        : launch_sliced_d<__bf16, DD, false>(                                  \
                              rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, Q, K, V, \
                              scaleLog2, out, ws, L, nHeads, ldIn, ldOut, mode, nTcb,    \
                              stream);                                                         \
  }
  F3S_FOR_EACH_HEAD_DIM(F3S_SLICED)
#undef F3S_SLICED
  return fail(-2, "f3s_attention: head dim %d unsupported (a multiple of 32 up to 256)", d);
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
                       scaleLog2, nullptr, out, nHeads, ldIn, ldOut, maxBlocks, longPrefix, 0);
  } else {
    if (int rc = allow_lds(f3s_fwd_unit_kernel<ET, D, SOFTMAX, false, false>, lds)) return rc;
    hipLaunchKernelGGL((f3s_fwd_unit_kernel<ET, D, SOFTMAX, false, false>), grid, block, lds,
                       stream, order, rwo, atox, bm, nullptr, 0, 0, N, (int)nRW, nTcb, q, k, v,
                       scaleLog2, nullptr, out, 1, D, D, maxBlocks, longPrefix, 0);
  }
  F3S_HIP_CHECK(hipGetLastError());
  return 0;
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
#define F3S_SHORT(DD)                                                                          \
  if (d == DD) {                                                                               \
    if (dtype == 0)                                                                            \
      return applySoftmax ? launch_short_d<_Float16, DD, true>(                                \
                                rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, Q, K,  \
                                V, scaleLog2, out, nHeads, ldIn, ldOut, maxBlocks,       \
                                longPrefix, nTcb, stream)                                      \
                          : launch_short_d<_Float16, DD, false>(                               \
                                rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, Q, K,  \
                                V, scaleLog2, out, nHeads, ldIn, ldOut, maxBlocks,       \
                                longPrefix, nTcb, stream);                                     \
    return applySoftmax ? launch_short_d<__bf16, DD, true>(                                    \
                              rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, Q, K, V, \
                              scaleLog2, out, nHeads, ldIn, ldOut, maxBlocks,            \
                              longPrefix, nTcb, stream)                                        \
                        : launch_short_d<__bf16, DD, false>(                                   \
                              rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, Q, K, V, \
                              scaleLog2, out, nHeads, ldIn, ldOut, maxBlocks,            \
                              longPrefix, nTcb, stream);                                       \
  }
  F3S_FOR_EACH_HEAD_DIM(F3S_SHORT)
#undef F3S_SHORT
  return fail(-2, "f3s_attention: head dim %d unsupported (a multiple of 32 up to 256)", d);
}

}  // namespace f3s
