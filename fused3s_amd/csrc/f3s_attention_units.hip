// Fused 3S attention with one wave per unit of work (gfx950). Same arithmetic per TC-block pair
// as f3s_fwd_kernel (f3s_attention.hip, which documents the register dataflow and the numerics);
// what differs is the decomposition. Two uses of the one kernel, f3s_fwd_unit_kernel:
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

#include "f3s_common.h"

namespace f3s {
namespace {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef int int4v __attribute__((ext_vector_type(4)));

constexpr int kXcds = 8;
constexpr int kMaxPhases = 16;
constexpr int kUnitWaves = 4;  // waves (= units) per workgroup; they do not cooperate

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float row_max4(float v) {
  v = fmaxf(v, __shfl_xor(v, 16));
  v = fmaxf(v, __shfl_xor(v, 32));
  return v;
}
__device__ __forceinline__ float row_sum4(float v) {
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 32);
  return v;
}
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// sliceStart[w * (S + 1) + s] = first TC block of window w whose first (smallest) column id is
// >= s * sliceWidth; entry S is the window's end. One thread per entry, binary search over the
// window's blocks (their first columns ascend).
__global__ void slice_index_kernel(const int32_t* __restrict__ rowWindowOffset,
                                   const int32_t* __restrict__ sparseAToXidx, int nRW, int S,
                                   int sliceWidth, int32_t* __restrict__ sliceStart) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
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

struct PairIndex {
  int meta;
};

// Partial result of a unit: D/4 + 2 dwords per lane, stored register by register so that every
// store and load is one coalesced 256-byte row: [o[0][0..3], ..., o[T-1][0..3], m, l][64 lanes].
template <int D>
constexpr int partial_dwords() {
  return (D / 4 + 2) * 64;
}

// Vectors of the 16-bit input type ET (_Float16 or __bf16) and the MFMA that contracts them.
template <typename ET, int L>
struct Vec {
  typedef ET type __attribute__((ext_vector_type(L)));
};
template <typename ET>
__device__ __forceinline__ float4v mfma_16x16x32(typename Vec<ET, 8>::type a,
                                                 typename Vec<ET, 8>::type b, float4v acc);
template <>
__device__ __forceinline__ float4v mfma_16x16x32<_Float16>(Vec<_Float16, 8>::type a,
                                                           Vec<_Float16, 8>::type b,
                                                           float4v acc) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc, 0, 0, 0);
}
template <>
__device__ __forceinline__ float4v mfma_16x16x32<__bf16>(Vec<__bf16, 8>::type a,
                                                         Vec<__bf16, 8>::type b, float4v acc) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
}

template <typename ET, int D>
struct UnitPair {
  typename Vec<ET, 8>::type kA[D / 32], kB[D / 32];
  typename Vec<ET, D / 16>::type vv[8];
  unsigned maskA, maskB;
};

constexpr int unit_waves_per_simd(int d, bool sliced) { return (!sliced && d <= 32) ? 4 : 2; }

// One wave per unit, four independent units per workgroup. A unit is
//   SLICED:  the TC blocks of one (window, column slice); the result is a partial (m, l, O);
//   !SLICED: one whole window (of one head, if HEADS); the result is the window's output rows.
//            Windows of more than maxBlocks TC blocks among the first longPrefix positions of
//            the order are left to f3s_fwd_kernel, whose four waves share a window and whose
//            grid covers exactly those positions (with a heavy-first order no long window lies
//            beyond them; with any other order such a window is simply computed here). Unit u = position * nHeads + head,
//            so the waves of a workgroup mostly work on the heads of one window and share its
//            column ids and bitmaps.
template <typename ET, int D, bool SOFTMAX, bool SLICED, bool HEADS>
__global__ __launch_bounds__(kUnitWaves * 64)
__attribute__((amdgpu_waves_per_eu(unit_waves_per_simd(D, SLICED),
                                   unit_waves_per_simd(D, SLICED)))) void
f3s_fwd_unit_kernel(const int32_t* __restrict__ windowOrder,
                    const int32_t* __restrict__ rowWindowOffset,
                    const int32_t* __restrict__ sparseAToXidx,
                    const uint8_t* __restrict__ bitmapBytes,
                    const int32_t* __restrict__ sliceStart, int S, int nGroups, int N, int nRW,
                    const ET* __restrict__ Q, const ET* __restrict__ K,
                    const ET* __restrict__ V, float scaleLog2, float* __restrict__ partial,
                    float* __restrict__ out, int nHeads, int ldIn, int ldOut, int maxBlocks,
                    int longPrefix) {
  typedef typename Vec<ET, 8>::type half8;
  constexpr int T = D / 16;
  constexpr int KS = D / 32;
  typedef typename Vec<ET, T>::type vrow_t;

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
    const int pos = (j - phase * nGroups) * kUnitWaves + wave;
    if (pos >= nRW) return;
    slice = phase * kXcds + xcd;
    w = uniform(windowOrder ? windowOrder[pos] : pos);
    if ((unsigned)w >= (unsigned)nRW) return;  // a corrupt order entry must not index out of range
    t0 = uniform(sliceStart[(int64_t)w * (S + 1) + slice]);
    t1 = uniform(sliceStart[(int64_t)w * (S + 1) + slice + 1]);
    if (t1 <= t0) return;  // empty unit: nothing is written, the merge skips it
  } else {
    const int64_t u = (int64_t)blockIdx.x * kUnitWaves + wave;
    const int pos = HEADS ? (int)(u / nHeads) : (int)u;
    head = HEADS ? (int)(u - (int64_t)pos * nHeads) : 0;
    if (pos >= nRW) return;
    w = uniform(windowOrder ? windowOrder[pos] : pos);
    if ((unsigned)w >= (unsigned)nRW) return;
    t0 = uniform(rowWindowOffset[w]);
    t1 = uniform(rowWindowOffset[w + 1]);
    if (t1 - t0 > maxBlocks && pos < longPrefix) return;  // f3s_fwd_kernel's
  }
  const int pitchIn = HEADS ? ldIn : D;
  const int pitchOut = HEADS ? ldOut : D;
  const uint32_t rowBytes = (uint32_t)pitchIn * 2u;
  Q += head * D;
  K += head * D;
  V += head * D;
  const int nPairs = (t1 - t0 + 1) >> 1;

  half8 qf[KS];
  {
    const int4v zero16 = {0, 0, 0, 0};
    const int64_t qrow = (int64_t)w * 16 + c;
    if (qrow < N) {
      const half8* qp = reinterpret_cast<const half8*>(Q + qrow * pitchIn) + g;
#pragma unroll
      for (int i = 0; i < KS; i++) qf[i] = qp[4 * i];
    } else {
#pragma unroll
      for (int i = 0; i < KS; i++) qf[i] = __builtin_bit_cast(half8, zero16);
    }
  }
  float m = 0.0f, l = 0.0f;
  float4v o[T];
#pragma unroll
  for (int jj = 0; jj < T; jj++) o[jj] = float4v{0.f, 0.f, 0.f, 0.f};

  const int maskByte = ((g >> 1) * 2 + (c >> 3)) * 8 + 7 - (c & 7);
  const int maskShift = 4 * (1 - (g & 1));
  const int permAddr = (4 * c + g) * 4;
  const char* Kb = reinterpret_cast<const char*>(K);
  const char* Vb = reinterpret_cast<const char*>(V);
  auto lane_read = [&](int v, int srcLane) { return __builtin_amdgcn_ds_bpermute(srcLane * 4, v); };
  // byte offset of a gathered row: 24-bit multiply for the pitched layout (N < 2^24 is checked
  // by the launcher), a shift for the contiguous one
  auto row_offset = [&](uint32_t row) {
    return HEADS ? __umul24(row, rowBytes) : row * (uint32_t)(D * 2);
  };

  auto load_index = [&](int p) {
    const int64_t tA = t0 + 2 * p;
    const bool hasB = (tA + 1) < t1;
    const int idSlot = (lane & 31) & (hasB ? 31 : 15);
    const int bmSlot = (lane & 15) & (hasB ? 15 : 7);
    const int32_t* src = (lane < 32)
                             ? sparseAToXidx + tA * 16 + idSlot
                             : reinterpret_cast<const int32_t*>(bitmapBytes) + tA * 8 + bmSlot;
    PairIndex ix;
    ix.meta = *src;
    return ix;
  };
  auto load_data = [&](const PairIndex& ix) {
    UnitPair<ET, D> pd;
    const uint32_t kRowA = (uint32_t)lane_read(ix.meta, lane >> 2);
    const uint32_t kRowB = (uint32_t)lane_read(ix.meta, 16 + (lane >> 2));
    const uint32_t koA = row_offset(kRowA) + (uint32_t)((lane & 3) * 16);
    const uint32_t koB = row_offset(kRowB) + (uint32_t)((lane & 3) * 16);
#pragma unroll
    for (int i = 0; i < KS; i++) {
      pd.kA[i] = *reinterpret_cast<const half8*>(Kb + koA + 64 * i);
      pd.kB[i] = *reinterpret_cast<const half8*>(Kb + koB + 64 * i);
    }
#pragma unroll
    for (int k = 0; k < 8; k++) {
      const uint32_t vRow = (uint32_t)lane_read(ix.meta, (k < 4 ? 0 : 16) + 4 * g + (k & 3));
      const uint32_t vo = row_offset(vRow) + (uint32_t)(c * T * 2);
      pd.vv[k] = *reinterpret_cast<const vrow_t*>(Vb + vo);
    }
    pd.maskA = ((unsigned)lane_read(ix.meta, 32 + (maskByte >> 2)) >> (8 * (maskByte & 3))) & 0xFFu;
    pd.maskB = ((unsigned)lane_read(ix.meta, 40 + (maskByte >> 2)) >> (8 * (maskByte & 3))) & 0xFFu;
    return pd;
  };
  auto to_mfma_layout = [&](half8 v) {
    int4v xv = __builtin_bit_cast(int4v, v);
#pragma unroll
    for (int k = 0; k < 4; k++) xv[k] = __builtin_amdgcn_ds_bpermute(permAddr, xv[k]);
    return __builtin_bit_cast(half8, xv);
  };
  auto compute = [&](const UnitPair<ET, D>& pd, int p) {
    const bool hasB = (t0 + 2 * p + 1) < t1;
    const unsigned bitsA = (pd.maskA >> maskShift) & 0xFu;
    const unsigned bitsB = hasB ? ((pd.maskB >> maskShift) & 0xFu) : 0u;
    float4v sA = {0.f, 0.f, 0.f, 0.f}, sB = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < KS; i++) {
      sA = mfma_16x16x32<ET>(to_mfma_layout(pd.kA[i]), qf[i], sA);
      sB = mfma_16x16x32<ET>(to_mfma_layout(pd.kB[i]), qf[i], sB);
    }
    float s[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      s[i] = ((bitsA >> (3 - i)) & 1u) ? sA[i] : 0.0f;
      s[4 + i] = ((bitsB >> (3 - i)) & 1u) ? sB[i] : 0.0f;
    }
    half8 pf;
    if constexpr (SOFTMAX) {
      float mx = m;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        s[i] *= scaleLog2;
        mx = fmaxf(mx, s[i]);
      }
      mx = row_max4(mx);
      const float alpha = fast_exp2(m - mx);
      m = mx;
      float sum = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const float ev = (s[i] == 0.0f) ? 0.0f : fast_exp2(s[i] - mx);
        sum += ev;
        pf[i] = (ET)ev;
      }
      l = fmaf(alpha, l, sum);
#pragma unroll
      for (int jj = 0; jj < T; jj++) o[jj] *= alpha;
    } else {
#pragma unroll
      for (int i = 0; i < 8; i++) pf[i] = (ET)s[i];
    }
#pragma unroll
    for (int jj = 0; jj < T; jj++) {
      half8 va;
#pragma unroll
      for (int k = 0; k < 8; k++) va[k] = pd.vv[k][jj];
      o[jj] = mfma_16x16x32<ET>(va, pf, o[jj]);
    }
  };

  // same pipeline as f3s_fwd_kernel: metadata four pairs ahead, K/V rows two pairs ahead
  if (nPairs > 0) {
    const int pLast = nPairs - 1;
    auto clamp_pair = [&](int q) { return q < pLast ? q : pLast; };
    int p = 0;
    PairIndex m0 = load_index(0);
    PairIndex m1 = load_index(clamp_pair(1));
    PairIndex m2 = load_index(clamp_pair(2));
    UnitPair<ET, D> pd0 = load_data(m0), pd1, pd2;
    m0 = load_index(clamp_pair(3));
    pd1 = load_data(m1);
#define F3S_STEP(CUR, FILL, MUSE, MFILL)  \
  MFILL = load_index(clamp_pair(p + 4));  \
  FILL = load_data(MUSE);                 \
  compute(CUR, p);                        \
  p += 1;                                 \
  if (p > pLast) break;
    while (true) {
      F3S_STEP(pd0, pd2, m2, m1)
      F3S_STEP(pd1, pd0, m0, m2)
      F3S_STEP(pd2, pd1, m1, m0)
    }
#undef F3S_STEP
  }

  if constexpr (SLICED) {
    float* dst = partial + ((int64_t)w * S + slice) * partial_dwords<D>() + lane;
#pragma unroll
    for (int jj = 0; jj < T; jj++)
#pragma unroll
      for (int i = 0; i < 4; i++) __builtin_nontemporal_store(o[jj][i], dst + (jj * 4 + i) * 64);
    __builtin_nontemporal_store(m, dst + (D / 4) * 64);
    __builtin_nontemporal_store(l, dst + (D / 4 + 1) * 64);
  } else {
    // lane (g, c) holds O[q = c][(4g + i) * T + j] in o[j][i]: 4T consecutive floats of row c
    float inv = 1.0f;
    if constexpr (SOFTMAX) {
      const float lAll = row_sum4(l);
      inv = (lAll == 0.0f) ? 0.0f : 1.0f / lAll;
    }
    const int64_t row = (int64_t)w * 16 + c;
    if (row < N) {
      float* dst = out + row * pitchOut + head * D + 4 * g * T;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        float4v v;
#pragma unroll
        for (int jj = 0; jj < 4; jj++) v[jj] = 0.f;
        if constexpr (T == 4) {
          v = float4v{o[0][i] * inv, o[1][i] * inv, o[2][i] * inv, o[3][i] * inv};
          *reinterpret_cast<float4v*>(dst + i * T) = v;
        } else {
#pragma unroll
          for (int jj = 0; jj < T; jj++) dst[i * T + jj] = o[jj][i] * inv;
        }
      }
    }
  }
}

// One wave per window: log-sum-exp merge of the window's unit partials, then the window's rows.
// Lane (g, c) holds O[q = c][(4g + i) * T + j] in o[j][i], as in the unit kernel.
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
      const float a = fast_exp2(M - mx), b = fast_exp2(ms - mx);
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
    const float lAll = row_sum4(L);
    inv = (lAll == 0.0f) ? 0.0f : 1.0f / lAll;
  }
  const int64_t row = (int64_t)w * 16 + c;
  if (row < N) {
    {
      float* dst = out + row * D + 4 * g * T;
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int jj = 0; jj < T; jj++) dst[i * T + jj] = O[jj * 4 + i] * inv;
    }
  }
}

// Phases P (S = 8 P slices). One slice's K + V rows are held to about 8 MiB: twice an XCD's L2,
// which already catches 4 of 5 accesses on the 233k-node benchmark graph (P = 1), while more and
// shorter units cost more than their higher hit rate returns (measured 1.99 / 2.23 / 2.48 ms at
// P = 1 / 2 / 3). F3S_SLICE_PHASES in the environment overrides the choice.
int choose_phases(int N, int d) {
  static const int forced = [] {
    const char* e = getenv("F3S_SLICE_PHASES");
    return e ? atoi(e) : 0;
  }();
  if (forced > 0) return forced > kMaxPhases ? kMaxPhases : forced;
  const int64_t bytes = (int64_t)N * d * 4;  // K + V
  const int64_t perPhase = (int64_t)kXcds * 8 * 1024 * 1024;
  int P = (int)((bytes + perPhase - 1) / perPhase);
  if (P < 1) P = 1;
  if (P > kMaxPhases) P = kMaxPhases;
  return P;
}

template <typename ET, int D, bool SOFTMAX>
int launch_sliced_d(const int32_t* rwo, const int32_t* order, const int32_t* atox,
                    const uint64_t* bitmap, int N, const void* Q, const void* K, const void* V,
                    float scaleLog2, float* out, int32_t* sliceStart, float* partial, int P,
                    hipStream_t stream) {
  const int nRW = (N + kWinRows - 1) / kWinRows;
  const int S = P * kXcds;
  const int sliceWidth = (N + S - 1) / S;
  const int64_t entries = (int64_t)nRW * (S + 1);
  hipLaunchKernelGGL(slice_index_kernel, dim3((unsigned)((entries + 255) / 256)), dim3(256), 0,
                     stream, rwo, atox, nRW, S, sliceWidth, sliceStart);
  F3S_HIP_CHECK(hipGetLastError());
  const int nGroups = (nRW + kUnitWaves - 1) / kUnitWaves;
  hipLaunchKernelGGL((f3s_fwd_unit_kernel<ET, D, SOFTMAX, true, false>),
                     dim3((unsigned)(P * nGroups * kXcds)), dim3(kUnitWaves * 64), 0, stream, order,
                     rwo, atox, reinterpret_cast<const uint8_t*>(bitmap), sliceStart, S, nGroups, N,
                     nRW, static_cast<const ET*>(Q), static_cast<const ET*>(K),
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
  return align256(nRW * (S + 1) * sizeof(int32_t)) + nRW * S * (size_t)(d / 4 + 2) * 64 * 4;
}

int launch_attention_sliced(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                            const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int d,
                            int dtype, const void* Q, const void* K, const void* V,
                            float scaleLog2, int applySoftmax, float* out, void* workspace,
                            size_t wsBytes, hipStream_t stream) {
  if (wsBytes < attention_sliced_workspace_bytes(N, d))
    return fail(-2, "f3s_attention_fwd: workspace %zu B < required %zu B", wsBytes,
                attention_sliced_workspace_bytes(N, d));
  const int P = choose_phases(N, d);
  const size_t nRW = (size_t)(N + kWinRows - 1) / kWinRows;
  int32_t* sliceStart = static_cast<int32_t*>(workspace);
  float* partial = reinterpret_cast<float*>(static_cast<char*>(workspace) +
                                            align256(nRW * ((size_t)P * kXcds + 1) * 4));
#define F3S_SLICED(ET, DD)                                                                     \
  case DD:                                                                                     \
    return applySoftmax ? launch_sliced_d<ET, DD, true>(rowWindowOffset, windowOrder,          \
                                                        sparseAToXidx, bitmap, N, Q, K, V,     \
                                                        scaleLog2, out, sliceStart, partial,   \
                                                        P, stream)                             \
                        : launch_sliced_d<ET, DD, false>(rowWindowOffset, windowOrder,         \
                                                         sparseAToXidx, bitmap, N, Q, K, V,    \
                                                         scaleLog2, out, sliceStart, partial,  \
                                                         P, stream);
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
                   int longPrefix, hipStream_t stream) {
  const int64_t nRW = ((int64_t)N + kWinRows - 1) / kWinRows;
  const int64_t units = nRW * (nHeads > 0 ? nHeads : 1);
  const dim3 grid((unsigned)((units + kUnitWaves - 1) / kUnitWaves)), block(kUnitWaves * 64);
  const auto* bm = reinterpret_cast<const uint8_t*>(bitmap);
  const auto* q = static_cast<const ET*>(Q);
  const auto* k = static_cast<const ET*>(K);
  const auto* v = static_cast<const ET*>(V);
  if (nHeads > 0)
    hipLaunchKernelGGL((f3s_fwd_unit_kernel<ET, D, SOFTMAX, false, true>), grid, block, 0, stream,
                       order, rwo, atox, bm, nullptr, 0, 0, N, (int)nRW, q, k, v, scaleLog2,
                       nullptr, out, nHeads, ldIn, ldOut, maxBlocks, longPrefix);
  else
    hipLaunchKernelGGL((f3s_fwd_unit_kernel<ET, D, SOFTMAX, false, false>), grid, block, 0, stream,
                       order, rwo, atox, bm, nullptr, 0, 0, N, (int)nRW, q, k, v, scaleLog2,
                       nullptr, out, 1, D, D, maxBlocks, longPrefix);
  F3S_HIP_CHECK(hipGetLastError());
  return 0;
}

template <typename ET>
int launch_short_et(const int32_t* rwo, const int32_t* order, const int32_t* atox,
                    const uint64_t* bitmap, int N, int d, const void* Q, const void* K,
                    const void* V, float scaleLog2, int applySoftmax, float* out, int nHeads,
                    int ldIn, int ldOut, int maxBlocks, int longPrefix, hipStream_t stream) {
#define F3S_SHORT(DD)                                                                          \
  case DD:                                                                                     \
    return applySoftmax ? launch_short_d<ET, DD, true>(rwo, order, atox, bitmap, N, Q, K, V,   \
                                                       scaleLog2, out, nHeads, ldIn, ldOut,    \
                                                       maxBlocks, longPrefix, stream)          \
                        : launch_short_d<ET, DD, false>(rwo, order, atox, bitmap, N, Q, K, V,  \
                                                        scaleLog2, out, nHeads, ldIn, ldOut,   \
                                                        maxBlocks, longPrefix, stream);
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
                                   hipStream_t stream) {
  return dtype == 0
             ? launch_short_et<_Float16>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, d,
                                         Q, K, V, scaleLog2, applySoftmax, out, nHeads, ldIn,
                                         ldOut, maxBlocks, longPrefix, stream)
             : launch_short_et<__bf16>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, d, Q,
                                       K, V, scaleLog2, applySoftmax, out, nHeads, ldIn, ldOut,
                                       maxBlocks, longPrefix, stream);
}

}  // namespace f3s
