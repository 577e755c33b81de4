// Fused 3S attention, column-band schedule (gfx950). Same arithmetic per TC-block pair as
// f3s_fwd_kernel (f3s_attention.hip, which documents the register dataflow and the numerics);
// what differs is who computes what, and when:
//
//   * a wave owns G whole row windows at a time and keeps their (m, l, O) and Q fragments in
//     registers, so there is no cross-wave merge and no LDS traffic for state;
//   * the column range is cut into bands, and every wave walks band 0 of all its windows, then
//     band 1, ...: at any moment all waves of the GPU gather K/V rows from about the same band.
//     A band's K+V rows fit in an XCD's 4 MiB L2, so a row is fetched from the memory side once
//     per XCD and sweep instead of once per window that names it.
//
// The reference has no counterpart of this schedule: its kernels (src/F3S_kernel.cu:1371-1583)
// walk one window per thread block from its first TC block to its last. The window order it
// sorts (src/utils.cu:400-436) is used here to deal windows to waves heavy-first.
#include "f3s_common.h"

namespace f3s {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef int int4v __attribute__((ext_vector_type(4)));

template <int T>
struct HalfVec {
  typedef _Float16 type __attribute__((ext_vector_type(T)));
};

constexpr int kMaxBands = 64;
constexpr int kBandWaves = 4;  // waves per workgroup (they do not cooperate)

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

// bandStart[w * (nBands + 1) + b] = first TC block of window w whose first (smallest) column id
// is >= b * bandWidth; entry nBands is the window's end. One thread per entry, binary search
// over the window's blocks (their first columns ascend).
__global__ void band_index_kernel(const int32_t* __restrict__ rowWindowOffset,
                                  const int32_t* __restrict__ sparseAToXidx, int nRW, int nBands,
                                  int bandWidth, int32_t* __restrict__ bandStart) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int per = nBands + 1;
  if (idx >= (int64_t)nRW * per) return;
  const int w = (int)(idx / per), b = (int)(idx % per);
  int lo = rowWindowOffset[w], hi = rowWindowOffset[w + 1];
  if (b == nBands) {
    bandStart[idx] = hi;
    return;
  }
  const int64_t limit = (int64_t)b * bandWidth;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (sparseAToXidx[(int64_t)mid * 16] < limit)
      lo = mid + 1;
    else
      hi = mid;
  }
  bandStart[idx] = lo;
}

template <int D>
struct PairData {
  half8 kA[D / 32], kB[D / 32];
  typename HalfVec<D / 16>::type vv[8];
  unsigned maskA, maskB;
  int desc;  // window slot | hasB << 8
};
struct PairIndex {
  int meta;
  int desc;
};

template <int S>
struct Slot {
  static constexpr int value = S;
};

template <int D, int G, bool SOFTMAX>
__global__ __launch_bounds__(kBandWaves * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void
f3s_fwd_band_kernel(const int32_t* __restrict__ windowOrder,
                    const int32_t* __restrict__ sparseAToXidx,
                    const uint8_t* __restrict__ bitmapBytes,
                    const int32_t* __restrict__ bandStart, int nBands, int N, int nRW,
                    const _Float16* __restrict__ Q, const _Float16* __restrict__ K,
                    const _Float16* __restrict__ V, float scaleLog2, float* __restrict__ out) {
  constexpr int T = D / 16;
  constexpr int KS = D / 32;
  typedef typename HalfVec<T>::type vrow_t;
  __shared__ int2 sSeg[kBandWaves][G * kMaxBands];

  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int g = lane >> 4;
  const int c = lane & 15;
  const int nWaves = gridDim.x * kBandWaves;
  const int gw = blockIdx.x * kBandWaves + wave;
  int2* seg = sSeg[wave];
  const int nSeg = G * nBands;

  const int maskByte = ((g >> 1) * 2 + (c >> 3)) * 8 + 7 - (c & 7);
  const int maskShift = 4 * (1 - (g & 1));
  const int permAddr = (4 * c + g) * 4;
  const char* Kb = reinterpret_cast<const char*>(K);
  const char* Vb = reinterpret_cast<const char*>(V);
  auto lane_read = [&](int v, int srcLane) { return __builtin_amdgcn_ds_bpermute(srcLane * 4, v); };

  // ---- sweeps: each takes the next nWaves * G windows of the order, dealt round-robin
  for (int base = 0; base < nRW; base += nWaves * G) {
    int win[G];
    half8 qf[G][KS];
    float m[G], l[G];
    float4v o[G][T];
#pragma unroll
    for (int k = 0; k < G; k++) {
      const int idx = base + k * nWaves + gw;
      int w = -1;
      if (idx < nRW) {
        w = uniform(windowOrder ? windowOrder[idx] : idx);
        if ((unsigned)w >= (unsigned)nRW) w = -1;  // corrupt order entry
      }
      win[k] = w;
      const int64_t qrow = (int64_t)w * 16 + c;
      if (w >= 0 && qrow < N) {
        const half8* qp = reinterpret_cast<const half8*>(Q + qrow * D) + g;
#pragma unroll
        for (int i = 0; i < KS; i++) qf[k][i] = qp[4 * i];
      } else {
#pragma unroll
        for (int i = 0; i < KS; i++) qf[k][i] = half8{0, 0, 0, 0, 0, 0, 0, 0};
      }
      m[k] = 0.0f;
      l[k] = 0.0f;
#pragma unroll
      for (int j = 0; j < T; j++) o[k][j] = float4v{0.f, 0.f, 0.f, 0.f};
    }

    // segment table of this wave, band-major: segment b*G + k = blocks of window k in band b
    int myPairs = 0;
    for (int s = lane; s < nSeg; s += 64) {
      const int b = s / G, k = s - b * G;
      int w = win[0];
#pragma unroll
      for (int kk = 1; kk < G; kk++) w = (k == kk) ? win[kk] : w;
      int tS = 0, tE = 0;
      if (w >= 0) {
        tS = bandStart[(int64_t)w * (nBands + 1) + b];
        tE = bandStart[(int64_t)w * (nBands + 1) + b + 1];
      }
      seg[s] = make_int2(tS, tE);
      myPairs += (tE - tS + 1) >> 1;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) myPairs += __shfl_xor(myPairs, off);
    const int totalPairs = uniform(myPairs);
    __builtin_amdgcn_wave_barrier();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");

    if (totalPairs > 0) {
      // cursor over the wave's pair sequence, kept in scalars; it saturates on the last pair
      int cs = -1, ct = 0, ce = 0;  // segment, first block of the current pair, segment end
      bool exhausted = false;
      auto next_segment = [&]() {
        // move to the next non-empty segment; false if there is none
        int s = cs;
        while (true) {
          s++;
          if (s >= nSeg) return false;
          const int2 v = seg[s];
          const int tS = uniform(v.x), tE = uniform(v.y);
          if (tE > tS) {
            cs = s;
            ct = tS;
            ce = tE;
            return true;
          }
        }
      };
      next_segment();
      auto advance = [&]() {
        if (exhausted) return;
        if (ct + 2 < ce) {
          ct += 2;
        } else if (!next_segment()) {
          exhausted = true;  // stay on the last pair: later loads repeat it and are never used
        }
      };

      auto load_index = [&]() {
        const int64_t tA = ct;
        const bool hasB = (ct + 1) < ce;
        const int idSlot = (lane & 31) & (hasB ? 31 : 15);
        const int bmSlot = (lane & 15) & (hasB ? 15 : 7);
        const int32_t* src = (lane < 32)
                                 ? sparseAToXidx + tA * 16 + idSlot
                                 : reinterpret_cast<const int32_t*>(bitmapBytes) + tA * 8 + bmSlot;
        PairIndex ix;
        ix.meta = *src;
        ix.desc = (cs % G) | ((hasB ? 1 : 0) << 8);
        advance();
        return ix;
      };
      auto load_data = [&](const PairIndex& ix) {
        PairData<D> pd;
        pd.desc = ix.desc;
        const uint32_t kRowA = (uint32_t)lane_read(ix.meta, lane >> 2);
        const uint32_t kRowB = (uint32_t)lane_read(ix.meta, 16 + (lane >> 2));
        const uint32_t koA = kRowA * (uint32_t)(D * 2) + (uint32_t)((lane & 3) * 16);
        const uint32_t koB = kRowB * (uint32_t)(D * 2) + (uint32_t)((lane & 3) * 16);
#pragma unroll
        for (int i = 0; i < KS; i++) {
          pd.kA[i] = *reinterpret_cast<const half8*>(Kb + koA + 64 * i);
          pd.kB[i] = *reinterpret_cast<const half8*>(Kb + koB + 64 * i);
        }
#pragma unroll
        for (int k = 0; k < 8; k++) {
          const uint32_t vRow = (uint32_t)lane_read(ix.meta, (k < 4 ? 0 : 16) + 4 * g + (k & 3));
          const uint32_t vo = vRow * (uint32_t)(D * 2) + (uint32_t)(c * T * 2);
          pd.vv[k] = *reinterpret_cast<const vrow_t*>(Vb + vo);
        }
        pd.maskA =
            ((unsigned)lane_read(ix.meta, 32 + (maskByte >> 2)) >> (8 * (maskByte & 3))) & 0xFFu;
        pd.maskB =
            ((unsigned)lane_read(ix.meta, 40 + (maskByte >> 2)) >> (8 * (maskByte & 3))) & 0xFFu;
        return pd;
      };
      auto to_mfma_layout = [&](half8 v) {
        int4v xv = __builtin_bit_cast(int4v, v);
#pragma unroll
        for (int k = 0; k < 4; k++) xv[k] = __builtin_amdgcn_ds_bpermute(permAddr, xv[k]);
        return __builtin_bit_cast(half8, xv);
      };
      auto compute_slot = [&](const PairData<D>& pd, auto slotTag) {
        constexpr int S = decltype(slotTag)::value;
        const bool hasB = (pd.desc >> 8) != 0;
        const unsigned bitsA = (pd.maskA >> maskShift) & 0xFu;
        const unsigned bitsB = hasB ? ((pd.maskB >> maskShift) & 0xFu) : 0u;
        float4v sA = {0.f, 0.f, 0.f, 0.f}, sB = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < KS; i++) {
          sA = __builtin_amdgcn_mfma_f32_16x16x32_f16(to_mfma_layout(pd.kA[i]), qf[S][i], sA, 0, 0,
                                                      0);
          sB = __builtin_amdgcn_mfma_f32_16x16x32_f16(to_mfma_layout(pd.kB[i]), qf[S][i], sB, 0, 0,
                                                      0);
        }
        float s[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
          s[i] = ((bitsA >> (3 - i)) & 1u) ? sA[i] : 0.0f;
          s[4 + i] = ((bitsB >> (3 - i)) & 1u) ? sB[i] : 0.0f;
        }
        half8 pf;
        if constexpr (SOFTMAX) {
          float mx = m[S];
#pragma unroll
          for (int i = 0; i < 8; i++) {
            s[i] *= scaleLog2;
            mx = fmaxf(mx, s[i]);
          }
          mx = row_max4(mx);
          const float alpha = fast_exp2(m[S] - mx);
          m[S] = mx;
          float sum = 0.0f;
#pragma unroll
          for (int i = 0; i < 8; i++) {
            const float ev = (s[i] == 0.0f) ? 0.0f : fast_exp2(s[i] - mx);
            sum += ev;
            pf[i] = (_Float16)ev;
          }
          l[S] = fmaf(alpha, l[S], sum);
#pragma unroll
          for (int j = 0; j < T; j++) o[S][j] *= alpha;
        } else {
#pragma unroll
          for (int i = 0; i < 8; i++) pf[i] = (_Float16)s[i];
        }
#pragma unroll
        for (int j = 0; j < T; j++) {
          half8 va;
#pragma unroll
          for (int k = 0; k < 8; k++) va[k] = pd.vv[k][j];
          o[S][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, pf, o[S][j], 0, 0, 0);
        }
      };
      auto compute = [&](const PairData<D>& pd) {
        const int slot = uniform(pd.desc & 0xFF);
        if (slot == 0) compute_slot(pd, Slot<0>{});
        if constexpr (G > 1)
          if (slot == 1) compute_slot(pd, Slot<1>{});
        if constexpr (G > 2)
          if (slot == 2) compute_slot(pd, Slot<2>{});
        if constexpr (G > 3)
          if (slot == 3) compute_slot(pd, Slot<3>{});
      };

      // same pipeline as f3s_fwd_kernel: metadata four pairs ahead, K/V two pairs ahead
      PairIndex m0 = load_index();
      PairIndex m1 = load_index();
      PairIndex m2 = load_index();
      PairData<D> pd0 = load_data(m0), pd1, pd2;
      m0 = load_index();
      pd1 = load_data(m1);
      int done = 0;
#define F3S_STEP(CUR, FILL, MUSE, MFILL) \
  MFILL = load_index();                  \
  FILL = load_data(MUSE);                \
  compute(CUR);                          \
  if (++done >= totalPairs) break;
      while (true) {
        F3S_STEP(pd0, pd2, m2, m1)
        F3S_STEP(pd1, pd0, m0, m2)
        F3S_STEP(pd2, pd1, m1, m0)
      }
#undef F3S_STEP
    }

    // ---- write the rows of this sweep's windows: lane (g, c) holds O[q=c][(4g+i)*T + j]
#pragma unroll
    for (int k = 0; k < G; k++) {
      if (win[k] < 0) continue;
      float inv = 1.0f;
      if constexpr (SOFTMAX) {
        const float lAll = row_sum4(l[k]);
        inv = (lAll == 0.0f) ? 0.0f : 1.0f / lAll;
      }
      const int64_t row = (int64_t)win[k] * 16 + c;
      if (row < N) {
        float* dst = out + row * D + 4 * g * T;
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
          for (int j = 0; j < T; j++) dst[i * T + j] = o[k][j][i] * inv;
      }
    }
    // the segment table is rewritten by the next sweep only after every lane is past its reads
    __builtin_amdgcn_wave_barrier();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
}

template <int D, bool SOFTMAX>
int launch_band_d(const int32_t* rwo, const int32_t* order, const int32_t* atox,
                  const uint64_t* bitmap, int N, const void* Q, const void* K, const void* V,
                  float scaleLog2, float* out, int32_t* bandStart, int nBands, int bandWidth,
                  hipStream_t stream) {
  constexpr int G = 2;
  const int nRW = (N + kWinRows - 1) / kWinRows;
  const int64_t entries = (int64_t)nRW * (nBands + 1);
  hipLaunchKernelGGL(band_index_kernel, dim3((unsigned)((entries + 255) / 256)), dim3(256), 0,
                     stream, rwo, atox, nRW, nBands, bandWidth, bandStart);
  F3S_HIP_CHECK(hipGetLastError());
  // two workgroups of four waves per CU = two waves per SIMD on all 256 CUs
  int grid = 512;
  const int needed = (nRW + kBandWaves * G - 1) / (kBandWaves * G);
  if (grid > needed) grid = needed;
  hipLaunchKernelGGL((f3s_fwd_band_kernel<D, G, SOFTMAX>), dim3(grid), dim3(kBandWaves * 64), 0,
                     stream, order, atox, reinterpret_cast<const uint8_t*>(bitmap), bandStart,
                     nBands, N, nRW, static_cast<const _Float16*>(Q),
                     static_cast<const _Float16*>(K), static_cast<const _Float16*>(V), scaleLog2,
                     out);
  F3S_HIP_CHECK(hipGetLastError());
  return 0;
}

// bands sized so that one band's K + V rows take about 1.5 MiB of an XCD's 4 MiB L2
int choose_bands(int N, int d, int* bandWidth) {
  const int64_t bandCols = (int64_t)(1536 * 1024) / (4 * d);
  int nBands = (int)((N + bandCols - 1) / bandCols);
  if (nBands < 1) nBands = 1;
  if (nBands > kMaxBands) nBands = kMaxBands;
  *bandWidth = (N + nBands - 1) / nBands;
  if (*bandWidth < 1) *bandWidth = 1;
  return nBands;
}

}  // namespace

size_t attention_workspace_bytes(int N, int d) {
  int bw;
  const int nBands = choose_bands(N, d, &bw);
  const size_t nRW = (size_t)(N + kWinRows - 1) / kWinRows;
  return nRW * (size_t)(nBands + 1) * sizeof(int32_t);
}

int launch_attention_band(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                          const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int d,
                          const void* Q, const void* K, const void* V, float scaleLog2,
                          int applySoftmax, float* out, void* workspace, size_t wsBytes,
                          hipStream_t stream) {
  if (wsBytes < attention_workspace_bytes(N, d))
    return fail(-2, "f3s_attention_fwd: workspace %zu B < required %zu B", wsBytes,
                attention_workspace_bytes(N, d));
  int bw;
  const int nBands = choose_bands(N, d, &bw);
  int32_t* bandStart = static_cast<int32_t*>(workspace);
#define F3S_BAND(DD)                                                                            \
  case DD:                                                                                      \
    return applySoftmax                                                                         \
               ? launch_band_d<DD, true>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, \
                                         Q, K, V, scaleLog2, out, bandStart, nBands, bw, stream) \
               : launch_band_d<DD, false>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap,  \
                                          N, Q, K, V, scaleLog2, out, bandStart, nBands, bw,    \
                                          stream);
  switch (d) {
    F3S_BAND(32)
    F3S_BAND(64)
    F3S_BAND(128)
    default:
      return fail(-2, "f3s_attention_fwd: head dim %d unsupported (32, 64, 128)", d);
  }
#undef F3S_BAND
}

}  // namespace f3s
