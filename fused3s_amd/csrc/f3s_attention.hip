// Fused SDDMM -> online softmax -> SpMM over 16x16 TC blocks for gfx950 (MI355X), wave64.
//
// Replaces the reference kernels f3sKernel1tb1rw / ...Scheduled / ...ScheduledPermutedQKV
// [ScaleQK] and f2sKernel1tb1rw (src/F3S_kernel.cu:997-1175, 1371-1800, 1999-2182, 2186-2327)
// and their launchers (src/F3S_kernel.cu:393-458, 581-671).
//
// One workgroup owns one 16-row window; its waves take the window's TC blocks two at a time
// (pair p -> wave p % NWAVES) and keep private running (m, l, O) in registers. One LDS merge
// per window combines the waves (log-sum-exp), instead of the reference's three block barriers
// per iteration.
//
// Register dataflow of one TC-block pair (lane = 16*g + c, g in 0..3, c in 0..15):
//   S^T = K_t Q^T   v_mfma_f32_16x16x32_f16, A = gathered K rows (lane: row slot c, features
//                   32i+8g..+7, one 16-byte load), B = Q (lane: query row c, same features).
//                   The accumulator leaves S[q=c][slot 4g+i], i<4, in this lane.
//   mask            one byte of the block's bitmap holds this lane's 4 bits.
//   softmax         row q=c lives in lanes c, c+16, c+32, c+48: 8 in-register values and two
//                   cross-lane steps.
//   O^T += V^T P^T  v_mfma_f32_16x16x32_f16 over the 32 keys of the pair, contraction index
//                   8g+k <-> (block A, slot 4g+k) for k<4, (block B, slot 4g+k-4) for k>=4, so
//                   the B operand is exactly the 8 probabilities this lane already holds.
//                   A = V^T: the lane reads D/16 contiguous halfs of each of its 8 key rows
//                   (16 lanes cover one whole V row: coalesced), element j feeds output tile j.
//                   Tile j therefore owns output columns {c*(D/16)+j}; after the MFMA lane
//                   (g,c) holds O[q=c][g*D/4 .. (g+1)*D/4), a contiguous run.
// Neither Q, K, V nor P touches LDS.
//
// Numerics follow the reference kernel (src/F3S_kernel.cu:1402-1406,1447-1451,1487-1499,
// 938-945,1560-1561): running max starts at 0 and masked zeros take part in it, an unmasked
// score that is exactly 0 is dropped like a masked one, the row sum uses un-rounded fp32
// exponentials while P is rounded to fp16 for the second MFMA, empty rows give 0.
#include <stdlib.h>
#include <string.h>

#include "f3s_common.h"

namespace f3s {
namespace {

typedef float float4v __attribute__((ext_vector_type(4)));

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

constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// max / sum over the four lanes {c, c+16, c+32, c+48} that share a query row
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

// Everything one TC-block pair needs from memory, as it sits in registers.
template <typename ET, int D>
struct PairData {
  typename Vec<ET, 8>::type kA[D / 32], kB[D / 32];  // K rows of the two blocks (A operand of S^T)
  typename Vec<ET, D / 16>::type vv[8];    // V pieces of this lane's 8 contraction slots
  unsigned maskA, maskB;                   // bitmap byte holding this lane's 4 bits per block
};
// Metadata of a pair, one dword per lane from a single load: lanes 0..31 hold the 32 column ids
// of blocks A and B, lanes 32..47 the 16 dwords of their bitmaps. Every lane later picks what it
// needs with cross-lane reads, which do not go through the memory pipeline.
struct PairIndex {
  int meta;
};

// Waves per SIMD the kernel is held to. Two at D >= 64: measured on the 233k-node benchmark
// graph 3.17 ms at one wave, 2.04 ms at two, 2.62 ms at three. The kernel is bound by instruction
// issue on the SIMDs with the vector L1 close behind, so a third wave has little to add, and the
// extra windows in flight per XCD spread the gather over more columns than the L2 holds.
constexpr int waves_per_simd(int d) { return d <= 32 ? 4 : 2; }

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
// blocks are laid out exactly like one 16x16 block, so the same pair pipeline runs over four
// 16x8 blocks per step; rowWindowOffset then counts 16x8 blocks, a window may end in the middle
// of a pair, and sddmm (if not null) receives the masked, unscaled scores, row-major 16x8 per
// block (saveSddmmResult, src/F3S_kernel.cu:99-115).
template <typename ET, int D, int NWAVES, bool SOFTMAX, bool CLOCKED, bool HEADS, bool W8>
__global__ __launch_bounds__(NWAVES * 64)
__attribute__((amdgpu_waves_per_eu(waves_per_simd(D), waves_per_simd(D)))) void f3s_fwd_kernel(
    const int32_t* __restrict__ rowWindowOffset, const int32_t* __restrict__ windowOrder,
    const int32_t* __restrict__ sparseAToXidx, const uint8_t* __restrict__ bitmapBytes, int N,
    int nRW, const ET* __restrict__ Q, const ET* __restrict__ K, const ET* __restrict__ V,
    float scaleLog2, float* __restrict__ out, unsigned long long* __restrict__ cuTimer,
    int nHeads, int ldIn, int ldOut, float* __restrict__ sddmm, int minBlocks) {
  typedef typename Vec<ET, 8>::type half8;
  constexpr int T = D / 16;   // output tiles == halfs read per lane per V row
  unsigned long long tBegin = 0;
  if constexpr (CLOCKED) tBegin = realtime_ticks();
  constexpr int KS = D / 32;  // MFMA k-steps of the score product
  constexpr int OSTRIDE = D + 4;
  typedef typename Vec<ET, T>::type vrow_t;

  __shared__ float sM[NWAVES][16];
  __shared__ float sL[NWAVES][16];
  __shared__ __align__(16) float sO[NWAVES][16][OSTRIDE];

  const int pos = HEADS ? (int)(blockIdx.x / (unsigned)nHeads) : (int)blockIdx.x;
  const int head = HEADS ? (int)(blockIdx.x - (unsigned)pos * (unsigned)nHeads) : 0;
  const int w = windowOrder ? windowOrder[pos] : pos;
  if ((unsigned)w >= (unsigned)nRW) return;  // a corrupt order entry must not index out of range
  // row pitches in elements / bytes; compile-time constants for the single-head layout
  const int pitchIn = HEADS ? ldIn : D;
  const int pitchOut = HEADS ? ldOut : D;
  const uint32_t rowBytes = (uint32_t)pitchIn * 2u;
  Q += head * D;
  K += head * D;
  V += head * D;
  out += head * D;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int g = lane >> 4;
  const int c = lane & 15;

  const int t0 = rowWindowOffset[w];
  const int t1 = rowWindowOffset[w + 1];
  // windows of at most minBlocks blocks belong to the wave-per-window kernel of the same call
  // (f3s_fwd_unit_kernel); -1 when this kernel computes every window
  if (t1 - t0 <= minBlocks) return;
  constexpr int BPP = W8 ? 4 : 2;  // blocks of the structure per pipeline step
  const int nPairs = (t1 - t0 + BPP - 1) / BPP;

  // B operand of the score product: this lane's query row, features 32i + 8g .. +7
  typedef int int4v __attribute__((ext_vector_type(4)));
  const int4v zero16 = {0, 0, 0, 0};
  half8 qf[KS];
  {
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

  float m = 0.0f;  // running row max (log2 domain when SOFTMAX), starts at 0 like the reference
  float l = 0.0f;  // this lane's share of the row sum
  float4v o[T];
#pragma unroll
  for (int j = 0; j < T; j++) o[j] = float4v{0.f, 0.f, 0.f, 0.f};

  const int maskByte = ((g >> 1) * 2 + (c >> 3)) * 8 + 7 - (c & 7);
  const int maskShift = 4 * (1 - (g & 1));

  // the second block of the window's last pair may not exist: it aliases the first one
  // (loads stay in bounds) and its bits are cleared at use
  auto load_index = [&](int p) {
    PairIndex ix;
    if constexpr (W8) {
      // 8 ids and 4 bitmap dwords per block; blocks past the window's end fold onto the first
      const int64_t tA = t0 + 4 * p;
      const int nValid = (t1 - tA) < 4 ? (int)(t1 - tA) : 4;
      int idSlot = lane & 31;
      if (idSlot >= nValid * 8) idSlot &= 7;
      int bmSlot = lane & 15;
      if (bmSlot >= nValid * 4) bmSlot &= 3;
      const int32_t* src = (lane < 32)
                               ? sparseAToXidx + tA * 8 + idSlot
                               : reinterpret_cast<const int32_t*>(bitmapBytes) + tA * 4 + bmSlot;
      ix.meta = *src;
    } else {
      const int64_t tA = t0 + 2 * p;
      const bool hasB = (tA + 1) < t1;
      // lane -> dword index inside the pair's 32 ids / 16 bitmap dwords (second block folded
      // onto the first when it does not exist)
      const int idSlot = (lane & 31) & (hasB ? 31 : 15);
      const int bmSlot = (lane & 15) & (hasB ? 15 : 7);
      const int32_t* src = (lane < 32)
                               ? sparseAToXidx + tA * 16 + idSlot
                               : reinterpret_cast<const int32_t*>(bitmapBytes) + tA * 8 + bmSlot;
      ix.meta = *src;
    }
    return ix;
  };
  auto lane_read = [&](int v, int srcLane) { return __builtin_amdgcn_ds_bpermute(srcLane * 4, v); };
  auto load_data = [&](const PairIndex& ix) {
    PairData<ET, D> pd;
    // 32-bit byte offsets from the uniform K / V bases (the launcher checks that K and V span
    // less than 4 GiB, and N < 2^24 for the pitched layout, whose row offset is a 24-bit
    // multiply): one address register per gathered row instead of a 64-bit pointer per load
    auto row_offset = [&](uint32_t row) {
      return HEADS ? __umul24(row, rowBytes) : row * (uint32_t)(D * 2);
    };
    const char* Kb = reinterpret_cast<const char*>(K);
    const char* Vb = reinterpret_cast<const char*>(V);
    // K is fetched with four adjacent lanes on one 64-byte piece of a row (lane -> slot lane/4,
    // 16-byte chunk lane%4): 16 cache-line touches per load instead of 64. compute() moves the
    // pieces to the MFMA layout (slot c, chunk g) with a cross-lane permute.
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
  // lane (g, c) takes the 16 bytes that lane 4c + g loaded
  const int permAddr = (4 * c + g) * 4;
  auto to_mfma_layout = [&](half8 v) {
    int4v x = __builtin_bit_cast(int4v, v);
#pragma unroll
    for (int k = 0; k < 4; k++) x[k] = __builtin_amdgcn_ds_bpermute(permAddr, x[k]);
    return __builtin_bit_cast(half8, x);
  };
  auto compute = [&](const PairData<ET, D>& pd, int p) {
    // this lane's slots 4g..4g+3 of block A / B exist? (16x8 structure: they belong to block
    // g/2 resp. 2 + g/2 of the step's four)
    const int tFirst = t0 + BPP * p;
    const bool validA = W8 ? (tFirst + (g >> 1)) < t1 : true;
    const bool validB = W8 ? (tFirst + 2 + (g >> 1)) < t1 : (tFirst + 1) < t1;
    const unsigned bitsA = validA ? ((pd.maskA >> maskShift) & 0xFu) : 0u;
    const unsigned bitsB = validB ? ((pd.maskB >> maskShift) & 0xFu) : 0u;
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
    if constexpr (W8) {
      if (sddmm) {
        // lane (g, c): row c, columns 4(g&1)..+3 of block tFirst + g/2 (A) and + 2 (B)
        float* dst = sddmm + ((size_t)(tFirst + (g >> 1)) * 16 + c) * 8 + 4 * (g & 1);
        if (validA) *reinterpret_cast<float4*>(dst) = float4{s[0], s[1], s[2], s[3]};
        if (validB) *reinterpret_cast<float4*>(dst + 256) = float4{s[4], s[5], s[6], s[7]};
      }
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
        const float e = (s[i] == 0.0f) ? 0.0f : fast_exp2(s[i] - mx);
        sum += e;
        pf[i] = (ET)e;
      }
      l = fmaf(alpha, l, sum);
#pragma unroll
      for (int j = 0; j < T; j++) o[j] *= alpha;
    } else {
#pragma unroll
      for (int i = 0; i < 8; i++) pf[i] = (ET)s[i];
    }
#pragma unroll
    for (int j = 0; j < T; j++) {
      half8 va;
#pragma unroll
      for (int k = 0; k < 8; k++) va[k] = pd.vv[k][j];
      o[j] = mfma_16x16x32<ET>(va, pf, o[j]);
    }
  };

  // Software pipeline per wave over its pairs p = wave, wave + NWAVES, ...: in the step of pair p
  // the metadata of pair p+4 is requested, the K/V loads of pair p+2 are issued (their metadata
  // was requested four steps earlier, so waiting for it never waits for younger K/V loads and
  // the cold HBM miss it usually is stays off the critical path), and pair p is computed.
  // Three data buffers and three metadata registers rotate; the loop is unrolled three times so
  // that every buffer has a fixed role in every copy of the body.
  if (wave < nPairs) {
    // loads past the wave's last pair are redirected to that pair (same lines again, no branch)
    const int pLast = wave + ((nPairs - 1 - wave) / NWAVES) * NWAVES;
    auto clamp_pair = [&](int q) { return q < pLast ? q : pLast; };
    int p = wave;
    PairIndex m0 = load_index(p);
    PairIndex m1 = load_index(clamp_pair(p + NWAVES));
    PairIndex m2 = load_index(clamp_pair(p + 2 * NWAVES));
    PairData<ET, D> pd0 = load_data(m0), pd1, pd2;
    m0 = load_index(clamp_pair(p + 3 * NWAVES));
    pd1 = load_data(m1);
#define F3S_STEP(CUR, FILL, MUSE, MFILL)              \
  MFILL = load_index(clamp_pair(p + 4 * NWAVES));      \
  FILL = load_data(MUSE);                              \
  compute(CUR, p);                                     \
  p += NWAVES;                                         \
  if (p > pLast) break;
    while (true) {
      F3S_STEP(pd0, pd2, m2, m1)
      F3S_STEP(pd1, pd0, m0, m2)
      F3S_STEP(pd2, pd1, m1, m0)
    }
#undef F3S_STEP
  }

  // ---- merge the waves' partial (m, l, O) and write the window's rows
  if constexpr (SOFTMAX) l = row_sum4(l);
  if (g == 0) {
    sM[wave][c] = m;
    sL[wave][c] = l;
  }
#pragma unroll
  for (int j = 0; j < T; j++)
#pragma unroll
    for (int i = 0; i < 4; i++) sO[wave][c][g * (D / 4) + i * T + j] = o[j][i];
  __syncthreads();

  constexpr int VEC_PER_ROW = D / 4;
  for (int idx = threadIdx.x; idx < 16 * VEC_PER_ROW; idx += NWAVES * 64) {
    const int q = idx / VEC_PER_ROW;
    const int cv = idx % VEC_PER_ROW;
    const int64_t row = (int64_t)w * 16 + q;
    if (row >= N) continue;
    float4 acc = {0.f, 0.f, 0.f, 0.f};
    if constexpr (SOFTMAX) {
      float mAll = sM[0][q];
#pragma unroll
      for (int v = 1; v < NWAVES; v++) mAll = fmaxf(mAll, sM[v][q]);
      float lAll = 0.0f;
#pragma unroll
      for (int v = 0; v < NWAVES; v++) {
        const float f = fast_exp2(sM[v][q] - mAll);
        lAll = fmaf(f, sL[v][q], lAll);
        const float4 ov = *reinterpret_cast<const float4*>(&sO[v][q][cv * 4]);
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
        const float4 ov = *reinterpret_cast<const float4*>(&sO[v][q][cv * 4]);
        acc.x += ov.x;
        acc.y += ov.y;
        acc.z += ov.z;
        acc.w += ov.w;
      }
    }
    *reinterpret_cast<float4*>(out + row * pitchOut + cv * 4) = acc;
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

struct HeadLayout {
  int nHeads;       // 0: contiguous [N, d] single head
  int ldIn;         // row pitch of Q/K/V in elements
  int ldOut;        // row pitch of out in floats
  int minBlocks;    // this kernel skips windows of at most minBlocks blocks (-1: none)
  int gridWindows;  // positions of the window order this launch covers (<= nRW)
};

template <typename ET, int D, bool SOFTMAX>
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
  if (hl.nHeads > 0)
    hipLaunchKernelGGL((f3s_fwd_kernel<ET, D, NWAVES, SOFTMAX, false, true, false>),
                       dim3(gw * (unsigned)hl.nHeads), block, 0, stream, rwo, order, atox, bm, N,
                       nRW, q, k, v, scaleLog2, out, cuTimer, hl.nHeads, hl.ldIn, hl.ldOut,
                       nullptr, hl.minBlocks);
  else if (cuTimer)
    hipLaunchKernelGGL((f3s_fwd_kernel<ET, D, NWAVES, SOFTMAX, true, false, false>), dim3(gw),
                       block, 0, stream, rwo, order, atox, bm, N, nRW, q, k, v, scaleLog2, out,
                       cuTimer, 1, D, D, nullptr, hl.minBlocks);
  else
    hipLaunchKernelGGL((f3s_fwd_kernel<ET, D, NWAVES, SOFTMAX, false, false, false>), dim3(gw),
                       block, 0, stream, rwo, order, atox, bm, N, nRW, q, k, v, scaleLog2, out,
                       cuTimer, 1, D, D, nullptr, hl.minBlocks);
  F3S_HIP_CHECK(hipGetLastError());
  return 0;
}

template <int D, bool SOFTMAX>
int launch_tcb8(const int32_t* rwo, const int32_t* order, const int32_t* atox,
                const uint64_t* bitmap, int N, const void* Q, const void* K, const void* V,
                float scaleLog2, float* out, float* sddmm, hipStream_t stream) {
  constexpr int NWAVES = 4;
  const int nRW = (N + kWinRows - 1) / kWinRows;
  if (nRW == 0) return 0;
  hipLaunchKernelGGL((f3s_fwd_kernel<_Float16, D, NWAVES, SOFTMAX, false, false, true>),
                     dim3(nRW), dim3(NWAVES * 64), 0, stream, rwo, order, atox,
                     reinterpret_cast<const uint8_t*>(bitmap), N, nRW,
                     static_cast<const _Float16*>(Q), static_cast<const _Float16*>(K),
                     static_cast<const _Float16*>(V), scaleLog2, out, nullptr, 1, D, D, sddmm, -1);
  F3S_HIP_CHECK(hipGetLastError());
  return 0;
}

template <typename ET>
int dispatch_d(const int32_t* rwo, const int32_t* order, const int32_t* atox,
               const uint64_t* bitmap, int N, int d, const void* Q, const void* K, const void* V,
               float scaleLog2, int applySoftmax, float* out, unsigned long long* cuTimer,
               HeadLayout hl, hipStream_t stream) {
#define F3S_DISPATCH(DD)                                                                        \
  case DD:                                                                                      \
    return applySoftmax ? launch_d<ET, DD, true>(rwo, order, atox, bitmap, N, Q, K, V,          \
                                                 scaleLog2, out, cuTimer, hl, stream)           \
                        : launch_d<ET, DD, false>(rwo, order, atox, bitmap, N, Q, K, V,         \
                                                  scaleLog2, out, cuTimer, hl, stream);
  switch (d) {
    F3S_DISPATCH(32)
    F3S_DISPATCH(64)
    F3S_DISPATCH(128)
    default:
      return fail(-2, "f3s_attention_fwd: head dim %d unsupported (32, 64, 128)", d);
  }
#undef F3S_DISPATCH
}

}  // namespace

// Graphs of short windows (a few TC blocks each) leave most of a four-wave workgroup idle and
// pay its LDS merge for nothing. With a window order such a call is split: windows of at most
// kShortWindowBlocks blocks go to the wave-per-window kernel, the others, with a heavy-first order
// a prefix of at most nTcb / kShortWindowBlocks positions, stay with f3s_fwd_kernel, which skips
// the short ones. An order that is not heavy-first stays correct (a long window outside the
// prefix is computed by one wave). The two kernels run one after the other, so the split only
// pays when long windows are rare: it is taken below 16 blocks per window on average (measured:
// 100k-node 8-head layer 0.164 -> 0.101 ms and 0.248 -> 0.176 ms; an R-MAT graph with 16.6 blocks
// per window and windows of up to 731 would go from 0.107 to 0.129 ms and is left alone).
// Without an order nothing is split. F3S_SHORT_WINDOWS=0 in the environment turns it off.
constexpr int kShortWindowBlocks = 32;
bool split_short_windows(const int32_t* windowOrder, int nRW, int64_t nTcb, HeadLayout* hl) {
  static const bool off = [] {
    const char* e = getenv("F3S_SHORT_WINDOWS");
    return e && strcmp(e, "0") == 0;
  }();
  if (off || !windowOrder || nRW < 1024 || nTcb >= (int64_t)16 * nRW) return false;
  hl->minBlocks = kShortWindowBlocks;
  const int64_t longMax = nTcb / (kShortWindowBlocks + 1) + 1;
  hl->gridWindows = (int)(longMax < nRW ? longMax : nRW);
  return true;
}

// The column-sliced schedule (f3s_attention_units.hip: (window, column slice) units, every XCD
// on one slice at a time so that its K/V rows stay in that XCD's L2, plus a merge kernel) pays off
// on graphs with long windows: on the 233k-node benchmark graph (475 TC blocks per window) it
// takes 1.66 / 1.94 / 3.67 ms at d = 32 / 64 / 128 against 2.27 / 2.11 / 6.05 ms for the
// workgroup-per-window kernel, with 6.5 GB instead of 15.1 GB of traffic beyond L2 at d = 64.
// Short windows would be cut into units of one or two blocks; they keep the window kernel.
// F3S_SCHEDULE=window / =sliced in the environment overrides the choice.
int attention_uses_workspace(int N, int64_t nTcb, int d, int dtype) {
  static const int forced = [] {
    const char* e = getenv("F3S_SCHEDULE");
    if (e && strcmp(e, "sliced") == 0) return 1;
    if (e && strcmp(e, "window") == 0) return -1;
    return 0;
  }();
  if ((dtype != 0 && dtype != 1) || (d != 32 && d != 64 && d != 128) || N <= 0) return 0;
  if (forced) return forced > 0;
  const int64_t nRW = ((int64_t)N + kWinRows - 1) / kWinRows;
  return nRW >= 2048 && nTcb >= 64 * nRW;
}

int launch_attention(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                     const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int64_t nTcb,
                     int d, int dtype, const void* Q, const void* K, const void* V,
                     float scalingFactor, int applySoftmax, float* out,
                     unsigned long long* cuTimer, void* workspace, size_t wsBytes,
                     hipStream_t stream) {
  if (dtype != 0 && dtype != 1)
    return fail(-3, "f3s_attention_fwd: dtype %d not supported (0 = fp16, 1 = bf16)", dtype);
  if (scalingFactor == 0.0f) return fail(-2, "f3s_attention_fwd: scalingFactor must be non-zero");
  if ((int64_t)N * d * 2 >= (int64_t)1 << 32)
    return fail(-2, "f3s_attention_fwd: K and V must each be smaller than 4 GiB (N*d*2 bytes)");
  // the reference divides unmasked scores by scalingFactor (src/F3S_kernel.cu:1666-1667);
  // exponentials are taken in base 2, so log2(e) is folded into the same multiplier
  const float scaleLog2 = applySoftmax ? kLog2e / scalingFactor : 1.0f;
  if (workspace && !cuTimer && attention_uses_workspace(N, nTcb, d, dtype))
    return launch_attention_sliced(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, d, dtype,
                                   Q, K, V, scaleLog2, applySoftmax, out, workspace, wsBytes,
                                   stream);
  const int nRWi = (N + kWinRows - 1) / kWinRows;
  HeadLayout single = {0, d, d, -1, nRWi};
  if (!cuTimer && split_short_windows(windowOrder, nRWi, nTcb, &single)) {
    const int rc = launch_attention_short_windows(rowWindowOffset, windowOrder, sparseAToXidx,
                                                  bitmap, N, d, dtype, Q, K, V, scaleLog2,
                                                  applySoftmax, out, 0, d, d, kShortWindowBlocks,
                                                  single.gridWindows, stream);
    if (rc != 0) return rc;
  }
  return dtype == 0 ? dispatch_d<_Float16>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N,
                                           d, Q, K, V, scaleLog2, applySoftmax, out, cuTimer,
                                           single, stream)
                    : dispatch_d<__bf16>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, d,
                                         Q, K, V, scaleLog2, applySoftmax, out, cuTimer, single,
                                         stream);
}

int launch_attention_tcb8(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                          const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int d,
                          const void* Q, const void* K, const void* V, int applySoftmax,
                          float* out, float* sddmm, hipStream_t stream) {
  if ((int64_t)N * d * 2 >= (int64_t)1 << 32)
    return fail(-2, "f3s_attention_fwd_tcb8: K and V must each be smaller than 4 GiB");
  // this path has no score scaling (src/F3S_kernel.cu:709-735)
  const float scaleLog2 = applySoftmax ? kLog2e : 1.0f;
#define F3S_DISPATCH(DD)                                                                      \
  case DD:                                                                                    \
    return applySoftmax ? launch_tcb8<DD, true>(rowWindowOffset, windowOrder, sparseAToXidx,  \
                                                bitmap, N, Q, K, V, scaleLog2, out, sddmm,    \
                                                stream)                                       \
                        : launch_tcb8<DD, false>(rowWindowOffset, windowOrder, sparseAToXidx, \
                                                 bitmap, N, Q, K, V, scaleLog2, out, sddmm,   \
                                                 stream);
  switch (d) {
    F3S_DISPATCH(32)
    F3S_DISPATCH(64)
    F3S_DISPATCH(128)
    default:
      return fail(-2, "f3s_attention_fwd_tcb8: head dim %d unsupported (32, 64, 128)", d);
  }
#undef F3S_DISPATCH
}

int launch_attention_heads(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                           const int32_t* sparseAToXidx, const uint64_t* bitmap, int N,
                           int64_t nTcb, int nHeads, int d, int dtype, const void* Q, const void* K,
                           const void* V, int64_t ldIn, float scalingFactor, int applySoftmax,
                           float* out, int64_t ldOut, hipStream_t stream) {
  if (dtype != 0 && dtype != 1)
    return fail(-3, "f3s_attention_fwd_heads: dtype %d not supported (0 = fp16, 1 = bf16)", dtype);
  if (scalingFactor == 0.0f)
    return fail(-2, "f3s_attention_fwd_heads: scalingFactor must be non-zero");
  if (nHeads < 1 || nHeads > 1024)
    return fail(-2, "f3s_attention_fwd_heads: nHeads %d out of range (1..1024)", nHeads);
  if (ldIn < (int64_t)nHeads * d || ldOut < (int64_t)nHeads * d)
    return fail(-2, "f3s_attention_fwd_heads: row pitches must be at least nHeads*d");
  if (ldIn % 8 != 0 || ldOut % 4 != 0)
    return fail(-2, "f3s_attention_fwd_heads: rows must stay 16-byte aligned (ldIn %% 8 == 0, "
                    "ldOut %% 4 == 0)");
  if (ldIn * 2 >= ((int64_t)1 << 24) || N >= (1 << 24))
    return fail(-2, "f3s_attention_fwd_heads: N and the row pitch in bytes must be below 2^24");
  if ((int64_t)N * ldIn * 2 >= (int64_t)1 << 32)
    return fail(-2, "f3s_attention_fwd_heads: K and V must each span less than 4 GiB");
  const int64_t nRW = ((int64_t)N + kWinRows - 1) / kWinRows;
  if (nRW * nHeads >= ((int64_t)1 << 31))
    return fail(-2, "f3s_attention_fwd_heads: too many (window, head) workgroups");
  const float scaleLog2 = applySoftmax ? kLog2e / scalingFactor : 1.0f;
  HeadLayout hl = {nHeads, (int)ldIn, (int)ldOut, -1, (int)nRW};
  if (split_short_windows(windowOrder, (int)nRW, nTcb, &hl)) {
    const int rc = launch_attention_short_windows(rowWindowOffset, windowOrder, sparseAToXidx,
                                                  bitmap, N, d, dtype, Q, K, V, scaleLog2,
                                                  applySoftmax, out, nHeads, (int)ldIn, (int)ldOut,
                                                  kShortWindowBlocks, hl.gridWindows, stream);
    if (rc != 0) return rc;
  }
  return dtype == 0 ? dispatch_d<_Float16>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N,
                                           d, Q, K, V, scaleLog2, applySoftmax, out, nullptr, hl,
                                           stream)
                    : dispatch_d<__bf16>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, d,
                                         Q, K, V, scaleLog2, applySoftmax, out, nullptr, hl,
                                         stream);
}

}  // namespace f3s
