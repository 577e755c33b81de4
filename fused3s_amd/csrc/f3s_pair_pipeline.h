// The inner loop of the fused SDDMM -> online softmax -> SpMM kernels for gfx950 (MI355X),
// wave64: one wave walks a run of consecutive TC blocks of one 16-row window, two 16x16 blocks
// (a "pair", 32 keys) per step, with running (m, l, O) in registers. Every kernel of the library
// (workgroup per window, wave per (window, column slice) unit, wave per short window, 16x8
// blocks, multi-head, timed) is this loop plus its own prologue and epilogue.
//
// Replaces the loop bodies of f3sKernel1tb1rw / ...Scheduled / ...ScheduledPermutedQKV[ScaleQK],
// f2sKernel1tb1rw and f3sKernel1tb1tcb (src/F3S_kernel.cu:1414-1558, 1040-1150, 2040-2160,
// 2230-2310, 702-853).
//
// Data path of one step (lane = 16*g + c, g in 0..3, c in 0..15):
//   metadata   column ids and bitmaps of four steps at a time: one 16-byte load per lane straight
//              into LDS (global_load_lds), 512 bytes of ids followed by 256 bytes of bitmaps.
//   K, V rows  gathered whole with 16 bytes per lane (D/8 adjacent lanes cover one row: every
//              HBM/L2 access is a full row) straight into this wave's LDS ring, K tile and V tile
//              of a pair side by side, 16-byte chunks XOR-swizzled by the choice of which chunk a
//              lane fetches. Nothing passes through registers on the way in, so the ring, not
//              the register file, holds the loads in flight.
//   S^T = K Q^T  v_mfma_f32_16x16x32, A = K rows read from LDS with one 16-byte read per k-step
//              and block (lane: key slot c, features 32i+8g..+7), B = Q, held in registers for
//              the whole window. The accumulator leaves S[q = c][slot 4g+i], i < 4, in this lane.
//   mask       this lane's 4 + 4 bits sit in one bitmap dword per block; a sign-extending bit
//              field extract turns each into an AND mask.
//   softmax    exponentials are taken against the running maximum m of the lane's row WITHOUT
//              looking for a new maximum first; m (which starts at 0 like the reference's) only
//              moves when a lane's sum of new exponentials exceeds 2^12, i.e. when some score
//              lies more than 12 (log2 units) above it. Then, and when an unmasked score is
//              exactly 0 (which the reference drops, see below), the wave takes the slow path:
//              true row maximum over the four lanes of a row, rescale of l and O, exact zero
//              test. The result is the same softmax (the shift cancels in O / l); P stays below
//              2^12 and keeps fp16's relative precision.
//   O^T += V^T P^T  v_mfma_f32_16x16x32 over the 32 keys of the pair; contraction index 8g+k <->
//              (block A, slot 4g+k) for k < 4, (block B, slot 4g+k-4) for k >= 4, so the B operand
//              is the 8 probabilities this lane already holds. A = V^T comes from LDS through
//              ds_read_b64_tr_b16, which hands lane (g, c) column 16j+c of four consecutive key
//              rows. Lane (g, c) accumulates O[q = c][16j + 4g .. +3] for output tile j.
//
// Numerics follow the reference kernel (src/F3S_kernel.cu:1402-1406,1447-1451,1487-1499,938-945,
// 1560-1561): masked entries do not contribute, an unmasked score that is exactly 0 is dropped
// like a masked one, the row sum uses un-rounded fp32 exponentials while P is rounded to fp16 for
// the second product, empty rows give 0. bf16 inputs (beyond the reference): P is split into a
// bf16 head and a bf16 tail (two products per tile), which keeps 16 bits of P, more than the
// reference's fp16.
#pragma once
#include "f3s_common.h"

namespace f3s {
namespace pipe {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef int int4v __attribute__((ext_vector_type(4)));
typedef int int2v __attribute__((ext_vector_type(2)));
typedef short short4v __attribute__((ext_vector_type(4)));

#define F3S_LDS __attribute__((address_space(3)))

// probe builds can drop one part of a step (results are then wrong on purpose)
#ifdef F3S_PROBE_NO_READ
#define F3S_ABL_READ(x) op = Operands{}
#else
#define F3S_ABL_READ(x) x
#endif
#ifdef F3S_PROBE_NO_GATHER
#define F3S_ABL_GATHER(x) (void)0
#else
#define F3S_ABL_GATHER(x) x
#endif
#ifdef F3S_PROBE_NO_COMPUTE
#define F3S_ABL_COMPUTE(x) consume(op)
#else
#define F3S_ABL_COMPUTE(x) x
#endif

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
// a lane's sum of new exponentials above this sends the wave to the slow path (new row maximum)
constexpr float kLazyLimit = 4096.0f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

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

// ---- LDS accesses the compiler does not see as memory operations. It orders every LDS access
// it knows about after ALL outstanding direct-to-LDS loads (a full vmcnt(0)), which would
// serialise the ring; these are issued by hand and completed by lds_wait().
template <int OFFSET>
__device__ __forceinline__ int4v lds_read_b128(unsigned byteAddr) {
  int4v v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(byteAddr), "n"(OFFSET) : "memory");
  return v;
}
template <int OFFSET0, int OFFSET1>  // offsets in dwords, 0..255
__device__ __forceinline__ int2v lds_read2_b32(unsigned byteAddr) {
  int2v v;
  asm volatile("ds_read2_b32 %0, %1 offset0:%2 offset1:%3"
               : "=v"(v)
               : "v"(byteAddr), "n"(OFFSET0), "n"(OFFSET1)
               : "memory");
  return v;
}
// 4 x 16 bit per lane, transposed inside each group of 16 lanes: lane 4e+x of a group addresses
// elements 4x..4x+3 of row e of a 4 x 16 matrix of 16-bit values and receives column 4e+x.
template <int OFFSET>
__device__ __forceinline__ short4v lds_read_tr16_b64(unsigned byteAddr) {
  short4v v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2"
               : "=v"(v)
               : "v"(byteAddr), "n"(OFFSET)
               : "memory");
  return v;
}
__device__ __forceinline__ void lds_wait() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
template <typename T>
__device__ __forceinline__ void pin(T& v) {
  asm volatile("" : "+v"(v));
}

// s_waitcnt vmcnt(N) only (expcnt / lgkmcnt unconstrained), N <= 63
template <int N>
__device__ __forceinline__ void vm_wait() {
  static_assert(N >= 0 && N <= 63, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
  __builtin_amdgcn_sched_barrier(0);
}

// ---- geometry of the per-wave LDS ring
// D: head dimension, any multiple of 32 up to 256 (the reference takes embeddingDim at run time,
// src/F3S_kernel.cu:601-604,1424,1522). The ring is laid out for DP, the next power of two: a row
// of the LDS tile is DP elements wide, of which the first D hold data; lanes whose chunk does not
// exist fetch nothing.
template <int D>
struct Geo {
  static_assert(D % 32 == 0 && D >= 32 && D <= 256, "head dimension: a multiple of 32 up to 256");
  static constexpr int DP = D <= 32 ? 32 : D <= 64 ? 64 : D <= 128 ? 128 : 256;
  static constexpr int T = D / 16;         // output tiles
  static constexpr int KS = D / 32;        // k-steps of the score product
  static constexpr int TG = DP / 16;       // gather instructions per 32-row tile
  static constexpr int ROW = DP * 2;       // bytes of a K / V row in LDS
  static constexpr int GROW = D * 2;       // bytes of a contiguous K / V row in memory
  static constexpr int CHUNKS = D / 8;     // 16-byte chunks of a row that exist
  static constexpr int CPR = DP / 8;       // 16-byte chunks per LDS row == lanes per gathered row
  static constexpr int RPI = 64 / CPR;     // rows per gather instruction
  static constexpr int TILE = 32 * ROW;    // K (or V) rows of one pair
  static constexpr int STAGE = 2 * TILE;   // one pair: K tile, then V tile
  static constexpr int NS = DP >= 128 ? 1 : 2;  // stages of the ring
  static constexpr int META_SLOT = 1024;   // metadata of four steps: 512 B ids, 256 B bitmaps
  static constexpr int META = 2 * META_SLOT;
  static constexpr int WAVE_BYTES = NS * STAGE + META;
};

// Which of the pair's 32 key slots lane-row rho of gather instruction i fetches, and its inverse
// (the row of the LDS tile a slot lands in: row i * RPI + rho). Chosen so that the slots a lane
// fetches are groups of four consecutive dwords of the metadata (one 16-byte LDS read yields four
// of its row ids). DP >= 64: slot = 4 * (rho + RPI * (i / 4)) + i % 4.
template <int DP>
__device__ __forceinline__ constexpr int slot_of(int i, int rho) {
  if constexpr (DP == 32) return 4 * (rho >> 1) + 2 * i + (rho & 1);
  constexpr int RPI = 512 / DP;
  return 4 * (rho + RPI * (i >> 2)) + (i & 3);
}
template <int DP>
__device__ __forceinline__ constexpr int lds_row_of(int s) {
  if constexpr (DP == 32) return ((s & 3) >> 1) * 16 + 2 * (s >> 2) + (s & 1);
  constexpr int RPI = 512 / DP;
  const int rho = (s >> 2) & (RPI - 1);
  const int q = (s >> 2) / RPI;
  return ((s & 3) + 4 * q) * RPI + rho;
}
// XOR applied to the 16-byte chunk index of slot s inside its LDS row: the K tile is read with
// one 16-byte read per lane (16 consecutive slots by 4 chunks), the V tile with transposing
// 8-byte reads (4 consecutive slots by 32 bytes); each pattern wants its rows on different banks.
template <int DP>
__device__ __forceinline__ constexpr int swz_k(int s) {
  const int c = s & 15;
  if constexpr (DP == 64) return (c & 3) | ((((c >> 2) ^ (c >> 3)) & 1) << 2);
  if constexpr (DP >= 128) return c;
  return ((c >> 1) & 1) | ((((c >> 2) ^ (c >> 3)) & 1) << 1);  // DP == 32
}
template <int DP>
__device__ __forceinline__ constexpr int swz_v(int s) {
  if constexpr (DP == 32) return ((s >> 1) & 1) << 1;
  return (s & 3) << 1;
}
// The chunk a lane fetches in gather instruction i depends on i only through i % NK (K) and
// i % NV (V), so that many byte offsets are kept per lane.
template <int DP>
constexpr int distinct_k_offsets() {
  return DP == 32 ? 2 : DP == 256 ? 8 : 4;
}
template <int DP>
constexpr int distinct_v_offsets() {
  return DP == 32 ? 2 : 4;
}
template <int DP>
constexpr bool gather_offsets_periodic() {
  constexpr int RPI = 512 / DP, TG = DP / 16;
  for (int i = 0; i < TG; i++)
    for (int rho = 0; rho < RPI; rho++) {
      if (swz_k<DP>(slot_of<DP>(i, rho)) !=
          swz_k<DP>(slot_of<DP>(i % distinct_k_offsets<DP>(), rho)))
        return false;
      if (swz_v<DP>(slot_of<DP>(i, rho)) !=
          swz_v<DP>(slot_of<DP>(i % distinct_v_offsets<DP>(), rho)))
        return false;
    }
  return true;
}
static_assert(gather_offsets_periodic<32>() && gather_offsets_periodic<64>() &&
                  gather_offsets_periodic<128>() && gather_offsets_periodic<256>(),
              "gather offsets must repeat with the stated periods");

// the two maps are inverse to each other for every power-of-two width
template <int DP>
constexpr bool slot_maps_consistent() {
  constexpr int RPI = 512 / DP, TG = DP / 16;
  for (int i = 0; i < TG; i++)
    for (int rho = 0; rho < RPI; rho++) {
      const int s = slot_of<DP>(i, rho);
      if (s < 0 || s >= 32 || lds_row_of<DP>(s) != i * RPI + rho) return false;
    }
  return true;
}
static_assert(slot_maps_consistent<32>() && slot_maps_consistent<64>() &&
                  slot_maps_consistent<128>() && slot_maps_consistent<256>(),
              "slot_of and lds_row_of must be inverse");

// Problem description shared by every kernel.
template <typename ET>
struct Problem {
  const int32_t* __restrict__ sparseAToXidx;
  const uint8_t* __restrict__ bitmapBytes;
  const ET* __restrict__ Q;
  const ET* __restrict__ K;
  const ET* __restrict__ V;
  int N;
  float scaleLog2;   // log2(e) / scalingFactor (1.0 without softmax)
  int pitchIn;       // row pitch of K/V in elements (D for the single-head layout)
  int pitchQ;        // row pitch of Q in elements
  int64_t nTcb;      // TC blocks in sparseAToXidx / bitmapBytes (bounds of the metadata loads)
  float* __restrict__ sddmm;  // 16x8 structure only: masked unscaled scores, or null
};

// ET: _Float16 or __bf16. HEADS: pitched rows (row offset by 24-bit multiply). W8: the structure
// comes from preprocessing with 8-column blocks; two consecutive 16x8 blocks are laid out like
// one 16x16 block, block indices and counts below are then in 16x8 blocks. WIDE: K or V spans
// 4 GiB or more (or a pitched layout exceeds the 24-bit multiply): row offsets in 64 bits.
template <typename ET, int D, bool SOFTMAX, bool HEADS, bool W8, bool WIDE = false>
struct PairPipeline {
  typedef Geo<D> G;
  typedef typename Vec<ET, 8>::type half8;
  static constexpr int T = G::T;
  static constexpr int KS = G::KS;
  static constexpr int NS = G::NS;
  static constexpr int TG = G::TG;
  static constexpr int DP = G::DP;
  static constexpr int NK = distinct_k_offsets<DP>();
  static constexpr int NV = distinct_v_offsets<DP>();
  static constexpr int NVA = T < 4 ? T : 4;  // V read addresses kept: tile j reads at
                                             // vReadAddr[j % 4] + (j / 4) * 128
  static constexpr int BPS = W8 ? 4 : 2;  // blocks of the structure per step
  static constexpr bool SPLIT_P = sizeof(ET) == 2 && !__is_same(ET, _Float16);  // bf16

  // running state
  float m, l;
  float4v o[T];

  // loop-invariant per-lane values
  half8 qf[KS];
  unsigned ring;        // LDS byte address of this wave's ring
  unsigned metaBase;    // LDS byte address of this wave's two metadata slots
  unsigned kReadAddr[2][KS];  // K tile: slot 16b + c, chunk 4i + g (swizzled)
  unsigned vReadAddr[NVA];  // V tile: transposing read of tiles 0..3, first key half
  unsigned idReadAddr;     // metadata: this lane's row ids
  unsigned maskReadAddr;   // metadata: the bitmap dword with this lane's bits of block A
  int keepPos[4];          // bit position of element i in that dword
  uint32_t gatherOffK[NK], gatherOffV[NV];  // byte offset inside the row this lane fetches
  uint32_t gatherLive;  // D < DP: bit i / bit 16 + i: the chunk of K / V instruction i exists
  int lane, g, c;

  __device__ __forceinline__ void init(const Problem<ET>& pb, int w, unsigned ringAddr, int head) {
    lane = threadIdx.x & 63;
    g = lane >> 4;
    c = lane & 15;
    ring = ringAddr;
    metaBase = ringAddr + NS * G::STAGE;
    m = 0.0f;
    l = 0.0f;
#pragma unroll
    for (int j = 0; j < T; j++) o[j] = float4v{0.f, 0.f, 0.f, 0.f};
    {
      const int4v zero16 = {0, 0, 0, 0};
      const int64_t qrow = (int64_t)w * 16 + c;
      if (qrow < pb.N) {
        const half8* qp =
            reinterpret_cast<const half8*>(pb.Q + qrow * pb.pitchQ + (HEADS ? head * D : 0)) + g;
#pragma unroll
        for (int i = 0; i < KS; i++) qf[i] = qp[4 * i];
      } else {
#pragma unroll
        for (int i = 0; i < KS; i++) qf[i] = __builtin_bit_cast(half8, zero16);
      }
    }
    // gather: in instruction i this lane fetches chunk (lane % CPR) ^ swizzle of slot
    // slot_of(i, lane / CPR); the chunk lands at ring + i * 1024 + lane * 16
    const int rho = lane / G::CPR;
    const int pos = lane % G::CPR;
    gatherLive = 0;
#pragma unroll
    for (int i = 0; i < TG; i++) {
      const int s = slot_of<DP>(i, rho);
      const int ck = pos ^ swz_k<DP>(s), cv = pos ^ swz_v<DP>(s);
      if (i < NK) gatherOffK[i] = (uint32_t)(ck * 16 + (HEADS ? head * D * 2 : 0));
      if (i < NV) gatherOffV[i] = (uint32_t)(cv * 16 + (HEADS ? head * D * 2 : 0));
      if (ck < G::CHUNKS) gatherLive |= 1u << i;
      if (cv < G::CHUNKS) gatherLive |= 1u << (16 + i);
    }
    // score product: lane (g, c) reads, for block b and k-step i, chunk 4i + g of slot 16b + c
#pragma unroll
    for (int b = 0; b < 2; b++) {
      const int s = 16 * b + c;
#pragma unroll
      for (int i = 0; i < KS; i++)
        kReadAddr[b][i] = ring + lds_row_of<DP>(s) * G::ROW + (((4 * i + g) ^ swz_k<DP>(s)) * 16);
    }
    // P V product: lane (g, c = 4e + x) addresses slot 16h + 4g + e, columns 16j + 4x .. +3:
    // chunk 2j + x/2 (swizzled), byte (x % 2) * 8 inside it. h = 1 is a fixed distance away.
    {
      const int e = c >> 2, x = c & 3;
      const int s = 4 * g + e;
#pragma unroll
      for (int j = 0; j < NVA; j++)
        vReadAddr[j] = ring + G::TILE + lds_row_of<DP>(s) * G::ROW +
                       (((2 * j + (x >> 1)) ^ swz_v<DP>(s)) * 16) + (x & 1) * 8;
    }
    // metadata slot: ids of step q at q * 128, bitmaps at 512 + q * 64
    if constexpr (DP == 32)
      idReadAddr = metaBase + (4 * (rho >> 1) + (rho & 1)) * 4;
    else
      idReadAddr = metaBase + rho * 16;
    const int maskByte = ((g >> 1) * 2 + (c >> 3)) * 8 + 7 - (c & 7);
    maskReadAddr = metaBase + 512 + (maskByte >> 2) * 4;
#pragma unroll
    for (int i = 0; i < 4; i++) keepPos[i] = 8 * (maskByte & 3) + 4 * (1 - (g & 1)) + 3 - i;
  }

  // ---- loads -------------------------------------------------------------------------------
  // Metadata of steps 4k .. 4k+3 of the run [t0, t1) into metadata slot k & 1. Lanes 0..31: the
  // 128 column ids (16 bytes each), lanes 32..47: the 64 bitmap dwords. Blocks past the end of
  // the run are folded onto its last block (the loads stay in bounds; their bits are never used).
  __device__ __forceinline__ void issue_meta(const Problem<ET>& pb, int t0, int t1, int k) {
    constexpr int IDS_PER_BLOCK = W8 ? 8 : 16;      // ids of one block of the structure
    constexpr int BM_BYTES = W8 ? 16 : 32;          // bitmap bytes of one block
    const int64_t first = (int64_t)t0 + (int64_t)k * 4 * BPS;
    const char* src;
    if (lane < 32) {
      int64_t blk = first + (lane * 4) / IDS_PER_BLOCK;
      const int within = (lane * 4) % IDS_PER_BLOCK;
      if (blk >= t1) blk = t1 - 1;
      src = reinterpret_cast<const char*>(pb.sparseAToXidx) + (blk * IDS_PER_BLOCK + within) * 4;
    } else {
      const int b = (lane - 32) & 15;  // lanes 48..63 repeat lanes 32..47 (their copy is unused)
      int64_t blk = first + (b * 16) / BM_BYTES;
      const int within = (b * 16) % BM_BYTES;
      if (blk >= t1) blk = t1 - 1;
      src = reinterpret_cast<const char*>(pb.bitmapBytes) + blk * BM_BYTES + within;
    }
    F3S_LDS int4v* dst =
        (F3S_LDS int4v*)(uintptr_t)(uniform((int)metaBase) + (k & 1) * G::META_SLOT);
    __builtin_amdgcn_global_load_lds(reinterpret_cast<const int4v*>(src), dst, 16, 0, 0);
  }

  // K and V rows of step p into ring stage `stage` (compile-time), row ids from metadata.
  template <int STAGE_IDX, int Q4>
  __device__ __forceinline__ void issue_gather(const Problem<ET>& pb, int metaSlot) {
    // row ids of this lane's TG slots: groups of four consecutive dwords of the step's 32 ids
    int rows[TG];
    const unsigned ida = idReadAddr + metaSlot * G::META_SLOT;
    if constexpr (DP == 32) {
      const int2v r = lds_read2_b32<Q4 * 32, Q4 * 32 + 2>(ida);
      lds_wait();
      rows[0] = r[0];
      rows[1] = r[1];
    } else {
      // group q of four slots starts RPI * 4 slots (RPI * 16 bytes) after group q - 1
      int4v r[TG / 4];
      r[0] = lds_read_b128<Q4 * 128>(ida);
      if constexpr (TG >= 8) r[1] = lds_read_b128<Q4 * 128 + 1 * G::RPI * 16>(ida);
      if constexpr (TG >= 16) {
        r[2] = lds_read_b128<Q4 * 128 + 2 * G::RPI * 16>(ida);
        r[3] = lds_read_b128<Q4 * 128 + 3 * G::RPI * 16>(ida);
      }
      lds_wait();
#pragma unroll
      for (int q = 0; q < TG / 4; q++)
#pragma unroll
        for (int i = 0; i < 4; i++) rows[4 * q + i] = r[q][i];
    }
    const char* Kb = reinterpret_cast<const char*>(pb.K);
    const char* Vb = reinterpret_cast<const char*>(pb.V);
    const uint32_t rowBytes = HEADS ? (uint32_t)pb.pitchIn * 2u : (uint32_t)G::GROW;
    const int ringU = uniform((int)ring);
#pragma unroll
    for (int i = 0; i < TG; i++) {
      pin(rows[i]);
#ifdef F3S_PROBE_ROWMASK
      rows[i] &= F3S_PROBE_ROWMASK;
#endif
    }
    // one gather instruction: 64 lanes x 16 bytes of K (V) rows into 1 KiB of the stage
    auto gather = [&](const char* src, bool live, int ldsOffset) {
      F3S_LDS int4v* dst = (F3S_LDS int4v*)(uintptr_t)(ringU + ldsOffset);
      if constexpr (D == DP) {
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const int4v*>(src), dst, 16, 0, 0);
      } else {
        if (live)
          __builtin_amdgcn_global_load_lds(reinterpret_cast<const int4v*>(src), dst, 16, 0, 0);
      }
    };
    if constexpr (WIDE) {
      // the reference indexes rows with int64_t (src/F3S_kernel.cu:1422-1423)
#pragma unroll
      for (int i = 0; i < TG; i++)
        gather(Kb + ((uint64_t)(uint32_t)rows[i] * rowBytes + gatherOffK[i % NK]),
               (gatherLive >> i) & 1u, STAGE_IDX * G::STAGE + i * 1024);
#pragma unroll
      for (int i = 0; i < TG; i++)
        gather(Vb + ((uint64_t)(uint32_t)rows[i] * rowBytes + gatherOffV[i % NV]),
               (gatherLive >> (16 + i)) & 1u, STAGE_IDX * G::STAGE + G::TILE + i * 1024);
    } else {
#pragma unroll
      for (int i = 0; i < TG; i++) {
        const uint32_t ro = HEADS ? __umul24((uint32_t)rows[i], rowBytes)
                                  : (uint32_t)rows[i] * rowBytes;
        gather(Kb + (ro + gatherOffK[i % NK]), (gatherLive >> i) & 1u,
               STAGE_IDX * G::STAGE + i * 1024);
      }
#pragma unroll
      for (int i = 0; i < TG; i++) {
        const uint32_t ro = HEADS ? __umul24((uint32_t)rows[i], rowBytes)
                                  : (uint32_t)rows[i] * rowBytes;
        gather(Vb + (ro + gatherOffV[i % NV]), (gatherLive >> (16 + i)) & 1u,
               STAGE_IDX * G::STAGE + G::TILE + i * 1024);
      }
    }
  }

  // ---- one step ------------------------------------------------------------------------------
  struct Operands {
    int4v k[2][KS];
    short4v v[T][2];
    int2v words;
  };

  template <int STAGE_IDX, int Q4>
  __device__ __forceinline__ void read_operands(int metaSlot, Operands& op) {
    constexpr int SO = STAGE_IDX * G::STAGE;
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int i = 0; i < KS; i++) op.k[b][i] = lds_read_b128<SO>(kReadAddr[b][i]);
    read_v_tile<SO, 0>(op);
    op.words = lds_read2_b32<Q4 * 16, Q4 * 16 + 8>(maskReadAddr + metaSlot * G::META_SLOT);
  }
  // tile J of the V operand: 128 bytes (eight chunks) per four tiles beyond tile J % 4
  template <int SO, int J>
  __device__ __forceinline__ void read_v_tile(Operands& op) {
    constexpr int OFF = SO + (J / 4) * 128;
    op.v[J][0] = lds_read_tr16_b64<OFF>(vReadAddr[J % 4]);
    op.v[J][1] = lds_read_tr16_b64<OFF + v_half_distance()>(vReadAddr[J % 4]);
    if constexpr (J + 1 < T) read_v_tile<SO, J + 1>(op);
  }
  // LDS distance between the rows of slot s and slot s + 16 of a tile
  static __device__ __forceinline__ constexpr int v_half_distance() {
    return (lds_row_of<DP>(16) - lds_row_of<DP>(0)) * G::ROW;
  }

  __device__ __forceinline__ void consume(Operands& op) {
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int i = 0; i < KS; i++) pin(op.k[b][i]);
#pragma unroll
    for (int j = 0; j < T; j++) {
      pin(op.v[j][0]);
      pin(op.v[j][1]);
    }
    pin(op.words);
  }

  // nValid: blocks of the structure that exist in this step (1..BPS); only the last step of a
  // run can have fewer than BPS.
  __device__ __forceinline__ void compute(const Problem<ET>& pb, Operands& op, int tFirst,
                                          int nValid) {
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int i = 0; i < KS; i++) pin(op.k[b][i]);
    float4v sA = {0.f, 0.f, 0.f, 0.f}, sB = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < KS; i++) {
      sA = mfma_16x16x32<ET>(__builtin_bit_cast(half8, op.k[0][i]), qf[i], sA);
      sB = mfma_16x16x32<ET>(__builtin_bit_cast(half8, op.k[1][i]), qf[i], sB);
    }
    pin(op.words);
    int wordA = op.words[0], wordB = op.words[1];
    if constexpr (W8) {
      // this lane's slots 4g..4g+3 belong to 16x8 block g/2 (A) resp. 2 + g/2 (B) of the step
      if ((g >> 1) >= nValid) wordA = 0;
      if (2 + (g >> 1) >= nValid) wordB = 0;
    } else {
      if (nValid < 2) wordB = 0;
    }
    int keep[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      keep[i] = __builtin_amdgcn_sbfe(wordA, keepPos[i], 1);  // 0 or -1
      keep[4 + i] = __builtin_amdgcn_sbfe(wordB, keepPos[i], 1);
    }
    float s[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      s[i] = sA[i];
      s[4 + i] = sB[i];
    }
    if constexpr (W8) {
      if (pb.sddmm) {
        // lane (g, c): row c, columns 4(g&1)..+3 of block tFirst + g/2 (A) and + 2 (B)
        float* dst = pb.sddmm + ((size_t)(tFirst + (g >> 1)) * 16 + c) * 8 + 4 * (g & 1);
        float4 a, b;
        a.x = __int_as_float(__float_as_int(s[0]) & keep[0]);
        a.y = __int_as_float(__float_as_int(s[1]) & keep[1]);
        a.z = __int_as_float(__float_as_int(s[2]) & keep[2]);
        a.w = __int_as_float(__float_as_int(s[3]) & keep[3]);
        b.x = __int_as_float(__float_as_int(s[4]) & keep[4]);
        b.y = __int_as_float(__float_as_int(s[5]) & keep[5]);
        b.z = __int_as_float(__float_as_int(s[6]) & keep[6]);
        b.w = __int_as_float(__float_as_int(s[7]) & keep[7]);
        if ((g >> 1) < nValid) *reinterpret_cast<float4*>(dst) = a;
        if (2 + (g >> 1) < nValid) *reinterpret_cast<float4*>(dst + 256) = b;
      }
    }
    float e[8];
    if constexpr (SOFTMAX) {
      // fast path: exponentials against the current maximum, masked ones cleared afterwards
      const float negM = -m;
      float sum = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const float ev = fast_exp2(fmaf(s[i], pb.scaleLog2, negM));
        e[i] = __int_as_float(__float_as_int(ev) & keep[i]);
        sum += e[i];
      }
      float zmin = fminf(fminf(fabsf(s[0]), fabsf(s[1])), fabsf(s[2]));
      zmin = fminf(fminf(zmin, fabsf(s[3])), fabsf(s[4]));
      zmin = fminf(fminf(zmin, fabsf(s[5])), fabsf(s[6]));
      zmin = fminf(zmin, fabsf(s[7]));
      // some lane saw a score far above its row's maximum (or a non-finite sum), or a score
      // that is exactly zero (masked or not): redo the step the careful way
      if (__builtin_amdgcn_ballot_w64(!(sum <= kLazyLimit) || zmin == 0.0f) != 0ull) {
        float sc[8];
        float mx = m;
#pragma unroll
        for (int i = 0; i < 8; i++) {
          sc[i] = __int_as_float(__float_as_int(s[i]) & keep[i]) * pb.scaleLog2;
          mx = fmaxf(mx, sc[i]);
        }
        mx = row_max4(mx);
        const float alpha = fast_exp2(m - mx);
        m = mx;
        sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
          e[i] = (sc[i] == 0.0f) ? 0.0f : fast_exp2(sc[i] - mx);
          sum += e[i];
        }
        l *= alpha;
#pragma unroll
        for (int j = 0; j < T; j++) o[j] *= alpha;
      }
      l += sum;
    } else {
#pragma unroll
      for (int i = 0; i < 8; i++) e[i] = __int_as_float(__float_as_int(s[i]) & keep[i]);
    }
    half8 pf;
#pragma unroll
    for (int i = 0; i < 8; i++) pf[i] = (ET)e[i];
#pragma unroll
    for (int j = 0; j < T; j++) {
      pin(op.v[j][0]);
      pin(op.v[j][1]);
    }
    if constexpr (SPLIT_P) {
      half8 pt;
#pragma unroll
      for (int i = 0; i < 8; i++) pt[i] = (ET)(e[i] - (float)pf[i]);
#pragma unroll
      for (int j = 0; j < T; j++) {
        const half8 va = __builtin_bit_cast(
            half8, __builtin_shufflevector(op.v[j][0], op.v[j][1], 0, 1, 2, 3, 4, 5, 6, 7));
        o[j] = mfma_16x16x32<ET>(va, pf, o[j]);
        o[j] = mfma_16x16x32<ET>(va, pt, o[j]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < T; j++) {
        const half8 va = __builtin_bit_cast(
            half8, __builtin_shufflevector(op.v[j][0], op.v[j][1], 0, 1, 2, 3, 4, 5, 6, 7));
        o[j] = mfma_16x16x32<ET>(va, pf, o[j]);
      }
    }
  }

  // ---- the loop over the run [t0, t1) of blocks of the structure ------------------------------
  // Ring discipline per step p (stage p % NS): wait until the step's K and V rows have landed
  // (vector loads complete in issue order), read all of its operands into registers, then reuse
  // the stage at once for step p + NS; the metadata of four steps at a time is requested at the
  // first of the four preceding steps.
  __device__ __forceinline__ void run(const Problem<ET>& pb, int t0, int t1) {
    const int nSteps = (t1 - t0 + BPS - 1) / BPS;
    if (nSteps <= 0) return;
    // prologue: metadata of the first four steps, then the first NS gathers
    issue_meta(pb, t0, t1, 0);
    vm_wait<0>();
    if constexpr (NS == 2) {
      issue_gather<0, 0>(pb, 0);
      if (nSteps > 1) issue_gather<1, 1>(pb, 0);
    } else {
      issue_gather<0, 0>(pb, 0);
    }
    int p = 0;
    bool metaIssued = false;  // the last first-of-four step requested the next four's metadata
    // One step; STAGE_IDX = p % NS and Q4 = p % 4 are compile-time. GQ4 = (p + NS) % 4 is the
    // position of the step whose gather is issued, in metadata slot ((p + NS) / 4) & 1.
#define F3S_PIPE_STEP(STAGE_IDX, Q4)                                                           \
  {                                                                                            \
    constexpr int GQ4 = (Q4 + NS) % 4;                                                         \
    const bool more = p + NS < nSteps;                                                         \
    /* loads issued after this step's gather: the later stages' gathers and, if one of those  \
       steps opened a group of four, its metadata load */                                     \
    if constexpr (NS == 2) {                                                                   \
      if (p + 1 < nSteps) {                                                                    \
        if (Q4 == 1 && metaIssued) vm_wait<2 * TG + 1>(); else vm_wait<2 * TG>();                \
      } else {                                                                                 \
        vm_wait<0>();                                                                          \
      }                                                                                        \
    } else {                                                                                   \
      vm_wait<0>();                                                                            \
    }                                                                                          \
    Operands op;                                                                               \
    F3S_ABL_READ((read_operands<STAGE_IDX, Q4>((p >> 2) & 1, op)));                            \
    lds_wait();                                                                                \
    __builtin_amdgcn_sched_barrier(0);                                                         \
    if constexpr (Q4 == 0) {                                                                   \
      metaIssued = (p >> 2) + 1 <= (nSteps - 1) >> 2;                                          \
      if (metaIssued) issue_meta(pb, t0, t1, (p >> 2) + 1);                                    \
    }                                                                                          \
    if (more) F3S_ABL_GATHER((issue_gather<STAGE_IDX, GQ4>(pb, ((p + NS) >> 2) & 1)));         \
    __builtin_amdgcn_sched_barrier(0);                                                         \
    {                                                                                          \
      const int tFirst = t0 + p * BPS;                                                         \
      const int left = t1 - tFirst;                                                            \
      F3S_ABL_COMPUTE(compute(pb, op, tFirst, left < BPS ? left : BPS));                       \
    }                                                                                          \
    p++;                                                                                       \
    if (p >= nSteps) break;                                                                    \
  }
    while (true) {
      F3S_PIPE_STEP(0, 0)
      F3S_PIPE_STEP(1 % NS, 1)
      F3S_PIPE_STEP(0, 2)
      F3S_PIPE_STEP(1 % NS, 3)
    }
#undef F3S_PIPE_STEP
  }
};

}  // namespace pipe
}  // namespace f3s
