// CSR -> 16-row windows of column-compacted TC blocks with per-block bitmaps, on gfx950.
//
// Replaces the reference's preprocessing pipeline (src/F3S.cpp:40-87, src/utils.cu:23-436):
// a global thrust::sort of (window, column) pairs followed by two kernels that walk each
// window with a single thread. Here a window never leaves its workgroup:
//
//   window_rank_radix_kernel / window_rank_small_kernel
//                        windows of <= 1024 edges, one WAVE per window, no workgroup barrier.
//                        Graphs of <= 2^22 nodes: stable LSD radix sort of (column, position)
//                        words in LDS, ranks of the distinct columns scattered back to the
//                        edges. Larger graphs: bitonic sort of the column ids, ballot / popcount
//                        compaction of the distinct ones, rank by binary search.
//   window_rank_kernel   larger windows, one workgroup per window. Column ids are OR-ed into an
//                        LDS bitset (a column range per pass when N exceeds the LDS range), a
//                        wave64 popcount prefix scan turns the bitset into ranks, and every edge
//                        reads its compacted column index back: the sorted unique column list
//                        (reference: sort + inplace_deduplication + binarysearch,
//                        src/utils.cu:102-153,281-289) is never materialised.
//   finalize_count_kernel one workgroup, every wave on its own chunk of the windows: inclusive
//                        scan of the per-window block counts (src/utils.cu:293-300) and a stable
//                        LSD radix sort of the windows by descending block count
//                        (src/utils.cu:400-436), ranks from wave ballots.
//   window_count_kernel, window_rank_fill_kernel
//                        graphs of long windows through the one-call entry: block counts, then
//                        ranks, rows, ids, bitmaps and tile ids of a window while its bitset sits
//                        in LDS.
//   window_fill_kernel   one workgroup (or one wave, on graphs of short windows) per window:
//                        bitmaps and per-(row, block) edge counts are accumulated in LDS, a scan
//                        yields the per-block offsets, and the tile ids are written per block
//                        from its bitmap when the window's rows ascend, else placed edge by edge
//                        in CSR order (src/utils.cu:173-224, 23-36, 53-65).
//
// All results are bit-identical to the reference's algorithm with edgeToRow[e] = row(e).

#include <mutex>

#include "f3s_common.h"

// Device scratch of f3s_preprocess_count_static, owned by the library instead of the caller: every
// GPU the library runs on holds its own copy (8 MiB) at its own address until the process ends.
// In host code the name below is only a handle for hipGetSymbolAddress, never an address.
static constexpr size_t kF3sStaticScratchBytes = (size_t)8 << 20;
static __device__ __align__(256) unsigned char scratch[kF3sStaticScratchBytes];

namespace f3s {
namespace {

constexpr int kBlock = 256;
constexpr int kRangeMax = 393216;  // columns per bitset pass: 48 KiB of bits + 12 KiB of prefixes
constexpr int kSortMax = 1024;     // windows up to this many edges are ranked by a per-wave LDS sort
// TC blocks held in LDS at once by window_fill_kernel: windows with strictly ascending rows (96
// bytes of LDS per 16x16 block) and windows with repeated or descending columns (96 bytes as
// well, but a second pass per chunk)
constexpr int kFillChunk = 640;
constexpr int kFillChunkGeneric = 512;
constexpr int kFillChunkSmall = 128;  // both, for graphs of short windows (one wave each)

// workspace header (bytes 0..255): int64 nTCB, int32 error flag, and the queue of windows too
// long for the wave-per-window kernel (filled by window_rank_small_kernel, drained by
// window_rank_kernel)
struct WsHeader {
  long long nTcb;
  int error;
  int nBig;     // entries in the queue of the bitset kernel (window_rank_kernel)
  int nextBig;  // next entry to hand out
  int maxCount; // largest per-window block count (multi-workgroup finalize)
  int nMed, nextMed;      // queue of window_rank_sort_kernel, windows of up to kMedMax edges
  int nLarge, nextLarge;  // the same for its launch over the windows of up to kLargeMax edges
};

// Where the wave-per-window kernels leave the windows that are too long for them: one queue per
// kernel that takes such windows, chosen by the window's edge count. big == nullptr: no queues
// (every long window is found by its own workgroup). medMax == 0: everything goes to `big`.
struct LongQueues {
  int32_t* med;
  int32_t* large;
  int32_t* big;
  int medMax, largeMax;
};
__device__ __forceinline__ void queue_long_window(const LongQueues& q, WsHeader* hdr, int w,
                                                  int nEdges) {
  if (!q.big) return;
  if (nEdges <= q.medMax)
    q.med[atomicAdd(&hdr->nMed, 1)] = w;
  else if (nEdges <= q.largeMax)
    q.large[atomicAdd(&hdr->nLarge, 1)] = w;
  else
    q.big[atomicAdd(&hdr->nBig, 1)] = w;
}
constexpr size_t kWsHeaderBytes = 256;

// Inclusive prefix sum over the wave's 64 lanes with data-parallel-primitive moves: shifts within
// rows of 16 lanes (lanes shifted in from outside a row read 0), then lane 15 of a row added to the
// whole next row and lane 31 to the upper half of the wave. Every lane of the wave must be active.
__device__ __forceinline__ unsigned wave_inclusive_scan(unsigned v, int /*lane*/) {
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, true);   // row_shr:1
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, true);   // row_shr:2
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, true);   // row_shr:4
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, true);   // row_shr:8
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);  // row_bcast:15
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);  // row_bcast:31
  return v;
}

// largest r in [0,15] with sRow[r] <= e (sRow[0] <= e < sRow[16])
__device__ __forceinline__ int row_of_edge(const int* sRow, int e) {
  int r = 0;
  if (sRow[r + 8] <= e) r += 8;
  if (sRow[r + 4] <= e) r += 4;
  if (sRow[r + 2] <= e) r += 2;
  if (sRow[r + 1] <= e) r += 1;
  return r;
}

// Writes a TC block's tile ids (row * W + column of every set bit, rows top to bottom, columns
// left to right) to dst[pos...]. words: the block's bitmap, 8x8 sub-blocks in column-major order,
// rows of a sub-block MSB first. The bitmap is first brought into row-major order as dwords whose
// bit 31 - p stands for tile id 32 q + p (two rows of 16 columns, or four of 8, per dword): for
// 16 columns that interleaves the bytes of the left and the right sub-block (two byte permutes
// per four rows), for 8 columns the words are in that order already.
template <int W>
__device__ __forceinline__ void walk_tile_ids(const unsigned long long (&words)[16 * W / 64],
                                              uint8_t* __restrict__ dst, unsigned pos) {
  constexpr int NQ = 16 * W / 32;
  unsigned rm[NQ];
  if constexpr (W == 16) {
#pragma unroll
    for (int half = 0; half < 2; half++) {  // rows 0-7 (sub-blocks 0 and 2), rows 8-15 (1 and 3)
      const unsigned long long left = words[half], right = words[2 + half];
#pragma unroll
      for (int k = 0; k < 2; k++) {  // rows 4k .. 4k+3 of the half: the dword from the top
        const unsigned a = k == 0 ? (unsigned)(left >> 32) : (unsigned)left;
        const unsigned c = k == 0 ? (unsigned)(right >> 32) : (unsigned)right;
        rm[4 * half + 2 * k] = __builtin_amdgcn_perm(a, c, 0x07030602u);      // rows +0, +1
        rm[4 * half + 2 * k + 1] = __builtin_amdgcn_perm(a, c, 0x05010400u);  // rows +2, +3
      }
    }
  } else {
#pragma unroll
    for (int k = 0; k < 2; k++) {
      rm[2 * k] = (unsigned)(words[k] >> 32);
      rm[2 * k + 1] = (unsigned)words[k];
    }
  }
#pragma unroll
  for (int q = 0; q < NQ; q++) {
    unsigned x = rm[q];
    while (x) {
      const int p = __builtin_clz(x);
      dst[pos++] = (uint8_t)(32 * q + p);
      x &= ~(0x80000000u >> p);
    }
  }
}

// ------------------------------------------------------------------ phase 1
// compiler-level ordering point between LDS phases of ONE wave (its LDS operations execute in
// program order, so no hardware barrier is needed)
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_wave_barrier();
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
}

// Windows of at most kSortMax edges: one WAVE per window, no workgroup barrier. The wave sorts
// the window's column ids in its LDS slice (bitonic network, 32 compare-exchanges per step and
// lane row), compacts the distinct ones with ballot + popcount prefixes, and ranks every edge by
// binary search in the distinct list.
template <int W>
__global__ __launch_bounds__(kBlock) void window_rank_small_kernel(
    const int32_t* __restrict__ rowPtr, const int32_t* __restrict__ colIdx, int N, int nRW,
    int32_t* __restrict__ blockPartition, int32_t* __restrict__ edgeToColumn,
    int32_t* __restrict__ edgeToRow, WsHeader* __restrict__ hdr, LongQueues queues) {
  constexpr int WAVES = kBlock / 64;
  __shared__ uint32_t sKeys[WAVES][kSortMax];
  __shared__ uint32_t sUniq[WAVES][kSortMax];
  __shared__ int sRowW[WAVES][17];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int w = blockIdx.x * WAVES + wave;
  if (w >= nRW) return;
  const int r0 = w * 16;
  int* sRow = sRowW[wave];
  if (lane < 17) sRow[lane] = rowPtr[min(r0 + lane, N)];
  wave_lds_sync();
  const int eS = sRow[0], eE = sRow[16];
  const int n = eE - eS;
  if (n == 0) {
    if (lane == 0) blockPartition[w] = 0;
    return;
  }
  if (n > kSortMax) {  // left to window_rank_kernel, through the queue if there is one
    if (lane == 0) queue_long_window(queues, hdr, w, n);
    return;
  }
  uint32_t* keys = sKeys[wave];
  uint32_t* uniq = sUniq[wave];
  int P = 64;
  while (P < n) P <<= 1;
  bool bad = false;
  for (int i = lane; i < P; i += 64) {
    uint32_t k = 0xFFFFFFFFu;  // padding sorts last
    if (i < n) {
      k = (uint32_t)colIdx[eS + i];
      if (k >= (uint32_t)N) {
        bad = true;
        k = 0xFFFFFFFEu;
      }
    }
    keys[i] = k;
  }
  if (bad) atomicOr(&hdr->error, 1);
  wave_lds_sync();
  for (int k = 2; k <= P; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      // all of the lane's compare-exchanges of this step: reads first, then writes, so the
      // LDS latencies overlap (at most kSortMax / 128 pairs per lane)
      constexpr int MAXP = kSortMax / 128;
      uint32_t va[MAXP], vb[MAXP];
      const int nPairsLane = P >> 7;  // P/2 pairs over 64 lanes (P >= 128), 0 when P == 64
      if (nPairsLane == 0) {
        if (lane < 32) {
          const int lo = ((lane & ~(j - 1)) << 1) | (lane & (j - 1));
          const int hi = lo | j;
          const uint32_t x = keys[lo], y = keys[hi];
          const bool up = (lo & k) == 0;
          if ((x > y) == up) {
            keys[lo] = y;
            keys[hi] = x;
          }
        }
      } else {
#pragma unroll
        for (int q = 0; q < MAXP; q++) {
          if (q < nPairsLane) {
            const int i = lane + 64 * q;
            const int lo = ((i & ~(j - 1)) << 1) | (i & (j - 1));
            va[q] = keys[lo];
            vb[q] = keys[lo | j];
          }
        }
#pragma unroll
        for (int q = 0; q < MAXP; q++) {
          if (q < nPairsLane) {
            const int i = lane + 64 * q;
            const int lo = ((i & ~(j - 1)) << 1) | (i & (j - 1));
            const bool up = (lo & k) == 0;
            const bool swap = (va[q] > vb[q]) == up;
            keys[lo] = swap ? vb[q] : va[q];
            keys[lo | j] = swap ? va[q] : vb[q];
          }
        }
      }
      wave_lds_sync();
    }
  }
  int nUniq = 0;
  const unsigned long long ltMask = (1ull << lane) - 1ull;
  for (int base = 0; base < P; base += 64) {
    const int i = base + lane;
    const uint32_t k = keys[i];
    const bool first = k < 0xFFFFFFFEu && (i == 0 || keys[i - 1] != k);
    const unsigned long long bal = __ballot(first);
    if (first) uniq[nUniq + __popcll(bal & ltMask)] = k;
    nUniq += __popcll(bal);
  }
  wave_lds_sync();
  for (int e = eS + lane; e < eE; e += 64) {
    const uint32_t col = (uint32_t)colIdx[e];
    int lo = 0, hi = nUniq - 1, found = 0;
    while (lo <= hi) {
      const int mid = (lo + hi) >> 1;
      const uint32_t v = uniq[mid];
      if (v == col) {
        found = mid;
        break;
      }
      if (v < col)
        lo = mid + 1;
      else
        hi = mid - 1;
    }
    edgeToColumn[e] = found;
    edgeToRow[e] = r0 + row_of_edge(sRow, e);
  }
  if (lane == 0) blockPartition[w] = (nUniq + W - 1) / W;
}

// One stable pass of a wave's LSD radix sort on a DB-bit digit: hist holds the first place of
// every digit; a lane's place is that plus the number of lanes before it in its group of 64 with
// the same digit (one ballot per digit bit).
template <int DB>
__device__ __forceinline__ void wave_scatter_in_order(const uint32_t* src, uint32_t* dst,
                                                      uint32_t* hist, int n, int shift, int lane) {
  const unsigned long long ltMask = (1ull << lane) - 1ull;
  for (int base = 0; base < n; base += 64) {
    const int i = base + lane;
    const bool valid = i < n;
    const uint32_t key = valid ? src[i] : 0u;
    const unsigned dgt = (key >> shift) & ((1u << DB) - 1u);
    unsigned long long peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < DB; b++) {
      const unsigned long long bal = __ballot((dgt >> b) & 1u);
      peers &= ((dgt >> b) & 1u) ? bal : ~bal;
    }
    if (valid) dst[hist[dgt] + __popcll(peers & ltMask)] = key;
    // the last peer advances the digit's position; the wave's LDS operations stay in order
    if (valid && (peers >> lane) == 1ull) hist[dgt] += __popcll(peers);
  }
}

// The same job for graphs of at most 2^22 nodes, where a column id and the edge's position in
// the window (< kSortMax = 2^10) fit one 32-bit word: a stable LSD radix sort of those words on
// the column bits, eight bits per pass, in the wave's LDS slice (histogram with LDS atomics,
// in-order scatter with wave ballots). The sorted words carry the edge positions along, so the
// rank of every distinct column is scattered straight back to its edges: no binary search, and
// a third of the instructions of the bitonic network.
template <int W>
__global__ __launch_bounds__(kBlock) void window_rank_radix_kernel(
    const int32_t* __restrict__ rowPtr, const int32_t* __restrict__ colIdx, int N, int nRW,
    int colBits, int32_t* __restrict__ blockPartition, int32_t* __restrict__ edgeToColumn,
    int32_t* __restrict__ edgeToRow, WsHeader* __restrict__ hdr, LongQueues queues) {
  constexpr int WAVES = kBlock / 64;
  constexpr int IDX_BITS = 10;
  static_assert(kSortMax <= (1 << IDX_BITS), "edge position must fit IDX_BITS");
  __shared__ uint32_t sBufA[WAVES][kSortMax];
  __shared__ uint32_t sBufB[WAVES][kSortMax];
  __shared__ __align__(16) uint32_t sHist[WAVES][256];
  __shared__ int sRowW[WAVES][17];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int w = blockIdx.x * WAVES + wave;
  if (w >= nRW) return;
  const int r0 = w * 16;
  int* sRow = sRowW[wave];
  if (lane < 17) sRow[lane] = rowPtr[min(r0 + lane, N)];
  wave_lds_sync();
  const int eS = sRow[0], eE = sRow[16];
  const int n = eE - eS;
  if (n == 0) {
    if (lane == 0) blockPartition[w] = 0;
    return;
  }
  if (n > kSortMax) {  // left to window_rank_kernel, through the queue if there is one
    if (lane == 0) queue_long_window(queues, hdr, w, n);
    return;
  }
  uint32_t* src = sBufA[wave];
  uint32_t* dst = sBufB[wave];
  uint32_t* hist = sHist[wave];
  const unsigned long long ltMask = (1ull << lane) - 1ull;
  bool bad = false;
  for (int i = lane; i < n; i += 64) {
    uint32_t col = (uint32_t)colIdx[eS + i];
    if (col >= (uint32_t)N) {
      bad = true;
      col = 0;
    }
    src[i] = (col << IDX_BITS) | (uint32_t)i;
    edgeToRow[eS + i] = r0 + row_of_edge(sRow, eS + i);
  }
  if (bad) atomicOr(&hdr->error, 1);
  // Digits: the first pass takes eight bits, the stable passes share the rest evenly (22 column
  // bits: 8 + 7 + 7; 18: 8 + 5 + 5), so that a stable pass spends one ballot per bit it needs.
  const int firstBits = colBits < 8 ? colBits : 8;
  const int restBits = colBits - firstBits;
  const int nStable = (restBits + 7) / 8;
  int shift = IDX_BITS;
  for (int pass = 0; pass <= nStable; pass++) {
    const int db = pass == 0 ? firstBits
                             : restBits / nStable + (pass <= restBits % nStable ? 1 : 0);
    const unsigned mask = (1u << db) - 1u;
#pragma unroll
    for (int k = 0; k < 4; k++) hist[lane + 64 * k] = 0;
    wave_lds_sync();
    for (int i = lane; i < n; i += 64) atomicAdd(&hist[(src[i] >> shift) & mask], 1u);
    wave_lds_sync();
    {
      // exclusive scan of the 256 counts: lane l owns bins 4l .. 4l+3
      const uint4 c = reinterpret_cast<uint4*>(hist)[lane];
      const unsigned sum = c.x + c.y + c.z + c.w;
      const unsigned excl = wave_inclusive_scan(sum, lane) - sum;
      reinterpret_cast<uint4*>(hist)[lane] =
          make_uint4(excl, excl + c.x, excl + c.x + c.y, excl + c.x + c.y + c.z);
    }
    wave_lds_sync();
    if (pass == 0) {
      // The first pass need not be stable: words with the same digit are put in order by the
      // later passes or name the same column, and equal columns only have to end up next to
      // each other. A returning LDS atomic hands out the places, a tenth of the instructions
      // of the in-order scatter below.
      for (int i = lane; i < n; i += 64) {
        const uint32_t key = src[i];
        dst[atomicAdd(&hist[(key >> shift) & mask], 1u)] = key;
      }
    } else {
      switch (db) {
        case 1: wave_scatter_in_order<1>(src, dst, hist, n, shift, lane); break;
        case 2: wave_scatter_in_order<2>(src, dst, hist, n, shift, lane); break;
        case 3: wave_scatter_in_order<3>(src, dst, hist, n, shift, lane); break;
        case 4: wave_scatter_in_order<4>(src, dst, hist, n, shift, lane); break;
        case 5: wave_scatter_in_order<5>(src, dst, hist, n, shift, lane); break;
        case 6: wave_scatter_in_order<6>(src, dst, hist, n, shift, lane); break;
        case 7: wave_scatter_in_order<7>(src, dst, hist, n, shift, lane); break;
        default: wave_scatter_in_order<8>(src, dst, hist, n, shift, lane); break;
      }
    }
    wave_lds_sync();
    uint32_t* t = src;
    src = dst;
    dst = t;
    shift += db;
  }
  // ranks of the distinct columns, scattered to their edges
  int nUniq = 0;
  for (int base = 0; base < n; base += 64) {
    const int i = base + lane;
    const bool valid = i < n;
    const uint32_t key = valid ? src[i] : 0u;
    const bool first = valid && (i == 0 || (src[i - 1] >> IDX_BITS) != (key >> IDX_BITS));
    const unsigned long long bal = __ballot(first);
    if (valid)
      edgeToColumn[eS + (int)(key & ((1u << IDX_BITS) - 1u))] =
          nUniq + __popcll(bal & (ltMask | (1ull << lane))) - 1;
    nUniq += __popcll(bal);
  }
  if (lane == 0) blockPartition[w] = (nUniq + W - 1) / W;
}

template <int W, int TB>
__global__ __launch_bounds__(TB) void window_rank_kernel(
    const int32_t* __restrict__ rowPtr, const int32_t* __restrict__ colIdx, int N, int range,
    int nPasses, int32_t* __restrict__ blockPartition,
    int32_t* __restrict__ edgeToColumn,
    int32_t* __restrict__ edgeToRow, WsHeader* __restrict__ hdr,
    const int32_t* __restrict__ bigList) {
  extern __shared__ __align__(16) uint32_t smem[];
  uint32_t* bits = smem;                 // range/32 words
  uint32_t* pref = smem + (range >> 5);  // range/128 group prefixes
  __shared__ int sRow[17];
  __shared__ unsigned sWaveTot[TB / 64];
  __shared__ int sTake;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  // Two ways to find work. With a queue (graphs of mostly short windows) the grid is a fixed
  // number of workgroups that drain it: an empty queue ends the kernel at once instead of one
  // workgroup per window holding this kernel's large LDS allocation. Without one (graphs of long
  // windows, where the appends to the queue would cost more than they save) workgroup b takes
  // window b.
  const int nBig = bigList ? hdr->nBig : 1;
  while (true) {
  __syncthreads();  // the previous window's reads of sRow / sTake are done
  if (tid == 0) sTake = bigList ? atomicAdd(&hdr->nextBig, 1) : 0;
  __syncthreads();
  if (sTake >= nBig) break;
  const int w = bigList ? bigList[sTake] : (int)blockIdx.x;
  const int r0 = w * 16;
  if (tid < 17) sRow[tid] = rowPtr[min(r0 + tid, N)];
  __syncthreads();
  const int eS = sRow[0], eE = sRow[16];
  if (!bigList && eE - eS <= kSortMax) break;  // ranked by window_rank_small_kernel
  const int nGroups = range >> 7;
  unsigned uniqueBefore = 0;
  for (int pass = 0; pass < nPasses; pass++) {
    const int lo = pass * range;
    for (int i = tid; i < nGroups; i += TB)
      reinterpret_cast<uint4*>(bits)[i] = make_uint4(0, 0, 0, 0);
    __syncthreads();
    // four edges per thread and step, loads first
    for (int e0 = eS + tid; e0 < eE; e0 += 4 * TB) {
      int cols[4];
#pragma unroll
      for (int u = 0; u < 4; u++) cols[u] = (e0 + u * TB < eE) ? colIdx[e0 + u * TB] : lo;
#pragma unroll
      for (int u = 0; u < 4; u++) {
        if (e0 + u * TB >= eE) continue;
        const int col = cols[u];
        if ((unsigned)col >= (unsigned)N) {
          atomicOr(&hdr->error, 1);
          continue;
        }
        const unsigned rel = (unsigned)(col - lo);
        if (rel < (unsigned)range) atomicOr(&bits[rel >> 5], 1u << (rel & 31));
      }
    }
    __syncthreads();
    unsigned carry = uniqueBefore;
    for (int gb = 0; gb < nGroups; gb += TB) {
      const int gi = gb + tid;
      unsigned cnt = 0;
      if (gi < nGroups) {
        const uint4 v = reinterpret_cast<const uint4*>(bits)[gi];
        cnt = __popc(v.x) + __popc(v.y) + __popc(v.z) + __popc(v.w);
      }
      const unsigned incl = wave_inclusive_scan(cnt, lane);
      if (lane == 63) sWaveTot[wave] = incl;
      __syncthreads();
      unsigned waveOff = 0, tileTot = 0;
#pragma unroll
      for (int v = 0; v < TB / 64; v++) {
        const unsigned t = sWaveTot[v];
        if (v < wave) waveOff += t;
        tileTot += t;
      }
      if (gi < nGroups) pref[gi] = carry + waveOff + incl - cnt;
      carry += tileTot;
      __syncthreads();
    }
    for (int e0 = eS + tid; e0 < eE; e0 += 4 * TB) {
      int cols[4];
#pragma unroll
      for (int u = 0; u < 4; u++) cols[u] = (e0 + u * TB < eE) ? colIdx[e0 + u * TB] : -1;
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int col = cols[u];
        const unsigned rel = (unsigned)(col - lo);
        if ((unsigned)col < (unsigned)N && rel < (unsigned)range) {
          // rank = set bits below this one: group prefix, then the whole 128-bit group read at
          // once and masked
          const unsigned wd = rel >> 5;
          const uint4 grp = reinterpret_cast<const uint4*>(bits)[wd >> 2];
          const unsigned words[4] = {grp.x, grp.y, grp.z, grp.w};
          unsigned rank = pref[wd >> 2];
#pragma unroll
          for (unsigned k = 0; k < 4; k++) {
            const unsigned keep = k < (wd & 3u) ? 0xFFFFFFFFu
                                  : (k == (wd & 3u) ? ((1u << (rel & 31)) - 1u) : 0u);
            rank += __popc(words[k] & keep);
          }
          edgeToColumn[e0 + u * TB] = (int)rank;
        }
      }
    }
    uniqueBefore = carry;
    __syncthreads();
  }
  for (int e = eS + tid; e < eE; e += TB) edgeToRow[e] = r0 + row_of_edge(sRow, e);
  if (tid == 0) blockPartition[w] = (int)((uniqueBefore + W - 1) / W);
  if (!bigList) break;
  }
}

// Windows of kSortMax < edges <= kMedMax on graphs whose column range needs several bitset passes
// (N > kRangeMax): one workgroup per queued window sorts the window's column ids, compacts the
// distinct ones and ranks every edge by binary search, instead of several passes over a 48 KiB
// bitset that such a window fills with a few thousand bits. The sort is the wave-level LSD radix
// sort of window_rank_radix_kernel widened to a workgroup: eight bits per pass, every wave on its
// own contiguous quarter of the keys (histogram with LDS atomics, one thread per digit turns the
// per-wave counts into start positions, in-order scatter with wave ballots), two LDS buffers.
// Two sizes: windows of up to kMedMax edges (256 threads, 32 KiB of buffers, four workgroups per
// CU), and the handful of windows of up to kLargeMax edges (1024 threads, 128 KiB), which would
// otherwise each walk the bitset passes alone at the end of the phase.
constexpr int kMedThreads = 256;
constexpr int kMedItems = 16;
constexpr int kMedMax = kMedThreads * kMedItems;
constexpr int kLargeThreads = 1024;
constexpr int kLargeItems = 16;
constexpr int kLargeMax = kLargeThreads * kLargeItems;

// takes the windows of `queue` (each of at most THREADS * ITEMS edges)
template <int W, int ITEMS, int THREADS>
__global__ __launch_bounds__(THREADS) void window_rank_sort_kernel(
    const int32_t* __restrict__ rowPtr, const int32_t* __restrict__ colIdx, int N, int colBits,
    int32_t* __restrict__ blockPartition, int32_t* __restrict__ edgeToColumn,
    int32_t* __restrict__ edgeToRow, WsHeader* __restrict__ hdr,
    const int32_t* __restrict__ queue, const int* __restrict__ queueLen,
    int* __restrict__ nextEntry) {
  constexpr int WAVES = THREADS / 64;
  constexpr int CAP = THREADS * ITEMS;
  static_assert(THREADS >= 256 && THREADS % 256 == 0, "the first 256 threads own one digit each");
  extern __shared__ __align__(16) uint32_t sBufDyn[];  // two buffers of CAP keys
  uint32_t* const sBuf0 = sBufDyn;
  uint32_t* const sBuf1 = sBufDyn + CAP;
  __shared__ uint32_t sHist[WAVES][256];
  __shared__ int sRow[17];
  __shared__ unsigned sWaveTot[WAVES];
  __shared__ int sTake;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const unsigned long long ltMask = (1ull << lane) - 1ull;
  const int nQueued = *queueLen;
  while (true) {
    __syncthreads();
    if (tid == 0) sTake = atomicAdd(nextEntry, 1);
    __syncthreads();
    if (sTake >= nQueued) break;
    const int w = queue[sTake];
    const int r0 = w * 16;
    if (tid < 17) sRow[tid] = rowPtr[min(r0 + tid, N)];
    __syncthreads();
    const int eS = sRow[0], eE = sRow[16];
    const int n = eE - eS;
    if (n > CAP) continue;  // cannot happen: the queue holds what fits
    bool bad = false;
    for (int i = tid; i < n; i += THREADS) {
      unsigned k = (unsigned)colIdx[eS + i];
      if (k >= (unsigned)N) {
        bad = true;
        k = 0u;
      }
      sBuf0[i] = k;
    }
    if (bad) atomicOr(&hdr->error, 1);
    // wave v sorts the keys [cb, ce) of every pass's input into their places of its output
    const int chunk = ((n + THREADS - 1) / THREADS) * 64;
    const int cb = min(n, wave * chunk), ce = min(n, cb + chunk);
    uint32_t* src = sBuf0;
    uint32_t* dst = sBuf1;
    uint32_t* hist = sHist[wave];
    for (int shift = 0; shift < colBits; shift += 8) {
#pragma unroll
      for (int k = 0; k < 4; k++) hist[lane + 64 * k] = 0;
      __syncthreads();  // the keys of this pass are in place, the counters are clear
      for (int i = cb + lane; i < ce; i += 64) atomicAdd(&hist[(src[i] >> shift) & 255u], 1u);
      __syncthreads();
      {
        // thread d < 256: keys with a smaller digit, then this digit's keys of the waves in front
        unsigned c[WAVES], tot = 0, incl = 0;
        if (tid < 256) {
#pragma unroll
          for (int v = 0; v < WAVES; v++) {
            c[v] = sHist[v][tid];
            tot += c[v];
          }
          incl = wave_inclusive_scan(tot, lane);
          if (lane == 63) sWaveTot[wave] = incl;
        }
        __syncthreads();
        if (tid < 256) {
          unsigned run = incl - tot;
#pragma unroll
          for (int v = 0; v < 4; v++)
            if (v < wave) run += sWaveTot[v];
#pragma unroll
          for (int v = 0; v < WAVES; v++) {
            sHist[v][tid] = run;
            run += c[v];
          }
        }
      }
      __syncthreads();
      if (shift == 0) {
        // the first pass need not be stable (equal columns only have to end up next to each
        // other): a returning LDS atomic hands out the places of the wave's keys
        for (int i = cb + lane; i < ce; i += 64) {
          const uint32_t key = src[i];
          dst[atomicAdd(&hist[key & 255u], 1u)] = key;
        }
      } else {
        wave_scatter_in_order<8>(src + cb, dst, hist, ce - cb, shift, lane);
      }
      uint32_t* t = src;
      src = dst;
      dst = t;
    }
    __syncthreads();
    // distinct columns: first occurrences, compacted in order into the other buffer (every wave
    // on its quarter [cb, ce) again: a count with ballots, the waves' totals, then the stores)
    uint32_t* uniq = dst;
    unsigned cnt = 0;
    for (int base = cb; base < ce; base += 64) {
      const int i = base + lane;
      const bool first = i < ce && (i == 0 || src[i - 1] != src[i]);
      cnt += (unsigned)__popcll(__ballot(first));
    }
    if (lane == 0) sWaveTot[wave] = cnt;
    __syncthreads();
    unsigned pos = 0, nUniq = 0;
#pragma unroll
    for (int v = 0; v < WAVES; v++) {
      const unsigned x = sWaveTot[v];
      if (v < wave) pos += x;
      nUniq += x;
    }
    for (int base = cb; base < ce; base += 64) {
      const int i = base + lane;
      const bool first = i < ce && (i == 0 || src[i - 1] != src[i]);
      const unsigned long long bal = __ballot(first);
      if (first) uniq[pos + (unsigned)__popcll(bal & ltMask)] = src[i];
      pos += (unsigned)__popcll(bal);
    }
    __syncthreads();
    for (int e = eS + tid; e < eE; e += THREADS) {
      unsigned col = (unsigned)colIdx[e];
      if (col >= (unsigned)N) col = 0u;
      int lo = 0, hi = (int)nUniq - 1, found = 0;
      while (lo <= hi) {
        const int mid = (lo + hi) >> 1;
        const unsigned v = uniq[mid];
        if (v == col) {
          found = mid;
          break;
        }
        if (v < col)
          lo = mid + 1;
        else
          hi = mid - 1;
      }
      edgeToColumn[e] = found;
      edgeToRow[e] = r0 + row_of_edge(sRow, e);
    }
    if (tid == 0) blockPartition[w] = (int)((nUniq + W - 1) / W);
  }
}

// ------------------------------------------------- scan + window ordering
constexpr int kFinBlock = 1024;
// windows the single-workgroup kernel takes: a window id fits kFinIdBits bits and a block count
// (at most 16 * kFinSingleMax / 8 + 1) the rest of a 32-bit word
constexpr int kFinSingleMax = 16384;
constexpr int kFinIdBits = 14;

__global__ __launch_bounds__(kFinBlock) void finalize_count_kernel(
    const int32_t* __restrict__ blockPartition, int nRW, int32_t* __restrict__ rowWindowOffset,
    int32_t* __restrict__ sortedRowWindows, WsHeader* __restrict__ hdr) {
  // One workgroup; every wave owns a contiguous chunk of the windows and walks it on its own
  // (wave-level scans and ballots only), so a pass over the array costs a handful of block
  // barriers instead of several per 1024 elements. The sort's two buffers are in LDS
  // (2 * kFinSingleMax words of dynamic LDS): a (key, window) pair is one word, key above
  // kFinIdBits bits of window id.
  extern __shared__ __align__(16) uint32_t finLds[];
  uint32_t* bufA = finLds;
  uint32_t* bufB = finLds + kFinSingleMax;
  constexpr int NW = kFinBlock / 64;
  __shared__ unsigned sWaveSum[NW];
  __shared__ int sWaveMax[NW];
  constexpr int DB = 6;               // digit bits per sorting pass: one bin per lane
  constexpr int NB = 1 << DB;
  static_assert(NB == 64, "the start computation gives every lane one bin");
  __shared__ unsigned sCnt[NW][NB];   // per wave: elements per digit, then its running position
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int chunk = (((nRW + NW - 1) / NW) + 63) & ~63;
  const int cBegin = min(wave * chunk, nRW);
  const int cEnd = min(cBegin + chunk, nRW);

  // ---- the counts into LDS first, every thread's loads in flight together: each later pass
  // walks its chunk group by group, and a global load per group would cost its full latency
  // every time
  {
    constexpr int U = 4;
    for (int i0 = tid; i0 < nRW; i0 += U * kFinBlock) {
      int v[U];
#pragma unroll
      for (int u = 0; u < U; u++) {
        const int i = i0 + u * kFinBlock;
        v[u] = i < nRW ? blockPartition[i] : 0;
      }
#pragma unroll
      for (int u = 0; u < U; u++) {
        const int i = i0 + u * kFinBlock;
        if (i < nRW) bufB[i] = (uint32_t)v[u];
      }
    }
  }
  __syncthreads();
  // ---- inclusive scan of the block counts into rowWindowOffset[1..], and their maximum
  {
    unsigned sum = 0;
    int mx = 0;
    for (int i = cBegin + lane; i < cEnd; i += 64) {
      const int v = (int)bufB[i];
      sum += (unsigned)v;
      mx = max(mx, v);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      sum += __shfl_xor(sum, off);
      mx = max(mx, __shfl_xor(mx, off));
    }
    if (lane == 0) {
      sWaveSum[wave] = sum;
      sWaveMax[wave] = mx;
    }
  }
  __syncthreads();
  unsigned carry = 0, total = 0;
  int maxC = 0;
#pragma unroll
  for (int k = 0; k < NW; k++) {
    const unsigned t = sWaveSum[k];
    if (k < wave) carry += t;
    total += t;
    maxC = max(maxC, sWaveMax[k]);
  }
  for (int base = cBegin; base < cEnd; base += 64) {
    const int i = base + lane;
    const unsigned v = (i < cEnd) ? bufB[i] : 0u;
    const unsigned incl = wave_inclusive_scan(v, lane);
    if (i < cEnd) rowWindowOffset[i + 1] = (int)(carry + incl);
    carry += __shfl(incl, 63);
  }
  if (tid == 0) {
    rowWindowOffset[0] = 0;
    hdr->nTcb = (long long)total;
  }

  // ---- stable sort by descending count == stable ascending LSD radix sort of (maxC - count),
  // six bits per pass
  int nBits = 0;
  while ((maxC >> nBits) != 0) nBits++;
  const int nPass = (nBits + DB - 1) / DB;
  if (nPass == 0) {
    for (int i = tid; i < nRW; i += kFinBlock) sortedRowWindows[i] = i;
    return;
  }
  const unsigned long long ltMask = (1ull << lane) - 1ull;
  for (int pass = 0; pass < nPass; pass++) {
    const int shift = kFinIdBits + pass * DB;
    const bool last = pass == nPass - 1;
    uint32_t* dst = (pass & 1) ? bufB : bufA;
    const uint32_t* src = (pass & 1) ? bufA : bufB;
    __syncthreads();  // the previous pass's writes are visible, its use of sCnt is over
    sCnt[wave][lane] = 0;
    // peers = lanes of this 64-element group with the same digit (one ballot per digit bit)
    auto digit_peers = [&](bool valid, int dgt) {
      unsigned long long peers = __ballot(valid);
#pragma unroll
      for (int b = 0; b < DB; b++) {
        const unsigned long long bal = __ballot((dgt >> b) & 1);
        peers &= ((dgt >> b) & 1) ? bal : ~bal;
      }
      return peers;
    };
    auto load_key = [&](int i) -> unsigned {
      if (i >= cEnd) return 0u;
      // the first pass finds the counts themselves in bufB
      return pass == 0 ? ((unsigned)(maxC - (int)src[i]) << kFinIdBits) | (unsigned)i : src[i];
    };
    // histogram of the wave's chunk: LDS atomics (the whole workgroup shares one CU's vector
    // ALUs, and a ballot per digit bit costs far more instructions than the atomic's conflicts)
    // Counts cluster (most windows of a skewed graph share a digit), and lanes that name the same
    // bin are served one after the other: the lanes that agree with the group's first one are
    // counted with one ballot and added once.
    wave_lds_sync();
    for (int base = cBegin; base < cEnd; base += 64) {
      const int i = base + lane;
      const bool valid = i < cEnd;
      const int dgt = (int)(load_key(i) >> shift) & (NB - 1);
      const int d0 = __builtin_amdgcn_readfirstlane(dgt);
      const unsigned long long same = __ballot(valid && dgt == d0);
      if (valid && dgt != d0) atomicAdd(&sCnt[wave][dgt], 1u);
      if (lane == 0) atomicAdd(&sCnt[wave][d0], (unsigned)__popcll(same));
    }
    __syncthreads();
    // start of (digit = lane, wave): all smaller digits, then the same digit in earlier waves
    unsigned digitTotal = 0, before = 0;
#pragma unroll
    for (int k = 0; k < NW; k++) {
      const unsigned cnt = sCnt[k][lane];
      digitTotal += cnt;
      if (k < wave) before += cnt;
    }
    const unsigned start = wave_inclusive_scan(digitTotal, lane) - digitTotal + before;
    __syncthreads();
    sCnt[wave][lane] = start;
    // scatter, in order (the next group's key is in flight during this one's)
    unsigned keyNext = load_key(cBegin + lane);
    for (int base = cBegin; base < cEnd; base += 64) {
      const int i = base + lane;
      const bool valid = i < cEnd;
      const unsigned key = keyNext;
      keyNext = load_key(i + 64);
      const int dgt = (int)(key >> shift) & (NB - 1);
      const unsigned long long peers = digit_peers(valid, dgt);
      if (valid) dst[sCnt[wave][dgt] + __popcll(peers & ltMask)] = key;
      // the last peer moves the digit's running position (the wave's LDS accesses stay in order)
      if (valid && (peers >> lane) == 1ull) sCnt[wave][dgt] += __popcll(peers);
    }
    if (last) {
      // the order leaves LDS as whole lines: scattered 4-byte stores from the last pass would
      // all go through this one CU's address unit, 64 lines per instruction
      __syncthreads();
      for (int i = tid; i < nRW; i += kFinBlock)
        sortedRowWindows[i] = (int)(dst[i] & ((1u << kFinIdBits) - 1u));
    }
  }
}

// ---- the same scan + stable sort spread over many workgroups, for graphs with many windows.
// Every WAVE of the grid owns a contiguous chunk of the windows (chunks in wave order), exactly as
// the waves of finalize_count_kernel do; what that kernel exchanges through LDS and block barriers
// goes through small global arrays and kernel boundaries here:
//   finalize_partials_kernel   per-wave sum and maximum of the block counts
//   finalize_scan_kernel       rowWindowOffset of the chunk (carry = sums of the earlier waves),
//                              total and maximum into the header, digit histogram of pass 0
//   finalize_scatter_kernel    one pass: start of (digit, wave) from every wave's histogram, then
//                              the in-order scatter of the chunk
//   finalize_histogram_kernel  digit histogram of the next pass (its input is the scattered
//                              order, complete only at the kernel boundary)
// The number of passes depends on the largest count, known on the device only: the host enqueues
// as many passes as the window count could need and the surplus kernels return at once.
constexpr int kFinDigitBits = 6;
constexpr int kFinBins = 1 << kFinDigitBits;

struct FinChunk {
  int begin, end;
};
__device__ __forceinline__ FinChunk fin_chunk(int nRW, int totalWaves, int gw) {
  const int chunk = (((nRW + totalWaves - 1) / totalWaves) + 63) & ~63;
  FinChunk c;
  c.begin = min(gw * chunk, nRW);
  c.end = min(c.begin + chunk, nRW);
  return c;
}
__device__ __forceinline__ unsigned long long fin_digit_peers(bool valid, int dgt) {
  unsigned long long peers = __ballot(valid);
#pragma unroll
  for (int b = 0; b < kFinDigitBits; b++) {
    const unsigned long long bal = __ballot((dgt >> b) & 1);
    peers &= ((dgt >> b) & 1) ? bal : ~bal;
  }
  return peers;
}
__device__ __forceinline__ int fin_passes(int maxC) {
  int nBits = 0;
  while ((maxC >> nBits) != 0) nBits++;
  return (nBits + kFinDigitBits - 1) / kFinDigitBits;
}

__global__ __launch_bounds__(256) void finalize_partials_kernel(
    const int32_t* __restrict__ blockPartition, int nRW, int totalWaves,
    unsigned* __restrict__ waveSum, int* __restrict__ waveMax) {
  const int lane = threadIdx.x & 63;
  const int gw = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (gw >= totalWaves) return;
  const FinChunk c = fin_chunk(nRW, totalWaves, gw);
  unsigned sum = 0;
  int mx = 0;
  for (int i = c.begin + lane; i < c.end; i += 64) {
    const int v = blockPartition[i];
    sum += (unsigned)v;
    mx = max(mx, v);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    sum += __shfl_xor(sum, off);
    mx = max(mx, __shfl_xor(mx, off));
  }
  if (lane == 0) {
    waveSum[gw] = sum;
    waveMax[gw] = mx;
  }
}

// digit histogram of a wave's chunk into hist[gw * 64 + digit]; sBins: 64 LDS counters of the wave
__device__ __forceinline__ void fin_histogram(const int32_t* __restrict__ keys, bool fromCounts,
                                              int maxC, FinChunk c, int shift, int lane,
                                              unsigned* sBins, unsigned* __restrict__ histRow) {
  sBins[lane] = 0;
  wave_lds_sync();
  const unsigned long long ltMask = (1ull << lane) - 1ull;
  int keyNext = (c.begin + lane < c.end) ? keys[c.begin + lane] : 0;
  for (int base = c.begin; base < c.end; base += 64) {
    const int i = base + lane;
    const bool valid = i < c.end;
    const int raw = keyNext;
    keyNext = (i + 64 < c.end) ? keys[i + 64] : 0;
    const int key = fromCounts ? maxC - raw : raw;
    const int dgt = (key >> shift) & (kFinBins - 1);
    const unsigned long long peers = fin_digit_peers(valid, dgt);
    // the first lane of every group of equal digits adds the group to its bin
    if (valid && (peers & ltMask) == 0ull) sBins[dgt] += __popcll(peers);
  }
  wave_lds_sync();
  histRow[lane] = sBins[lane];
}

__global__ __launch_bounds__(256) void finalize_scan_kernel(
    const int32_t* __restrict__ blockPartition, int nRW, int totalWaves,
    const unsigned* __restrict__ waveSum, const int* __restrict__ waveMax,
    int32_t* __restrict__ rowWindowOffset, unsigned* __restrict__ hist,
    WsHeader* __restrict__ hdr) {
  __shared__ unsigned sBins[4][kFinBins];
  const int lane = threadIdx.x & 63;
  const int gw = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (gw >= totalWaves) return;
  const FinChunk c = fin_chunk(nRW, totalWaves, gw);
  unsigned carry = 0, total = 0;
  int maxC = 0;
#pragma unroll 4
  for (int k = lane; k < totalWaves; k += 64) {
    const unsigned t = waveSum[k];
    if (k < gw) carry += t;
    total += t;
    maxC = max(maxC, waveMax[k]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    carry += __shfl_xor(carry, off);
    total += __shfl_xor(total, off);
    maxC = max(maxC, __shfl_xor(maxC, off));
  }
  for (int base = c.begin; base < c.end; base += 64) {
    const int i = base + lane;
    const unsigned v = (i < c.end) ? (unsigned)blockPartition[i] : 0u;
    const unsigned incl = wave_inclusive_scan(v, lane);
    if (i < c.end) rowWindowOffset[i + 1] = (int)(carry + incl);
    carry += __shfl(incl, 63);
  }
  if (gw == 0 && lane == 0) {
    rowWindowOffset[0] = 0;
    hdr->nTcb = (long long)total;
    hdr->maxCount = maxC;
  }
  fin_histogram(blockPartition, true, maxC, c, 0, lane, sBins[threadIdx.x >> 6],
                hist + (size_t)gw * kFinBins);
}

__global__ __launch_bounds__(256) void finalize_histogram_kernel(
    int nRW, int totalWaves, int pass, const int32_t* __restrict__ keysA,
    const int32_t* __restrict__ keysB, unsigned* __restrict__ hist,
    const WsHeader* __restrict__ hdr) {
  __shared__ unsigned sBins[4][kFinBins];
  const int lane = threadIdx.x & 63;
  const int gw = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (gw >= totalWaves) return;
  const int maxC = hdr->maxCount;
  const int nPass = fin_passes(maxC);
  if (pass >= nPass) return;
  // the keys this pass reads are the ones the previous pass wrote
  const bool prevToOut = ((nPass - pass) & 1) == 0;
  const int32_t* kSrc = prevToOut ? keysA : keysB;
  fin_histogram(kSrc, false, maxC, fin_chunk(nRW, totalWaves, gw), pass * kFinDigitBits, lane,
                sBins[threadIdx.x >> 6], hist + (size_t)gw * kFinBins);
}

__global__ __launch_bounds__(256) void finalize_scatter_kernel(
    const int32_t* __restrict__ blockPartition, int nRW, int totalWaves, int pass,
    int32_t* __restrict__ sortedRowWindows, int32_t* __restrict__ keysA,
    int32_t* __restrict__ keysB, int32_t* __restrict__ valsTmp, const unsigned* __restrict__ hist,
    const WsHeader* __restrict__ hdr) {
  __shared__ unsigned sPos[4][kFinBins];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int gw = blockIdx.x * 4 + wave;
  if (gw >= totalWaves) return;
  const FinChunk c = fin_chunk(nRW, totalWaves, gw);
  const int maxC = hdr->maxCount;
  const int nPass = fin_passes(maxC);
  if (nPass == 0) {  // every window is empty: the order is the identity
    if (pass == 0)
      for (int i = c.begin + lane; i < c.end; i += 64) sortedRowWindows[i] = i;
    return;
  }
  if (pass >= nPass) return;
  const int shift = pass * kFinDigitBits;
  const bool toOut = ((nPass - 1 - pass) & 1) == 0;
  int32_t* kDst = toOut ? keysA : keysB;
  int32_t* vDst = toOut ? sortedRowWindows : valsTmp;
  const int32_t* kSrc = toOut ? keysB : keysA;
  const int32_t* vSrc = toOut ? valsTmp : sortedRowWindows;
  // start of (digit = lane, this wave): all smaller digits, then the same digit in earlier waves
  unsigned digitTotal = 0, before = 0;
#pragma unroll 8
  for (int k = 0; k < totalWaves; k++) {
    const unsigned cnt = hist[(size_t)k * kFinBins + lane];
    digitTotal += cnt;
    before += (k < gw) ? cnt : 0u;
  }
  const unsigned start = wave_inclusive_scan(digitTotal, lane) - digitTotal + before;
  sPos[wave][lane] = start;
  wave_lds_sync();
  const unsigned long long ltMask = (1ull << lane) - 1ull;
  auto load_key = [&](int i) {
    return (i < c.end) ? ((pass == 0) ? (maxC - blockPartition[i]) : kSrc[i]) : 0;
  };
  auto load_val = [&](int i) { return (i < c.end) ? ((pass == 0) ? i : vSrc[i]) : 0; };
  int keyNext = load_key(c.begin + lane);
  int valNext = load_val(c.begin + lane);
  for (int base = c.begin; base < c.end; base += 64) {
    const int i = base + lane;
    const bool valid = i < c.end;
    const int key = keyNext, val = valNext;
    keyNext = load_key(i + 64);
    valNext = load_val(i + 64);
    const int dgt = (key >> shift) & (kFinBins - 1);
    const unsigned long long peers = fin_digit_peers(valid, dgt);
    if (valid) {
      const unsigned pos = sPos[wave][dgt] + __popcll(peers & ltMask);
      kDst[pos] = key;
      vDst[pos] = val;
    }
    // the last peer moves the digit's running position (the wave's LDS accesses stay in order)
    if (valid && (peers >> lane) == 1ull) sPos[wave][dgt] += __popcll(peers);
  }
}

// ------------------------------------------------------------------ phase 2
// Any window, TC blocks at a time: rows may hold repeated or descending columns. sCnt
// ([TC * 16]) and sBm ([TC * WPT]) are the caller's LDS; sRow holds the window's 17 row pointers;
// *sUnsorted must be 0 on entry. Every thread of the workgroup calls this.
template <int W, int TB>
__device__ __forceinline__ void fill_window_generic(
    const int32_t* __restrict__ colIdx, const int32_t* __restrict__ edgeToColumn, int w, int base,
    int nb, const int TC, int32_t* __restrict__ tcblockRowid, uint8_t* __restrict__ tcblocktileId,
    int32_t* __restrict__ tcblockOffset, int32_t* __restrict__ sparseAToXidx,
    unsigned long long* __restrict__ bitmap, unsigned* sCnt, unsigned long long* sBm,
    const int* sRow, unsigned* sWaveTot, unsigned* sUnsortedPtr) {
  constexpr int WPT = 16 * W / 64;  // bitmap words per TC block
  constexpr int LOGW = (W == 16) ? 4 : 3;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int eS = sRow[0], eE = sRow[16];
  const unsigned long long ltMask = (1ull << lane) - 1ull;
  unsigned carry = (unsigned)eS;  // absolute edge position where the next TC block starts

  for (int tc0 = 0; tc0 < nb; tc0 += TC) {
    const int nt = min(TC, nb - tc0);
    for (int i = tid; i < nt * 16; i += TB) sCnt[i] = 0;
    for (int i = tid; i < nt * WPT; i += TB) sBm[i] = 0ull;
    __syncthreads();
    // four edges per thread and step, loads first: the LDS atomics of one edge then overlap the
    // memory latency of the next ones
    for (int e0 = eS + tid; e0 < eE; e0 += 4 * TB) {
      int ecs[4], cols[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int e = e0 + u * TB;
        ecs[u] = (e < eE) ? edgeToColumn[e] : -1;
        cols[u] = (e < eE) ? colIdx[e] : 0;
      }
      if (tc0 == 0) {
        // once per window: which rows are strictly ascending (every edge against its left
        // neighbour in the same row)
#pragma unroll
        for (int u = 0; u < 4; u++) {
          const int e = e0 + u * TB;
          if (e < eE && e > eS) {
            const int r = row_of_edge(sRow, e);
            if (e > sRow[r] && colIdx[e - 1] >= cols[u]) atomicOr(sUnsortedPtr, 1u << r);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int e = e0 + u * TB;
        const int ec = ecs[u];
        const int t = (ec >> LOGW) - tc0;
        if (ec >= 0 && (unsigned)t < (unsigned)nt) {
          const int r = row_of_edge(sRow, e);
          const int cl = ec & (W - 1);
          atomicAdd(&sCnt[t * 16 + r], 1u);
          // 8x8 sub-blocks in column-major order, row-major and MSB-first inside
          const int sub = (cl >> 3) * (W / 8) + (r >> 3);
          atomicOr(&sBm[t * WPT + sub], 1ull << (63 - ((r & 7) * 8 + (cl & 7))));
          sparseAToXidx[(int64_t)(base + tc0 + t) * W + cl] = cols[u];
        }
      }
    }
    __syncthreads();
    for (int tb = 0; tb < nt; tb += TB) {
      const int t = tb + tid;
      unsigned nnz = 0;
      if (t < nt) {
#pragma unroll
        for (int r = 0; r < 16; r++) nnz += sCnt[t * 16 + r];
      }
      const unsigned incl = wave_inclusive_scan(nnz, lane);
      if (lane == 63) sWaveTot[wave] = incl;
      __syncthreads();
      unsigned waveOff = 0, tileTot = 0;
#pragma unroll
      for (int v = 0; v < TB / 64; v++) {
        const unsigned x = sWaveTot[v];
        if (v < wave) waveOff += x;
        tileTot += x;
      }
      if (t < nt) {
        const int64_t gt = (int64_t)base + tc0 + t;
        unsigned run = carry + waveOff + incl - nnz;
        tcblockOffset[gt] = (int)run;
        tcblockRowid[gt] = w;
        if (*sUnsortedPtr == 0u) {
          // Every row of the window is strictly ascending, so the block's tile ids are its set
          // bits read row by row, left to right (src/utils.cu:213-223 walks the edges in that
          // order): this thread writes them all, next to the previous block's.
          unsigned long long words[WPT];
#pragma unroll
          for (int k = 0; k < WPT; k++) words[k] = sBm[t * WPT + k];
          walk_tile_ids<W>(words, tcblocktileId, run);
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const unsigned c = sCnt[t * 16 + r];
          sCnt[t * 16 + r] = run;
          run += c;
        }
        // bitmap words out; a compacted slot that no edge named keeps column id 0
        unsigned colMask = 0;  // bit cl set <=> slot cl holds a column
#pragma unroll
        for (int k = 0; k < WPT; k++) {
          const unsigned long long word = sBm[t * WPT + k];
          bitmap[gt * WPT + k] = word;
          unsigned long long x = word;
          x |= x >> 32;
          x |= x >> 16;
          x |= x >> 8;
          const unsigned rowOr = (unsigned)(x & 0xFFull);  // bit (7 - cl%8)
          const int colHalf = (W == 16) ? (k >> 1) : 0;
#pragma unroll
          for (int b = 0; b < 8; b++)
            if (rowOr & (0x80u >> b)) colMask |= 1u << (colHalf * 8 + b);
        }
#pragma unroll
        for (int cl = 0; cl < W; cl++)
          if (!((colMask >> cl) & 1u)) sparseAToXidx[gt * W + cl] = 0;
      }
      carry += tileTot;
      __syncthreads();
    }
    // Windows with some row that is not strictly ascending. Tile ids sit in CSR edge order
    // inside a TC block (src/utils.cu:213-223): position = start of (block, row) + number of
    // earlier edges of that row in the block. In a strictly ascending row those are exactly the
    // bits left of the edge's own bit in the block's bitmap row, so every edge of such a row
    // finds its place on its own; the other rows are replayed in order below.
    const unsigned unsorted = *sUnsortedPtr;
    for (int e = eS + tid; unsorted != 0u && e < eE; e += TB) {
      const int ec = edgeToColumn[e];
      const int t = (ec >> LOGW) - tc0;
      if ((unsigned)t >= (unsigned)nt) continue;
      const int r = row_of_edge(sRow, e);
      if ((unsorted >> r) & 1u) continue;
      const int cl = ec & (W - 1);
      const int shift = 8 * (7 - (r & 7));
      unsigned before = 0;
      if (W == 16 && cl >= 8)
        before = __popc((unsigned)(sBm[t * WPT + (r >> 3)] >> shift) & 0xFFu);
      const unsigned own =
          (unsigned)(sBm[t * WPT + (cl >> 3) * (W / 8) + (r >> 3)] >> shift) & 0xFFu;
      before += __popc(own >> (8 - (cl & 7)));
      tcblocktileId[sCnt[t * 16 + r] + before] = (uint8_t)(r * W + cl);
    }
    // rows with repeated or descending columns: a wave replays the whole row in order
    for (int r = wave; r < 16; r += TB / 64) {
      if (!((unsorted >> r) & 1u)) continue;
      const int rs = sRow[r], re = sRow[r + 1];
      int ecNext = (rs + lane < re) ? edgeToColumn[rs + lane] : 0;
      for (int eb = rs; eb < re; eb += 64) {
        const int e = eb + lane;
        const bool valid = e < re;
        const int ec = ecNext;
        ecNext = (e + 64 < re) ? edgeToColumn[e + 64] : 0;  // next batch, in flight during this one
        const int t = (ec >> LOGW) - tc0;
        const bool inr = valid && (unsigned)t < (unsigned)nt;
        unsigned long long peers = __ballot(inr);
        if (peers == 0ull) continue;
        // lanes whose edges fall into the same block: agree on every bit of t (t < TC)
        for (int b = 0; ((TC - 1) >> b) != 0; b++) {
          const unsigned long long bal = __ballot((t >> b) & 1);
          peers &= ((t >> b) & 1) ? bal : ~bal;
        }
        unsigned pos = 0;
        if (inr) pos = sCnt[t * 16 + r] + __popcll(peers & ltMask);
        if (inr) tcblocktileId[pos] = (uint8_t)(r * W + (ec & (W - 1)));
        // the highest peer lane advances the running position of (block, row)
        if (inr && (peers >> lane) == 1ull) sCnt[t * 16 + r] += __popcll(peers);
      }
    }
    __syncthreads();
  }
}


// One workgroup (or one wave) per window. Windows whose rows are all strictly ascending (every
// CSR that is sorted and free of repeated entries) take the short way: every edge sets its bit in
// the LDS bitmaps and drops its column id into the LDS copy of the block's id slots; a block's
// non-zero count is then the population count of its bitmap, its tile ids are its set bits read
// row by row (src/utils.cu:213-223 walks the edges in exactly that order), and bitmaps and ids
// leave LDS as contiguous runs. A window with a repeated or descending column is handed to
// fill_window_generic. TC blocks of LDS at a time on the short way, TCG on the general one.
template <int W, int TB, int TC, int TCG>
__device__ __forceinline__ void fill_one_window(
    int w, int nRW, const int32_t* __restrict__ rowPtr, const int32_t* __restrict__ colIdx, int N,
    int E, const int32_t* __restrict__ edgeToColumn, const int32_t* __restrict__ rowWindowOffset,
    const WsHeader* __restrict__ hdr, int32_t* __restrict__ tcblockRowid,
    uint8_t* __restrict__ tcblocktileId, int32_t* __restrict__ tcblockOffset,
    int32_t* __restrict__ sparseAToXidx, unsigned long long* __restrict__ bitmap, int minBlocks,
    int maxBlocks) {
  constexpr int WPT = 16 * W / 64;  // bitmap words per TC block
  constexpr int LOGW = (W == 16) ? 4 : 3;
  constexpr int FAST_BYTES = TC * (WPT * 8 + W * 4);
  constexpr int GEN_BYTES = TCG * (16 * 4 + WPT * 8);
  constexpr int RAW_BYTES = FAST_BYTES > GEN_BYTES ? FAST_BYTES : GEN_BYTES;
  __shared__ __align__(16) unsigned char sRaw[RAW_BYTES];
  __shared__ int sRow[17];
  __shared__ unsigned sWaveTot[TB / 64];
  __shared__ unsigned sUnsorted;  // bit r: row r's columns are not strictly ascending
  unsigned long long* sBm = reinterpret_cast<unsigned long long*>(sRaw);       // [TC * WPT]
  int32_t* sIds = reinterpret_cast<int32_t*>(sRaw + TC * WPT * 8);             // [TC * W]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  // launched right behind phase 1 (no host in between): a column index outside [0, N) left
  // edgeToColumn unwritten, so nothing here may run
  if (hdr && hdr->error) return;
  if (tid == 0) sUnsorted = 0u;
  if (w == 0 && tid == 0) tcblockOffset[rowWindowOffset[nRW]] = E;
  const int base = rowWindowOffset[w];
  const int nb = rowWindowOffset[w + 1] - base;
  // a launch may be one of two that share the windows by length: [minBlocks, maxBlocks]
  if (nb == 0 || nb < minBlocks || nb > maxBlocks) return;
  const int r0 = w * 16;
  if (tid < 17) sRow[tid] = rowPtr[min(r0 + tid, N)];
  __syncthreads();
  const int eS = sRow[0], eE = sRow[16];
  unsigned carry = (unsigned)eS;  // absolute edge position where the next TC block starts

  for (int tc0 = 0; tc0 < nb; tc0 += TC) {
    const int nt = min(TC, nb - tc0);
    for (int i = tid; i < nt * WPT; i += TB) sBm[i] = 0ull;
    for (int i = tid; i < nt * W; i += TB) sIds[i] = 0;
    __syncthreads();
    // Four CONSECUTIVE edges per thread (one 16-byte load of ranks, one of column ids, from a
    // 16-byte aligned index). Consecutive edges of a row fall into the same bitmap byte (row r
    // of an 8-column sub-block) up to eight at a time, so a thread first ORs its edges' bits
    // together per byte and then issues one 32-bit LDS atomic per distinct byte.
    unsigned* sBmWords = reinterpret_cast<unsigned*>(sBm);
    for (int e0 = (eS & ~3) + 4 * tid; e0 < eE; e0 += 4 * TB) {
      int ecs[4], cols[4];
      if (e0 + 4 <= E) {
        const int4 a = *reinterpret_cast<const int4*>(edgeToColumn + e0);
        const int4 b = *reinterpret_cast<const int4*>(colIdx + e0);
        ecs[0] = a.x; ecs[1] = a.y; ecs[2] = a.z; ecs[3] = a.w;
        cols[0] = b.x; cols[1] = b.y; cols[2] = b.z; cols[3] = b.w;
      } else {
#pragma unroll
        for (int u = 0; u < 4; u++) {
          ecs[u] = (e0 + u < E) ? edgeToColumn[e0 + u] : 0;
          cols[u] = (e0 + u < E) ? colIdx[e0 + u] : 0;
        }
      }
      int left = (tc0 == 0 && e0 > eS) ? colIdx[e0 - 1] : -1;
      const int eLo = e0 > eS ? e0 : eS;
      const int eHi = (e0 + 3 < eE - 1) ? e0 + 3 : eE - 1;
      const int rLo = row_of_edge(sRow, eLo);
      const int rHi = row_of_edge(sRow, eHi);
      int curKey = -1;
      unsigned curMask = 0;
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int e = e0 + u;
        const bool valid = e >= eS && e < eE;
        const int r = (rLo == rHi) ? rLo : (valid ? row_of_edge(sRow, e) : rLo);
        // once per window: is every edge right of its left neighbour in the same row?
        if (tc0 == 0 && valid && e > sRow[r] && left >= cols[u]) atomicOr(&sUnsorted, 1u << r);
        left = cols[u];
        const int t = (ecs[u] >> LOGW) - tc0;
        if (valid && (unsigned)t < (unsigned)nt) {
          const int cl = ecs[u] & (W - 1);
          sIds[t * W + cl] = cols[u];
          // 8x8 sub-blocks in column-major order; byte 7 - r%8 of the sub-block's word is row
          // r%8, MSB first
          const int sub = (cl >> 3) * (W / 8) + (r >> 3);
          const int key = (t * WPT + sub) * 8 + 7 - (r & 7);
          const unsigned m8 = 0x80u >> (cl & 7);
          if (key == curKey) {
            curMask |= m8;
          } else {
            if (curKey >= 0) atomicOr(&sBmWords[curKey >> 2], curMask << (8 * (curKey & 3)));
            curKey = key;
            curMask = m8;
          }
        }
      }
      if (curKey >= 0) atomicOr(&sBmWords[curKey >> 2], curMask << (8 * (curKey & 3)));
    }
    __syncthreads();
    if (sUnsorted != 0u) break;  // known after the first pass over the window's edges
    for (int tb = 0; tb < nt; tb += TB) {
      const int t = tb + tid;
      unsigned long long words[WPT];
      unsigned nnz = 0;
      if (t < nt) {
#pragma unroll
        for (int k = 0; k < WPT; k++) {
          words[k] = sBm[t * WPT + k];
          nnz += __popcll(words[k]);
        }
      }
      const unsigned incl = wave_inclusive_scan(nnz, lane);
      if (lane == 63) sWaveTot[wave] = incl;
      __syncthreads();
      unsigned waveOff = 0, tileTot = 0;
#pragma unroll
      for (int v = 0; v < TB / 64; v++) {
        const unsigned x = sWaveTot[v];
        if (v < wave) waveOff += x;
        tileTot += x;
      }
      if (t < nt) {
        const int64_t gt = (int64_t)base + tc0 + t;
        unsigned pos = carry + waveOff + incl - nnz;
        tcblockOffset[gt] = (int)pos;
        tcblockRowid[gt] = w;
        // tile ids: the block's set bits read row by row (each lane walks its own block; the
        // byte stores of neighbouring lanes fall next to each other)
        walk_tile_ids<W>(words, tcblocktileId, pos);
      }
      carry += tileTot;
      __syncthreads();
    }
    // bitmaps and column ids of the chunk as contiguous runs (unused id slots stay 0)
    {
      unsigned long long* bmDst = bitmap + ((int64_t)base + tc0) * WPT;
      for (int i = tid; i < nt * WPT; i += TB) bmDst[i] = sBm[i];
      int32_t* idDst = sparseAToXidx + ((int64_t)base + tc0) * W;
      for (int i = tid; i < nt * W; i += TB) idDst[i] = sIds[i];
    }
    __syncthreads();
  }
  if (sUnsorted != 0u) {
    // repeated or descending columns somewhere in the window: start over on the general way
    __syncthreads();
    if (tid == 0) sUnsorted = 0u;
    __syncthreads();
    unsigned* gCnt = reinterpret_cast<unsigned*>(sRaw);                                  // [TCG*16]
    unsigned long long* gBm = reinterpret_cast<unsigned long long*>(sRaw + TCG * 64);    // [TCG*WPT]
    fill_window_generic<W, TB>(colIdx, edgeToColumn, w, base, nb, TCG, tcblockRowid,
                               tcblocktileId, tcblockOffset, sparseAToXidx, bitmap, gCnt, gBm, sRow,
                               sWaveTot, &sUnsorted);
  }
}

template <int W, int TB, int TC, int TCG>
__global__ __launch_bounds__(TB) void window_fill_kernel(
    const int32_t* __restrict__ rowPtr, const int32_t* __restrict__ colIdx, int N, int E,
    const int32_t* __restrict__ edgeToColumn, const int32_t* __restrict__ rowWindowOffset,
    const WsHeader* __restrict__ hdr, int32_t* __restrict__ tcblockRowid,
    uint8_t* __restrict__ tcblocktileId, int32_t* __restrict__ tcblockOffset,
    int32_t* __restrict__ sparseAToXidx, unsigned long long* __restrict__ bitmap, int minBlocks,
    int maxBlocks) {
  fill_one_window<W, TB, TC, TCG>((int)blockIdx.x, (int)gridDim.x, rowPtr, colIdx, N, E,
                                  edgeToColumn, rowWindowOffset, hdr, tcblockRowid, tcblocktileId,
                                  tcblockOffset, sparseAToXidx, bitmap, minBlocks, maxBlocks);
}

// The few long windows of a graph of short ones (more than minBlocks - 1 TC blocks): a grid of a
// few hundred workgroups looks through the block counts, 256 windows at a time per workgroup,
// and fills the long ones it finds one after the other. One workgroup per window, as
// window_fill_kernel has it, would start a hundred thousand workgroups of 60 KiB of LDS each to
// find that nearly all of them have nothing to do.
template <int W, int TB, int TC, int TCG>
__global__ __launch_bounds__(TB) void window_fill_long_kernel(
    const int32_t* __restrict__ rowPtr, const int32_t* __restrict__ colIdx, int N, int E, int nRW,
    const int32_t* __restrict__ edgeToColumn, const int32_t* __restrict__ rowWindowOffset,
    const WsHeader* __restrict__ hdr, int32_t* __restrict__ tcblockRowid,
    uint8_t* __restrict__ tcblocktileId, int32_t* __restrict__ tcblockOffset,
    int32_t* __restrict__ sparseAToXidx, unsigned long long* __restrict__ bitmap, int minBlocks) {
  static_assert(TB == 256, "one candidate window per thread and round");
  __shared__ int sList[TB];
  __shared__ int sListLen;
  for (int base = (int)blockIdx.x * TB; base < nRW; base += (int)gridDim.x * TB) {
    __syncthreads();  // the list of the 256 windows before these has been worked through
    if (threadIdx.x == 0) sListLen = 0;
    __syncthreads();
    const int w = base + (int)threadIdx.x;
    if (w < nRW && rowWindowOffset[w + 1] - rowWindowOffset[w] >= minBlocks)
      sList[atomicAdd(&sListLen, 1)] = w;
    __syncthreads();
    const int len = sListLen;
    for (int k = 0; k < len; k++) {
      __syncthreads();  // the window before this one has left the LDS arrays
      fill_one_window<W, TB, TC, TCG>(sList[k], nRW, rowPtr, colIdx, N, E, edgeToColumn,
                                      rowWindowOffset, hdr, tcblockRowid, tcblocktileId,
                                      tcblockOffset, sparseAToXidx, bitmap, minBlocks, 0x7FFFFFFF);
    }
  }
}

// ------------------------------------------------------------------ both phases, one call
// Graphs of long windows whose column range fits one bitset (N <= kRangeMax) when the caller has
// sized the block arrays by an upper bound instead of waiting for the count: the window's bitset
// is built twice (window_count_kernel for the block counts, window_rank_fill_kernel after the
// scan) and everything else happens while it sits in LDS, so edgeToColumn is written once and
// never read back and the column ids are read from memory once (the second and third reads of a
// window's 30 KB come from the L2).
//
// Neither kernel is bound by memory (on a 115 M-edge graph the vector ALUs are busy about half of
// the time and HBM a quarter), so they are written for few instructions per edge: a window's edges are split into whole groups of four consecutive edges
// from a 4-aligned index (no per-edge range checks, 16-byte loads and stores) and at most six
// edges at the window's two ends, which single threads handle one by one.

// Workgroup barrier that orders LDS traffic only: unlike __syncthreads() it does not wait for the
// wave's outstanding global loads and stores, which then overlap the next phase. For phases that
// talk to each other through LDS and never through global memory.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// The window's edges [eS, eE) as whole 4-aligned groups [gA, gB) plus the edges in front of and
// behind them (at most three each).
struct EdgeSplit {
  int gA, gB;      // whole groups: e0 = gA, gA + 4, ... < gB
  int headEnd;     // loose edges [eS, headEnd) and [tailBegin, eE)
  int tailBegin;
};
__device__ __forceinline__ EdgeSplit split_edges(int eS, int eE) {
  EdgeSplit sp;
  const int up = (eS + 3) & ~3, down = eE & ~3;
  sp.headEnd = min(up, eE);
  sp.tailBegin = max(down, sp.headEnd);
  sp.gA = up;
  sp.gB = max(down, up);
  return sp;
}
// the i-th loose edge (i = 0..5), or -1
__device__ __forceinline__ int loose_edge(const EdgeSplit& sp, int eS, int eE, int i) {
  const int nHead = sp.headEnd - eS;
  const int e = i < nHead ? eS + i : sp.tailBegin + (i - nHead);
  return (i < 6 && e < eE) ? e : -1;
}

// Sets the bits of the window's column ids in `bits` (32-bit words). Returns false (for the
// calling thread) when it met a column outside [0, N). U groups per thread and step, loads first.
template <int TB, int U>
__device__ __forceinline__ bool set_column_bits(const int32_t* __restrict__ colIdx, int eS, int eE,
                                                const EdgeSplit& sp, unsigned N, uint32_t* bits) {
  const int tid = threadIdx.x;
  bool ok = true;
  for (int e0 = sp.gA + 4 * tid; e0 < sp.gB; e0 += 4 * U * TB) {
    int4 c[U];
#pragma unroll
    for (int g = 0; g < U; g++) {
      // a group past the end repeats the first one (its bits are set already)
      const int e = e0 + 4 * g * TB < sp.gB ? e0 + 4 * g * TB : e0;
      c[g] = *reinterpret_cast<const int4*>(colIdx + e);
    }
#pragma unroll
    for (int g = 0; g < U; g++) {
      const unsigned col[4] = {(unsigned)c[g].x, (unsigned)c[g].y, (unsigned)c[g].z,
                               (unsigned)c[g].w};
#pragma unroll
      for (int u = 0; u < 4; u++) {
        if (col[u] < N)
          atomicOr(&bits[col[u] >> 5], 1u << (col[u] & 31));
        else
          ok = false;
      }
    }
  }
  const int e = loose_edge(sp, eS, eE, tid);
  if (e >= 0) {
    const unsigned c = (unsigned)colIdx[e];
    if (c < N)
      atomicOr(&bits[c >> 5], 1u << (c & 31));
    else
      ok = false;
  }
  return ok;
}

template <int W, int TB>
__global__ __launch_bounds__(TB) void window_count_kernel(
    const int32_t* __restrict__ rowPtr, const int32_t* __restrict__ colIdx, int N, int range,
    int32_t* __restrict__ blockPartition, WsHeader* __restrict__ hdr) {
  extern __shared__ __align__(16) uint32_t smem[];
  uint32_t* bits = smem;  // range/32 words
  __shared__ unsigned sWaveTot[TB / 64];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int w = blockIdx.x;
  const int eS = rowPtr[min(w * 16, N)], eE = rowPtr[min(w * 16 + 16, N)];
  if (eE <= eS) {
    if (tid == 0) blockPartition[w] = 0;
    return;
  }
  const int nGroups = range >> 7;
  for (int i = tid; i < nGroups; i += TB)
    reinterpret_cast<uint4*>(bits)[i] = make_uint4(0, 0, 0, 0);
  lds_barrier();
  const EdgeSplit sp = split_edges(eS, eE);
  if (!set_column_bits<TB, 4>(colIdx, eS, eE, sp, (unsigned)N, bits)) atomicOr(&hdr->error, 1);
  lds_barrier();
  unsigned cnt = 0;
  for (int gi = tid; gi < nGroups; gi += TB) {
    const uint4 v = reinterpret_cast<const uint4*>(bits)[gi];
    cnt += __popc(v.x) + __popc(v.y) + __popc(v.z) + __popc(v.w);
  }
  const unsigned incl = wave_inclusive_scan(cnt, lane);
  if (lane == 63) sWaveTot[wave] = incl;
  lds_barrier();
  if (tid == 0) {
    unsigned total = 0;
#pragma unroll
    for (int v = 0; v < TB / 64; v++) total += sWaveTot[v];
    blockPartition[w] = (int)((total + W - 1) / W);
  }
}

constexpr int kRankFillThreads = 768;
// 64-bit bitset words per thread of window_rank_fill_kernel at the largest column range
constexpr int kRankFillPerMax = (kRangeMax / 64 + kRankFillThreads - 1) / kRankFillThreads;

// Dynamic LDS: bitset (range/64 64-bit words) | set bits before each word (range/64 32-bit words)
// | chunkBytes of TC-block bitmaps. A window with a repeated or descending column is handed to
// fill_window_generic once its edgeToColumn entries are written, with the whole of the dynamic LDS
// as that routine's arrays.
template <int W, int TB>
__global__ __launch_bounds__(TB) __attribute__((amdgpu_waves_per_eu(6, 6)))
void window_rank_fill_kernel(
    const int32_t* __restrict__ rowPtr, const int32_t* __restrict__ colIdx, int N, int E,
    int range, int chunkBytes, const int32_t* __restrict__ rowWindowOffset,
    const int32_t* __restrict__ order, const WsHeader* __restrict__ hdr, int32_t* edgeToColumn,
    int32_t* __restrict__ edgeToRow,
    int32_t* __restrict__ tcblockRowid, uint8_t* __restrict__ tcblocktileId,
    int32_t* __restrict__ tcblockOffset, int32_t* __restrict__ sparseAToXidx,
    unsigned long long* __restrict__ bitmap) {
  constexpr int WPT = 16 * W / 64;  // bitmap words per TC block
  constexpr int LOGW = (W == 16) ? 4 : 3;
  constexpr int NWAVE = TB / 64;
  constexpr int PER = kRankFillPerMax;
  static_assert(TB == kRankFillThreads, "PER is computed for this workgroup size");
  extern __shared__ __align__(16) uint32_t smem[];
  const int nW64 = range >> 6;  // even: range is a multiple of 128
  unsigned long long* bits64 = reinterpret_cast<unsigned long long*>(smem);
  uint32_t* bits = smem;
  uint32_t* pref = smem + 2 * nW64;
  const int bitsetWords = (3 * nW64 + 3) & ~3;  // 32-bit words of bitset + prefixes, 16-byte padded
  unsigned long long* sBm = reinterpret_cast<unsigned long long*>(smem + bitsetWords);
  const int TC = chunkBytes / (WPT * 8);
  __shared__ int sRow[17];
  __shared__ unsigned sWaveTot[NWAVE];
  __shared__ unsigned sTot[PER * NWAVE];  // set bits per (round, wave), then their exclusive scan
  __shared__ unsigned sUnsorted;          // bit r: row r's columns are not strictly ascending

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  // windows start in the heavy-first order that the scan kernel has just written: the longest
  // ones first, so that none of them is still running alone when the others are done
  const int w = order[blockIdx.x];
  if (hdr->error) return;  // a column index outside [0, N): the caller gets the error, no output
  if (w == 0 && tid == 0) tcblockOffset[rowWindowOffset[gridDim.x]] = E;
  const int base = rowWindowOffset[w];
  const int nb = rowWindowOffset[w + 1] - base;
  const int r0 = w * 16;
  if (tid < 17) sRow[tid] = rowPtr[min(r0 + tid, N)];
  if (tid == 0) sUnsorted = 0u;
  for (int i = tid; i < (nW64 >> 1); i += TB)
    reinterpret_cast<uint4*>(bits)[i] = make_uint4(0, 0, 0, 0);
  lds_barrier();
  const int eS = sRow[0], eE = sRow[16];
  if (eE <= eS) return;
  const EdgeSplit sp = split_edges(eS, eE);

  // ---- the window's distinct columns as a bitset (validated by window_count_kernel)
  set_column_bits<TB, 2>(colIdx, eS, eE, sp, (unsigned)N, bits);
  lds_barrier();

  // ---- set bits before every 64-bit word; the compacted column ids, which are the set bits in
  // ascending order. Thread t owns the words t, t + TB, ... (neighbouring lanes, neighbouring
  // words): a wave-level scan per round, one scan of the (round, wave) totals by the first wave.
  const int per = (nW64 + TB - 1) / TB;  // <= PER
#pragma unroll
  for (int k = 0; k < PER; k++) {
    if (k < per) {
      const int i = k * TB + tid;
      const unsigned cnt = i < nW64 ? (unsigned)__popcll(bits64[i]) : 0u;
      const unsigned incl = wave_inclusive_scan(cnt, lane);
      if (i < nW64) pref[i] = incl - cnt;  // within the wave's 64 words for now
      if (lane == 63) sTot[k * NWAVE + wave] = incl;
    }
  }
  lds_barrier();
  if (wave == 0) {
    // exclusive scan of the per * NWAVE totals in (round, wave) order, two per lane
    static_assert(PER * NWAVE <= 128, "two totals per lane");
    const int n = per * NWAVE;
    const unsigned a = (2 * lane < n) ? sTot[2 * lane] : 0u;
    const unsigned b = (2 * lane + 1 < n) ? sTot[2 * lane + 1] : 0u;
    const unsigned inc = wave_inclusive_scan(a + b, lane);
    if (2 * lane < n) sTot[2 * lane] = inc - a - b;
    if (2 * lane + 1 < n) sTot[2 * lane + 1] = inc - b;
    if (lane == 63) sWaveTot[0] = inc;
  }
  lds_barrier();
  const unsigned nCols = sWaveTot[0];
  {
    int32_t* idDst = sparseAToXidx + (int64_t)base * W;
    char* idBytes = reinterpret_cast<char*>(idDst);
    for (int k = 0; k < per; k++) {
      const int i = k * TB + tid;
      if (i < nW64) {
        unsigned pos = sTot[k * NWAVE + wave] + pref[i];
        pref[i] = pos;
#ifdef F3S_PROBE_PRE_NO_IDS
        continue;
#endif
        // 32 bits at a time, with a 32-bit byte offset from the window's first id slot
        const unsigned long long x = bits64[i];
        unsigned off = pos * 4u;
#pragma unroll
        for (int h = 0; h < 2; h++) {
          unsigned half = h ? (unsigned)(x >> 32) : (unsigned)x;
          const int idBase = i * 64 + 32 * h;
          while (half) {
            *reinterpret_cast<int32_t*>(idBytes + off) = idBase + __builtin_ctz(half);
            off += 4u;
            half &= half - 1u;
          }
        }
      }
    }
    // the slots that the last block leaves unused hold 0
    for (int i = (int)nCols + tid; i < nb * W; i += TB) idDst[i] = 0;
  }

  // ---- ranks, rows and bitmaps. The first chunk of TC blocks also writes edgeToColumn /
  // edgeToRow; a window with more blocks ranks its edges again per chunk (the bitset stays in
  // LDS).
  auto rank_of = [&](int col) -> int {
    const unsigned wd = (unsigned)col >> 6;
    const unsigned long long below = bits64[wd] & ((1ull << (col & 63)) - 1ull);
    return (int)(pref[wd] + (unsigned)__popcll(below));
  };
  unsigned carry = (unsigned)eS;  // absolute edge position where the next TC block starts
  unsigned* sBmWords = reinterpret_cast<unsigned*>(sBm);
  const int stageBytes = ((bitsetWords * 4) / NWAVE) & ~15;
  for (int tc0 = 0; tc0 < nb; tc0 += TC) {
    const int nt = min(TC, nb - tc0);
    const bool lastChunk = tc0 + TC >= nb;
    const bool first = tc0 == 0;
    lds_barrier();  // ranks are read after the prefixes are written (and the previous chunk is out)
    for (int i = tid; i < nt * WPT; i += TB) sBm[i] = 0ull;
    lds_barrier();
    // one edge: rank, row, bit (the window's loose ends and groups that straddle rows)
    auto one_edge = [&](int e, int col, int r) {
      const int ec = rank_of(col);
      if (first) {
        edgeToColumn[e] = ec;
        edgeToRow[e] = r0 + r;
        if (e > sRow[r] && colIdx[e - 1] >= col) atomicOr(&sUnsorted, 1u << r);
      }
      const int t = (ec >> LOGW) - tc0;
      if ((unsigned)t < (unsigned)nt) {
        const int cl = ec & (W - 1);
        const int sub = (cl >> 3) * (W / 8) + (r >> 3);
        const int key = (t * WPT + sub) * 8 + 7 - (r & 7);
        atomicOr(&sBmWords[key >> 2], (0x80u >> (cl & 7)) << (8 * (key & 3)));
      }
    };
    // a whole group of four edges
    auto group = [&](int e0, const int4& c4, int left) {
      const int cols[4] = {c4.x, c4.y, c4.z, c4.w};
      const int r = row_of_edge(sRow, e0);
      if (e0 + 3 >= sRow[r + 1]) {  // the group straddles rows
#pragma unroll
        for (int u = 0; u < 4; u++) one_edge(e0 + u, cols[u], row_of_edge(sRow, e0 + u));
        return;
      }
      int ecs[4];
#pragma unroll
      for (int u = 0; u < 4; u++) ecs[u] = rank_of(cols[u]);
      if (first) {
#ifndef F3S_PROBE_PRE_NO_EDGE_STORES
        *reinterpret_cast<int4*>(edgeToColumn + e0) = make_int4(ecs[0], ecs[1], ecs[2], ecs[3]);
        *reinterpret_cast<int4*>(edgeToRow + e0) = make_int4(r0 + r, r0 + r, r0 + r, r0 + r);
#endif
        const bool bad = (e0 > sRow[r] && left >= cols[0]) || cols[0] >= cols[1] ||
                         cols[1] >= cols[2] || cols[2] >= cols[3];
        if (bad) atomicOr(&sUnsorted, 1u << r);
      }
      // Bits of one row. A TC block's bitmap is WPT 64-bit words, one per 8x8 sub-block (column
      // halves first); byte 7 - r%8 of a word is row r%8, MSB first. With rank = 16 t + cl (or
      // 8 t + cl) the 64-bit word of (t, cl, r) is 2 (rank >> 3) + (r >> 3) for both widths, and
      // the bit inside the row's byte is 0x80 >> (rank & 7). Consecutive edges of a row fall into
      // the same byte up to eight at a time: OR the bits of equal bytes together, then one
      // 32-bit LDS atomic per byte.
      const int byte = 7 - (r & 7);
      const int wordBias = (r >> 3) * 2 + (byte >> 2) - tc0 * (WPT * 2);  // in 32-bit words
      const unsigned rowBit = 0x80u << (8 * (byte & 3));
      int word[4];
      unsigned m[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        word[u] = (ecs[u] >> 3) * 4 + wordBias;
        m[u] = rowBit >> (ecs[u] & 7);
        if ((unsigned)((ecs[u] >> LOGW) - tc0) >= (unsigned)nt) m[u] = 0u;
      }
#pragma unroll
      for (int u = 1; u < 4; u++) {
        if (word[u] == word[u - 1]) {
          m[u] |= m[u - 1];
          m[u - 1] = 0u;
        }
      }
#pragma unroll
      for (int u = 0; u < 4; u++)
        if (m[u]) atomicOr(&sBmWords[word[u]], m[u]);
    };
    // two groups per thread and step, loads first
#ifdef F3S_PROBE_PRE_NO_FILL
    if (nb < 0)
#endif
    for (int e0 = sp.gA + 4 * tid; e0 < sp.gB; e0 += 8 * TB) {
      const int e1 = e0 + 4 * TB;
      const bool two = e1 < sp.gB;
      const int4 a = *reinterpret_cast<const int4*>(colIdx + e0);
      int4 b = a;
      if (two) b = *reinterpret_cast<const int4*>(colIdx + e1);
      int leftA = -1, leftB = -1;
      if (first) {
        if (e0 > eS) leftA = colIdx[e0 - 1];
        if (two) leftB = colIdx[e1 - 1];
      }
      group(e0, a, leftA);
      if (two) group(e1, b, leftB);
    }
    {
      const int e = loose_edge(sp, eS, eE, tid);
      if (e >= 0) one_edge(e, colIdx[e], row_of_edge(sRow, e));
    }
    lds_barrier();
    if (sUnsorted != 0u) break;  // known after the first pass over the window's edges
    for (int tb = 0; tb < nt; tb += TB) {
      const int t = tb + tid;
      unsigned long long words[WPT];
      unsigned nnz = 0;
      if (t < nt) {
#pragma unroll
        for (int k = 0; k < WPT; k++) {
          words[k] = sBm[t * WPT + k];
          nnz += __popcll(words[k]);
        }
      }
      const unsigned inc = wave_inclusive_scan(nnz, lane);
      if (lane == 63) sWaveTot[wave] = inc;
      lds_barrier();
      unsigned waveOff = 0, tileTot = 0;
#pragma unroll
      for (int v = 0; v < NWAVE; v++) {
        const unsigned x = sWaveTot[v];
        if (v < wave) waveOff += x;
        tileTot += x;
      }
      // tile ids: a block's set bits read row by row (src/utils.cu:213-223 walks the edges of a
      // window with ascending rows in exactly that order). In the window's last chunk the bitset
      // is no longer needed: each wave then collects the bytes of its 64 blocks in its slice of
      // that LDS and writes them out as whole dwords.
      const unsigned waveTot = __shfl(inc, 63);
      const unsigned wavePos0 = carry + waveOff;
      const unsigned a0 = wavePos0 & ~3u;
      const bool staged = lastChunk && waveTot + 3u <= (unsigned)stageBytes;
      uint8_t* stage = reinterpret_cast<uint8_t*>(smem) + wave * stageBytes;
      if (t < nt) {
        const int64_t gt = (int64_t)base + tc0 + t;
        const unsigned pos = wavePos0 + inc - nnz;
        tcblockOffset[gt] = (int)pos;
        tcblockRowid[gt] = w;
        // two calls, so that each store knows its address space (LDS or global)
#ifndef F3S_PROBE_PRE_NO_TILEIDS
        if (staged)
          walk_tile_ids<W>(words, stage, pos - a0);
        else
          walk_tile_ids<W>(words, tcblocktileId, pos);
#endif
      }
      if (staged && waveTot != 0u) {
        wave_lds_sync();
        const unsigned end = wavePos0 + waveTot;
        const unsigned d0 = min((wavePos0 + 3u) & ~3u, end);  // first whole dword
        const unsigned d1 = max(end & ~3u, d0);                // end of the whole dwords
        for (unsigned i = wavePos0 + lane; i < d0; i += 64) tcblocktileId[i] = stage[i - a0];
        for (unsigned i = d0 + 4u * lane; i < d1; i += 256u)
          *reinterpret_cast<uint32_t*>(tcblocktileId + i) =
              *reinterpret_cast<const uint32_t*>(stage + (i - a0));
        for (unsigned i = d1 + lane; i < end; i += 64) tcblocktileId[i] = stage[i - a0];
        wave_lds_sync();
      }
      carry += tileTot;
      lds_barrier();
    }
    {
      unsigned long long* bmDst = bitmap + ((int64_t)base + tc0) * WPT;
      for (int i = tid; i < nt * WPT; i += TB) bmDst[i] = sBm[i];
    }
  }
  if (sUnsorted != 0u) {
    // repeated or descending columns somewhere in the window: the general way, from the
    // edgeToColumn entries written above (visible to the whole workgroup after the barrier)
    __syncthreads();
    if (tid == 0) sUnsorted = 0u;
    __syncthreads();
    const int dynBytes = bitsetWords * 4 + chunkBytes;
    const int tcg = dynBytes / (64 + WPT * 8);
    unsigned* gCnt = reinterpret_cast<unsigned*>(smem);                                // [tcg*16]
    unsigned long long* gBm = reinterpret_cast<unsigned long long*>(smem + tcg * 16);  // [tcg*WPT]
    fill_window_generic<W, TB>(colIdx, edgeToColumn, w, base, nb, tcg, tcblockRowid,
                               tcblocktileId, tcblockOffset, sparseAToXidx, bitmap, gCnt, gBm, sRow,
                               sWaveTot, &sUnsorted);
  }
}

__global__ void set_tail_kernel(int32_t* tcblockOffset, long long nTcb, int E) {
  tcblockOffset[nTcb] = E;
}

__global__ void clear_header_kernel(WsHeader* hdr) {
  hdr->nTcb = 0;
  hdr->error = 0;
  hdr->nBig = 0;
  hdr->nextBig = 0;
  hdr->maxCount = 0;
  hdr->nMed = 0;
  hdr->nextMed = 0;
  hdr->nLarge = 0;
  hdr->nextLarge = 0;
}

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

}  // namespace

// waves of the multi-workgroup finalize (0: the single-workgroup kernel is used)
int finalize_waves(int nRW) {
  if (nRW <= kFinSingleMax) return 0;
  const int w = (nRW + 511) / 512;
  return w < 4096 ? w : 4096;
}

size_t preprocess_workspace_bytes(int N, int /*E*/) {
  const size_t nRW = (size_t)(N + kWinRows - 1) / kWinRows;
  const size_t fin = (size_t)finalize_waves((int)nRW) * (2 + kFinBins) * sizeof(int32_t);
  return kWsHeaderBytes + 3 * align256(nRW * sizeof(int32_t)) + align256(fin);
}

namespace {

// Scan of the block counts and the window order, after the kernels that write blockPartition.
int enqueue_finalize(int N, int W, const int32_t* blockPartition, int32_t* rowWindowOffset,
                     int32_t* sortedRowWindows, char* ws, hipStream_t stream) {
  const int nRW = (N + kWinRows - 1) / kWinRows;
  WsHeader* hdr = reinterpret_cast<WsHeader*>(ws);
  const size_t seg = align256((size_t)nRW * sizeof(int32_t));
  int32_t* keysA = reinterpret_cast<int32_t*>(ws + kWsHeaderBytes);
  int32_t* keysB = reinterpret_cast<int32_t*>(ws + kWsHeaderBytes + seg);
  int32_t* valsTmp = reinterpret_cast<int32_t*>(ws + kWsHeaderBytes + 2 * seg);
  const int finWaves = finalize_waves(nRW);
  if (finWaves == 0) {
    constexpr int ldsBytes = 2 * kFinSingleMax * (int)sizeof(uint32_t);
    F3S_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&finalize_count_kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, ldsBytes));
    hipLaunchKernelGGL(finalize_count_kernel, dim3(1), dim3(kFinBlock), ldsBytes, stream,
                       blockPartition, nRW, rowWindowOffset, sortedRowWindows, hdr);
    F3S_HIP_CHECK(hipGetLastError());
    return 0;
  }
  unsigned* waveSum = reinterpret_cast<unsigned*>(ws + kWsHeaderBytes + 3 * seg);
  int* waveMax = reinterpret_cast<int*>(waveSum + finWaves);
  unsigned* hist = waveSum + 2 * (size_t)finWaves;
  const dim3 grid((unsigned)((finWaves + 3) / 4)), block(256);
  hipLaunchKernelGGL(finalize_partials_kernel, grid, block, 0, stream, blockPartition, nRW,
                     finWaves, waveSum, waveMax);
  hipLaunchKernelGGL(finalize_scan_kernel, grid, block, 0, stream, blockPartition, nRW, finWaves,
                     waveSum, waveMax, rowWindowOffset, hist, hdr);
  // a window holds at most ceil(N / W) blocks: that bounds the passes that can be needed
  int maxBits = 0;
  while ((((int64_t)N + W - 1) / W >> maxBits) != 0) maxBits++;
  const int maxPass = (maxBits + kFinDigitBits - 1) / kFinDigitBits;
  for (int pass = 0; pass < (maxPass > 0 ? maxPass : 1); pass++) {
    if (pass > 0)
      hipLaunchKernelGGL(finalize_histogram_kernel, grid, block, 0, stream, nRW, finWaves, pass,
                         keysA, keysB, hist, hdr);
    hipLaunchKernelGGL(finalize_scatter_kernel, grid, block, 0, stream, blockPartition, nRW,
                       finWaves, pass, sortedRowWindows, keysA, keysB, valsTmp, hist, hdr);
  }
  F3S_HIP_CHECK(hipGetLastError());
  return 0;
}

// Enqueues every kernel of phase 1 on `stream`; `ws` is device scratch of
// preprocess_workspace_bytes(N, E) bytes whose header ends up holding the TC-block total and the
// error flag.
int enqueue_count(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int W,
                  int32_t* blockPartition, int32_t* edgeToColumn, int32_t* edgeToRow,
                  int32_t* rowWindowOffset, int32_t* sortedRowWindows, char* ws,
                  hipStream_t stream) {
  const int nRW = (N + kWinRows - 1) / kWinRows;
  WsHeader* hdr = reinterpret_cast<WsHeader*>(ws);
  const size_t seg = align256((size_t)nRW * sizeof(int32_t));
  // the three buffers the window order later sorts in hold the queues of long windows until then
  int32_t* keysA = reinterpret_cast<int32_t*>(ws + kWsHeaderBytes);
  int32_t* keysB = reinterpret_cast<int32_t*>(ws + kWsHeaderBytes + seg);
  int32_t* valsTmp = reinterpret_cast<int32_t*>(ws + kWsHeaderBytes + 2 * seg);

  hipLaunchKernelGGL(clear_header_kernel, dim3(1), dim3(1), 0, stream, hdr);
  if (nRW > 0) {
    int range = ((N + 127) / 128) * 128;
    if (range > kRangeMax) range = kRangeMax;
    const int nPasses = (N + range - 1) / range;
    const size_t lds = (size_t)(range / 32 + range / 128) * sizeof(uint32_t);
    const int smallGrid = (nRW + kBlock / 64 - 1) / (kBlock / 64);
    const bool big = (int64_t)E >= (int64_t)nRW * 2048;  // long windows on average
    int32_t* queue = big ? nullptr : valsTmp;
    // queued windows of a few thousand edges on a graph that needs several bitset passes are
    // sorted (window_rank_sort_kernel) instead of walking every pass; the others go to the
    // bitset kernel
    const bool sortMedium = queue != nullptr && nPasses >= 2;
    const LongQueues queues = {keysA, keysB, queue, sortMedium ? kMedMax : 0,
                               sortMedium ? kLargeMax : 0};
    // short windows: radix sort of packed (column, position) words when the column ids leave
    // room for the position, else the bitonic network on bare column ids
    int colBits = 0;
    while (colBits < 31 && ((int64_t)1 << colBits) < (int64_t)N) colBits++;
    if (colBits <= 22) {
      if (W == 16)
        hipLaunchKernelGGL(window_rank_radix_kernel<16>, dim3(smallGrid), dim3(kBlock), 0, stream,
                           rowPtr, colIdx, N, nRW, colBits, blockPartition, edgeToColumn,
                           edgeToRow, hdr, queues);
      else
        hipLaunchKernelGGL(window_rank_radix_kernel<8>, dim3(smallGrid), dim3(kBlock), 0, stream,
                           rowPtr, colIdx, N, nRW, colBits, blockPartition, edgeToColumn,
                           edgeToRow, hdr, queues);
    } else if (W == 16) {
      hipLaunchKernelGGL(window_rank_small_kernel<16>, dim3(smallGrid), dim3(kBlock), 0, stream,
                         rowPtr, colIdx, N, nRW, blockPartition, edgeToColumn, edgeToRow, hdr,
                         queues);
    } else {
      hipLaunchKernelGGL(window_rank_small_kernel<8>, dim3(smallGrid), dim3(kBlock), 0, stream,
                         rowPtr, colIdx, N, nRW, blockPartition, edgeToColumn, edgeToRow, hdr,
                         queues);
    }
    F3S_HIP_CHECK(hipGetLastError());
    if (sortMedium) {
      // two launches: up to kMedMax edges with 32 KiB of sort buffers (four workgroups per CU),
      // then the few windows up to kLargeMax with 128 KiB (one per CU)
#define F3S_SORT(WW, ITEMS, THREADS, GRID, QUEUE, LEN, COUNTER)                                 \
  do {                                                                                          \
    constexpr size_t ldsSort = (size_t)2 * THREADS * ITEMS * sizeof(uint32_t);                  \
    if (ldsSort > 48 * 1024)                                                                    \
      F3S_HIP_CHECK(hipFuncSetAttribute(                                                        \
          reinterpret_cast<const void*>(&window_rank_sort_kernel<WW, ITEMS, THREADS>),          \
          hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsSort));                           \
    hipLaunchKernelGGL((window_rank_sort_kernel<WW, ITEMS, THREADS>), dim3(GRID), dim3(THREADS),\
                       ldsSort, stream, rowPtr, colIdx, N, colBits, blockPartition,             \
                       edgeToColumn, edgeToRow, hdr, QUEUE, LEN, COUNTER);                      \
    F3S_HIP_CHECK(hipGetLastError());                                                           \
  } while (0)
      const int medGrid = nRW < 1024 ? nRW : 1024;
      const int largeGrid = nRW < 256 ? nRW : 256;
      if (W == 16) {
        F3S_SORT(16, kMedItems, kMedThreads, medGrid, keysA, &hdr->nMed, &hdr->nextMed);
        F3S_SORT(16, kLargeItems, kLargeThreads, largeGrid, keysB, &hdr->nLarge, &hdr->nextLarge);
      } else {
        F3S_SORT(8, kMedItems, kMedThreads, medGrid, keysA, &hdr->nMed, &hdr->nextMed);
        F3S_SORT(8, kLargeItems, kLargeThreads, largeGrid, keysB, &hdr->nLarge, &hdr->nextLarge);
      }
#undef F3S_SORT
    }
#define F3S_RANK(WW, TBB)                                                                     \
  hipLaunchKernelGGL((window_rank_kernel<WW, TBB>), dim3(rankGrid), dim3(TBB), lds, stream,   \
                     rowPtr, colIdx, N, range, nPasses, blockPartition,                       \
                     edgeToColumn, edgeToRow, hdr, queue)
    // the queue lives in the buffer finalize_count_kernel later uses for its values and is
    // drained by at most two workgroups per CU (2048 of them took 25 us to find an empty queue)
    const int rankGrid = big ? nRW : (nRW < 512 ? nRW : 512);
    if (W == 16) {
      if (big) F3S_RANK(16, 512); else F3S_RANK(16, 256);
    } else {
      if (big) F3S_RANK(8, 512); else F3S_RANK(8, 256);
    }
#undef F3S_RANK
    F3S_HIP_CHECK(hipGetLastError());
  }
  return enqueue_finalize(N, W, blockPartition, rowWindowOffset, sortedRowWindows, ws, stream);
}

int check_count_args(const char* who, int N, int E, int H, int W) {
  if (H != 16 || (W != 16 && W != 8))
    return fail(-2, "%s: block %dx%d unsupported (16x16 or 16x8)", who, H, W);
  if (N < 0 || E < 0) return fail(-2, "%s: negative size", who);
  return 0;
}

}  // namespace

int launch_preprocess_count(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int H,
                            int W, int32_t* blockPartition, int32_t* edgeToColumn,
                            int32_t* edgeToRow, int32_t* rowWindowOffset,
                            int32_t* sortedRowWindows, void* workspace, size_t wsBytes,
                            int64_t* nTcbHost, hipStream_t stream) {
  if (int rc = check_count_args("f3s_preprocess_count", N, E, H, W)) return rc;
  if (wsBytes < preprocess_workspace_bytes(N, E))
    return fail(-2, "f3s_preprocess_count: workspace %zu B < required %zu B", wsBytes,
                preprocess_workspace_bytes(N, E));
  char* ws = static_cast<char*>(workspace);
  if (int rc = enqueue_count(rowPtr, colIdx, N, E, W, blockPartition, edgeToColumn, edgeToRow,
                             rowWindowOffset, sortedRowWindows, ws, stream))
    return rc;
  WsHeader host;
  F3S_HIP_CHECK(hipMemcpyAsync(&host, ws, sizeof(WsHeader), hipMemcpyDeviceToHost, stream));
  F3S_HIP_CHECK(hipStreamSynchronize(stream));
  if (host.error) return fail(-4, "f3s_preprocess_count: column index outside [0, %d)", N);
  *nTcbHost = host.nTcb;
  return 0;
}

// ------------------------------------------------------- phase 1 without any allocation
// The scratch is the file-scope array `scratch` at the top of this file; host code reaches it
// through the per-device address hipGetSymbolAddress returns, looked up once per device.
constexpr size_t kStaticScratchBytes = kF3sStaticScratchBytes;

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratchMutex;
void* g_scratchPtr[kMaxDevices] = {};

int static_scratch(char** out) {
  int dev = -1;
  F3S_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(-2, "f3s_preprocess_count_static: device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratchMutex);
  if (!g_scratchPtr[dev]) {
    void* ptr = nullptr;
    F3S_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    g_scratchPtr[dev] = ptr;
  }
  *out = static_cast<char*>(g_scratchPtr[dev]);
  return 0;
}

__global__ void publish_result_kernel(const WsHeader* __restrict__ hdr,
                                      long long* __restrict__ result) {
  result[0] = hdr->nTcb;
  result[1] = (long long)hdr->error;
}

}  // namespace

size_t preprocess_static_scratch_bytes() { return kStaticScratchBytes; }

int launch_preprocess_count_static(const int32_t* rowPtr, const int32_t* colIdx, int N, int E,
                                   int H, int W, int32_t* blockPartition, int32_t* edgeToColumn,
                                   int32_t* edgeToRow, int32_t* rowWindowOffset,
                                   int32_t* sortedRowWindows, int64_t* resultDev,
                                   hipStream_t stream) {
  if (int rc = check_count_args("f3s_preprocess_count_static", N, E, H, W)) return rc;
  if (preprocess_workspace_bytes(N, E) > kStaticScratchBytes)
    return fail(-5, "f3s_preprocess_count_static: a graph of %d nodes needs %zu B of scratch, the "
                    "library's own buffer holds %zu B; use f3s_preprocess_count with a workspace",
                N, preprocess_workspace_bytes(N, E), kStaticScratchBytes);
  char* ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  // every kernel below starts from a header it clears itself and overwrites whatever else it
  // reads of the buffer, so nothing of an earlier call survives into this one
  if (int rc = enqueue_count(rowPtr, colIdx, N, E, W, blockPartition, edgeToColumn, edgeToRow,
                             rowWindowOffset, sortedRowWindows, ws, stream))
    return rc;
  hipLaunchKernelGGL(publish_result_kernel, dim3(1), dim3(1), 0, stream,
                     reinterpret_cast<const WsHeader*>(ws),
                     reinterpret_cast<long long*>(resultDev));
  F3S_HIP_CHECK(hipGetLastError());
  return 0;
}

namespace {

// Enqueues phase 2. `hdr` (may be null) is the header phase 1 left on the device: with it the
// kernels do nothing after a column index error, so that phase 2 can follow phase 1 on the stream
// without the host in between.
int enqueue_fill(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int W,
                 const int32_t* edgeToColumn, const int32_t* rowWindowOffset, const WsHeader* hdr,
                 int32_t* tcblockRowid, uint8_t* tcblocktileId, int32_t* tcblockOffset,
                 int32_t* sparseAToXidx, uint64_t* bitmap, hipStream_t stream) {
  const int nRW = (N + kWinRows - 1) / kWinRows;
  auto bm = reinterpret_cast<unsigned long long*>(bitmap);
  // Windows with thousands of edges get eight waves and 512 TC blocks of LDS at a time. Graphs
  // of short windows get one wave per window and 128 blocks of LDS, so that a CU works on a
  // dozen windows at once instead of three with most of their waves idle; their few windows of
  // more than 128 blocks are left to a second launch with four waves per window.
#define F3S_FILL(WW, TBB, TCC, TCG, LO, HI)                                                    \
  hipLaunchKernelGGL((window_fill_kernel<WW, TBB, TCC, TCG>), dim3(nRW), dim3(TBB), 0, stream, \
                     rowPtr, colIdx, N, E, edgeToColumn, rowWindowOffset, hdr, tcblockRowid,   \
                     tcblocktileId, tcblockOffset, sparseAToXidx, bm, LO, HI)
  // the long windows of a graph of short ones: at most two workgroups per CU look for them
#define F3S_FILL_LONG(WW)                                                                       \
  hipLaunchKernelGGL((window_fill_long_kernel<WW, 256, kFillChunk, kFillChunkGeneric>),         \
                     dim3((unsigned)min(512, (nRW + 255) / 256)), dim3(256), 0, stream, rowPtr, \
                     colIdx, N, E, nRW, edgeToColumn, rowWindowOffset, hdr, tcblockRowid,       \
                     tcblocktileId, tcblockOffset, sparseAToXidx, bm, kFillChunkSmall + 1)
  const bool big = (int64_t)E >= (int64_t)nRW * 2048;
  constexpr int kAll = 0x7FFFFFFF;
  if (W == 16) {
    if (big) {
      F3S_FILL(16, 512, kFillChunk, kFillChunkGeneric, 0, kAll);
    } else {
      F3S_FILL(16, 64, kFillChunkSmall, kFillChunkSmall, 0, kFillChunkSmall);
      F3S_HIP_CHECK(hipGetLastError());
      F3S_FILL_LONG(16);
    }
  } else {
    if (big) {
      F3S_FILL(8, 512, kFillChunk, kFillChunkGeneric, 0, kAll);
    } else {
      F3S_FILL(8, 64, kFillChunkSmall, kFillChunkSmall, 0, kFillChunkSmall);
      F3S_HIP_CHECK(hipGetLastError());
      F3S_FILL_LONG(8);
    }
  }
#undef F3S_FILL
#undef F3S_FILL_LONG
  F3S_HIP_CHECK(hipGetLastError());
  return 0;
}

}  // namespace

int launch_preprocess_fill(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int H,
                           int W, const int32_t* edgeToColumn, const int32_t* rowWindowOffset,
                           int64_t nTcb, int32_t* tcblockRowid, uint8_t* tcblocktileId,
                           int32_t* tcblockOffset, int32_t* sparseAToXidx, uint64_t* bitmap,
                           hipStream_t stream) {
  if (H != 16 || (W != 16 && W != 8))
    return fail(-2, "f3s_preprocess_fill: block %dx%d unsupported (16x16 or 16x8)", H, W);
  const int nRW = (N + kWinRows - 1) / kWinRows;
  if (nRW == 0) {
    hipLaunchKernelGGL(set_tail_kernel, dim3(1), dim3(1), 0, stream, tcblockOffset,
                       (long long)nTcb, E);
    F3S_HIP_CHECK(hipGetLastError());
    return 0;
  }
  return enqueue_fill(rowPtr, colIdx, N, E, W, edgeToColumn, rowWindowOffset, nullptr, tcblockRowid,
                      tcblocktileId, tcblockOffset, sparseAToXidx, bitmap, stream);
}

// ------------------------------------------------------- both phases behind one call
int64_t preprocess_capacity(int N, int64_t E, int W) {
  // a window of e edges names at most e distinct columns: ceil(e / W) <= e / W + 1 blocks
  const int64_t nRW = ((int64_t)N + kWinRows - 1) / kWinRows;
  return (E + W - 1) / W + nRW;
}

int launch_preprocess(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int H, int W,
                      int32_t* blockPartition, int32_t* edgeToColumn, int32_t* edgeToRow,
                      int32_t* rowWindowOffset, int32_t* sortedRowWindows, int64_t capacity,
                      int32_t* tcblockRowid, uint8_t* tcblocktileId, int32_t* tcblockOffset,
                      int32_t* sparseAToXidx, uint64_t* bitmap, void* workspace, size_t wsBytes,
                      int64_t* nTcbHost, hipStream_t stream) {
  if (int rc = check_count_args("f3s_preprocess", N, E, H, W)) return rc;
  if (wsBytes < preprocess_workspace_bytes(N, E))
    return fail(-2, "f3s_preprocess: workspace %zu B < required %zu B", wsBytes,
                preprocess_workspace_bytes(N, E));
  if (capacity < preprocess_capacity(N, E, W))
    return fail(-2, "f3s_preprocess: block arrays sized for %lld TC blocks, the bound for this "
                    "graph is %lld (f3s_preprocess_capacity)",
                (long long)capacity, (long long)preprocess_capacity(N, E, W));
  char* ws = static_cast<char*>(workspace);
  WsHeader* hdr = reinterpret_cast<WsHeader*>(ws);
  const int nRW = (N + kWinRows - 1) / kWinRows;
  const bool aligned16 =
      ((reinterpret_cast<uintptr_t>(colIdx) | reinterpret_cast<uintptr_t>(edgeToColumn) |
        reinterpret_cast<uintptr_t>(edgeToRow) | reinterpret_cast<uintptr_t>(sparseAToXidx) |
        reinterpret_cast<uintptr_t>(tcblocktileId)) & 15u) == 0;
  // long windows, one bitset pass: the kernels that keep a window's bitset in LDS for both phases
  const bool fused = nRW > 0 && (int64_t)E >= (int64_t)nRW * 2048 && N <= kRangeMax && aligned16;
  if (fused) {
    const int range = ((N + 127) / 128) * 128;
    const int bitsetBytes = ((3 * (range / 64) + 3) & ~3) * 4;  // bitset + per-word prefixes
    // two workgroups of twelve waves per CU (registers allow no more): half of the CU's LDS each
    int chunkBytes = (160 * 1024) / 2 - 1024 - bitsetBytes;
    chunkBytes &= ~255;
    const size_t ldsCount = (size_t)(range / 32) * 4;
    const size_t ldsFill = (size_t)bitsetBytes + chunkBytes;
    hipLaunchKernelGGL(clear_header_kernel, dim3(1), dim3(1), 0, stream, hdr);
#define F3S_ONECALL(WW)                                                                        \
  do {                                                                                         \
    if (ldsFill > 64 * 1024)                                                                   \
      F3S_HIP_CHECK(hipFuncSetAttribute(                                                       \
          reinterpret_cast<const void*>(&window_rank_fill_kernel<WW, kRankFillThreads>),                    \
          hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsFill));                          \
    hipLaunchKernelGGL((window_count_kernel<WW, 512>), dim3(nRW), dim3(512), ldsCount, stream, \
                       rowPtr, colIdx, N, range, blockPartition, hdr);                      \
    F3S_HIP_CHECK(hipGetLastError());                                                          \
    if (int rc = enqueue_finalize(N, W, blockPartition, rowWindowOffset, sortedRowWindows, ws, \
                                  stream))                                                     \
      return rc;                                                                               \
    hipLaunchKernelGGL((window_rank_fill_kernel<WW, kRankFillThreads>), dim3(nRW),            \
                       dim3(kRankFillThreads), ldsFill,                                          \
                       stream, rowPtr, colIdx, N, E, range, chunkBytes, rowWindowOffset,       \
                       sortedRowWindows, hdr,                                                  \
                       edgeToColumn, edgeToRow, tcblockRowid, tcblocktileId, tcblockOffset,    \
                       sparseAToXidx, reinterpret_cast<unsigned long long*>(bitmap));          \
    F3S_HIP_CHECK(hipGetLastError());                                                          \
  } while (0)
    if (W == 16) F3S_ONECALL(16); else F3S_ONECALL(8);
#undef F3S_ONECALL
  } else {
    if (int rc = enqueue_count(rowPtr, colIdx, N, E, W, blockPartition, edgeToColumn, edgeToRow,
                               rowWindowOffset, sortedRowWindows, ws, stream))
      return rc;
    if (nRW == 0) {
      hipLaunchKernelGGL(set_tail_kernel, dim3(1), dim3(1), 0, stream, tcblockOffset, 0ll, E);
      F3S_HIP_CHECK(hipGetLastError());
    } else if (int rc = enqueue_fill(rowPtr, colIdx, N, E, W, edgeToColumn, rowWindowOffset, hdr,
                                     tcblockRowid, tcblocktileId, tcblockOffset, sparseAToXidx,
                                     bitmap, stream)) {
      return rc;
    }
  }
  WsHeader host;
  F3S_HIP_CHECK(hipMemcpyAsync(&host, ws, sizeof(WsHeader), hipMemcpyDeviceToHost, stream));
  F3S_HIP_CHECK(hipStreamSynchronize(stream));
  if (host.error) return fail(-4, "f3s_preprocess: column index outside [0, %d)", N);
  *nTcbHost = host.nTcb;
  return 0;
}

}  // namespace f3s
