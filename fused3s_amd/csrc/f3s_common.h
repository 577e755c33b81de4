// Shared declarations of the MI355X Fused3S library (internal; the public C ABI is
// include/f3s_amd.h).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace f3s {

constexpr int kWave = 64;       // CDNA4 wavefront width
constexpr int kWinRows = 16;    // rows per row window (reference BLK_H / BLK_M)

// Head dimensions the attention kernels are built for: every multiple of 32 up to 256 (the
// reference takes embeddingDim at run time, src/F3S_kernel.cu:601-604,1424,1522).
#define F3S_FOR_EACH_HEAD_DIM(X) X(32) X(64) X(96) X(128) X(160) X(192) X(224) X(256)
inline bool head_dim_supported(int d) { return d >= 32 && d <= 256 && d % 32 == 0; }

// 1 when the K/V gathers have to form row offsets in 64 bits: rows of `pitchBytes` bytes whose
// array spans 4 GiB or more, or (pitched rows) a row count or pitch beyond the 24-bit multiply
// of the narrow path.
inline int gather_needs_wide_offsets(int64_t N, int64_t pitchBytes, bool pitched) {
  if (N * pitchBytes >= ((int64_t)1 << 32)) return 1;
  if (pitched && (N >= (1 << 24) || pitchBytes >= (1 << 24))) return 1;
  return 0;
}

// Records a message retrievable through f3s_last_error() and returns `code`.
int fail(int code, const char* fmt, ...);

#define F3S_HIP_CHECK(expr)                                                          \
  do {                                                                               \
    hipError_t e__ = (expr);                                                         \
    if (e__ != hipSuccess)                                                           \
      return ::f3s::fail(-100, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e__), \
                         __FILE__, __LINE__);                                        \
  } while (0)

// attention (f3s_attention.hip)
int launch_attention(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                     const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int64_t nTcb,
                     int d, int dtype, const void* Q, const void* K, const void* V,
                     float scalingFactor, int applySoftmax, float* out,
                     unsigned long long* cuTimer, void* workspace, size_t wsBytes, int prepared,
                     hipStream_t stream);

int launch_attention_heads(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                           const int32_t* sparseAToXidx, const uint64_t* bitmap, int N,
                           int64_t nTcb, int nHeads, int d, int dtype, const void* Q, const void* K,
                           const void* V, int64_t ldIn, float scalingFactor, int applySoftmax,
                           float* out, int64_t ldOut, void* workspace, size_t wsBytes,
                           int prepared, hipStream_t stream);

int launch_attention_prepare(const int32_t* rowWindowOffset, const int32_t* sparseAToXidx, int N,
                             int64_t nTcb, int d, int nHeads, void* workspace, size_t wsBytes,
                             hipStream_t stream);

int launch_attention_tcb8(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                          const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int d,
                          const void* Q, const void* K, const void* V, int applySoftmax,
                          float* out, float* sddmm, int64_t nTcb8, hipStream_t stream);

int attention_uses_workspace(int N, int64_t nTcb, int d, int dtype);

// column-sliced schedule (f3s_attention_units.hip)
// nHeads = 0: contiguous single head. mode 0: attention call; 1: build the slice index only;
// 2: attention call on a prepared workspace
size_t attention_sliced_workspace_bytes(int N, int d, int nHeads);
int launch_attention_sliced(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                            const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int d,
                            int dtype, const void* Q, const void* K, const void* V,
                            float scaleLog2, int applySoftmax, float* out, void* workspace,
                            size_t wsBytes, int64_t nTcb, int nHeads, int ldIn, int ldOut,
                            int mode, hipStream_t stream);

int launch_attention_short_windows(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                                   const int32_t* sparseAToXidx, const uint64_t* bitmap, int N,
                                   int d, int dtype, const void* Q, const void* K, const void* V,
                                   float scaleLog2, int applySoftmax, float* out, int nHeads,
                                   int ldIn, int ldOut, int maxBlocks, int longPrefix,
                                   int64_t nTcb, hipStream_t stream);

// The workgroup-per-window kernel built with 64-bit row offsets in its gathers, for K / V of
// 4 GiB and more (f3s_attention_wide.hip). nHeads = 0: contiguous single head.
int launch_window_wide(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                       const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int d,
                       int dtype, const void* Q, const void* K, const void* V, float scaleLog2,
                       int applySoftmax, float* out, unsigned long long* cuTimer, int nHeads,
                       int ldIn, int ldOut, int64_t nTcb, hipStream_t stream);
int launch_tcb8_wide(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                     const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int d,
                     const void* Q, const void* K, const void* V, float scaleLog2,
                     int applySoftmax, float* out, float* sddmm, int64_t nTcb8,
                     hipStream_t stream);

// preprocessing (f3s_preprocess.hip)
size_t preprocess_workspace_bytes(int N, int E);
int launch_preprocess_count(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int H,
                            int W, int32_t* blockPartition, int32_t* edgeToColumn,
                            int32_t* edgeToRow, int32_t* rowWindowOffset,
                            int32_t* sortedRowWindows, void* workspace, size_t wsBytes,
                            int64_t* nTcbHost, hipStream_t stream);
size_t preprocess_static_scratch_bytes();
int launch_preprocess_count_static(const int32_t* rowPtr, const int32_t* colIdx, int N, int E,
                                   int H, int W, int32_t* blockPartition, int32_t* edgeToColumn,
                                   int32_t* edgeToRow, int32_t* rowWindowOffset,
                                   int32_t* sortedRowWindows, int64_t* resultDev,
                                   hipStream_t stream);
int launch_preprocess_fill(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int H,
                           int W, const int32_t* edgeToColumn, const int32_t* rowWindowOffset,
                           int64_t nTcb, int32_t* tcblockRowid, uint8_t* tcblocktileId,
                           int32_t* tcblockOffset, int32_t* sparseAToXidx, uint64_t* bitmap,
                           hipStream_t stream);

int64_t preprocess_capacity(int N, int64_t E, int W);
int launch_preprocess(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int H, int W,
                      int32_t* blockPartition, int32_t* edgeToColumn, int32_t* edgeToRow,
                      int32_t* rowWindowOffset, int32_t* sortedRowWindows, int64_t capacity,
                      int32_t* tcblockRowid, uint8_t* tcblocktileId, int32_t* tcblockOffset,
                      int32_t* sparseAToXidx, uint64_t* bitmap, void* workspace, size_t wsBytes,
                      int64_t* nTcbHost, hipStream_t stream);

}  // namespace f3s
