// C ABI of libf3s_amd.so (declared in include/f3s_amd.h): argument checks, error text,
// dispatch into the HIP launchers.
#include <stdarg.h>
#include <stdio.h>

#include "../../include/f3s_amd.h"
#include "f3s_common.h"

namespace f3s {
namespace {
thread_local char g_error[512] = "";
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

namespace {
bool misaligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }
}  // namespace
}  // namespace f3s

extern "C" {

int f3s_abi_version(void) { return 2; }

const char* f3s_last_error(void) { return f3s::g_error; }

size_t f3s_preprocess_workspace_bytes(int N, int E) {
  if (N < 0) N = 0;
  return f3s::preprocess_workspace_bytes(N, E);
}

int f3s_preprocess_count(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int H, int W,
                         int32_t* blockPartition, int32_t* edgeToColumn, int32_t* edgeToRow,
                         int32_t* rowWindowOffset, int32_t* sortedRowWindows, void* workspace,
                         size_t ws_bytes, int64_t* nTCB_host, void* stream) {
  if (!rowPtr || !rowWindowOffset || !workspace || !nTCB_host)
    return f3s::fail(-1, "f3s_preprocess_count: null pointer");
  if (N > 0 && (!blockPartition || !sortedRowWindows))
    return f3s::fail(-1, "f3s_preprocess_count: null window output");
  if (E > 0 && (!colIdx || !edgeToColumn || !edgeToRow))
    return f3s::fail(-1, "f3s_preprocess_count: null edge array");
  if (f3s::misaligned(workspace, 256))
    return f3s::fail(-1, "f3s_preprocess_count: workspace must be 256-byte aligned");
  return f3s::launch_preprocess_count(rowPtr, colIdx, N, E, H, W, blockPartition, edgeToColumn,
                                      edgeToRow, rowWindowOffset, sortedRowWindows, workspace,
                                      ws_bytes, nTCB_host, static_cast<hipStream_t>(stream));
}

size_t f3s_preprocess_static_scratch_bytes(void) { return f3s::preprocess_static_scratch_bytes(); }

int f3s_preprocess_count_static(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int H,
                                int W, int32_t* blockPartition, int32_t* edgeToColumn,
                                int32_t* edgeToRow, int32_t* rowWindowOffset,
                                int32_t* sortedRowWindows, int64_t* result_dev, void* stream) {
  if (!rowPtr || !rowWindowOffset || !result_dev)
    return f3s::fail(-1, "f3s_preprocess_count_static: null pointer");
  if (N > 0 && (!blockPartition || !sortedRowWindows))
    return f3s::fail(-1, "f3s_preprocess_count_static: null window output");
  if (E > 0 && (!colIdx || !edgeToColumn || !edgeToRow))
    return f3s::fail(-1, "f3s_preprocess_count_static: null edge array");
  if (f3s::misaligned(result_dev, 8))
    return f3s::fail(-1, "f3s_preprocess_count_static: result_dev must be 8-byte aligned");
  return f3s::launch_preprocess_count_static(rowPtr, colIdx, N, E, H, W, blockPartition,
                                             edgeToColumn, edgeToRow, rowWindowOffset,
                                             sortedRowWindows, result_dev,
                                             static_cast<hipStream_t>(stream));
}

int f3s_preprocess_fill(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int H, int W,
                        const int32_t* edgeToColumn, const int32_t* rowWindowOffset, int64_t nTCB,
                        int32_t* tcblockRowid, uint8_t* tcblocktileId, int32_t* tcblockOffset,
                        int32_t* sparseAToXidx, uint64_t* tcbBitMap, void* stream) {
  if (!rowPtr || !rowWindowOffset || !tcblockOffset)
    return f3s::fail(-1, "f3s_preprocess_fill: null pointer");
  if (nTCB < 0 || N < 0 || E < 0) return f3s::fail(-2, "f3s_preprocess_fill: negative size");
  if (nTCB > 0 && (!tcblockRowid || !sparseAToXidx || !tcbBitMap || !colIdx || !edgeToColumn ||
                   !tcblocktileId))
    return f3s::fail(-1, "f3s_preprocess_fill: null output");
  if (f3s::misaligned(tcbBitMap, 16) || f3s::misaligned(sparseAToXidx, 16))
    return f3s::fail(-1, "f3s_preprocess_fill: tcbBitMap and sparseAToXidx must be 16-byte "
                         "aligned (the attention kernels fetch them 16 bytes per lane)");
  return f3s::launch_preprocess_fill(rowPtr, colIdx, N, E, H, W, edgeToColumn, rowWindowOffset,
                                     nTCB, tcblockRowid, tcblocktileId, tcblockOffset,
                                     sparseAToXidx, tcbBitMap, static_cast<hipStream_t>(stream));
}

int64_t f3s_preprocess_capacity(int N, int64_t E, int W) {
  if (N < 0) N = 0;
  if (E < 0) E = 0;
  if (W != 8) W = 16;
  return f3s::preprocess_capacity(N, E, W);
}

int f3s_preprocess(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int H, int W,
                   int32_t* blockPartition, int32_t* edgeToColumn, int32_t* edgeToRow,
                   int32_t* rowWindowOffset, int32_t* sortedRowWindows, int64_t capacity,
                   int32_t* tcblockRowid, uint8_t* tcblocktileId, int32_t* tcblockOffset,
                   int32_t* sparseAToXidx, uint64_t* tcbBitMap, void* workspace, size_t ws_bytes,
                   int64_t* nTCB_host, void* stream) {
  if (!rowPtr || !rowWindowOffset || !workspace || !nTCB_host || !tcblockOffset)
    return f3s::fail(-1, "f3s_preprocess: null pointer");
  if (N > 0 && (!blockPartition || !sortedRowWindows))
    return f3s::fail(-1, "f3s_preprocess: null window output");
  if (E > 0 && (!colIdx || !edgeToColumn || !edgeToRow || !tcblocktileId || !tcblockRowid ||
                !sparseAToXidx || !tcbBitMap))
    return f3s::fail(-1, "f3s_preprocess: null edge or block array");
  if (f3s::misaligned(workspace, 256))
    return f3s::fail(-1, "f3s_preprocess: workspace must be 256-byte aligned");
  if (f3s::misaligned(tcbBitMap, 16) || f3s::misaligned(sparseAToXidx, 16))
    return f3s::fail(-1, "f3s_preprocess: tcbBitMap and sparseAToXidx must be 16-byte aligned "
                         "(the attention kernels fetch them 16 bytes per lane)");
  return f3s::launch_preprocess(rowPtr, colIdx, N, E, H, W, blockPartition, edgeToColumn,
                                edgeToRow, rowWindowOffset, sortedRowWindows, capacity,
                                tcblockRowid, tcblocktileId, tcblockOffset, sparseAToXidx,
                                tcbBitMap, workspace, ws_bytes, nTCB_host,
                                static_cast<hipStream_t>(stream));
}

size_t f3s_attention_workspace_bytes(int N, int d) {
  if (N < 0) N = 0;
  if (d < 32) d = 32;
  return f3s::attention_sliced_workspace_bytes(N, d, 0);
}

size_t f3s_attention_heads_workspace_bytes(int N, int nHeads, int d) {
  if (N < 0) N = 0;
  if (d < 32) d = 32;
  if (nHeads < 1) nHeads = 1;
  return f3s::attention_sliced_workspace_bytes(N, d, nHeads);
}

int f3s_attention_uses_workspace(int N, int64_t nTCB, int d, int dtype) {
  return f3s::attention_uses_workspace(N, nTCB, d, dtype);
}

int f3s_attention_uses_wide_offsets(int64_t N, int64_t pitch_bytes, int pitched) {
  if (N < 0 || pitch_bytes < 0) return 0;
  return f3s::gather_needs_wide_offsets(N, pitch_bytes, pitched != 0);
}

int f3s_attention_prepare(const int32_t* rowWindowOffset, const int32_t* sparseAToXidx, int N,
                          int64_t nTCB, int d, int nHeads, void* workspace, size_t ws_bytes,
                          void* stream) {
  if (N <= 0 || nTCB < 0) return f3s::fail(-2, "f3s_attention_prepare: N must be positive");
  if (!rowWindowOffset || !workspace || (nTCB > 0 && !sparseAToXidx))
    return f3s::fail(-1, "f3s_attention_prepare: null pointer");
  if (f3s::misaligned(workspace, 256) || f3s::misaligned(sparseAToXidx, 16))
    return f3s::fail(-1, "f3s_attention_prepare: workspace needs 256-byte, sparseAToXidx 16-byte "
                         "alignment");
  return f3s::launch_attention_prepare(rowWindowOffset, sparseAToXidx, N, nTCB, d, nHeads,
                                       workspace, ws_bytes,
                                       static_cast<hipStream_t>(stream));
}

int f3s_attention_fwd(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                      const int32_t* sparseAToXidx, const uint64_t* tcbBitMap, int N, int64_t nTCB,
                      int d, int dtype, const void* Q, const void* K, const void* V,
                      float scalingFactor, int applySoftmax, float* out,
                      unsigned long long* cuTimer, void* workspace, size_t ws_bytes, int prepared,
                      void* stream) {
  if (N < 0) return f3s::fail(-2, "f3s_attention_fwd: negative N");
  if (N == 0) return 0;
  if (!rowWindowOffset || !Q || !K || !V || !out)
    return f3s::fail(-1, "f3s_attention_fwd: null pointer");
  if (f3s::misaligned(Q, 16) || f3s::misaligned(K, 16) || f3s::misaligned(V, 16) ||
      f3s::misaligned(out, 16) || f3s::misaligned(sparseAToXidx, 16) ||
      f3s::misaligned(tcbBitMap, 16))
    return f3s::fail(-1, "f3s_attention_fwd: Q/K/V/out/sparseAToXidx/tcbBitMap need 16-byte "
                         "alignment");
  if (nTCB < 0) return f3s::fail(-2, "f3s_attention_fwd: negative nTCB");
  if (nTCB > 0 && (!sparseAToXidx || !tcbBitMap))
    return f3s::fail(-1, "f3s_attention_fwd: null TC-block arrays");
  if (workspace && f3s::misaligned(workspace, 256))
    return f3s::fail(-1, "f3s_attention_fwd: workspace must be 256-byte aligned");
  return f3s::launch_attention(rowWindowOffset, windowOrder, sparseAToXidx, tcbBitMap, N, nTCB, d,
                               dtype, Q, K, V, scalingFactor, applySoftmax, out, cuTimer,
                               workspace, ws_bytes, prepared, static_cast<hipStream_t>(stream));
}

int f3s_attention_fwd_heads(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                            const int32_t* sparseAToXidx, const uint64_t* tcbBitMap, int N,
                            int64_t nTCB, int nHeads, int d, int dtype, const void* Q,
                            const void* K, const void* V, int64_t ldIn, float scalingFactor,
                            int applySoftmax, float* out, int64_t ldOut, void* workspace,
                            size_t ws_bytes, int prepared, void* stream) {
  if (N < 0) return f3s::fail(-2, "f3s_attention_fwd_heads: negative N");
  if (N == 0) return 0;
  if (!rowWindowOffset || !Q || !K || !V || !out)
    return f3s::fail(-1, "f3s_attention_fwd_heads: null pointer");
  if (f3s::misaligned(Q, 16) || f3s::misaligned(K, 16) || f3s::misaligned(V, 16) ||
      f3s::misaligned(out, 16) || f3s::misaligned(sparseAToXidx, 16) ||
      f3s::misaligned(tcbBitMap, 16))
    return f3s::fail(-1, "f3s_attention_fwd_heads: Q/K/V/out/sparseAToXidx/tcbBitMap need "
                         "16-byte alignment");
  if (nTCB < 0) return f3s::fail(-2, "f3s_attention_fwd_heads: negative nTCB");
  if (nTCB > 0 && (!sparseAToXidx || !tcbBitMap))
    return f3s::fail(-1, "f3s_attention_fwd_heads: null TC-block arrays");
  if (workspace && f3s::misaligned(workspace, 256))
    return f3s::fail(-1, "f3s_attention_fwd_heads: workspace must be 256-byte aligned");
  return f3s::launch_attention_heads(rowWindowOffset, windowOrder, sparseAToXidx, tcbBitMap, N,
                                     nTCB, nHeads, d, dtype, Q, K, V, ldIn, scalingFactor,
                                     applySoftmax, out, ldOut, workspace, ws_bytes, prepared,
                                     static_cast<hipStream_t>(stream));
}

int f3s_attention_fwd_tcb8(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                           const int32_t* sparseAToXidx, const uint64_t* tcbBitMap, int N,
                           int64_t nTCB, int d, const void* Q, const void* K, const void* V,
                           int applySoftmax, float* out, float* sddmmResult, void* stream) {
  if (N < 0) return f3s::fail(-2, "f3s_attention_fwd_tcb8: negative N");
  if (N == 0) return 0;
  if (!rowWindowOffset || !Q || !K || !V || !out)
    return f3s::fail(-1, "f3s_attention_fwd_tcb8: null pointer");
  if (f3s::misaligned(Q, 16) || f3s::misaligned(K, 16) || f3s::misaligned(V, 16) ||
      f3s::misaligned(out, 16) || f3s::misaligned(sparseAToXidx, 16) ||
      f3s::misaligned(tcbBitMap, 16) || f3s::misaligned(sddmmResult, 16))
    return f3s::fail(-1, "f3s_attention_fwd_tcb8: Q/K/V/out/sparseAToXidx/tcbBitMap/sddmmResult "
                         "need 16-byte alignment");
  if (nTCB < 0) return f3s::fail(-2, "f3s_attention_fwd_tcb8: negative nTCB");
  if (nTCB > 0 && (!sparseAToXidx || !tcbBitMap))
    return f3s::fail(-1, "f3s_attention_fwd_tcb8: null TC-block arrays");
  return f3s::launch_attention_tcb8(rowWindowOffset, windowOrder, sparseAToXidx, tcbBitMap, N, d,
                                    Q, K, V, applySoftmax, out, sddmmResult, nTCB,
                                    static_cast<hipStream_t>(stream));
}

}  // extern "C"
