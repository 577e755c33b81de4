// Launchers of every attention entry point of the MI355X Fused3S library (gfx950): argument
// rules, the choice of schedule (workgroup per window, wave per short window, column-sliced
// units), and the hand-off to the kernels with 64-bit row offsets for K / V of 4 GiB and more.
// The kernel with one workgroup per window is f3s_window_kernel.h; this translation unit builds
// it with 32-bit row offsets.
#include <stdlib.h>
#include <string.h>

#include "f3s_common.h"
#include "f3s_window_kernel.h"

namespace f3s {

using pipe::kLog2e;
using window::HeadLayout;


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
  const char* e = getenv("F3S_SHORT_WINDOWS");  // read per call, like every other switch
  const bool off = e && strcmp(e, "0") == 0;
  if (off || !windowOrder || nRW < 1024 || nTcb >= (int64_t)16 * nRW) return false;
  hl->minBlocks = kShortWindowBlocks;
  const int64_t longMax = nTcb / (kShortWindowBlocks + 1) + 1;
  hl->gridWindows = (int)(longMax < nRW ? longMax : nRW);
  return true;
}

// The column-sliced schedule (f3s_attention_units.hip: (window, column slice) units, every XCD
// on one slice at a time so that its K/V rows stay in that XCD's L2, plus a merge kernel) pays off
// on graphs with long windows: on the 233k-node benchmark graph (450 TC blocks per window) it
// takes 1.54 ms at d = 64 against 2.48 ms for the workgroup-per-window kernel, with 7.1 GB
// instead of 17.7 GB of traffic beyond L2.
// Short windows would be cut into units of one or two blocks; they keep the window kernel.
// F3S_SCHEDULE=window / =sliced in the environment overrides the choice.
int attention_uses_workspace(int N, int64_t nTcb, int d, int dtype) {
  const char* e = getenv("F3S_SCHEDULE");  // read per call
  const int forced = (e && strcmp(e, "sliced") == 0) ? 1 : (e && strcmp(e, "window") == 0) ? -1 : 0;
  if ((dtype != 0 && dtype != 1) || !head_dim_supported(d) || N <= 0) return 0;
  if (forced) return forced > 0;
  const int64_t nRW = ((int64_t)N + kWinRows - 1) / kWinRows;
  return nRW >= 2048 && nTcb >= 64 * nRW;
}

int launch_attention(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                     const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int64_t nTcb,
                     int d, int dtype, const void* Q, const void* K, const void* V,
                     float scalingFactor, int applySoftmax, float* out,
                     unsigned long long* cuTimer, void* workspace, size_t wsBytes, int prepared,
                     hipStream_t stream) {
  if (dtype != 0 && dtype != 1)
    return fail(-3, "f3s_attention_fwd: dtype %d not supported (0 = fp16, 1 = bf16)", dtype);
  if (scalingFactor == 0.0f) return fail(-2, "f3s_attention_fwd: scalingFactor must be non-zero");
  if (!head_dim_supported(d))
    return fail(-2, "f3s_attention_fwd: head dim %d unsupported (a multiple of 32 up to 256)", d);
  // the reference divides unmasked scores by scalingFactor (src/F3S_kernel.cu:1666-1667);
  // exponentials are taken in base 2, so log2(e) is folded into the same multiplier
  const float scaleLog2 = applySoftmax ? kLog2e / scalingFactor : 1.0f;
  // K / V of 4 GiB and more: every window goes to the window kernel built with 64-bit row
  // offsets (the other schedules exist with 32-bit offsets only)
  if (gather_needs_wide_offsets(N, (int64_t)d * 2, false))
    return launch_window_wide(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, d, dtype, Q,
                              K, V, scaleLog2, applySoftmax, out, cuTimer, 0, d, d, nTcb, stream);
  if (workspace && !cuTimer && attention_uses_workspace(N, nTcb, d, dtype))
    return launch_attention_sliced(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, d, dtype,
                                   Q, K, V, scaleLog2, applySoftmax, out, workspace, wsBytes,
                                   nTcb, 0, d, d, prepared ? 2 : 0, stream);
  const int nRWi = (N + kWinRows - 1) / kWinRows;
  HeadLayout single = {0, d, d, -1, nRWi, nTcb};
  if (!cuTimer && split_short_windows(windowOrder, nRWi, nTcb, &single)) {
    const int rc = launch_attention_short_windows(rowWindowOffset, windowOrder, sparseAToXidx,
                                                  bitmap, N, d, dtype, Q, K, V, scaleLog2,
                                                  applySoftmax, out, 0, d, d, kShortWindowBlocks,
                                                  single.gridWindows, nTcb, stream);
    if (rc != 0) return rc;
  }
  return dtype == 0 ? window::dispatch_d<_Float16, false>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N,
                                           d, Q, K, V, scaleLog2, applySoftmax, out, cuTimer,
                                           single, stream)
                    : window::dispatch_d<__bf16, false>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, d,
                                         Q, K, V, scaleLog2, applySoftmax, out, cuTimer, single,
                                         stream);
}

// Builds the column-sliced schedule's index (slice boundaries) in `workspace` and marks it as
// belonging to these arrays, so that attention calls with the same arrays skip that step.
// nHeads = 0: the single-head layout.
int launch_attention_prepare(const int32_t* rowWindowOffset, const int32_t* sparseAToXidx, int N,
                             int64_t nTcb, int d, int nHeads, void* workspace, size_t wsBytes,
                             hipStream_t stream) {
  if (!head_dim_supported(d))
    return fail(-2, "f3s_attention_prepare: head dim %d unsupported (a multiple of 32 up to 256)",
                d);
  if (nHeads < 0 || nHeads > 1024)
    return fail(-2, "f3s_attention_prepare: nHeads %d out of range (0..1024)", nHeads);
  return launch_attention_sliced(rowWindowOffset, nullptr, sparseAToXidx, nullptr, N, d, 0,
                                 nullptr, nullptr, nullptr, 1.0f, 1, nullptr, workspace, wsBytes,
                                 nTcb, nHeads, nHeads * d, nHeads * d, 1, stream);
}

int launch_attention_tcb8(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                          const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int d,
                          const void* Q, const void* K, const void* V, int applySoftmax,
                          float* out, float* sddmm, int64_t nTcb8, hipStream_t stream) {
  // this path has no score scaling (src/F3S_kernel.cu:709-735)
  const float scaleLog2 = applySoftmax ? kLog2e : 1.0f;
  if (gather_needs_wide_offsets(N, (int64_t)d * 2, false))
    return launch_tcb8_wide(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, d, Q, K, V,
                            scaleLog2, applySoftmax, out, sddmm, nTcb8, stream);
#define F3S_DISPATCH(DD)                                                                      \
  if (d == DD)                                                                                \
    return applySoftmax                                                                       \
               ? window::launch_tcb8<DD, true, false>(rowWindowOffset, windowOrder,           \
                                                      sparseAToXidx, bitmap, N, Q, K, V,      \
                                                      scaleLog2, out, sddmm, nTcb8, stream)   \
               : window::launch_tcb8<DD, false, false>(rowWindowOffset, windowOrder,          \
                                                       sparseAToXidx, bitmap, N, Q, K, V,     \
                                                       scaleLog2, out, sddmm, nTcb8, stream);
  F3S_FOR_EACH_HEAD_DIM(F3S_DISPATCH)
#undef F3S_DISPATCH
  return fail(-2, "f3s_attention_fwd_tcb8: head dim %d unsupported (a multiple of 32 up to 256)",
              d);
}

int launch_attention_heads(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                           const int32_t* sparseAToXidx, const uint64_t* bitmap, int N,
                           int64_t nTcb, int nHeads, int d, int dtype, const void* Q, const void* K,
                           const void* V, int64_t ldIn, float scalingFactor, int applySoftmax,
                           float* out, int64_t ldOut, void* workspace, size_t wsBytes,
                           int prepared, hipStream_t stream) {
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
  if (!head_dim_supported(d))
    return fail(-2, "f3s_attention_fwd_heads: head dim %d unsupported (a multiple of 32 up to 256)",
                d);
  if (ldIn >= ((int64_t)1 << 31) || ldOut >= ((int64_t)1 << 31))
    return fail(-2, "f3s_attention_fwd_heads: row pitches must be below 2^31 elements");
  const int64_t nRW = ((int64_t)N + kWinRows - 1) / kWinRows;
  if (nRW * nHeads >= ((int64_t)1 << 31))
    return fail(-2, "f3s_attention_fwd_heads: too many (window, head) workgroups");
  const float scaleLog2 = applySoftmax ? kLog2e / scalingFactor : 1.0f;
  if (gather_needs_wide_offsets(N, ldIn * 2, true))
    return launch_window_wide(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, d, dtype, Q,
                              K, V, scaleLog2, applySoftmax, out, nullptr, nHeads, (int)ldIn,
                              (int)ldOut, nTcb, stream);
  if (workspace && attention_uses_workspace(N, nTcb, d, dtype))
    return launch_attention_sliced(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, d, dtype,
                                   Q, K, V, scaleLog2, applySoftmax, out, workspace, wsBytes,
                                   nTcb, nHeads, (int)ldIn, (int)ldOut, prepared ? 2 : 0, stream);
  HeadLayout hl = {nHeads, (int)ldIn, (int)ldOut, -1, (int)nRW, nTcb};
  if (split_short_windows(windowOrder, (int)nRW, nTcb, &hl)) {
    const int rc = launch_attention_short_windows(rowWindowOffset, windowOrder, sparseAToXidx,
                                                  bitmap, N, d, dtype, Q, K, V, scaleLog2,
                                                  applySoftmax, out, nHeads, (int)ldIn, (int)ldOut,
                                                  kShortWindowBlocks, hl.gridWindows, nTcb,
                                                  stream);
    if (rc != 0) return rc;
  }
  return dtype == 0 ? window::dispatch_d<_Float16, false>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N,
                                           d, Q, K, V, scaleLog2, applySoftmax, out, nullptr, hl,
                                           stream)
                    : window::dispatch_d<__bf16, false>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap, N, d,
                                         Q, K, V, scaleLog2, applySoftmax, out, nullptr, hl,
                                         stream);
}

}  // namespace f3s
