// The workgroup-per-window attention kernel (f3s_window_kernel.h) built with 64-bit row offsets in
// its K / V gathers: for arrays of 4 GiB and more, and for pitched multi-head layouts whose row
// count or pitch exceeds the 24-bit multiply of the narrow kernels. The reference indexes rows
// with int64_t throughout (src/F3S_kernel.cu:1422-1423). Every window of such a problem is
// computed by this kernel (no column-sliced units, no wave-per-window split): a translation unit
// of its own, so that the common kernels do not carry a second address form.
#include "f3s_common.h"
#include "f3s_window_kernel.h"

namespace f3s {

int launch_window_wide(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                       const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int d,
                       int dtype, const void* Q, const void* K, const void* V, float scaleLog2,
                       int applySoftmax, float* out, unsigned long long* cuTimer, int nHeads,
                       int ldIn, int ldOut, int64_t nTcb, hipStream_t stream) {
  const int nRW = (N + kWinRows - 1) / kWinRows;
  const window::HeadLayout hl = {nHeads, ldIn, ldOut, -1, nRW, nTcb};
  return dtype == 0
             ? window::dispatch_d<_Float16, true>(rowWindowOffset, windowOrder, sparseAToXidx,
                                                  bitmap, N, d, Q, K, V, scaleLog2, applySoftmax,
                                                  out, cuTimer, hl, stream)
             : window::dispatch_d<__bf16, true>(rowWindowOffset, windowOrder, sparseAToXidx, bitmap,
                                                N, d, Q, K, V, scaleLog2, applySoftmax, out,
                                                cuTimer, hl, stream);
}

int launch_tcb8_wide(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                     const int32_t* sparseAToXidx, const uint64_t* bitmap, int N, int d,
                     const void* Q, const void* K, const void* V, float scaleLog2,
                     int applySoftmax, float* out, float* sddmm, int64_t nTcb8,
                     hipStream_t stream) {
#define F3S_DISPATCH(DD)                                                                      \
  if (d == DD)                                                                                \
    return applySoftmax                                                                       \
               ? window::launch_tcb8<DD, true, true>(rowWindowOffset, windowOrder,            \
                                                     sparseAToXidx, bitmap, N, Q, K, V,       \
                                                     scaleLog2, out, sddmm, nTcb8, stream)    \
               : window::launch_tcb8<DD, false, true>(rowWindowOffset, windowOrder,           \
                                                      sparseAToXidx, bitmap, N, Q, K, V,      \
                                                      scaleLog2, out, sddmm, nTcb8, stream);
  F3S_FOR_EACH_HEAD_DIM(F3S_DISPATCH)
#undef F3S_DISPATCH
  return fail(-2, "f3s_attention_fwd_tcb8: head dim %d unsupported (a multiple of 32 up to 256)",
              d);
}

}  // namespace f3s
