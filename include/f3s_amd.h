/*
 * f3s_amd.h -- C ABI of the MI355X (gfx950) Fused3S library, libf3s_amd.so.
 *
 * Plain pointers and sizes only. Unless stated otherwise every pointer is DEVICE memory on the
 * current HIP device, int32 arrays are 4-byte aligned, sparseAToXidx / tcbBitMap / Q / K / V / out are
 * 16-byte aligned, and `stream` is a hipStream_t passed as void* (NULL = default stream).
 * Every entry point returns 0 on success and a negative code on failure; the message is then
 * available from f3s_last_error() (per thread). Nothing here calls exit(): the reference's
 * printf + exit(-1) error path (src/utils.cu:72-77, src/F3S_kernel.cu:662-666) becomes a status.
 *
 * Citations are to the HPCForge/Fused3S sources each entry point replaces.
 */
#ifndef F3S_AMD_H
#define F3S_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define F3S_DTYPE_F16 0
#define F3S_DTYPE_BF16 1

/* ABI version of this header (bumped on incompatible change). */
int f3s_abi_version(void);

/* Message of the last failure on the calling thread ("" if none). Never NULL. */
const char* f3s_last_error(void);

/*
 * Bytes of device scratch f3s_preprocess_count needs for a graph of N nodes and E edges.
 * Replaces the thrust::device_vector temporaries of seg_sort_dequ and
 * sort_row_windows_by_tcb_count (src/utils.cu:281-284, 297-298, 404-405): the caller owns
 * the allocation instead of the library.
 */
size_t f3s_preprocess_workspace_bytes(int N, int E);

/*
 * Phase 1 of F3S.preprocess_gpu (src/F3S.cpp:40-87): everything whose size is known up front.
 * Replaces fill_edgeToRow_cuda (src/utils.cu:343-368, with edgeToRow[e] = row(e) for every
 * edge -- the reference's grid-stride slip at :348 is not reproduced), fill_segment_cuda +
 * thrust::sort + generate_edgetocolumn_cuda (src/utils.cu:371-396, 281-292, 131-170), the
 * inclusive scan into rowWindowOffset (src/utils.cu:293-300) and
 * sort_row_windows_by_tcb_count (src/utils.cu:400-436; equal counts keep ascending window id).
 *
 *   rowPtr  [N+1], colIdx [E]      CSR, int32; columns of a row may be unsorted or repeated
 *   H, W                           TC-block height (16) and width (16, or 8 for the 16x8 layout)
 *   blockPartition   [ceil(N/H)]   out: TC blocks per row window
 *   edgeToColumn     [E]           out: rank of the edge's column among the window's sorted
 *                                  unique columns
 *   edgeToRow        [E]           out: row of each edge
 *   rowWindowOffset  [ceil(N/H)+1] out: exclusive prefix of blockPartition
 *   sortedRowWindows [ceil(N/H)]   out: windows by descending TC-block count
 *   workspace, ws_bytes            device scratch of f3s_preprocess_workspace_bytes(N, E)
 *   nTCB_host                      HOST pointer, out: total TC blocks (the reference's D->H
 *                                  copy at src/utils.cu:307-309); the call synchronises `stream`
 * Outputs are fully written; they need not be zeroed by the caller.
 */
int f3s_preprocess_count(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int H, int W,
                         int32_t* blockPartition, int32_t* edgeToColumn, int32_t* edgeToRow,
                         int32_t* rowWindowOffset, int32_t* sortedRowWindows, void* workspace,
                         size_t ws_bytes, int64_t* nTCB_host, void* stream);

/*
 * f3s_preprocess_count for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference. Same
 * inputs and outputs as f3s_preprocess_count, with two differences:
 *   - the scratch is a buffer the library owns, a static device array of
 *     f3s_preprocess_static_scratch_bytes() = 8 MiB per GPU that lives until the process ends;
 *     graphs needing more (f3s_preprocess_workspace_bytes(N, E) > 8 MiB, i.e. above about
 *     10.7 million nodes) are rejected with status -5 and a message;
 *   - nothing is copied to the host and the stream is not synchronised: result_dev is a DEVICE
 *     pointer to two int64, out: {total TC blocks, 1 if a column index lay outside [0, N) else 0}.
 * The call makes no hipMalloc / hipFree and uses no allocating library routine; everything is
 * enqueued on `stream` (kernels only, no memset nodes). Every call on a GPU shares that GPU's
 * buffer: calls that overlap on one GPU (different streams, different threads) race; calls that
 * follow each other on one stream, or are otherwise ordered, are safe, and each call clears what
 * it needs cleared. The first call on a device looks up the buffer's address
 * (hipGetSymbolAddress) and may set a kernel attribute (hipFuncSetAttribute): make that call
 * outside stream capture; the calls after it only launch kernels.
 */
size_t f3s_preprocess_static_scratch_bytes(void);
int f3s_preprocess_count_static(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int H,
                                int W, int32_t* blockPartition, int32_t* edgeToColumn,
                                int32_t* edgeToRow, int32_t* rowWindowOffset,
                                int32_t* sortedRowWindows, int64_t* result_dev, void* stream);

/*
 * Phase 2 of F3S.preprocess_gpu: the outputs sized by nTCB. Replaces
 * generate_tcblock_rowid_cuda (src/utils.cu:53-78), generate_tcoffset_id_atob_cuda with
 * update_bitmap (src/utils.cu:23-36, 173-267) and the inclusive scan into tcblock_offset
 * (src/utils.cu:333-337). No limit on TC blocks per window (the reference exits above
 * 25 599, src/utils.cu:235-239).
 *
 *   edgeToColumn, rowWindowOffset  as produced by f3s_preprocess_count
 *   tcblockRowid   [nTCB]          out: row window of each TC block
 *   tcblocktileId  [E]  (uint8)    out: row_local*W + col_local, grouped by TC block, CSR order
 *   tcblockOffset  [nTCB+1]        out: exclusive prefix of per-block nnz
 *   sparseAToXidx  [nTCB*W]        out: original column of each compacted slot, 0 when unused
 *   tcbBitMap      [nTCB*H*W/64] (uint64)  out: 8x8 sub-blocks in column-major order,
 *                                  row-major and MSB-first inside a sub-block
 * sparseAToXidx and tcbBitMap must be 16-byte aligned (here and in f3s_preprocess), as the
 * attention entry points require of them.
 * Asynchronous on `stream`. Outputs are fully written.
 */
int f3s_preprocess_fill(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int H, int W,
                        const int32_t* edgeToColumn, const int32_t* rowWindowOffset, int64_t nTCB,
                        int32_t* tcblockRowid, uint8_t* tcblocktileId, int32_t* tcblockOffset,
                        int32_t* sparseAToXidx, uint64_t* tcbBitMap, void* stream);

/*
 * All of F3S.preprocess_gpu (src/F3S.cpp:40-87) behind one call, for callers that size the
 * nTCB-long outputs by an upper bound instead of waiting for the count: both phases are enqueued
 * back to back and the host reads the block total once, at the end. The reference allocates its
 * block arrays between the phases (src/F3S.cpp:62-70 around the copy at src/utils.cu:307-309);
 * a caller of this entry allocates them for f3s_preprocess_capacity(N, E, W) blocks beforehand
 * and uses the first nTCB entries.
 *
 *   capacity       TC blocks the four nTCB-sized arrays below have room for; at least
 *                  f3s_preprocess_capacity(N, E, W) = ceil(E / W) + ceil(N / 16), which bounds
 *                  the total of any graph with these sizes
 *   tcblockRowid [capacity], tcblocktileId [E], tcblockOffset [capacity+1],
 *   sparseAToXidx [capacity*W], tcbBitMap [capacity*H*W/64]
 *                  out: entries of the first nTCB blocks as f3s_preprocess_fill writes them
 *                  (tcblockOffset: nTCB + 1 entries); the rest is left untouched
 *   every other argument as in f3s_preprocess_count
 * On graphs of long windows whose column range fits one LDS bitset (E >= 128 N, N <= 393 216)
 * a window's ranking bitset stays in LDS for both phases, so edgeToColumn is written once and
 * not read back. Synchronises `stream` before returning. Returns 0 or a negative status; after a
 * column index outside [0, N) (-4) the outputs are undefined.
 */
int64_t f3s_preprocess_capacity(int N, int64_t E, int W);
int f3s_preprocess(const int32_t* rowPtr, const int32_t* colIdx, int N, int E, int H, int W,
                   int32_t* blockPartition, int32_t* edgeToColumn, int32_t* edgeToRow,
                   int32_t* rowWindowOffset, int32_t* sortedRowWindows, int64_t capacity,
                   int32_t* tcblockRowid, uint8_t* tcblocktileId, int32_t* tcblockOffset,
                   int32_t* sparseAToXidx, uint64_t* tcbBitMap, void* workspace, size_t ws_bytes,
                   int64_t* nTCB_host, void* stream);

/*
 * Fused SDDMM -> softmax -> SpMM over 16x16 TC blocks. Replaces f3sCuda1tb1rw,
 * f3sCuda1tb1rwScheduled (src/F3S_kernel.cu:393-458, 581-671) and the kernels they launch
 * (f3sKernel1tb1rw :997-1175, f3sKernel1tb1rwScheduled :1999-2182,
 * f3sKernel1tb1rwScheduledPermutedQKV[ScaleQK] :1371-1800, f2sKernel1tb1rw :2186-2327).
 *
 *   rowWindowOffset [nRW+1], sparseAToXidx [nTCB*16], tcbBitMap [nTCB*4]   from preprocessing
 *   windowOrder [nRW] or NULL      launch order of the row windows: sortedRowWindows for the
 *                                  heavy-first schedule, NULL for natural order
 *   N, nTCB, d                     nodes; TC blocks (rowWindowOffset[nRW]); head dimension: a
 *                                  multiple of 32 up to 256 (the reference takes embeddingDim
 *                                  at run time, src/F3S_kernel.cu:601-604,1424,1522)
 *   dtype                          F3S_DTYPE_F16 (the reference's only type) or F3S_DTYPE_BF16
 *                                  (bf16 MFMA; the probabilities then enter the second product as
 *                                  the sum of two bf16 terms, 16 bits of mantissa instead of the
 *                                  11 of the reference's fp16 rounding)
 *   Q, K, V [N*d]                  row-major, contiguous; any size (row offsets are formed in
 *                                  64 bits once an array reaches 4 GiB, as the reference's
 *                                  int64_t offsets are, src/F3S_kernel.cu:1422-1423)
 *   scalingFactor                  unmasked scores are DIVIDED by it (src/F3S_kernel.cu:1666-1667);
 *                                  1.0 = unscaled (:612-613)
 *   applySoftmax                   0 = SDDMM -> SpMM only (src/F3S_kernel.cu:420-443)
 *   out [N*d] float                fully written (rows without edges get 0)
 *   cuTimer                        NULL, or 3*nRW uint64 {begin, end, cu id} per workgroup
 *                                  (the Clocked variants, src/F3S_kernel.cu:1178-1368, 1803-1997)
 *   workspace, ws_bytes            NULL / 0, or device scratch of
 *                                  f3s_attention_workspace_bytes(N, d) bytes (256-byte aligned).
 *                                  With it, graphs for which f3s_attention_uses_workspace()
 *                                  returns 1 are computed by the column-sliced schedule: per
 *                                  (window, column slice) partial results that a second kernel
 *                                  merges in slice order. Results agree with the default
 *                                  schedule within the tolerance of the summation order.
 *                                  Ignored with cuTimer. Calls that share a workspace must not
 *                                  overlap. Its contents need not be initialised.
 *   prepared                       0, or 1 when f3s_attention_prepare was called on this workspace
 *                                  for these arrays: the schedule's index is then not rebuilt
 *                                  (the call checks on the device that the workspace's header
 *                                  names these arrays and rebuilds the index otherwise)
 * Asynchronous on `stream` (kernel launches only: no host wait, no copy, no allocation).
 */
int f3s_attention_fwd(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                      const int32_t* sparseAToXidx, const uint64_t* tcbBitMap, int N, int64_t nTCB,
                      int d, int dtype, const void* Q, const void* K, const void* V,
                      float scalingFactor, int applySoftmax, float* out,
                      unsigned long long* cuTimer, void* workspace, size_t ws_bytes, int prepared,
                      void* stream);

/*
 * Bytes of device scratch f3s_attention_fwd / f3s_attention_fwd_heads can use for a graph of N
 * nodes at head dimension d (a header, the slice boundaries of every window, plus one partial
 * (m, l, O) per window, head and slice: about 4.6 KB * ceil(N/16) * slices at d = 64; for the
 * single-head call at d = 64 also 512 * N bytes for copies of K and V with 256-byte rows, which
 * the call makes itself and gathers from instead: rows that start on even 128-byte lines are
 * served faster than rows on the odd lines in between). The reference's launchers
 * (src/F3S_kernel.cu:581-671) need no scratch; passing workspace = NULL keeps that behaviour.
 */
size_t f3s_attention_workspace_bytes(int N, int d);
size_t f3s_attention_heads_workspace_bytes(int N, int nHeads, int d);

/*
 * Optional: builds the part of the column-sliced schedule that depends only on the TC-block
 * structure (the slice boundaries of every window) in `workspace` once, so that the attention
 * calls that follow (with prepared = 1) do not rebuild it. It has no counterpart in the reference
 * (whose launchers keep no state between calls). The workspace then belongs to exactly these
 * arrays (rowWindowOffset, sparseAToXidx: same pointers, same N, nTCB, d and head count; nHeads =
 * 0 for f3s_attention_fwd, the head count for f3s_attention_fwd_heads): the caller must not
 * change their contents, nor write to the workspace, while it passes prepared = 1. A call with
 * prepared = 0, or with other arrays, on the same workspace rebuilds the index and ends the
 * preparation. Asynchronous on `stream`.
 */
int f3s_attention_prepare(const int32_t* rowWindowOffset, const int32_t* sparseAToXidx, int N,
                          int64_t nTCB, int d, int nHeads, void* workspace, size_t ws_bytes,
                          void* stream);

/*
 * 1 if f3s_attention_fwd would use a workspace for this problem (at least 2048 row windows with
 * 64 or more TC blocks each on average), else 0: callers can skip the allocation.
 * F3S_SCHEDULE=window or =sliced in the environment (read at every call) forces 0 or 1.
 */
int f3s_attention_uses_workspace(int N, int64_t nTCB, int d, int dtype);

/*
 * 1 if the attention kernels form 64-bit row offsets for K / V arrays of N rows with a row pitch
 * of pitch_bytes (pitched = 1: the multi-head layout): the array spans 4 GiB or more, or, with
 * pitched rows, N or the pitch reaches 2^24. Informational; the entry points decide by
 * themselves. The reference always uses int64_t offsets (src/F3S_kernel.cu:1422-1423).
 */
int f3s_attention_uses_wide_offsets(int64_t N, int64_t pitch_bytes, int pitched);

/*
 * The same fused kernel over nHeads attention heads in one launch: Q, K, V are [N, nHeads, d]
 * with a row pitch of ldIn elements (head h of node i starts at element i*ldIn + h*d), out is
 * [N, nHeads*d] fp32 with a row pitch of ldOut floats, i.e. the per-head results already
 * concatenated. All heads share one graph (one TC-block structure). The reference has no
 * multi-head entry: its callers run f3s_1tb1rw_scheduled_permuteV_scaleQK (src/F3S.cpp:247-270)
 * once per head on contiguous per-head copies and concatenate; this call returns what that loop
 * returns. ldIn % 8 == 0, ldOut % 4 == 0, both below 2^31.
 * workspace, ws_bytes: NULL / 0, or f3s_attention_heads_workspace_bytes(N, nHeads, d) bytes of
 * device scratch (256-byte aligned); with it, graphs for which f3s_attention_uses_workspace()
 * returns 1 take the column-sliced schedule with (window, slice, head) units, as in
 * f3s_attention_fwd; prepared as there. Asynchronous on `stream`.
 */
int f3s_attention_fwd_heads(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                            const int32_t* sparseAToXidx, const uint64_t* tcbBitMap, int N,
                            int64_t nTCB, int nHeads, int d, int dtype, const void* Q,
                            const void* K, const void* V, int64_t ldIn, float scalingFactor,
                            int applySoftmax, float* out, int64_t ldOut, void* workspace,
                            size_t ws_bytes, int prepared, void* stream);

/*
 * Fused SDDMM -> softmax -> SpMM over 16x8 TC blocks: replaces f3sCuda1tb1tcb and
 * f3sKernel1tb1tcb (src/F3S_kernel.cu:325-391, 677-877), the path behind F3S.f3s_1tb1tcb
 * (src/F3S.cpp:272-296).
 *
 *   rowWindowOffset [nRW+1], sparseAToXidx [nTCB*8], tcbBitMap [nTCB*2]   from preprocessing
 *                                  with H = 16, W = 8
 *   windowOrder [nRW] or NULL      launch order (the reference launches in natural order)
 *   Q, K, V [N*d]                  fp16, row-major, contiguous; d a multiple of 32 up to 256
 *   applySoftmax                   0 = SDDMM -> SpMM only; scores are never scaled on this path
 *   out [N*d] float                fully written
 *   sddmmResult                    NULL, or nTCB*128 floats: the masked scores of every block,
 *                                  row-major 16x8 (saveSddmmResult, src/F3S_kernel.cu:99-115);
 *                                  fully written
 * Asynchronous on `stream`.
 */
int f3s_attention_fwd_tcb8(const int32_t* rowWindowOffset, const int32_t* windowOrder,
                           const int32_t* sparseAToXidx, const uint64_t* tcbBitMap, int N,
                           int64_t nTCB, int d, const void* Q, const void* K, const void* V,
                           int applySoftmax, float* out, float* sddmmResult, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* F3S_AMD_H */
