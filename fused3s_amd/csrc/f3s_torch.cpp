// Python operator module `F3S`: the reference's pybind surface (src/F3S.cpp:298-305) re-created
// on top of the C ABI of libf3s_amd.so. Host-only C++: tensors are allocated here, every kernel
// is reached through include/f3s_amd.h. Same function names, argument order and return tuples
// as the reference; differences are listed in the comments of each function.
#include <ATen/hip/HIPContext.h>
#include <c10/core/DeviceGuard.h>
#include <hip/hip_runtime_api.h>
#include <torch/extension.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iomanip>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/f3s_amd.h"

namespace {

#define F3S_CHECK_DEVICE(x) TORCH_CHECK(x.device().is_cuda(), #x " must be a CUDA tensor")
#define F3S_CHECK_CONTIGUOUS(x) TORCH_CHECK(x.is_contiguous(), #x " must be contiguous")
#define F3S_CHECK_INPUT(x) \
  F3S_CHECK_DEVICE(x);     \
  F3S_CHECK_CONTIGUOUS(x)

void check_status(int rc, const char* what) {
  TORCH_CHECK(rc == 0, what, " failed: ", f3s_last_error(), " (status ", rc, ")");
}

void* current_stream() { return static_cast<void*>(at::hip::getCurrentHIPStream().stream()); }

bool verbose() {
  const char* v = std::getenv("F3S_VERBOSE");
  return v && v[0] != '\0' && v[0] != '0';
}

// F3S_PREPROCESS=two_phase: count, exact allocations, fill, as the reference does; default: one
// call with the block arrays allocated for a bound on the block total (read per call)
bool two_phase() {
  const char* v = std::getenv("F3S_PREPROCESS");
  return v && std::strcmp(v, "two_phase") == 0;
}

// F3S.preprocess_gpu (src/F3S.cpp:40-87). The three caller tensors are filled in place as in
// the reference; they need not be zeroed. The "GPU Preprocess time" / "TC_Blocks" lines the
// reference prints (src/F3S.cpp:73-75,82) appear only when F3S_VERBOSE=1.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
           torch::Tensor, torch::Tensor, int>
preprocess_gpu(torch::Tensor edgeList, torch::Tensor nodePointer, int num_nodes, int blockSize_h,
               int blockSize_w, torch::Tensor blockPartition, torch::Tensor edgeToColumn,
               torch::Tensor edgeToRow) {
  F3S_CHECK_INPUT(edgeList);
  F3S_CHECK_INPUT(nodePointer);
  F3S_CHECK_INPUT(blockPartition);
  F3S_CHECK_INPUT(edgeToColumn);
  F3S_CHECK_INPUT(edgeToRow);
  TORCH_CHECK(edgeList.scalar_type() == torch::kInt32 &&
                  nodePointer.scalar_type() == torch::kInt32 &&
                  blockPartition.scalar_type() == torch::kInt32 &&
                  edgeToColumn.scalar_type() == torch::kInt32 &&
                  edgeToRow.scalar_type() == torch::kInt32,
              "preprocess_gpu: all index tensors must be int32");
  TORCH_CHECK(num_nodes >= 0 && nodePointer.numel() == (int64_t)num_nodes + 1,
              "preprocess_gpu: nodePointer must have num_nodes + 1 entries");
  TORCH_CHECK(blockSize_h > 0 && blockSize_w > 0, "preprocess_gpu: block sizes must be positive");
  const int64_t E = edgeList.numel();
  const int64_t nRW = ((int64_t)num_nodes + blockSize_h - 1) / blockSize_h;
  TORCH_CHECK(blockPartition.numel() == nRW, "preprocess_gpu: blockPartition must have ", nRW,
              " entries");
  TORCH_CHECK(edgeToColumn.numel() == E && edgeToRow.numel() == E,
              "preprocess_gpu: edgeToColumn / edgeToRow must have one entry per edge");
  c10::DeviceGuard guard(edgeList.device());
  auto i32 = torch::TensorOptions().dtype(torch::kInt32).device(edgeList.device());
  auto start = std::chrono::high_resolution_clock::now();
  auto rowWindowOffset = torch::empty({nRW + 1}, i32);
  auto sortedRowWindows = torch::empty({nRW}, i32);
  const size_t wsBytes = f3s_preprocess_workspace_bytes(num_nodes, (int)E);
  auto workspace = torch::empty({(int64_t)wsBytes}, i32.dtype(torch::kUInt8));
  int64_t nTcb = 0;
  auto tcblocktileId = torch::empty({E}, i32.dtype(torch::kUInt8));
  torch::Tensor tcblockRowid, tcblockOffset, sparseAToXidx, tcbBitMap;
  const int64_t bmWords = (int64_t)blockSize_h * blockSize_w / 64;
  if (two_phase()) {
    // the reference's sequence: count, allocate exactly, fill
    check_status(
        f3s_preprocess_count(nodePointer.data_ptr<int>(), edgeList.data_ptr<int>(), num_nodes,
                             (int)E, blockSize_h, blockSize_w, blockPartition.data_ptr<int>(),
                             edgeToColumn.data_ptr<int>(), edgeToRow.data_ptr<int>(),
                             rowWindowOffset.data_ptr<int>(), sortedRowWindows.data_ptr<int>(),
                             workspace.data_ptr(), wsBytes, &nTcb, current_stream()),
        "f3s_preprocess_count");
    tcblockRowid = torch::empty({nTcb}, i32);
    tcblockOffset = torch::empty({nTcb + 1}, i32);
    sparseAToXidx = torch::empty({nTcb * blockSize_w}, i32);
    tcbBitMap = torch::empty({nTcb * bmWords}, i32.dtype(torch::kUInt64));
    check_status(
        f3s_preprocess_fill(nodePointer.data_ptr<int>(), edgeList.data_ptr<int>(), num_nodes,
                            (int)E, blockSize_h, blockSize_w, edgeToColumn.data_ptr<int>(),
                            rowWindowOffset.data_ptr<int>(), nTcb, tcblockRowid.data_ptr<int>(),
                            tcblocktileId.data_ptr<uint8_t>(), tcblockOffset.data_ptr<int>(),
                            sparseAToXidx.data_ptr<int>(),
                            reinterpret_cast<uint64_t*>(tcbBitMap.data_ptr()), current_stream()),
        "f3s_preprocess_fill");
  } else {
    // one call: the nTCB-sized arrays are allocated for the bound on the block total and returned as
    // views of their first nTcb entries, so the host waits for the device once, at the end
    TORCH_CHECK(blockSize_h == 16 && (blockSize_w == 16 || blockSize_w == 8),
                "preprocess_gpu: block ", blockSize_h, "x", blockSize_w,
                " unsupported (16x16 or 16x8)");
    const int64_t cap = f3s_preprocess_capacity(num_nodes, E, blockSize_w);
    tcblockRowid = torch::empty({cap}, i32);
    tcblockOffset = torch::empty({cap + 1}, i32);
    sparseAToXidx = torch::empty({cap * blockSize_w}, i32);
    tcbBitMap = torch::empty({cap * bmWords}, i32.dtype(torch::kUInt64));
    check_status(
        f3s_preprocess(nodePointer.data_ptr<int>(), edgeList.data_ptr<int>(), num_nodes, (int)E,
                       blockSize_h, blockSize_w, blockPartition.data_ptr<int>(),
                       edgeToColumn.data_ptr<int>(), edgeToRow.data_ptr<int>(),
                       rowWindowOffset.data_ptr<int>(), sortedRowWindows.data_ptr<int>(), cap,
                       tcblockRowid.data_ptr<int>(), tcblocktileId.data_ptr<uint8_t>(),
                       tcblockOffset.data_ptr<int>(), sparseAToXidx.data_ptr<int>(),
                       reinterpret_cast<uint64_t*>(tcbBitMap.data_ptr()), workspace.data_ptr(),
                       wsBytes, &nTcb, current_stream()),
        "f3s_preprocess");
    tcblockRowid = tcblockRowid.narrow(0, 0, nTcb);
    tcblockOffset = tcblockOffset.narrow(0, 0, nTcb + 1);
    sparseAToXidx = sparseAToXidx.narrow(0, 0, nTcb * blockSize_w);
    tcbBitMap = tcbBitMap.narrow(0, 0, nTcb * bmWords);
    if (nTcb * 2 < cap) {
      // rows of a window that share columns: far fewer blocks than the bound. The views would keep
      // the whole allocation alive for as long as the caller keeps the structure, so it gets
      // exact-size copies instead (at most half of what was allocated is copied).
      tcblockRowid = tcblockRowid.clone();
      tcblockOffset = tcblockOffset.clone();
      sparseAToXidx = sparseAToXidx.clone();
      tcbBitMap = tcbBitMap.clone();
    }
  }
  if (verbose()) {
    TORCH_CHECK(hipStreamSynchronize(at::hip::getCurrentHIPStream().stream()) == hipSuccess);
    std::chrono::duration<double> dt = std::chrono::high_resolution_clock::now() - start;
    std::printf("\t GPU Preprocess time: %f seconds\nTC_Blocks:\t%d\n", dt.count(), (int)nTcb);
  }
  return std::make_tuple(rowWindowOffset, sortedRowWindows, tcblockRowid, tcblocktileId,
                         tcblockOffset, sparseAToXidx, tcbBitMap, (int)nTcb);
}

// Folds {begin, end, cu} triples into one "[first begin] [last end]" line per CU, in
// milliseconds with 15 decimals -- the format of the reference's printSMTime
// (src/F3S_kernel.cu:43-75), with one line per CU that ran a workgroup instead of a fixed
// NUM_SM_GPU. Ticks are 10 ns.
void write_cu_time(const torch::Tensor& timer, int64_t nBlocks, const std::string& filename) {
  auto host = timer.cpu();
  const auto* t = reinterpret_cast<const unsigned long long*>(host.data_ptr());
  std::map<unsigned long long, std::pair<unsigned long long, unsigned long long>> span;
  for (int64_t b = 0; b < nBlocks; b++) {
    const unsigned long long begin = t[3 * b], end = t[3 * b + 1], cu = t[3 * b + 2];
    if (end == 0) continue;  // workgroup never ran (cannot happen for a completed launch)
    auto it = span.find(cu);
    if (it == span.end()) {
      span[cu] = {begin, end};
    } else {
      it->second.first = std::min(it->second.first, begin);
      it->second.second = std::max(it->second.second, end);
    }
  }
  std::ofstream out(filename);
  if (!out.is_open()) return;
  out << std::fixed << std::setprecision(15);
  for (const auto& kv : span)
    out << (double)kv.second.first / 1e5 << " " << (double)kv.second.second / 1e5 << std::endl;
}

// Runs `launch(stream)` on PyTorch's current stream between two events, blocks on the stop event
// like the reference's launchers (src/F3S_kernel.cu:436-451) and returns the elapsed ms.
template <typename F>
float timed_launch(const char* what, F&& launch) {
  hipStream_t stream = at::hip::getCurrentHIPStream().stream();
  hipEvent_t start, stop;
  TORCH_CHECK(hipEventCreate(&start) == hipSuccess && hipEventCreate(&stop) == hipSuccess);
  TORCH_CHECK(hipEventRecord(start, stream) == hipSuccess);
  const int rc = launch(static_cast<void*>(stream));
  hipError_t e1 = hipEventRecord(stop, stream);
  hipError_t e2 = hipEventSynchronize(stop);
  float ms = 0.f;
  hipError_t e3 = hipEventElapsedTime(&ms, start, stop);
  (void)hipEventDestroy(start);
  (void)hipEventDestroy(stop);
  check_status(rc, what);
  TORCH_CHECK(e1 == hipSuccess && e2 == hipSuccess && e3 == hipSuccess, "HIP event timing failed: ",
              hipGetErrorString(e2 != hipSuccess ? e2 : (e1 != hipSuccess ? e1 : e3)));
  return ms;
}

struct Launch {
  const torch::Tensor* order;  // nullptr = natural window order
  float scalingFactor;
  bool applySoftmax;
  const char* timerFile;  // non-null: record per-CU active time into this file
};

// Scratch of the column-sliced schedule: one tensor per device, kept between calls and grown when
// a call needs more. A call holds the lock from the moment it takes the tensor until its kernels
// are done (every entry point blocks on its stop event, see timed_launch), so two host threads
// never compute into the same scratch. F3S.release_workspace() drops the tensors.
std::mutex g_wsMutex;
std::map<int, torch::Tensor> g_wsCache;

struct WorkspaceLease {
  std::unique_lock<std::mutex> lock;
  torch::Tensor tensor;
  WorkspaceLease(bool wanted, size_t bytes, const c10::Device& device) {
    if (!wanted) return;
    lock = std::unique_lock<std::mutex>(g_wsMutex);
    torch::Tensor& cached = g_wsCache[(int)device.index()];
    if (!cached.defined() || (size_t)cached.numel() < bytes)
      cached = torch::empty({(int64_t)bytes},
                            torch::TensorOptions().dtype(torch::kUInt8).device(device));
    tensor = cached;
  }
};

// F3S.release_workspace(): frees the cached scratch of every device (beyond the reference's
// surface, whose launchers keep nothing between calls). Returns the number of bytes released.
int64_t releaseWorkspace() {
  std::lock_guard<std::mutex> lock(g_wsMutex);
  int64_t bytes = 0;
  for (auto& kv : g_wsCache)
    if (kv.second.defined()) bytes += kv.second.numel();
  g_wsCache.clear();
  return bytes;
}

// Common host path of every 1tb1rw entry point: f3sCuda1tb1rw / f3sCuda1tb1rwScheduled and the
// Clocked launchers (src/F3S_kernel.cu:393-671). Returns {time_ms (0-d CPU fp32), out fp32[N,d],
// empty fp32 sddmmResult} like the reference. `out` is allocated [N, d] (the reference
// allocates it padded to 16 rows and returns a [:N] view). The launch goes to PyTorch's current
// stream (the reference uses the legacy default stream), and the host blocks on the stop event.
std::vector<torch::Tensor> run_1tb1rw(const torch::Tensor& rowWindowOffset,
                                      const torch::Tensor& sparseAToXidx,
                                      const torch::Tensor& tcbBitMap, int nNodes,
                                      const torch::Tensor& Q, const torch::Tensor& K,
                                      const torch::Tensor& V, int nWarpPerBlock, const Launch& L) {
  TORCH_CHECK(Q.dim() == 2 && K.dim() == 2 && V.dim() == 2, "Q, K, V must be [N, d]");
  TORCH_CHECK((Q.scalar_type() == torch::kHalf || Q.scalar_type() == torch::kBFloat16) &&
                  K.scalar_type() == Q.scalar_type() && V.scalar_type() == Q.scalar_type(),
              "Q, K, V must all be float16 (the reference's type) or all bfloat16");
  TORCH_CHECK(Q.is_cuda() && K.is_cuda() && V.is_cuda() && rowWindowOffset.is_cuda() &&
                  sparseAToXidx.is_cuda() && tcbBitMap.is_cuda(),
              "all tensors must be CUDA tensors");
  TORCH_CHECK(Q.is_contiguous() && K.is_contiguous() && V.is_contiguous() &&
                  rowWindowOffset.is_contiguous() && sparseAToXidx.is_contiguous() &&
                  tcbBitMap.is_contiguous(),
              "all tensors must be contiguous");
  const int64_t d = Q.size(1);
  TORCH_CHECK(K.size(1) == d && V.size(1) == d, "Q, K, V must share the embedding dimension");
  TORCH_CHECK(Q.size(0) >= nNodes && K.size(0) >= nNodes && V.size(0) >= nNodes,
              "Q, K, V need at least nNodes rows");
  const int64_t nRW = rowWindowOffset.numel() - 1;
  TORCH_CHECK(nRW == ((int64_t)nNodes + 15) / 16,
              "rowWindowOffset does not match nNodes (expected ceil(nNodes/16)+1 entries)");
  TORCH_CHECK(nWarpPerBlock >= 2 && nWarpPerBlock % 2 == 0,
              "nWarpPerBlock must be even and >= 2 (accepted for compatibility; the wave count "
              "per window is fixed by this implementation)");
  if (L.order) {
    TORCH_CHECK(L.order->is_cuda() && L.order->is_contiguous() && L.order->numel() == nRW &&
                    L.order->scalar_type() == torch::kInt32,
                "sortedRowWindows must be a contiguous int32 CUDA tensor with one entry per window");
  }
  c10::DeviceGuard guard(Q.device());
  auto f32 = torch::TensorOptions().dtype(torch::kFloat32).device(Q.device());
  auto out = torch::empty({(int64_t)nNodes, d}, f32);
  auto sddmmResult = torch::zeros({0}, f32);
  torch::Tensor timer;
  unsigned long long* timerPtr = nullptr;
  if (L.timerFile) {
    timer = torch::zeros({3 * nRW}, f32.dtype(torch::kInt64));
    timerPtr = reinterpret_cast<unsigned long long*>(timer.data_ptr());
  }
  const int dtype = Q.scalar_type() == torch::kHalf ? F3S_DTYPE_F16 : F3S_DTYPE_BF16;
  // scratch of the column-sliced schedule, allocated only for the graphs the library uses it on
  const bool sliced = !L.timerFile && f3s_attention_uses_workspace(
                                          nNodes, sparseAToXidx.numel() / 16, (int)d, dtype) != 0;
  const size_t wsBytes = sliced ? f3s_attention_workspace_bytes(nNodes, (int)d) : 0;
  WorkspaceLease lease(sliced, wsBytes, Q.device());
  torch::Tensor& workspace = lease.tensor;
  const float ms = timed_launch("f3s_attention_fwd", [&](void* stream) {
    return f3s_attention_fwd(
        rowWindowOffset.data_ptr<int>(), L.order ? L.order->data_ptr<int>() : nullptr,
        sparseAToXidx.data_ptr<int>(), reinterpret_cast<const uint64_t*>(tcbBitMap.data_ptr()),
        nNodes, sparseAToXidx.numel() / 16, (int)d, dtype, Q.data_ptr(), K.data_ptr(),
        V.data_ptr(), L.scalingFactor, L.applySoftmax ? 1 : 0, out.data_ptr<float>(), timerPtr,
        sliced ? workspace.data_ptr() : nullptr, wsBytes, 0, stream);
  });
  if (L.timerFile) write_cu_time(timer, nRW, L.timerFile);
  auto time = torch::tensor(ms, torch::TensorOptions().dtype(torch::kFloat32));
  return {time, out, sddmmResult};
}

// Multi-head call, beyond the reference's surface: its graph-transformer callers run
// f3s_1tb1rw_scheduled_permuteV_scaleQK (src/F3S.cpp:247-270) once per head and concatenate.
// Q, K, V are [N, nHeads, d] (heads contiguous inside a row, rows may be pitched), fp16 or bf16;
// returns {time_ms, out fp32[N, nHeads*d], empty} from ONE launch over all (window, head) pairs.
std::vector<torch::Tensor> f3sMultiHeadScaleQK(torch::Tensor rowWindowOffset,
                                               torch::Tensor sortedRowWindows,
                                               torch::Tensor sparseAToXidx,
                                               torch::Tensor tcbBitMap, int nNodes,
                                               torch::Tensor Q, torch::Tensor K, torch::Tensor V,
                                               float scalingFactor) {
  TORCH_CHECK(Q.dim() == 3 && K.sizes() == Q.sizes() && V.sizes() == Q.sizes(),
              "Q, K, V must be [N, nHeads, d] with identical shapes");
  TORCH_CHECK((Q.scalar_type() == torch::kHalf || Q.scalar_type() == torch::kBFloat16) &&
                  K.scalar_type() == Q.scalar_type() && V.scalar_type() == Q.scalar_type(),
              "Q, K, V must all be float16 or all bfloat16");
  const int64_t nHeads = Q.size(1), d = Q.size(2);
  for (const torch::Tensor* t : {&Q, &K, &V})
    TORCH_CHECK(t->is_cuda() && t->stride(2) == 1 && t->stride(1) == d &&
                    t->stride(0) == Q.stride(0),
                "Q, K, V must be CUDA tensors with heads contiguous inside a row and one row "
                "pitch");
  for (const torch::Tensor* t : {&rowWindowOffset, &sortedRowWindows, &sparseAToXidx, &tcbBitMap})
    TORCH_CHECK(t->is_cuda() && t->is_contiguous(), "TC-block tensors must be contiguous CUDA "
                                                    "tensors");
  TORCH_CHECK(Q.size(0) >= nNodes, "Q, K, V need at least nNodes rows");
  const int64_t nRW = rowWindowOffset.numel() - 1;
  TORCH_CHECK(nRW == ((int64_t)nNodes + 15) / 16,
              "rowWindowOffset does not match nNodes (expected ceil(nNodes/16)+1 entries)");
  TORCH_CHECK(sortedRowWindows.numel() == nRW && sortedRowWindows.scalar_type() == torch::kInt32,
              "sortedRowWindows must be int32 with one entry per window");
  c10::DeviceGuard guard(Q.device());
  auto f32 = torch::TensorOptions().dtype(torch::kFloat32).device(Q.device());
  auto out = torch::empty({(int64_t)nNodes, nHeads * d}, f32);
  const int dtype = Q.scalar_type() == torch::kHalf ? F3S_DTYPE_F16 : F3S_DTYPE_BF16;
  // graphs of long windows take the column-sliced schedule here as in the single-head calls
  const bool sliced =
      f3s_attention_uses_workspace(nNodes, sparseAToXidx.numel() / 16, (int)d, dtype) != 0;
  const size_t wsBytes =
      sliced ? f3s_attention_heads_workspace_bytes(nNodes, (int)nHeads, (int)d) : 0;
  WorkspaceLease lease(sliced, wsBytes, Q.device());
  const float ms = timed_launch("f3s_attention_fwd_heads", [&](void* stream) {
    return f3s_attention_fwd_heads(
        rowWindowOffset.data_ptr<int>(), sortedRowWindows.data_ptr<int>(),
        sparseAToXidx.data_ptr<int>(), reinterpret_cast<const uint64_t*>(tcbBitMap.data_ptr()),
        nNodes, sparseAToXidx.numel() / 16, (int)nHeads, (int)d, dtype, Q.data_ptr(),
        K.data_ptr(), V.data_ptr(), Q.stride(0), scalingFactor, 1, out.data_ptr<float>(),
        out.stride(0), sliced ? lease.tensor.data_ptr() : nullptr, wsBytes, 0, stream);
  });
  auto time = torch::tensor(ms, torch::TensorOptions().dtype(torch::kFloat32));
  return {time, out, torch::zeros({0}, f32)};
}

// F3S.f3s_1tb1rw (src/F3S.cpp:145-183)
std::vector<torch::Tensor> f3s1tb1rw(torch::Tensor rowWindowOffset, torch::Tensor sparseAToXidx,
                                     torch::Tensor tcbBitMap, int nNodes, torch::Tensor Q,
                                     torch::Tensor K, torch::Tensor V, int nWarpPerBlock,
                                     bool applySoftmax, bool checkSMActiveTime) {
  F3S_CHECK_INPUT(rowWindowOffset);
  F3S_CHECK_INPUT(sparseAToXidx);
  F3S_CHECK_INPUT(tcbBitMap);
  F3S_CHECK_INPUT(Q);
  F3S_CHECK_INPUT(K);
  F3S_CHECK_INPUT(V);
  // the reference's timed variant always applies the softmax (src/F3S.cpp:164-171)
  Launch L{nullptr, 1.0f, checkSMActiveTime ? true : applySoftmax,
           checkSMActiveTime ? "SM_time_f3s1tb1rw.csv" : nullptr};
  return run_1tb1rw(rowWindowOffset, sparseAToXidx, tcbBitMap, nNodes, Q, K, V, nWarpPerBlock, L);
}

// F3S.f3s_1tb1rw_scheduled (src/F3S.cpp:185-219)
std::vector<torch::Tensor> f3s1tb1rwScheduled(torch::Tensor rowWindowOffset,
                                              torch::Tensor sortedRowWindows,
                                              torch::Tensor sparseAToXidx, torch::Tensor tcbBitMap,
                                              int nNodes, torch::Tensor Q, torch::Tensor K,
                                              torch::Tensor V, int nWarpPerBlock,
                                              bool checkSMActiveTime) {
  Launch L{&sortedRowWindows, 1.0f, true,
           checkSMActiveTime ? "SM_time_f3s1tb1rw_scheduled.csv" : nullptr};
  return run_1tb1rw(rowWindowOffset, sparseAToXidx, tcbBitMap, nNodes, Q, K, V, nWarpPerBlock, L);
}

// F3S.f3s_1tb1rw_scheduled_permuteV (src/F3S.cpp:222-244). The reference's "permute" is a
// register-layout choice of its kernel; here the one kernel already gathers K and V with wide
// coalesced loads, so this entry differs from f3s_1tb1rw_scheduled only by name.
std::vector<torch::Tensor> f3s1tb1rwScheduledPermuteV(torch::Tensor rowWindowOffset,
                                                      torch::Tensor sortedRowWindows,
                                                      torch::Tensor sparseAToXidx,
                                                      torch::Tensor tcbBitMap, int nNodes,
                                                      torch::Tensor Q, torch::Tensor K,
                                                      torch::Tensor V, int nWarpPerBlock) {
  Launch L{&sortedRowWindows, 1.0f, true, nullptr};
  return run_1tb1rw(rowWindowOffset, sparseAToXidx, tcbBitMap, nNodes, Q, K, V, nWarpPerBlock, L);
}

// F3S.f3s_1tb1rw_scheduled_permuteV_scaleQK (src/F3S.cpp:247-270): scores are divided by
// scalingFactor; 1.0 selects the unscaled path (src/F3S_kernel.cu:612-613).
std::vector<torch::Tensor> f3s1tb1rwScheduledPermuteVScaleQK(
    torch::Tensor rowWindowOffset, torch::Tensor sortedRowWindows, torch::Tensor sparseAToXidx,
    torch::Tensor tcbBitMap, int nNodes, torch::Tensor Q, torch::Tensor K, torch::Tensor V,
    float scalingFactor, int nWarpPerBlock) {
  Launch L{&sortedRowWindows, scalingFactor, true, nullptr};
  return run_1tb1rw(rowWindowOffset, sparseAToXidx, tcbBitMap, nNodes, Q, K, V, nWarpPerBlock, L);
}

// F3S.f3s_1tb1tcb (src/F3S.cpp:272-296; launcher src/F3S_kernel.cu:325-391): 16x8 TC blocks from
// preprocess_gpu(..., blockSize_w = 8), natural window order, no score scaling; with
// saveSddmmResult the third tensor holds the masked scores, 16x8 row-major per block.
std::vector<torch::Tensor> f3s1tb1tcb(torch::Tensor rowWindowOffset, torch::Tensor sparseAToXidx,
                                      torch::Tensor tcbBitMap, int nNodes, torch::Tensor Q,
                                      torch::Tensor K, torch::Tensor V, bool applySoftmax,
                                      bool saveSddmmResult) {
  F3S_CHECK_INPUT(Q);
  F3S_CHECK_INPUT(K);
  F3S_CHECK_INPUT(V);
  F3S_CHECK_INPUT(rowWindowOffset);
  F3S_CHECK_INPUT(sparseAToXidx);
  F3S_CHECK_INPUT(tcbBitMap);
  TORCH_CHECK(Q.dim() == 2 && K.sizes() == Q.sizes() && V.sizes() == Q.sizes(),
              "Q, K, V must be [N, d] with identical shapes");
  TORCH_CHECK(Q.scalar_type() == torch::kHalf && K.scalar_type() == torch::kHalf &&
                  V.scalar_type() == torch::kHalf,
              "Q, K, V must be float16");
  TORCH_CHECK(Q.size(0) >= nNodes, "Q, K, V need at least nNodes rows");
  const int64_t d = Q.size(1);
  const int64_t nRW = rowWindowOffset.numel() - 1;
  TORCH_CHECK(nRW == ((int64_t)nNodes + 15) / 16,
              "rowWindowOffset does not match nNodes (expected ceil(nNodes/16)+1 entries)");
  const int64_t nTcb = sparseAToXidx.numel() / 8;
  TORCH_CHECK(tcbBitMap.numel() == 2 * nTcb,
              "tcbBitMap must hold two words per 16x8 block (preprocess_gpu with blockSize_w = 8)");
  c10::DeviceGuard guard(Q.device());
  auto f32 = torch::TensorOptions().dtype(torch::kFloat32).device(Q.device());
  auto out = torch::empty({(int64_t)nNodes, d}, f32);
  auto sddmmResult = torch::empty({saveSddmmResult ? nTcb * 128 : 0}, f32);
  const float ms = timed_launch("f3s_attention_fwd_tcb8", [&](void* stream) {
    return f3s_attention_fwd_tcb8(
        rowWindowOffset.data_ptr<int>(), nullptr, sparseAToXidx.data_ptr<int>(),
        reinterpret_cast<const uint64_t*>(tcbBitMap.data_ptr()), nNodes, nTcb, (int)d,
        Q.data_ptr(), K.data_ptr(), V.data_ptr(), applySoftmax ? 1 : 0, out.data_ptr<float>(),
        saveSddmmResult ? sddmmResult.data_ptr<float>() : nullptr, stream);
  });
  auto time = torch::tensor(ms, torch::TensorOptions().dtype(torch::kFloat32));
  return {time, out, sddmmResult};
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("preprocess_gpu", &preprocess_gpu, "CSR -> TC blocks (HIP)");
  m.def("f3s_1tb1tcb", &f3s1tb1tcb, "fused3S 1tb1tcb");
  m.def("f3s_1tb1rw", &f3s1tb1rw, "fused3S 1tb1rw");
  m.def("f3s_1tb1rw_scheduled", &f3s1tb1rwScheduled, "fused3S 1tb1rw scheduled");
  m.def("f3s_1tb1rw_scheduled_permuteV", &f3s1tb1rwScheduledPermuteV,
        "fused3S 1tb1rw scheduled permuteV");
  m.def("f3s_1tb1rw_scheduled_permuteV_scaleQK", &f3s1tb1rwScheduledPermuteVScaleQK,
        "fused3S 1tb1rw scheduled permuteV scaleQK");
  m.def("f3s_multihead_scaleQK", &f3sMultiHeadScaleQK,
        "fused3S over [N, heads, d] Q/K/V in one launch (fp16 or bf16), heavy-first order");
  m.def("release_workspace", &releaseWorkspace,
        "free the cached scratch of the column-sliced schedule; returns the bytes released");
}
