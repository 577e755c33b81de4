"""MI355X-native Fused3S: TC-block preprocessing and fused SDDMM -> softmax -> SpMM attention.

Layout
  csrc/            hand-written HIP kernels (gfx950) + the C ABI of libf3s_amd.so + the torch
                   extension source that re-creates the reference's `F3S` operator module
  capi.py          ctypes binding of the C ABI on torch device tensors
  synth.py         synthetic graphs / features of the benchmark configurations
  build.py         in-tree build (hipcc, g++)
After `python -m fused3s_amd.build`, `from fused3s_amd import F3S` gives the drop-in operator
module (preprocess_gpu, f3s_1tb1rw, f3s_1tb1rw_scheduled, f3s_1tb1rw_scheduled_permuteV,
f3s_1tb1rw_scheduled_permuteV_scaleQK, f3s_1tb1tcb).
"""
__all__ = ["capi", "synth", "build"]
