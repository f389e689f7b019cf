"""MI355X (gfx950) native kernels for the quantized-linear hot path of LLMQRT.

Layout:
  csrc/            HIP kernels + C ABI (include/llmq.h) -> lib/libllmq_gfx950.so
  _abi.py          ctypes loader (no fallback: a missing library raises)
  quantize.py      activation quantizers (reference names)
  norm.py          RMSNorm, alone or fused with the per-token quantizer
  sq_fp8_kernels   drop-in for runtime.sq_fp8_kernels
  awq_kernels      drop-in for runtime.triton_kernels.awq_kernels
  linear/          quantized Linear modules + registry
  fused_utils.py   fuse q/k/v or gate/up sibling modules into one
  checkpoint.py    QuantConfig, nn.Linear replacement and by-name loading of safetensors checkpoints
  workloads.py     seeded synthetic inputs of the benchmark configurations
"""
__version__ = "0.1.0"
