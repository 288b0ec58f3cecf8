"""hot_amd -- MI355X-native (gfx950) HOT linear-layer backward.

Layout:
  csrc/            HIP kernels and the C ABI (built into libhot_gfx950.so)
  _lib.py          ctypes binding of the C ABI
  ops.py           tensor-level wrappers of each entry point
  hadamard_matmul  transform helpers with the reference's names
  args             module-global options with the reference's names
  quant_matmul     FLinearQ / HQ_Linear on the native path
  HLQ_backward     backward(Go, W, X, ...) drop-in op
"""
__version__ = "0.1.0"
