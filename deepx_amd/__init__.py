"""deepx op-mem-hip: an MI355X-native deepxIR executor.

  csrc/       hand-written HIP kernels + the C ABI (libdxhip.so, include/dxhip.h)
  executor/   the C++ host: deepxIR parser, TfFactory, Mem, UDP server (deepx-executor-hip)
  lib.py      ctypes view of the C ABI for harnesses
"""
__all__ = ["lib"]
