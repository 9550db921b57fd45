"""MI355X-native `hip` backend for the `mops` operator library of nano_vllm_ninetoothed.

Layout
  csrc/      hand-written gfx950 HIP kernels and the C-ABI launchers (include/mops_hip.h)
  build.py   hipcc driver producing lib/libmops_hip.so in-tree
  _capi.py   ctypes binding of the C ABI (no fallback: missing library is an error)
  mops/      host-side mirror of the reference's op registry with the `hip` backend registered
"""
__version__ = "0.1.0"
