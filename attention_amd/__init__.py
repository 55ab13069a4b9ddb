"""attention_amd: MI355X (gfx950) FlashAttention-forward and PagedAttention-decode kernels.

The product is two shared libraries built from this directory:
  lib/libahpc_hip.so       the HIP kernels behind the C ABI of include/ahpc_hip.h
  lib/libattention_hpc.so  the C++ host classes (AttentionInterface / BackendFactory /
                           PagedAttention sequence API) that call that C ABI
`attention_amd.hip` is a thin ctypes view of the C ABI for Python harnesses (tests, bench).
There is no CPU fallback: loading fails loudly when the library has not been built.
"""
from . import hip  # noqa: F401
