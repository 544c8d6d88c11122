"""byteir_amd -- MI355X-native op-kernel provider for ByteIR's runtime (BRT).

The package is a thin Python host layer over three in-tree shared libraries:

  lib/libbrt_rocm_kernels.so  HIP kernels + device plumbing behind a C ABI (include/brt_rocm_kernels.h)
  lib/libflash_attn.so        drop-in for the reference's flash-attention custom library
                              (VERSION, run_flash_attn_fwd, run_flash_attn_bwd; include/flash_api.h)
  lib/libbrt.so               BRT-shaped C++ host runtime: ByRE text reader, kernel registry, ROCm
                              execution provider, session / request context (include/brt_c_api.h)

There is no CPU fallback: every entry point raises if its library is missing.
"""
from . import _lib  # noqa: F401

__all__ = ["_lib"]
