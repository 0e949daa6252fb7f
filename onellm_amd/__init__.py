"""MI355X (gfx950) backend for oneLLM's per-token decode hot path.

The product is two shared libraries built from `csrc/`:
  libonellm_hip.so        the C ABI declared in include/onellm_hip.h (hand-written HIP kernels)
  libonellm_launchers.so  oneLLM's six launch* functions, same signatures, over that C ABI
`capi` binds the C ABI with ctypes for tests and benchmarks; it raises if the library is missing
and has no fallback path.
"""
from . import capi  # noqa: F401

__all__ = ["capi"]
