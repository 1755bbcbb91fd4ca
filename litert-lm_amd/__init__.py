"""MI355X-native attention path for LiteRT-LM style executors.

The directory name carries a hyphen, so the package is loaded by path (see
``__graft_entry__.load_package``) and registers itself as ``litert_lm_amd``.

    attn      ctypes binding of libmi355_attn.so (the C ABI in include/mi355_attn.h)
    executor  ctypes binding of the C++ HipLlmExecutor test surface
    sampler   ctypes binding of libmi355_sampler.so (the C ABI in include/mi355_sampler.h)
"""
from . import attn  # noqa: F401
from . import executor  # noqa: F401
from . import sampler  # noqa: F401

__all__ = ["attn", "executor", "sampler"]
