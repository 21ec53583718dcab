"""MI355X-native mixture-of-experts layer forward (HIP, gfx950) behind a C ABI.

The product is `libatenia_moe_hip.so` (sources in `csrc/`, interface in
`include/atenia_moe_hip.h`).  `capi` is a thin ctypes binding of that C ABI used by
the tests and the benchmark; it adds no arithmetic of its own.
"""
from . import capi  # noqa: F401

__all__ = ["capi"]
