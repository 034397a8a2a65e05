"""inferspore_amd -- MI355X (gfx950) implementation of InferSpore's fused per-layer kernels.

The product is the C-ABI shared library `lib/libinferspore_amd.so` (declared in
include/inferspore_amd.h) plus the C++ `launch*` shims in `lib/libinferspore_launch.so`.  This Python
package is plumbing over that ABI: `capi` loads the library with ctypes, `ops` calls it on torch
tensors (torch supplies device memory and streams only).  There is no CPU or eager fallback: if the
library is missing or no GPU is present, calls raise.
"""
from . import capi  # noqa: F401

__all__ = ["capi", "ops"]


def __getattr__(name):
    if name == "ops":
        import importlib
        return importlib.import_module(".ops", __name__)
    raise AttributeError(name)
