"""MI355X-native diagonal-sparse (DIA) matrix products behind CUV's interface.

The compute lives in lib/libcuvdia.so (hand-written HIP for gfx950, C ABI in
include/cuvdia.h).  `cuv_amd.dia` is the Python surface, `cuv_amd/include/cuv`
the C++ one; `cuv_amd.workloads` generates the measured configurations and `cuv_amd.io`
saves and loads DIA matrices.
"""
from . import _lib  # noqa: F401

__all__ = ["_lib", "dia", "io", "workloads"]
