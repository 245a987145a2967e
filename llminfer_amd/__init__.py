"""MI355X (gfx950) decode-phase grouped-query attention: HIP kernels behind a C ABI.

The product is libllmi_hip.so (see include/llmi_hip.h); this package holds its
sources (csrc/), the build recipe, a ctypes binding and a thin torch front end
used by the tests and the benchmark.
"""
from . import _binding  # noqa: F401
from ._binding import (KV_LAYOUT_HEAD_MAJOR, KV_LAYOUT_POS_MAJOR, PATH_AUTO, PATH_SINGLE_PASS,  # noqa: F401
                       PATH_SPLIT, PATH_SPLIT_FUSED, LlmiError, lib)

__all__ = ["lib", "LlmiError", "KV_LAYOUT_POS_MAJOR", "KV_LAYOUT_HEAD_MAJOR", "PATH_AUTO",
           "PATH_SINGLE_PASS", "PATH_SPLIT", "PATH_SPLIT_FUSED"]
