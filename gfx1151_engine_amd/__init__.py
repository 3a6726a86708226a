"""MI355X-native routed-expert MoE layer behind gfx1151-engine's MoE entry points.

The product is libmi355moe.so (HIP kernels + C++ host code, C ABI in include/mi355_moe.h);
this package only builds it and binds it for the tests and the benchmark.
"""
from .build import LIB, LIB_TIMING, build, build_all  # noqa: F401
