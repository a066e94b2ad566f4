"""hiptensor_amd: an MI355X (gfx950) implementation of hipTensor's tensor-contraction path.

The product is libhiptensor_amd.so (hand-written HIP kernels + host planner, C++ API
compatible with hipTensor 1.4 and a flat C ABI); this package is its Python binding plus
the definitions of the benchmark workloads.
"""
from .api import *  # noqa: F401,F403
from . import api, workloads  # noqa: F401
