"""Profiler for the version-2 id table (kairos/perf_profiler_v2.py).

The reference's v2 adds a pre-pass that chooses between two resident W4A16 packings (its own and Marlin's) and two
third-party candidates.  There is a single resident packing and a single W4A16 GEMM here, so v2 differs from v1 in
the id table it records, in the linear class it times and in one more candidate: `w4a8_qserve` (id 7), the W4A8 lane.
"""
from . import perf_profiler as _v1
from .dynamic_linear_v2 import COMP_TYPE_NAME, DynamicLinear
from .perf_profiler import LUT, compress_segments, test_perf  # noqa: F401  (same helpers, re-exported)


class Profiler(_v1.Profiler):
    comp_type_name = COMP_TYPE_NAME
    linear_cls = DynamicLinear
    comp_types = _v1.DEFAULT_COMP_TYPES + ['w4a8_qserve']
