"""DynamicLinear, version-2 id table (kairos/dynamic_linear_v2.py:11-13,43-228).

Version 2 of the reference adds two third-party candidates: `w4a16_marlin` (6), a second W4A16 tensor-core kernel,
and `w4a8_qserve` (7), int8 activations against int4 weights (a re-pack of the resident tensor on every call plus a
third-party GEMM with its own second-level quantiser).  On this hardware there is one W4A16 MFMA GEMM, so id 6 runs
it (tables profiled upstream stay loadable), and id 7 is this library's W4A8 lane: the activation quantiser and an
int8 MFMA GEMM that decodes the resident int4 weight to exactly the int8 weight of the W8A8 lane while staging it --
no re-pack, no converted copy, results bit-identical to the W8A8 lane.  Both ids are handled by the base class.
"""
import torch

from . import dynamic_linear as _v1

COMP_TYPE_NAME = {'w4a16_gemm': 0, 'w4a16_gemv': 1, 'w8a8': 2,
                  'w8a16_gemm': 3, 'w8a16_gemv': 4,
                  'fp16': 5, 'w4a16_marlin': 6, 'w4a8_qserve': 7}


class DynamicLinear(_v1.DynamicLinear):
    prof = None

    @torch.no_grad()
    def _trans_weight_to_8(self):
        self._cache().invalidate()
        return self._converted('i8')[0]

    @torch.no_grad()
    def _trans_weight_to_16(self):
        self._cache().invalidate()
        return self._converted('f16')[0]
