"""DynamicLinear, version-2 id table (kairos/dynamic_linear_v2.py:11-13,43-228).

Version 2 of the reference adds two third-party candidates: `w4a16_marlin` (6), a second W4A16
tensor-core kernel, and `w4a8_qserve` (7).  On this hardware there is one W4A16 MFMA GEMM, so id 6
runs it (tables profiled upstream stay loadable); id 7 has no kernel here and is rejected.
"""
import torch

from . import dynamic_linear as _v1

COMP_TYPE_NAME = {'w4a16_gemm': 0, 'w4a16_gemv': 1, 'w8a8': 2,
                  'w8a16_gemm': 3, 'w8a16_gemv': 4,
                  'fp16': 5, 'w4a16_marlin': 6, 'w4a8_qserve': 7}


class DynamicLinear(_v1.DynamicLinear):
    prof = None

    @torch.no_grad()
    def _forward(self, input, batch_token_len, comp_type):
        if comp_type == COMP_TYPE_NAME['w4a16_marlin']:
            comp_type = COMP_TYPE_NAME['w4a16_gemm']
        elif comp_type == COMP_TYPE_NAME['w4a8_qserve']:
            raise NotImplementedError("w4a8_qserve has no kernel in this build")
        return super()._forward(input, batch_token_len, comp_type)

    @torch.no_grad()
    def _trans_weight_to_8(self):
        self._cache().invalidate()
        return self._converted('i8')[0]

    @torch.no_grad()
    def _trans_weight_to_16(self):
        self._cache().invalidate()
        return self._converted('f16')[0]
