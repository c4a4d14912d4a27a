"""SwitchLinear: the keep-everything-resident variant (kairos/switch_linear.py:43-213).

Same interface as DynamicLinear, but the int8 and fp16 copies of the weight are produced once in
from_module and stay in HBM, so no lane pays a conversion at call time (the "oracle" ablation of the
reference: fastest, largest footprint).
"""
import torch

from . import ops
from .dynamic_linear_v2 import COMP_TYPE_NAME, DynamicLinear


class SwitchLinear(DynamicLinear):
    prof = None

    @classmethod
    @torch.no_grad()
    def from_module(cls, linear, device, return_dtype=torch.float16, init_only=False, name=''):
        q = super().from_module(linear, device, return_dtype, init_only, name)
        if init_only:
            return q
        tiled = q._tileable()
        q.smq_weight = torch.empty(q.shape, dtype=torch.int8, device=device)
        ops.dequant_interleaved_int4_to_int8(q.smq_weight, q.qweight, q.scales_to8, q.scaled_zeros_to8, 128, tiled=tiled)
        q.ori_weight = torch.empty(q.shape, dtype=torch.float16, device=device)
        ops.dequant_interleaved_int4_to_fp16(q.ori_weight, q.qweight, q.scales, q.scaled_zeros, 128, tiled=tiled)
        q._resident_tiled = tiled
        if tiled:       # the W8A16 lane reads row-major int8
            q.smq_weight_rowmajor = torch.empty(q.shape, dtype=torch.int8, device=device)
            ops.dequant_interleaved_int4_to_int8(q.smq_weight_rowmajor, q.qweight, q.scales_to8, q.scaled_zeros_to8, 128)
        return q

    def _converted(self, fmt, tiled=None):
        if fmt == 'i8' and tiled is False and self._resident_tiled:
            return self.smq_weight_rowmajor, False
        return (self.smq_weight if fmt == 'i8' else self.ori_weight), self._resident_tiled
