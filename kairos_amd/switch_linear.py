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
    resident_copies = True

    def init(self):
        super().init()
        self._resident = None           # (int8 weight, fp16 weight, tiled), built on first use
        self._w8_rows = None            # row-major int8 for the W8A16 lane, built when that lane is first asked for

    def _ensure_resident(self):
        """The int8 and fp16 copies are derived data: not part of state_dict, rebuilt after a load or a move."""
        if getattr(self, "_resident", None) is None:
            dev, tiled = self.qweight.device, self._tileable()
            w8 = torch.empty(self.shape, dtype=torch.int8, device=dev)
            ops.dequant_interleaved_int4_to_int8(w8, self.qweight, self.scales_to8, self.scaled_zeros_to8, 128, tiled=tiled)
            w16 = torch.empty(self.shape, dtype=torch.float16, device=dev)
            ops.dequant_interleaved_int4_to_fp16(w16, self.qweight, self.scales, self.scaled_zeros, 128, tiled=tiled)
            self._resident = (w8, w16, tiled)
        return self._resident

    def resident_bytes(self):
        """Bytes of HBM this layer holds: the packed weight and its tables plus every converted copy built so far."""
        held = [getattr(self, k) for k in ("qweight", "scales", "scaled_zeros", "scales_to8", "scaled_zeros_to8", "scales_1", "bias")]
        held += list(getattr(self, "_resident", None) or ())[:2] + [getattr(self, "_w8_rows", None)]
        return sum(t.numel() * t.element_size() for t in held if isinstance(t, torch.Tensor))

    @property
    def smq_weight(self):               # names of the reference's attributes (kairos/switch_linear.py:43-213)
        return self._ensure_resident()[0]

    @property
    def ori_weight(self):
        return self._ensure_resident()[1]

    @classmethod
    @torch.no_grad()
    def from_module(cls, linear, device, return_dtype=torch.float16, init_only=False, name=''):
        q = super().from_module(linear, device, return_dtype, init_only, name)
        if not init_only and torch.device(device).type == 'cuda':
            q._ensure_resident()
        return q

    def _converted(self, fmt, tiled=None):
        w8, w16, res_tiled = self._ensure_resident()
        if fmt == 'i8' and tiled is False and res_tiled:    # the W8A16 lane reads row-major int8
            if getattr(self, "_w8_rows", None) is None:
                self._w8_rows = torch.empty(self.shape, dtype=torch.int8, device=self.qweight.device)
                ops.dequant_interleaved_int4_to_int8(self._w8_rows, self.qweight, self.scales_to8, self.scaled_zeros_to8, 128)
            return self._w8_rows, False
        return (w8 if fmt == 'i8' else w16), res_tiled
