"""DynamicLinear, version-2 id table (kairos/dynamic_linear_v2.py:11-13,43-228).

Version 2 of the reference adds two third-party candidates: `w4a16_marlin` (6), a second W4A16 tensor-core kernel,
and `w4a8_qserve` (7), int8 activations against int4 weights (a re-pack of the resident tensor on every call plus a
third-party GEMM with its own second-level quantiser).  On this hardware there is one W4A16 MFMA GEMM, so id 6 runs
it (tables profiled upstream stay loadable), and id 7 is this library's W4A8 lane: the activation quantiser and an
int8 MFMA GEMM that decodes the resident int4 weight to exactly the int8 weight of the W8A8 lane while staging it --
no re-pack, no converted copy, results bit-identical to the W8A8 lane.  Both ids are handled by the base class.

`from_module(..., qserve_factors=True)` keeps the reference's own operands for id 7 instead: the integer per-group
factors and the per-channel scale of its second quantiser (kairos/dynamic_linear_v2.py:103 -> thirdparty/Qserve/
w4a8_linear.py:175-262), three more buffers, and id 7 then multiplies the resident nibbles with them exactly as the
reference's GEMM does (`kmi_gemm_w4a8_int`) -- still without the re-pack in front.
"""
import torch

from . import dynamic_linear as _v1
from . import ops
from .weight_prep import qserve_factor_tables

QSERVE_KEYS = ("qserve_s1_scales", "qserve_s2_scales", "qserve_s2_zeros")

COMP_TYPE_NAME = {'w4a16_gemm': 0, 'w4a16_gemv': 1, 'w8a8': 2,
                  'w8a16_gemm': 3, 'w8a16_gemv': 4,
                  'fp16': 5, 'w4a16_marlin': 6, 'w4a8_qserve': 7}


class DynamicLinear(_v1.DynamicLinear):
    prof = None

    def __init__(self, in_features, out_features, bias, device, group_size):
        super().__init__(in_features, out_features, bias, device, group_size)
        for key in QSERVE_KEYS:                  # None unless from_module(qserve_factors=True) or a state dict fills them
            self.register_buffer(key, None)

    @classmethod
    @torch.no_grad()
    def from_module(cls, linear, device, return_dtype=torch.float16, init_only=False, name='', qserve_factors=False):
        q_linear = super().from_module(linear, device, return_dtype, init_only, name)
        if qserve_factors:
            N, K = q_linear.shape
            if init_only:
                q_linear.qserve_s1_scales = torch.empty((N,), dtype=torch.float16, device=device)
                q_linear.qserve_s2_scales = torch.empty((K // 128, N), dtype=torch.int8, device=device)
                q_linear.qserve_s2_zeros = torch.empty((K // 128, N), dtype=torch.int8, device=device)
            else:
                # on the host: elementwise fp32 division on the GPU is not correctly rounded, which would flip ties
                t = qserve_factor_tables(linear.weight.data, group_size=128)
                q_linear.qserve_s1_scales = t["s1_scales"].to(device)
                q_linear.qserve_s2_scales = t["s2_scales"].to(device)
                q_linear.qserve_s2_zeros = t["s2_zeros"].to(device)
        return q_linear

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        for key in QSERVE_KEYS:                  # plain constructor: take the tensors' shapes from the file
            if getattr(self, key) is None and prefix + key in state_dict:
                src = state_dict[prefix + key]
                dev = self.qweight.device if self.qweight is not None else (src.device if self.bias is None else self.bias.device)
                setattr(self, key, torch.empty_like(src, device=dev))
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    def _w4a8(self, x, int_x, scale_x):
        if self.qserve_s2_scales is None:
            return super()._w4a8(x, int_x, scale_x)
        N, K = self.shape
        if int_x is None:
            int_x = torch.empty_like(x, dtype=torch.int8)
            scale_x = torch.empty((x.shape[0],), device=x.device, dtype=torch.float16)
            ops.quant_fp16_to_int8(int_x, x, scale_x)
        out = torch.empty((int_x.shape[0], N), device=int_x.device, dtype=torch.float16)
        ops.w4a8_int_gemm_forward(int_x, self.qweight, self.qserve_s2_scales, self.qserve_s2_zeros, self.qserve_s1_scales,
                                  scale_x, out, bias=self.bias)
        return out

    @torch.no_grad()
    def _trans_weight_to_8(self):
        self._cache().invalidate()
        return self._converted('i8')[0]

    @torch.no_grad()
    def _trans_weight_to_16(self):
        self._cache().invalidate()
        return self._converted('f16')[0]
