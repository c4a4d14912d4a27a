"""Activation matching: the operator in front of a switched linear produces the activation format that the
linear's lane needs (README.md:23-27 of the reference: "Kairos propagates the required precision to the
quantization operator to directly produce the needed format ... When the target precision matches the original
FP16, the quantization step is simply skipped").

The reference's modules quantise inside `_forward` (kairos/dynamic_linear.py:150-152); here the decoder's RMSNorm
asks its consumers which lane they will take for this token count and emits fp16, int8 + per-token scales, or
both, from one read of the hidden state (`kmi_rmsnorm_quant_act`); the SiLU(gate) * up in front of the down
projection does the same (`kmi_silu_mul_quant_act`).  A `MatchedActivation` carries the result to
`DynamicLinear.forward`, which skips its own quantiser when the int8 form is already there.
"""
import torch

from . import ops
from .dynamic_linear import _W4A8, _W8A8, DynamicLinear


class MatchedActivation:
    """Output of MatchedRMSNorm: `f16` (fp16 [..., K]) and / or `int_x` (int8 [..., K]) with `scale_x` (fp16 [tokens])."""
    __slots__ = ("f16", "int_x", "scale_x", "shape")

    def __init__(self, f16, int_x, scale_x):
        self.f16, self.int_x, self.scale_x = f16, int_x, scale_x
        self.shape = (f16 if f16 is not None else int_x).shape

    def numel(self):
        return (self.f16 if self.f16 is not None else self.int_x).numel()


def _formats_for(consumers, m):
    """(want_f16, want_i8) for m tokens: int8 if a consumer's lane takes int8 activations (W8A8, W4A8), fp16 if one is anything else."""
    want_f16 = want_i8 = False
    for lin in consumers:
        comp = type(lin).prof.get_comp_type(lin.shape, m) if isinstance(lin, DynamicLinear) else None
        if comp in (_W8A8, _W4A8):
            want_i8 = True
        else:
            want_f16 = True
    return want_f16, want_i8


class MatchedRMSNorm(torch.nn.Module):
    """RMSNorm whose output format follows its consumers' lanes.

    norm: a module with `.weight` and `.variance_epsilon` or `.eps` (Llama / Qwen RMSNorm); consumers: the switched
    linears that read this norm's output (q/k/v or gate/up).  forward(x, residual=None) returns
    (MatchedActivation, h) with h = fp16(x + residual) (None without a residual).
    """

    def __init__(self, weight, eps, consumers):
        super().__init__()
        self.weight = weight
        self.eps = float(eps)
        self.consumers = list(consumers)          # a plain list: the linears stay owned by their parent modules

    @classmethod
    def from_module(cls, norm, consumers):
        eps = getattr(norm, "variance_epsilon", None)
        if eps is None:
            eps = norm.eps
        return cls(norm.weight, eps, consumers)

    def formats_for(self, m):
        return _formats_for(self.consumers, m)

    @torch.no_grad()
    def forward(self, x, residual=None):
        K = x.shape[-1]
        want_f16, want_i8 = self.formats_for(x.numel() // K)
        y, int_x, scale_x, h = ops.rmsnorm_quant(x, self.weight, self.eps, residual, want_f16, want_i8)
        return MatchedActivation(y, int_x, scale_x), h


class MatchedSiluMul(torch.nn.Module):
    """SiLU(gate) * up in front of the down projection, in the format of that projection's lane.
    forward(gate_up [..., 2*I], gate first) -> MatchedActivation [..., I]."""

    def __init__(self, consumers):
        super().__init__()
        self.consumers = list(consumers)

    def formats_for(self, m):
        return _formats_for(self.consumers, m)

    @torch.no_grad()
    def forward(self, gate_up):
        want_f16, want_i8 = self.formats_for(gate_up.numel() // gate_up.shape[-1])
        return MatchedActivation(*ops.silu_mul_quant(gate_up, want_f16, want_i8))
