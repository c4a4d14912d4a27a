"""Linear-type registry of the model surgery (kairos/quant_config.py:20-60).

The reference registers its own two layers next to five third-party baselines (SmoothQuant, AWQ, Marlin,
QServe, QQQ linears).  Only the switched layers are part of this build; the baseline names are recognised
and refused with a message that says so.
"""
import torch

from .dynamic_linear import DynamicLinear
from .switch_linear import SwitchLinear

THIRD_PARTY_BASELINES = ("W8A8Linear", "W4A16Linear", "W4A16Linear_Marlin", "W4A8Linear", "W4A8Linear_QQQ")


class TensorQuantConfig:
    @torch.no_grad()
    def __init__(self, q_bit, qtype=None, group_size=-1):
        self.bit = q_bit
        self.qtype = qtype          # 'A'symmetric or 'S'ymmetric
        self.group_size = group_size


class LinearQuantConfig:
    @torch.no_grad()
    def __init__(self, quant_type, version='1'):
        self.x = TensorQuantConfig(8, 'S')
        self.w = TensorQuantConfig(4, 'A', group_size=128)
        if quant_type == 'DynamicLinear':
            if str(version) == '2':
                from .dynamic_linear_v2 import DynamicLinear as DynamicLinearV2
                self.from_module = DynamicLinearV2.from_module
            else:
                self.from_module = DynamicLinear.from_module
        elif quant_type == 'SwitchLinear':
            self.from_module = SwitchLinear.from_module
        elif quant_type in THIRD_PARTY_BASELINES:
            raise NotImplementedError(f"{quant_type} is a third-party baseline of the reference, not part of this build "
                                      f"(available: DynamicLinear, SwitchLinear)")
        else:
            raise ValueError(f"No Supported Linear Type: {quant_type}.")
