"""Applying stored smoothing scales before quantisation (kairos/smooth_scale.py:33-63).

The reference searches per-input-channel scales on calibration data (`smooth_scale`, a grid search over simulated
quantisers that needs a tokenizer, a dataset and the third-party fake-quant layers) and stores them as
`scales_meta_data[layer] = [(prev_op_name, [linear names], scales[1, K]), ...]` (dumped as q_scales.pt,
kairos/main.py:88).  Only the deterministic half is part of this build: folding such scales into the weights,
W' = W * s for the listed linears and prev' = prev / s for the operator that feeds them, which leaves the fp16
function of the layer unchanged and is what runs right before `quantize_model`.  The search itself is not built.
"""
import torch

from .quant_model import get_name_linears


@torch.no_grad()
def get_op_by_name(module, op_name):
    for name, m in module.named_modules():
        if name == op_name:
            return m
    raise ValueError(f"Cannot find op {op_name} in module {module}")


def _is_norm(op):
    return isinstance(op, torch.nn.LayerNorm) or type(op).__name__.endswith("RMSNorm")


@torch.no_grad()
def _apply_scale_block(layer, prev_op, child_names, best_scales):
    prev = get_op_by_name(layer, prev_op)
    name2linears = get_name_linears(layer)
    for name in child_names:
        linear = name2linears[name]
        s = best_scales.to(device=linear.weight.device, dtype=linear.weight.dtype)
        linear.weight.mul_(s.view(1, -1))
        if torch.isnan(linear.weight).any():
            raise ValueError(f"NaN in {name} after scaling")
    s = best_scales.to(device=prev.weight.device, dtype=prev.weight.dtype).view(-1)
    if isinstance(prev, torch.nn.Linear):
        prev.weight.div_(s.view(-1, 1))
        if prev.bias is not None:
            prev.bias.div_(s)
    elif _is_norm(prev):
        prev.weight.div_(s)
        if getattr(prev, "bias", None) is not None:
            prev.bias.div_(s)
    else:
        raise NotImplementedError(f"Prev_op {type(prev)} not supported yet.")
    for w in prev.parameters():
        if torch.isnan(w).any():
            raise ValueError(f"NaN in {prev_op} after scaling")


@torch.no_grad()
def apply_scale(model, scales_meta_data):
    """Folds stored scales into `model` in place; call before `quantize_model`."""
    for layer, blocks in zip(model.model.layers, scales_meta_data):
        for prev_op, child_names, scales in blocks:
            _apply_scale_block(layer, prev_op, child_names, scales)
