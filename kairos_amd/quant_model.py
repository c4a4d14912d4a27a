"""Model surgery: every torch.nn.Linear inside the decoder layers becomes a switched linear
(kairos/quant_model.py:8-56).

`quantize_model(model)` quantises in place and returns the per-layer {linear name: type} list that the
reference dumps as quant_config.json; `quantize_model(model, init_only=True, _quant_config=cfg)` rebuilds the
same module tree with empty resident tensors, the target of `load_state_dict` / `load_checkpoint_in_model`
(utils/load_model.py:15-29).  The type is chosen per call (`quant_strategy`) instead of from a process-wide
command-line global.
"""
import gc

import torch

from .quant_config import LinearQuantConfig


@torch.no_grad()
def get_name_linears(module):
    return {name: m for name, m in module.named_modules() if isinstance(m, torch.nn.Linear)}


@torch.no_grad()
def set_op_by_name(layer, name, new_module):
    levels = name.split(".")
    mod_ = layer
    for level in levels[:-1]:
        mod_ = mod_[int(level)] if level.isdigit() else getattr(mod_, level)
    setattr(mod_, levels[-1], new_module)


@torch.no_grad()
def quantize_model(model, init_only=False, _quant_config=None, quant_strategy='DynamicLinear', version='1'):
    """Replaces the linears of `model.model.layers[i]`; returns [{name: quant_type}] per layer."""
    quant_config = []
    device = model.device
    for layer_idx, layer in enumerate(model.model.layers):
        quant_config.append({})
        for name, module in get_name_linears(layer).items():
            quant_type = _quant_config[layer_idx][name] if _quant_config is not None else quant_strategy
            quant_config[layer_idx][name] = quant_type
            q_linear = LinearQuantConfig(quant_type, version).from_module(module, device, init_only=init_only)
            if init_only is False:
                module.cpu()
            set_op_by_name(layer, name, q_linear)
        if device.type == 'cuda':
            torch.cuda.empty_cache()
        gc.collect()
    return quant_config
