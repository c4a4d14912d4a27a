"""Activation-aware smoothing before quantisation (kairos/smooth_scale.py).

`smooth_scale(model, inputs)` searches, layer by layer on calibration activations, per-input-channel scales s that
move quantisation difficulty from the activations into the weights: for the three blocks of a decoder layer
(q/k/v behind the input norm, gate/up behind the post-attention norm, down behind up_proj) it tries
s = mean|x|^r, r = 0, 1/20 .. 19/20, normalised by sqrt(max * min), runs the block with the listed linears replaced by
quantised probes computing q(W * s) . (x / s), and keeps the r with the smallest squared error against the
unquantised block (kairos/smooth_scale.py:66-160).  The result, `scales_meta_data[layer] = [(prev_op_name,
[linear names], scales[1, K]), ...]` (dumped upstream as q_scales.pt, kairos/main.py:88), is what `apply_scale` folds
into the model: W' = W * s for the listed linears and prev' = prev / s for the operator that feeds them, which
leaves the fp16 function of the layer unchanged and runs right before `quantize_model`.

The probe.  Upstream the probe is a third-party simulated W4A8 layer; here it is the library's own quantised linear:
`DynamicLinear.from_module` of the scaled weight, evaluated through one fixed lane with int8 activations (the W4A8
lane by default: the operand precisions smoothing is meant for), so the search minimises the error of the kernels
that will run.  `make_probe` replaces it, e.g. by `fake_quant_probe` (plain torch arithmetic of the same scheme:
per-token int8 activations, group-wise asymmetric int4 weights) where no GPU is present.
"""
import functools

import torch

from .quant_model import get_name_linears, set_op_by_name


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


# ---- the search (kairos/smooth_scale.py:66-160) -----------------------------------------------------------------------
N_GRID = 20


class _Probe(torch.nn.Module):
    """q(W * s) applied to x / s (kairos/simu_quant.py:4-31)."""

    def __init__(self, proj, scales):
        super().__init__()
        self.proj, self.scales = proj, scales

    @torch.no_grad()
    def forward(self, x):
        return self.proj(x / self.scales.to(dtype=x.dtype, device=x.device))


def library_probe(linear, scales, lane='w4a8_qserve'):
    """The library's quantised linear of the scaled weight, pinned to one lane (default: int8 activations against the
    int4 weight).  Needs the GPU the linear lives on."""
    from .dynamic_linear_v2 import COMP_TYPE_NAME, DynamicLinear
    scaled = torch.nn.Linear(linear.in_features, linear.out_features, bias=linear.bias is not None,
                             dtype=linear.weight.dtype, device=linear.weight.device)
    scaled.weight.data.copy_(linear.weight.data * scales.to(device=linear.weight.device, dtype=linear.weight.dtype))
    if linear.bias is not None:
        scaled.bias.data.copy_(linear.bias.data)
    q = DynamicLinear.from_module(scaled, linear.weight.device)
    cid = COMP_TYPE_NAME[lane]

    def run(x):
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1]).to(torch.float16).contiguous()
        return q._forward(x2, x2.shape[0], cid).reshape(*lead, -1).to(x.dtype)
    return _Probe(run, scales)


def fake_quant_probe(linear, scales, group_size=128):
    """The same scheme in plain torch arithmetic (no kernels): weights to asymmetric int4 per group of `group_size`
    input channels and back, activations to symmetric int8 per token and back, product in the linear's own dtype."""
    w = (linear.weight.data * scales.to(device=linear.weight.device, dtype=linear.weight.dtype)).float()
    N, K = w.shape
    g = w.reshape(N, K // group_size, group_size)
    lo, hi = g.amin(-1, keepdim=True), g.amax(-1, keepdim=True)
    step = ((hi - lo).clamp(min=1e-5) / 15)
    wq = (torch.clamp(torch.round((g - lo) / step), 0, 15) * step + lo).reshape(N, K).to(linear.weight.dtype)
    bias = linear.bias

    def run(x):
        xf = x.float()
        s = xf.abs().amax(-1, keepdim=True).clamp(min=1e-7) / 127
        xq = (torch.clamp(torch.round(xf / s), -128, 127) * s).to(x.dtype)
        return torch.nn.functional.linear(xq, wq.to(x.dtype), bias)
    return _Probe(run, scales)


@torch.no_grad()
def _smooth_scale_block(layer, prev_op, child_names, input, detected_module, detected_input=None, kwargs=None,
                        make_probe=library_probe):
    """One block: -> (name of prev_op, child names, best scales [1, K]) (kairos/smooth_scale.py:66-104)."""
    kwargs = kwargs or {}
    act_magnitude = input.abs().reshape(-1, input.shape[-1]).float().mean(0)
    if detected_input is None:
        detected_input = input
    ref_out = detected_module(detected_input, **kwargs)
    if isinstance(ref_out, tuple):
        ref_out = ref_out[0]
    name2linears = get_name_linears(layer)
    best_loss, best_scales = float("inf"), None
    try:
        for ratio in range(N_GRID):
            scales = act_magnitude.pow(ratio / N_GRID).clamp(min=1e-4).view(-1)
            scales = (scales / (scales.max() * scales.min()).sqrt()).view(1, -1)
            for name in child_names:
                set_op_by_name(layer, name, make_probe(name2linears[name], scales))
            cur_out = detected_module(detected_input, **kwargs)
            if isinstance(cur_out, tuple):
                cur_out = cur_out[0]
            loss = (ref_out.reshape(-1) - cur_out.reshape(-1)).float().pow(2).mean().item()
            if loss < best_loss:
                best_loss, best_scales = loss, scales
    finally:
        for name in child_names:                       # the original linears come back whatever happened
            set_op_by_name(layer, name, name2linears[name])
    prev_name = next(name for name, m in layer.named_modules() if m is prev_op)
    return prev_name, list(child_names), best_scales


@torch.no_grad()
def smooth_scale_layer(layer, layer_kwargs, activations, make_probe=library_probe):
    """The three blocks of a Llama / Qwen decoder layer (kairos/smooth_scale.py:106-132)."""
    block = functools.partial(_smooth_scale_block, layer, make_probe=make_probe)
    return [
        block(layer.input_layernorm, ['self_attn.q_proj', 'self_attn.k_proj', 'self_attn.v_proj'],
              activations['self_attn.q_proj'], layer.self_attn, kwargs=layer_kwargs),
        block(layer.post_attention_layernorm, ['mlp.gate_proj', 'mlp.up_proj'], activations['mlp.gate_proj'], layer.mlp),
        block(layer.mlp.up_proj, ['mlp.down_proj'], activations['mlp.down_proj'], layer.mlp,
              detected_input=activations['mlp.gate_proj']),
    ]


class _Caught(Exception):
    pass


@torch.no_grad()
def catch_embedding_output(model, inputs):
    """Hidden states and keyword arguments that reach the first decoder layer (kairos/catch_tensor.py:9-31)."""
    caught = {}

    def hook(module, args, kwargs):
        caught["hidden"] = args[0] if args else kwargs["hidden_states"]
        caught["kwargs"] = {k: v for k, v in kwargs.items() if k != "hidden_states"}
        raise _Caught

    handle = model.model.layers[0].register_forward_pre_hook(hook, with_kwargs=True)
    try:
        model(**inputs)
    except _Caught:
        pass
    finally:
        handle.remove()
    return caught["hidden"], caught["kwargs"]


@torch.no_grad()
def smooth_scale(model, inputs, make_probe=library_probe):
    """Searches the smoothing scales of every decoder layer on `inputs` (a dict for `model(**inputs)`, e.g.
    {"input_ids": ids}); returns scales_meta_data for `apply_scale` (kairos/smooth_scale.py:134-176).  The model is
    left unchanged; with the default probe it must live on a GPU."""
    hidden, layer_kwargs = catch_embedding_output(model, inputs)
    if "use_cache" in layer_kwargs:
        layer_kwargs["use_cache"] = False
    for key in ("past_key_value", "past_key_values"):
        if key in layer_kwargs:
            layer_kwargs[key] = None
    scales_meta_data = []
    for layer in model.model.layers:
        activations, handles = {}, []
        for name, lin in get_name_linears(layer).items():
            handles.append(lin.register_forward_hook(
                lambda module, args, output, name=name: activations.__setitem__(name, args[0])))
        try:
            out = layer(hidden, **layer_kwargs)
        finally:
            for h in handles:
                h.remove()
        hidden = out[0] if isinstance(out, tuple) else out
        scales_meta_data.append(smooth_scale_layer(layer, layer_kwargs, activations, make_probe=make_probe))
    return scales_meta_data
