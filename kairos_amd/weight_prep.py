"""Host-side weight preparation: fp16 -> per-channel int8 -> asymmetric uint4 (float zero-point) ->
the resident packed format and its scale tables.  Runs once per layer, offline, as torch tensor
ops on whatever device the weight lives on.

Mirrors kairos/quantization.py:112-141 (quantize_tensor_int8), kairos/dynamic_linear_v2.py:15-41
(kairos_quantize_tensor_int4) and thirdparty/AWQ/awq_method.py:5-75 (pack_int_awq,
calculate_zeros_width, trans_qfactor_layout_awq): same names, arguments and results.  The second
quantiser whose integer factors the version-2 `w4a8_qserve` candidate multiplies with
(thirdparty/Qserve/quantization.py:4-36, tables of thirdparty/Qserve/w4a8_linear.py:215-262) is
here as well: qserve_quantize_tensor_int8 / _int4 and qserve_factor_tables.
"""
import torch


@torch.no_grad()
def quantize_tensor_int8(x, q_type="S", group_size=-1, return_dtype=torch.float16, max_int=-1):
    """Symmetric per-channel (group_size=-1) or per-tensor (-2) int8; returns (int8 tensor, config dict)."""
    if q_type != "S":
        raise NotImplementedError("only the symmetric scheme lies on the switched-linear path")
    shape = x.shape
    flat = x.reshape(1, -1) if group_size == -2 else x.reshape(-1, shape[-1])
    flat = flat.to(torch.float32)
    if max_int == -1:
        max_int = 127
    amax = flat.abs().amax(dim=1, keepdim=True).clamp(min=1e-7)
    scale = amax / max_int
    q = torch.round(flat / scale).to(torch.int8)
    return q.reshape(shape), {"q_type": q_type, "scale": scale.to(return_dtype),
                              "zero_pt": torch.tensor([0]).to(return_dtype)}


@torch.no_grad()
def kairos_quantize_tensor_int4(x, group_size=-1):
    """int8 -> uint4 with an UNROUNDED floating zero-point, per group along the last axis.

    Order of operations is part of the format: x/s, then +z, then round-half-even, then clamp.
    """
    shape = x.shape
    if group_size < 0:
        g = x.reshape(-1, shape[-1])
    else:
        if shape[-1] % group_size:
            raise ValueError(f"last dimension {shape[-1]} is not a multiple of group_size {group_size}")
        g = x.reshape(-1, group_size)
    g = g.to(torch.float32)
    hi = g.amax(dim=1, keepdim=True)
    lo = g.amin(dim=1, keepdim=True)
    scale_f = (hi - lo).clamp(min=1e-5) / 15
    zero_pt_f = -(lo / scale_f)
    q = torch.clamp(torch.round(g / scale_f + zero_pt_f), 0, 15)
    if torch.isnan(q).any():
        raise ValueError("NaN while quantising to int4")
    return q.reshape(shape).to(torch.int8), {
        "scale_f": scale_f.to(torch.float16), "scale_i": torch.floor(scale_f).to(torch.int8),
        "zero_pt_f": zero_pt_f.to(torch.float16), "zero_pt_i": torch.round(zero_pt_f).to(torch.int8),
        "group_size": group_size}


@torch.no_grad()
def pack_int_awq(unpacked_qweight, interleave=4, kstride=64):
    """uint4 [N, K] -> int16 [N/4, K].

    Element (n, k) goes to word (n/4)*K + (k/64)*64 + (n%4)*16 + ((k%64)/32)*8 + k%8, nibble
    (k%32)/8: view K as (block64, half, nibble, word8), move the nibble axis last, fold it.
    """
    if interleave != 4 or kstride != 64:
        raise NotImplementedError("the resident format is fixed: interleave 4, kstride 64")
    N, K = unpacked_qweight.shape
    if N % 4 or K % 64:
        raise ValueError(f"need N%4==0 and K%64==0, got {N}x{K}")
    v = unpacked_qweight.to(torch.int32).reshape(N // 4, 4, K // 64, 2, 4, 8)   # quad, row, blk, half, nib, word
    v = v.permute(0, 2, 1, 3, 5, 4)                                               # quad, blk, row, half, word, nib
    shifts = torch.tensor([0, 4, 8, 12], dtype=torch.int32, device=v.device)
    words = ((v & 0xF) << shifts).sum(dim=-1)                                     # disjoint bits: sum == or
    words = torch.where(words >= 32768, words - 65536, words)                     # two's complement into int16
    return words.to(torch.int16).reshape(N // 4, K).contiguous()


@torch.no_grad()
def unpack_int_awq(packed):
    """Inverse of pack_int_awq: int16 [N/4, K] -> uint8-valued int8 [N, K]."""
    N4, K = packed.shape
    w = packed.to(torch.int32) & 0xFFFF
    shifts = torch.tensor([0, 4, 8, 12], dtype=torch.int32, device=w.device)
    nib = (w.reshape(N4, K // 64, 4, 2, 8, 1) >> shifts) & 0xF                    # quad, blk, row, half, word, nib
    return nib.permute(0, 2, 1, 3, 5, 4).reshape(N4 * 4, K).to(torch.int8)


def calculate_zeros_width(in_features, group_size=128, pack_num=8):
    if group_size >= 128:
        mult = 1
    elif group_size == 64:
        mult = 2
    elif group_size == 32:
        mult = 4
    else:
        raise NotImplementedError
    width = -(-(in_features // group_size) // pack_num)
    return -(-width // mult) * mult


@torch.no_grad()
def trans_qfactor_layout_awq(scales, zeros, group_size, method="AWQ"):
    """[N, K/G] scales and zero-points -> ([Gp, N] scales, [Gp, N] scaled zeros = -fp16(s*z)), zero padded."""
    N, ng = scales.shape
    gp = calculate_zeros_width(ng * group_size, group_size) * 8
    s16 = scales.to(torch.float16)
    if method == "AWQ":
        zeros = zeros.to(torch.int32)
    qs = torch.zeros((gp, N), dtype=torch.float16, device=scales.device)
    sz = torch.zeros((gp, N), dtype=torch.float16, device=scales.device)
    qs[:ng] = s16.t()
    sz[:ng] = (-(s16.to(torch.float32) * zeros.to(torch.float32)).to(torch.float16)).t()
    return qs.contiguous(), sz.contiguous()


@torch.no_grad()
def prepare_linear_weight(weight, group_size=128):
    """The three steps of DynamicLinear.from_module (kairos/dynamic_linear.py:95-111) on a weight tensor."""
    w = weight.detach().to(torch.float16)
    N, K = w.shape
    w8, cfg1 = quantize_tensor_int8(w, max_int=127)
    scale_1 = cfg1["scale"]
    q4, cfg2 = kairos_quantize_tensor_int4(w8, group_size=group_size)
    scale_2 = cfg2["scale_f"].reshape(N, -1)
    zero_2 = cfg2["zero_pt_f"].reshape(N, -1)
    scales_to8, scaled_zeros_to8 = trans_qfactor_layout_awq(scale_2, zero_2, group_size, method="kairos")
    scale_f = scale_2 * scale_1                                   # fp16 * fp16 -> fp16
    scales, scaled_zeros = trans_qfactor_layout_awq(scale_f, zero_2, group_size, method="kairos")
    return {"qweight": pack_int_awq(q4), "scales": scales, "scaled_zeros": scaled_zeros,
            "scales_to8": scales_to8, "scaled_zeros_to8": scaled_zeros_to8,
            "scales_1": scale_1.reshape(-1).contiguous()}


@torch.no_grad()
def qserve_quantize_tensor_int8(x, return_dtype=torch.float16):
    """Per-row symmetric int8 inside the protective range +-119 (thirdparty/Qserve/quantization.py:4-15)."""
    shape = x.shape
    rows = x.reshape(-1, shape[-1]).to(torch.float32)
    step = rows.abs().amax(dim=1, keepdim=True).clamp(min=1e-7) / 119
    q = torch.round(rows / step).to(torch.int8)
    if torch.isnan(rows).any():
        raise ValueError("NaN while quantising to int8")
    return q.reshape(shape), {"scale": step.to(return_dtype)}


@torch.no_grad()
def qserve_quantize_tensor_int4(x, group_size=-1):
    """int8 -> uint4 per group with whole-number scale and zero point (thirdparty/Qserve/quantization.py:17-36):
    scale = round(range / 15) (0 becomes 1), zero = round(-min / scale), q = clamp(round(x / scale + zero), 0, 15)."""
    shape = x.shape
    if group_size < 0:
        g = x.reshape(-1, shape[-1])
    else:
        if shape[-1] % group_size:
            raise ValueError(f"last dimension {shape[-1]} is not a multiple of group_size {group_size}")
        g = x.reshape(-1, group_size)
    g = g.to(torch.float32)
    lo = g.amin(dim=1, keepdim=True)
    step = torch.round((g.amax(dim=1, keepdim=True) - lo).clamp(min=1e-7) / 15)
    step[step == 0] = 1
    zero = torch.round(-(lo / step))
    q = torch.clamp(torch.round(g / step + zero), 0, 15)
    return q.reshape(shape).to(torch.int8), {"scale": step.to(torch.int8), "zero_pt": zero.to(torch.int8),
                                             "group_size": group_size}


@torch.no_grad()
def qserve_factor_tables(weight, group_size=128):
    """The operands that W4A8Linear.from_module derives beside its own nibbles (thirdparty/Qserve/w4a8_linear.py:182-262)
    and that the version-2 layer hands to the W4A8 GEMM with the RESIDENT nibbles (kairos/dynamic_linear_v2.py:103,
    161-179): s1_scales fp16 [N], s2_scales int8 [K/G, N], s2_zeros int8 [K/G, N] = -(zero * scale) as a
    two's-complement byte.  Plain column order: the shuffle inside blocks of 32 columns that the reference applies is
    the fragment order of its CUDA kernel and has no meaning for the MFMA kernel that reads these tables."""
    w = weight.detach().to(torch.float16).cpu()
    N, K = w.shape
    w8, cfg1 = qserve_quantize_tensor_int8(w)
    _, cfg2 = qserve_quantize_tensor_int4(w8, group_size=group_size)
    s2 = cfg2["scale"].reshape(N, K // group_size).t().contiguous()
    z2 = cfg2["zero_pt"].reshape(N, K // group_size).t().contiguous()
    zs = (-(z2.to(torch.int32) * s2.to(torch.int32))).to(torch.int8)          # wraps like the reference's int8 store
    return {"s1_scales": cfg1["scale"].reshape(N).contiguous(), "s2_scales": s2, "s2_zeros": zs}
