"""CPU oracle for the switched mixed-precision linear path.  TEST INFRASTRUCTURE ONLY.

This module restates, in numpy, the arithmetic of the reference's switched linear layer so that
the HIP kernels can be checked against it.  Only the test-suite, the smoke check and the
benchmark's CPU-baseline leg may import it; the shipped package never does.

Every function cites the reference file:line it follows (paths relative to the reference root).

Pinning status (what, other than this file agreeing with itself, fixes each function):

  pack_int_awq / unpack_int_awq   two independent statements of the layout in the reference
                                  (step-by-step thirdparty/AWQ/awq_method.py:5-38, closed-form
                                  reshape/permute test/depacking.py:8-19 and its inverse :22-38)
                                  re-typed in tests/test_oracle_layout.py plus brute-force enumeration.
  qfactor_layout                  closed form + width table (awq_method.py:40-75); hand cases.
  quantize_int8 / quantize_int4   closed forms; invariants (range, reconstruction error bound).
  dequant_to_f16 / dequant_to_i8  exact fp16 FMA rule; s=1,z=0 reduces to pure unpack; integer
                                  zero-point reduces to textbook (q-z)*s dequantisation.
  quant_act_i8                    hand cases (zeros, +-amax, half-way ties); the reference builds with
                                  fast-math so its division may differ by one step on exact ties:
                                  the specification here is IEEE fp32 division.
  gemm_w8a8                       exact integer matmul + fixed epilogue order.
  gemm_f16 / gemm_w4a16           parity unpinned by the reference (its fp16 GEMM is cuBLAS, its
                                  W4A16 kernels accumulate in fp16); oracle = dequantise then fp32
                                  accumulated matmul, tolerance 1e-2 max-abs-rel.
  gemm_w8a16                      parity unpinned: the reference declares the id but has no
                                  implementation (kairos/dynamic_linear.py:8-9).
  switched_forward, id 7          the build's default W4A8 lane is DEFINED as the W8A8 lane's product (same int8
                                  weight, decoded inside the GEMM), so its oracle is the pinned W8A8 chain, bit for
                                  bit.  The reference's own `w4a8_qserve` candidate (kairos/dynamic_linear_v2.py:
                                  161-179) feeds the resident nibbles to a CUDA GEMM with integer per-group factors
                                  of a second quantiser; that arithmetic is restated below:
  qserve_quantize_int8 / _int4    closed forms of thirdparty/Qserve/quantization.py:4-36; hand cases, the protective
                                  range (|w8| <= 119 keeps q*s - z*s inside int8, so the byte-wise wrap never
                                  fires), reconstruction error <= s/2 per element.
  dequant_w4a8_int / gemm_w4a8_   the kernel's register arithmetic (thirdparty/Qserve/qserve_kernels/csrc/qgemm/
  int                             w4a8_per_group/gemm_cuda.cu:299-329: byte-wise q*s + z') and its epilogue
                                  (:620-627); pinned by textbook (q - zero) * scale on the quantiser's own output,
                                  by wrap-around hand cases, and by the exact integer matmul.  No output of the
                                  CUDA kernel exists in the reference to compare with (it cannot be built here).
  pack_int_w4a8 / trans_layout_   the reference states the layout twice (test/test_trans_layout.py:8-14 in one
  c16_to_c8                       permutation, thirdparty/Qserve/w4a8_linear.py:187-205 in two) and its own test
                                  demands trans(pack_awq(A)) == pack_w4a8(A) bit for bit (test_trans_layout.py:46-52);
                                  both statements re-typed in tests/test_oracle_layout.py plus the index formula
                                  by brute force.
  rmsnorm_f16                     parity unpinned by the reference (its modules run the eager PyTorch norm of the
                                  checkpoint, which is not importable here): pinned by closed-form rows (constant
                                  magnitude, so the sum, the root and the reciprocal are exact), by torch's own
                                  CPU ops composed as the eager module composes them, and by the float64 sum
                                  (at most one fp16 step apart, equal on almost every element).
  silu_mul_f16                    parity unpinned by the reference (eager activation of the checkpoint's module);
                                  pinned by torch's CPU silu and multiply (one fp16 step: the exponential is not
                                  correctly rounded in any of the libraries), exact points (0, large |g|) and the
                                  identity silu(g) - silu(-g) = g.
  LUT                             reference C++ header compiled into oracle/_ref (see Makefile) and
                                  the two shipped table files.
"""
from __future__ import annotations

import json
import numpy as np

GROUP = 128
INTERLEAVE = 4
KSTRIDE = 64

# kairos/dynamic_linear.py:8-9 (v1) and kairos/dynamic_linear_v2.py:11-13 (v2 adds 6 and 7)
COMP_TYPE_NAME = {
    "w4a16_gemm": 0, "w4a16_gemv": 1, "w8a8": 2, "w8a16_gemm": 3, "w8a16_gemv": 4, "fp16": 5,
    "w4a16_marlin": 6, "w4a8_qserve": 7,
}


# ----------------------------------------------------------------------------------------------
# F: resident int4 format                                   thirdparty/AWQ/awq_method.py:5-38
# ----------------------------------------------------------------------------------------------
def awq_position(n, k, K):
    """(flat int16 index, nibble) that holds element (n, k) of an [N, K] uint4 matrix.

    Derived from the three permutations of awq_method.py:10-37: inside every 32-wide K block the
    nibble is (k%32)//8; inside a 64-wide K block the four rows of a row-quad are laid side by
    side, 16 int16 words each, and the word index inside those 16 is ((k%64)//32)*8 + k%8.
    """
    n = np.asarray(n, dtype=np.int64)
    k = np.asarray(k, dtype=np.int64)
    word = (n // 4) * K + (k // 64) * 64 + (n % 4) * 16 + ((k % 64) // 32) * 8 + (k % 8)
    nib = (k % 32) // 8
    return word, nib


def pack_int_awq(q):
    """uint4 [N, K] (any integer dtype, values 0..15) -> int16 [N/4, K].

    Vectorised form of awq_position(): K splits as (block64, half, nibble, word8); the nibble axis is
    folded into the bits of the word.  tests/test_oracle_layout.py checks it against the index
    formula, against both statements of the reference and by brute force.
    """
    q = np.asarray(q)
    N, K = q.shape
    assert N % INTERLEAVE == 0 and K % KSTRIDE == 0
    v = (q.astype(np.uint16) & 0xF).reshape(N // 4, 4, K // 64, 2, 4, 8)      # quad,row,blk,half,nib,word
    v = v.transpose(0, 2, 1, 3, 5, 4)                                          # quad,blk,row,half,word,nib
    w = v[..., 0] | (v[..., 1] << 4) | (v[..., 2] << 8) | (v[..., 3] << 12)
    return np.ascontiguousarray(w).reshape(N // 4, K).view(np.int16)


def pack_int_awq_by_index(q):
    """Same result through awq_position() element by element (slow; the definition)."""
    q = np.asarray(q)
    N, K = q.shape
    nn, kk = np.meshgrid(np.arange(N), np.arange(K), indexing="ij")
    word, nib = awq_position(nn, kk, K)
    out = np.zeros(N // 4 * K, dtype=np.uint16)
    np.bitwise_or.at(out, word.ravel(), ((q.astype(np.uint16) & 0xF) << (4 * nib).astype(np.uint16)).ravel())
    return out.view(np.int16).reshape(N // 4, K)


def unpack_int_awq(packed):
    """int16 [N/4, K] -> uint8 [N, K] with values 0..15 (inverse of pack_int_awq)."""
    packed = np.ascontiguousarray(packed)
    N4, K = packed.shape
    w = packed.view(np.uint16).reshape(N4, K // 64, 4, 2, 8)                   # quad,blk,row,half,word
    nib = np.stack([(w >> s) & 0xF for s in (0, 4, 8, 12)], axis=-1)           # ... ,nib
    return np.ascontiguousarray(nib.transpose(0, 2, 1, 3, 5, 4)).reshape(N4 * 4, K).astype(np.uint8)


def unpack_int_awq_by_index(packed):
    packed = np.ascontiguousarray(packed)
    N4, K = packed.shape
    flat = packed.view(np.uint16).ravel()
    nn, kk = np.meshgrid(np.arange(N4 * 4), np.arange(K), indexing="ij")
    word, nib = awq_position(nn, kk, K)
    return ((flat[word] >> (4 * nib).astype(np.uint16)) & 0xF).astype(np.uint8)


# ----------------------------------------------------------------------------------------------
# W4A8 operand layout of the v2 candidate and the re-pack into it      test/test_trans_layout.py:8-52
# ----------------------------------------------------------------------------------------------
def w4a8_position(n, k, K):
    """(flat byte index, nibble) of element (n, k) in the [N, K/2] int8 W4A8 operand.

    32x32 blocks of 512 bytes, block order (n/32, k/32).  Inside a block the byte index is
    (n%8)*64 + ((k%16)//4)*16 + ((k%32)//16)*8 + ((n%16)//8)*4 + k%4, and rows n and n+16 of the block share a
    byte: low nibble (n%32) < 16, high nibble otherwise.
    """
    n = np.asarray(n, dtype=np.int64)
    k = np.asarray(k, dtype=np.int64)
    block = (n // 32) * (K // 32) + k // 32
    byte = block * 512 + (n % 8) * 64 + ((k % 16) // 4) * 16 + ((k % 32) // 16) * 8 + ((n % 16) // 8) * 4 + k % 4
    return byte, (n % 32) // 16


def pack_int_w4a8(q):
    """uint4 [N, K] -> int8 [N, K/2] (pack_int_qserve, test/test_trans_layout.py:8-14)."""
    q = np.asarray(q)
    N, K = q.shape
    assert N % 32 == 0 and K % 32 == 0
    v = (q.astype(np.uint8) & 0xF).reshape(N // 32, 2, 2, 8, K // 32, 2, 4, 4)
    v = v.transpose(0, 4, 3, 6, 5, 2, 7, 1)
    return np.ascontiguousarray((v[..., 1] << 4) + v[..., 0]).reshape(N, K // 2).view(np.int8)


def pack_int_w4a8_by_index(q):
    q = np.asarray(q)
    N, K = q.shape
    nn, kk = np.meshgrid(np.arange(N), np.arange(K), indexing="ij")
    byte, nib = w4a8_position(nn, kk, K)
    out = np.zeros(N * K // 2, dtype=np.uint8)
    np.bitwise_or.at(out, byte.ravel(), ((q.astype(np.uint8) & 0xF) << (4 * nib).astype(np.uint8)).ravel())
    return out.view(np.int8).reshape(N, K // 2)


def trans_layout_c16_to_c8(packed):
    """Resident packed int4 [N/4, K] -> W4A8 operand [N, K/2]: the same nibbles, re-ordered
    (trans_layout_c16_to_c8_awq, kernels/csrc/kairos_kernel/trans_layout/trans_layout_marlin_c16_to_c8.cu:183-205;
    contract: test/test_trans_layout.py:46-52)."""
    return pack_int_w4a8(unpack_int_awq(packed))


# ----------------------------------------------------------------------------------------------
# S: scale / scaled-zero tables                             thirdparty/AWQ/awq_method.py:40-75
# ----------------------------------------------------------------------------------------------
def calculate_zeros_width(in_features, group_size=GROUP, pack_num=8):
    """awq_method.py:40-54: number of 8-wide column packs the [K/G] axis is padded to."""
    if group_size >= 128:
        mult = 1
    elif group_size == 64:
        mult = 2
    elif group_size == 32:
        mult = 4
    else:
        raise NotImplementedError(group_size)
    ceil_div = lambda c, d: (c + d - 1) // d
    return ceil_div(ceil_div(in_features // group_size, pack_num), mult) * mult


def padded_groups(K, group_size=GROUP):
    return calculate_zeros_width(K, group_size) * 8


def qfactor_layout(scales, zeros, group_size=GROUP):
    """fp16 [N, K/G] x2 -> (scales_t, scaled_zeros_t) fp16 [Gp, N]   (awq_method.py:56-75, 'kairos').

    scaled_zeros = -fp16( fp32(scale_fp16) * fp32(zero) ); padded rows are zero.
    """
    scales = np.asarray(scales, dtype=np.float16)
    zeros = np.asarray(zeros)
    N, ng = scales.shape
    Gp = padded_groups(ng * group_size, group_size)
    qs = np.zeros((N, Gp), dtype=np.float16)
    qs[:, :ng] = scales
    sz = np.zeros((N, Gp), dtype=np.float16)
    prod = qs[:, :ng].astype(np.float32) * zeros.astype(np.float32)
    sz[:, :ng] = -(prod.astype(np.float16))
    return np.ascontiguousarray(qs.T), np.ascontiguousarray(sz.T)


# ----------------------------------------------------------------------------------------------
# Q8 / Q4 / P: weight preparation
# ----------------------------------------------------------------------------------------------
def quantize_int8(w):
    """kairos/quantization.py:112-141 with q_type='S', group_size=-1, max_int=127.

    fp16 [N, K] -> (int8 [N, K], scale fp16 [N, 1]); all arithmetic in fp32.
    """
    x = np.asarray(w, dtype=np.float16).astype(np.float32)
    amax = np.maximum(np.abs(x).max(axis=1, keepdims=True), np.float32(1e-7))
    scale = amax / np.float32(127)
    q = np.rint(x / scale)  # round half to even, as torch.round_
    return q.astype(np.int8), scale.astype(np.float16)


def quantize_int4_kairos(w8, group_size=GROUP):
    """kairos/dynamic_linear_v2.py:15-41 (eager order; same maths as dynamic_linear.py:13-37).

    int8 [N, K] -> (uint4-in-int8 [N, K], scale fp16 [N*K/G, 1], zero fp16 [N*K/G, 1]).
    The zero-point is kept unrounded; the order of operations is x/s, + z, round, clamp.
    """
    w8 = np.asarray(w8)
    shape = w8.shape
    assert shape[-1] % group_size == 0
    x = w8.reshape(-1, group_size).astype(np.float32)
    mx = x.max(axis=1, keepdims=True)
    mn = x.min(axis=1, keepdims=True)
    scale = np.maximum(mx - mn, np.float32(1e-5)) / np.float32(15)
    zero = -(mn / scale)
    q = np.clip(np.rint(x / scale + zero), 0, 15)
    with np.errstate(over="ignore"):   # a constant group makes zero overflow fp16, as in the reference
        return q.reshape(shape).astype(np.int8), scale.astype(np.float16), zero.astype(np.float16)


def quantize_int4_int_factors(w8, group_size=GROUP):
    """The integer second-level factors that the version-2 quantiser also returns (kairos/dynamic_linear_v2.py:36-41):
    scale_i = floor(scale_f), zero_pt_i = round_half_even(zero_pt_f), both taken from the fp32 values (before their
    fp16 rounding) and stored as int8.  The reference computes them and nothing in its tree reads them; they describe
    the W4A8 operand a per-group integer dequantiser would use.  Groups whose zero-point leaves the int8 range (constant
    groups: scale 1e-5 / 15) have no defined int8 value there (the cast of an out-of-range float); they are returned
    saturated and flagged in the third result.  -> (scale_i int8 [G,1], zero_pt_i int8 [G,1], in_range bool [G,1])"""
    w8 = np.asarray(w8)
    assert w8.shape[-1] % group_size == 0
    x = w8.reshape(-1, group_size).astype(np.float32)
    mx = x.max(axis=1, keepdims=True)
    mn = x.min(axis=1, keepdims=True)
    scale = np.maximum(mx - mn, np.float32(1e-5)) / np.float32(15)
    zero = -(mn / scale)
    zi = np.rint(zero)
    in_range = (zi >= -128) & (zi <= 127)
    return np.floor(scale).astype(np.int8), np.clip(zi, -128, 127).astype(np.int8), in_range


def prepare_weights(w, group_size=GROUP):
    """kairos/dynamic_linear.py:86-115 (from_module): fp16 [N, K] -> dict of resident tensors."""
    w = np.asarray(w, dtype=np.float16)
    N, K = w.shape
    w8, scale_1 = quantize_int8(w)
    q4, scale_2, zero_2 = quantize_int4_kairos(w8, group_size)
    scale_2 = scale_2.reshape(N, -1)
    zero_2 = zero_2.reshape(N, -1)
    scales_to8, scaled_zeros_to8 = qfactor_layout(scale_2, zero_2, group_size)
    # fp16 * fp16 -> fp16 (dynamic_linear.py:108): exact product, one rounding
    scale_f = (scale_2.astype(np.float32) * scale_1.astype(np.float32)).astype(np.float16)
    scales, scaled_zeros = qfactor_layout(scale_f, zero_2, group_size)
    return {
        "qweight": pack_int_awq(q4),
        "scales": scales, "scaled_zeros": scaled_zeros,
        "scales_to8": scales_to8, "scaled_zeros_to8": scaled_zeros_to8,
        "scales_1": scale_1.reshape(-1),
        "q4": q4, "w8_step1": w8,
    }


# ----------------------------------------------------------------------------------------------
# C16 / C8: on-demand conversion
# ----------------------------------------------------------------------------------------------
def _fma_f16(q, s, z):
    """Single-rounding fp16 FMA: the exact value q*s+z fits in fp64, so one cast rounds once."""
    return (q.astype(np.float64) * s.astype(np.float64) + z.astype(np.float64)).astype(np.float16)


def dequant_to_f16(qweight, scales, scaled_zeros, group_size=GROUP):
    """kernels/csrc/kairos_kernel/dequant_awq_format/dequant_i4_to_f16.cu:14-36,40-151.

    W16[n, k] = fma_f16(q[n, k], scales[k/G, n], scaled_zeros[k/G, n]) -> fp16 [N, K] row-major.
    """
    qweight = np.ascontiguousarray(qweight)
    N, K = qweight.shape[0] * 4, qweight.shape[1]
    ng = K // group_size
    out = np.empty((N, K), dtype=np.float16)
    step = 2048                                                 # rows per slab: bounds the fp64 temporaries
    for r0 in range(0, N, step):
        r1 = min(N, r0 + step)
        q = unpack_int_awq(qweight[r0 // 4:r1 // 4]).reshape(r1 - r0, ng, group_size)
        s = np.asarray(scales)[:ng, r0:r1].T[:, :, None]
        z = np.asarray(scaled_zeros)[:ng, r0:r1].T[:, :, None]
        out[r0:r1] = _fma_f16(q, s, z).reshape(r1 - r0, K)
    return out


def dequant_to_i8(qweight, scales_to8, scaled_zeros_to8, group_size=GROUP):
    """kernels/csrc/kairos_kernel/dequant_awq_format/dequant_i4_to_i8.cu:14-36,143-146.

    W8[n, k] = (int8) fma_f16(q, s, sz): the C cast truncates toward zero.  Values outside
    [-128, 127] cannot arise from prepare_weights(); they are clipped here.
    """
    f = dequant_to_f16(qweight, scales_to8, scaled_zeros_to8, group_size).astype(np.float32)
    f = np.where(np.isnan(f), np.float32(0), f)
    return np.clip(np.trunc(f), -128, 127).astype(np.int8)


# ----------------------------------------------------------------------------------------------
# The reference's own id-7 operands: integer per-group factors on top of a per-channel int8 level
# ----------------------------------------------------------------------------------------------
def qserve_quantize_int8(w):
    """thirdparty/Qserve/quantization.py:4-15: per-row symmetric int8 with the protective range 119.
    fp [N, K] -> (int8 [N, K], scale fp16 [N, 1]); the division uses the fp32 scale, the fp16 one is what is stored."""
    x = np.asarray(w).astype(np.float32)
    mx = np.maximum(np.abs(x).max(axis=1, keepdims=True), np.float32(1e-7))
    scale = (mx / np.float32(119)).astype(np.float32)
    return np.rint(x / scale).astype(np.int8), scale.astype(np.float16)


def qserve_quantize_int4(w8, group_size=GROUP):
    """thirdparty/Qserve/quantization.py:17-36: int8 -> uint4 per group with WHOLE-NUMBER scale and zero point.
    scale = round((max - min).clamp(1e-7) / 15), 0 -> 1; zero = round(-min / scale); q = clamp(round(x / scale + zero)).
    -> (uint4-in-int8 [N, K], scale int8 [N*K/G, 1], zero int8 [N*K/G, 1])"""
    w8 = np.asarray(w8)
    shape = w8.shape
    assert shape[-1] % group_size == 0
    x = w8.reshape(-1, group_size).astype(np.float32)
    mx = x.max(axis=1, keepdims=True)
    mn = x.min(axis=1, keepdims=True)
    scale = np.rint(np.maximum(mx - mn, np.float32(1e-7)) / np.float32(15))
    scale[scale == 0] = 1
    zero = np.rint(-(mn / scale))
    q = np.clip(np.rint(x / scale + zero), 0, 15)
    return q.reshape(shape).astype(np.int8), scale.astype(np.int8), zero.astype(np.int8)


def qserve_tables(scale_i, zero_i, N, group_size=GROUP):
    """thirdparty/Qserve/w4a8_linear.py:215-262 without the 32-column shuffle the CUDA fragments want: per-group tables
    [K/G, N] in plain column order, s2_scales = scale, s2_zeros = int8(-zero * scale) (two's complement, wrapping)."""
    s = np.asarray(scale_i).reshape(N, -1).T.astype(np.int32)
    z = np.asarray(zero_i).reshape(N, -1).T.astype(np.int32)
    return s.astype(np.int8), ((-z * s) & 0xFF).astype(np.uint8).view(np.int8)


def dequant_w4a8_int(qweight, s2_scales, s2_zeros, group_size=GROUP):
    """gemm_cuda.cu:299-329 of the per-group W4A8 kernel: every weight byte is (q * scale + zeros') modulo 256, read
    as int8 -- a packed 32-bit multiply by the scale byte (no carry between bytes while 15 * scale < 256, which the
    quantiser guarantees) and a byte-wise wrapping add of the pre-multiplied zero.  Here each byte is taken modulo
    256 on its own, for any scale byte (read as unsigned, as the kernel's mask does)."""
    N, K = qweight.shape[0] * 4, qweight.shape[1]
    ng = K // group_size
    q = unpack_int_awq(qweight).reshape(N, ng, group_size).astype(np.int32)
    s = (np.asarray(s2_scales)[:ng].astype(np.int32) & 0xFF).T[:, :, None]
    z = (np.asarray(s2_zeros)[:ng].astype(np.int32) & 0xFF).T[:, :, None]
    return ((q * s + z) & 0xFF).astype(np.uint8).view(np.int8).reshape(N, K)


def gemm_w4a8_int(a8, qweight, s2_scales, s2_zeros, wscales, ascales, group_size=GROUP):
    """The reference's id-7 product (kairos/dynamic_linear_v2.py:161-179; epilogue gemm_cuda.cu:620-627, the same
    order as the W8A8 kernel's): int32 accumulators and fp16 output."""
    return gemm_w8a8(a8, dequant_w4a8_int(qweight, s2_scales, s2_zeros, group_size), wscales, ascales)


# ----------------------------------------------------------------------------------------------
# A: per-token activation quantiser
# ----------------------------------------------------------------------------------------------
def quant_act_i8(x):
    """kernels/csrc/kairos_kernel/quant/quant_f16_to_i8.cu:45-81 + quant/utils.cuh:77-82.

    fp16 [M, K] -> (int8 [M, K], scale fp16 [M]).  amax in fp32; scale = fp16(amax/127);
    t = 127/amax (IEEE fp32); q = sat_s8(round_half_even(fp32(x)*t)); NaN (0*inf) converts to 0.
    """
    xf = np.asarray(x, dtype=np.float16).astype(np.float32)
    amax = np.abs(xf).max(axis=1, keepdims=True).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        scale = (amax / np.float32(127)).astype(np.float16)
        t = np.float32(127) / amax
        p = xf * t
    p = np.where(np.isnan(p), np.float32(0), p)
    q = np.clip(np.rint(p), -128, 127).astype(np.int8)
    return q, scale.reshape(-1)


# ----------------------------------------------------------------------------------------------
# RMSNorm in front of the quantiser ("activation matching", README.md:23-27)
# ----------------------------------------------------------------------------------------------
def rmsnorm_f16(x, gamma, eps, residual=None, exact_sum=False):
    """The fp16 RMSNorm of the decoder modules the reference quantises (transformers LlamaRMSNorm /
    Qwen2RMSNorm, which kairos/smooth_scale.py:112-119 addresses as input_layernorm / post_attention_layernorm),
    every intermediate rounded as the eager module rounds it:
        h = fp16(x + residual);  var = mean(float(h)^2);  y = gamma * fp16(float(h) * rsqrt(var + eps)).
    fp16 [M, K] -> (y fp16 [M, K], h fp16 [M, K]).

    The fp32 sum of squares depends on the order of addition.  exact_sum=False follows the order of the HIP
    kernel (256 threads per token; thread t owns the 8-element chunks t, t+256, ..; per thread in order;
    butterfly over each 64-lane wave with xor 32, 16, .., 1; then (w0 + w1) + (w2 + w3)), which makes the
    comparison with the kernel bit-exact.  exact_sum=True sums in float64 (exact for these inputs up to one final rounding) and is
    the order-free statement the other one is checked against.
    """
    h = np.asarray(x, dtype=np.float16)
    if residual is not None:
        h = (h + np.asarray(residual, dtype=np.float16)).astype(np.float16)      # numpy adds fp16 with one rounding
    M, K = h.shape
    hf = h.astype(np.float32)
    if exact_sum:
        total = (hf.astype(np.float64) ** 2).sum(axis=1).astype(np.float32)
    else:
        nchunk = K // 8
        tpt = 256                                                                 # threads per token
        cpt = (nchunk + tpt - 1) // tpt
        sq = np.zeros((M, cpt * tpt, 8), dtype=np.float32)
        sq[:, :nchunk, :] = (hf * hf).reshape(M, nchunk, 8)                       # exact: 22-bit products
        sq = sq.reshape(M, cpt, tpt, 8)
        ss = np.zeros((M, tpt), dtype=np.float32)
        for i in range(cpt):
            for e in range(8):
                ss = ss + sq[:, i, :, e]
        ss = ss.reshape(M, tpt // 64, 64)
        lanes = np.arange(64)
        for off in (32, 16, 8, 4, 2, 1):
            ss = ss + ss[:, :, lanes ^ off]
        w = ss[:, :, 0]
        total = (w[:, 0] + w[:, 1]) + (w[:, 2] + w[:, 3])
    var = total / np.float32(K)
    with np.errstate(divide="ignore"):
        r = np.float32(1) / np.sqrt(var + np.float32(eps), dtype=np.float32)
    t = (hf * r[:, None]).astype(np.float16)
    y = (np.asarray(gamma, dtype=np.float16).astype(np.float32)[None, :] * t.astype(np.float32)).astype(np.float16)
    return y, h


def rmsnorm_quant_act(x, gamma, eps, residual=None):
    """rmsnorm_f16 followed by quant_act_i8: what the fused kernel must equal bit for bit.
    -> (int8 [M, K], scale fp16 [M], y fp16 [M, K], h fp16 [M, K])."""
    y, h = rmsnorm_f16(x, gamma, eps, residual)
    q, s = quant_act_i8(y)
    return q, s, y, h


def silu_mul_f16(gate_up):
    """The eager fp16 MLP activation in front of the down projection (transformers LlamaMLP / Qwen2MLP:
    act_fn(gate_proj(x)) * up_proj(x) with act_fn = SiLU), on a fused [M, 2*I] input, gate first:
        s = fp16(g / (1 + exp(-g))) evaluated in fp32;  y = fp16(float(s) * float(u)).
    The exponential is not correctly rounded anywhere (numpy, torch and the GPU each have their own), so
    comparisons against this function allow one fp16 step; everything behind y is exact again."""
    gu = np.asarray(gate_up, dtype=np.float16)
    I = gu.shape[1] // 2
    g = gu[:, :I].astype(np.float32)
    u = gu[:, I:].astype(np.float32)
    with np.errstate(over="ignore"):
        s = (g / (np.float32(1) + np.exp(-g, dtype=np.float32))).astype(np.float16)
    return (s.astype(np.float32) * u).astype(np.float16)


# ----------------------------------------------------------------------------------------------
# GEMMs
# ----------------------------------------------------------------------------------------------
def gemm_i8_acc(a8, w8):
    """Exact int8 x int8 -> int32 accumulators, a8 [M, K], w8 [N, K] (both K-contiguous)."""
    acc = np.asarray(a8).astype(np.float64) @ np.asarray(w8).astype(np.float64).T  # exact: |acc| < 2^53
    return acc.astype(np.int64).astype(np.int32)


def w8a8_epilogue(acc, wscales, ascales):
    """thirdparty/AWQ/kernels/csrc/w8a8/w8a8_gemm_cuda.cu:889-902.

    out = fp16_rn( float_rn(acc) * (float(ws[n]) * float(as[m])) ), every step rounded to fp32.
    """
    ws = np.asarray(wscales, dtype=np.float16).astype(np.float32).reshape(1, -1)
    as_ = np.asarray(ascales, dtype=np.float16).astype(np.float32).reshape(-1, 1)
    s = (ws * as_).astype(np.float32)
    with np.errstate(over="ignore"):
        return (acc.astype(np.float32) * s).astype(np.float32).astype(np.float16)


def gemm_w8a8(a8, w8, wscales, ascales):
    acc = gemm_i8_acc(a8, w8)
    return acc, w8a8_epilogue(acc, wscales, ascales)


def gemm_f16(x, w16):
    """Oracle for kairos/dynamic_linear.py:163 (`input @ tmp_weight.T`): fp32 accumulation, fp16 result."""
    with np.errstate(over="ignore"):
        return (np.asarray(x, dtype=np.float16).astype(np.float32)
                @ np.asarray(w16, dtype=np.float16).astype(np.float32).T).astype(np.float16)


def gemm_w4a16(x, qweight, scales, scaled_zeros, group_size=GROUP):
    """Oracle for gemv_forward_cuda_new / gemm_forward_cuda_new: dequantise (C16) then fp16 matmul."""
    return gemm_f16(x, dequant_to_f16(qweight, scales, scaled_zeros, group_size))


def gemm_w8a16(x, w8, scales_1):
    """Build-defined W8A16: out = fp16( (x . W8^T) * scales_1[n] ), fp32 accumulation."""
    acc = np.asarray(x, dtype=np.float16).astype(np.float32) @ np.asarray(w8).astype(np.float32).T
    with np.errstate(over="ignore"):
        return (acc * np.asarray(scales_1, dtype=np.float16).astype(np.float32).reshape(1, -1)).astype(np.float16)


def switched_forward(x, prep, comp_type, bias=None):
    """kairos/dynamic_linear.py:133-172 (_forward): x fp16 [M, K] -> fp16 [M, N] for one comp id."""
    name = {v: k for k, v in COMP_TYPE_NAME.items()}[comp_type]
    if name in ("w4a16_gemv", "w4a16_gemm", "fp16", "w4a16_marlin"):
        out = gemm_w4a16(x, prep["qweight"], prep["scales"], prep["scaled_zeros"])
    elif name in ("w8a8", "w4a8_qserve"):      # id 7: the build's W4A8 lane, defined as the W8A8 product without a copy
        w8 = dequant_to_i8(prep["qweight"], prep["scales_to8"], prep["scaled_zeros_to8"])
        a8, sx = quant_act_i8(x)
        out = gemm_w8a8(a8, w8, prep["scales_1"], sx)[1]
    elif name in ("w8a16_gemm", "w8a16_gemv"):
        w8 = dequant_to_i8(prep["qweight"], prep["scales_to8"], prep["scaled_zeros_to8"])
        out = gemm_w8a16(x, w8, prep["scales_1"])
    else:
        raise ValueError(f"no oracle for comp_type {comp_type}")
    if bias is not None:
        out = (out.astype(np.float32) + np.asarray(bias, np.float16).astype(np.float32)).astype(np.float16)
    return out


def max_abs_rel(out, ref):
    """The fp16-output tolerance metric: max|out-ref| / max|ref|."""
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.abs(out - ref).max() / max(np.abs(ref).max(), 1e-30))


# ----------------------------------------------------------------------------------------------
# L: interval lookup table
# ----------------------------------------------------------------------------------------------
class LUT:
    """kernels/csrc/kairos_kernel/lut/lut.h:8-45 semantics (the C++ variant, memo initialised to -1).

    record(r, c) appends the right edge r; get(m) is c of the first segment with m <= r, and the
    last segment's c for every m beyond the last edge.
    """

    def __init__(self):
        self.edges = []
        self.comps = []

    def record(self, r, comp):
        self.edges.append(int(r))
        self.comps.append(int(comp))

    def get(self, m):
        for r, c in zip(self.edges, self.comps):
            if m <= r:
                return c
        return self.comps[-1]


def load_seg_perf_list(path):
    """kairos/perf_profiler.py:76-81 + utils/util.py:29-30: the table file is JSON text."""
    with open(path) as f:
        return json.load(f)


# ----------------------------------------------------------------------------------------------
# synthetic inputs shared by tests and the benchmark's CPU leg
# ----------------------------------------------------------------------------------------------
def synth_weights(N, K, seed=10):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.02)).astype(np.float16)


def synth_acts(M, K, seed=11, outlier_frac=0.01, outlier_gain=20.0):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, K), dtype=np.float32)
    n_out = int(outlier_frac * K)
    if n_out:
        cols = rng.choice(K, size=n_out, replace=False)
        x[:, cols] *= np.float32(outlier_gain)
    return x.astype(np.float16)
