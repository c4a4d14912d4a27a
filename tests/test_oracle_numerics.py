"""Pins the oracle's arithmetic rows (Q8, Q4, C16, C8, A, G8) through closed forms, invariants and
hand cases chosen so that a dropped term, a wrong sign/index or a wrong rounding mode fails."""
import numpy as np
import pytest

from oracle import kairos_oracle as O


# ---------------------------------------------------------------- Q8 (kairos/quantization.py:112-141)
def test_quantize_int8_hand_cases():
    w = np.array([[1.0, -0.5, 0.25, 0.0], [0.0, 0.0, 0.0, 0.0]], dtype=np.float16)
    q, s = O.quantize_int8(w)
    assert q.dtype == np.int8 and s.dtype == np.float16 and s.shape == (2, 1)
    assert q[0].tolist() == [127, -64, 32, 0]          # 63.5 -> 64 (even), 31.75 -> 32
    assert s[0, 0] == np.float16(np.float32(1.0) / np.float32(127))
    assert q[1].tolist() == [0, 0, 0, 0]               # all-zero row: clamp(1e-7) keeps it finite


def test_quantize_int8_invariants():
    w = O.synth_weights(64, 512, seed=3)
    q, s = O.quantize_int8(w)
    assert np.abs(q).max() == 127 and (np.abs(q).max(axis=1) == 127).all()
    s32 = (np.abs(w.astype(np.float32)).max(axis=1, keepdims=True) / np.float32(127))
    assert np.abs(q * s32 - w.astype(np.float32)).max() <= s32.max() * 0.5 * (1 + 1e-6)


# ---------------------------------------------------------------- Q4 (kairos/dynamic_linear_v2.py:15-41)
def test_quantize_int4_hand_case():
    # group with min=-30, max=45: s=5, z=6 -> q=(x/5+6) rounded half-even
    x = np.zeros((1, 128), dtype=np.int8)
    x[0, :6] = [-30, 45, 0, 2, 3, -3]
    x[0, 6:] = 5
    q, s, z = O.quantize_int4_kairos(x)
    assert s[0, 0] == np.float16(5.0) and z[0, 0] == np.float16(6.0)
    assert q[0, :7].tolist() == [0, 15, 6, 6, 7, 5, 7]  # 6.4->6, 6.6->7, 5.4->5


def test_quantize_int4_float_zero_point_and_range():
    rng = np.random.default_rng(5)
    w8 = rng.integers(-127, 128, size=(16, 512)).astype(np.int8)
    q, s, z = O.quantize_int4_kairos(w8)
    assert q.min() >= 0 and q.max() <= 15
    g = w8.reshape(-1, 128).astype(np.float32)
    s32 = (g.max(1) - g.min(1)) / np.float32(15)
    z32 = -(g.min(1) / s32)
    assert np.array_equal(s.ravel(), s32.astype(np.float16))
    assert np.array_equal(z.ravel(), z32.astype(np.float16))
    assert (np.abs(z32 - np.rint(z32)) > 1e-3).any()       # the zero-point is NOT rounded
    recon = (q.reshape(-1, 128) - z32[:, None]) * s32[:, None]
    assert np.abs(recon - g).max() <= s32.max() * 0.5 * (1 + 1e-5)
    # group extremes map to the ends of the range
    qq = q.reshape(-1, 128)
    assert (qq[np.arange(len(g)), g.argmin(1)] == 0).all() and (qq[np.arange(len(g)), g.argmax(1)] == 15).all()


def test_constant_group_uses_clamp():
    x = np.full((1, 128), 7, dtype=np.int8)
    q, s, z = O.quantize_int4_kairos(x)
    assert np.isfinite(s.astype(np.float32)).all()
    assert q.min() >= 0 and q.max() <= 15


# ---------------------------------------------------------------- C16 / C8
def _fma_f16_bruteforce(q, s, z):
    """Exact rational arithmetic on the fp16 bit patterns, rounded once (ties to even)."""
    from fractions import Fraction
    exact = Fraction(int(q)) * Fraction(float(s)) + Fraction(float(z))
    f = np.float64(exact)   # exact: <= 30 significant bits
    assert Fraction(float(f)) == exact
    return np.float16(f)


def test_dequant_identity_scale_is_pure_unpack():
    N, K = 8, 256
    rng = np.random.default_rng(1)
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    pk = O.pack_int_awq(q)
    ones = np.ones((8, N), np.float16)
    zeros = np.zeros((8, N), np.float16)
    assert np.array_equal(O.dequant_to_f16(pk, ones, zeros), q.astype(np.float16))
    assert np.array_equal(O.dequant_to_i8(pk, ones, zeros), q.astype(np.int8))


def test_dequant_group_and_row_indexing():
    """scale depends on (k//128, n) only: a table that encodes its own index must come back."""
    N, K = 8, 384
    q = np.ones((N, K), dtype=np.uint8)
    pk = O.pack_int_awq(q)
    tab = np.zeros((8, N), np.float16)
    for g in range(3):
        for n in range(N):
            tab[g, n] = 16 * g + n
    w = O.dequant_to_f16(pk, tab, np.zeros_like(tab))
    for n in range(N):
        for k in range(K):
            assert w[n, k] == 16 * (k // 128) + n


def test_dequant_integer_zero_point_is_textbook():
    """With integer zero z the rule reduces to (q - z) * s (thirdparty/AWQ/awq_method.py:105-116)."""
    N, K = 8, 128
    rng = np.random.default_rng(2)
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    s = np.full((N, 1), 0.25, np.float16)
    z = np.full((N, 1), 8, np.float16)
    st, szt = O.qfactor_layout(s, z)
    w = O.dequant_to_f16(O.pack_int_awq(q), st, szt)
    assert np.array_equal(w, ((q.astype(np.float32) - 8) * 0.25).astype(np.float16))


def test_dequant_single_rounding_vs_rationals():
    rng = np.random.default_rng(7)
    for _ in range(300):
        q = rng.integers(0, 16)
        s = np.float16(rng.uniform(1e-3, 20))
        z = np.float16(-rng.uniform(0, 15) * float(s))
        got = O._fma_f16(np.array([q]), np.array([s]), np.array([z]))[0]
        assert got == _fma_f16_bruteforce(q, s, z)
    # a case where mul-then-add (two roundings) differs from the fused result
    found = False
    for _ in range(2000):
        q = rng.integers(1, 16)
        s = np.float16(rng.uniform(1e-3, 20))
        z = np.float16(-rng.uniform(0, 15) * float(s))
        two_step = np.float16(np.float32(np.float16(np.float32(q) * np.float32(s))) + np.float32(z))
        fused = O._fma_f16(np.array([q]), np.array([s]), np.array([z]))[0]
        assert fused == _fma_f16_bruteforce(q, s, z)
        found |= bool(two_step != fused)
    assert found   # the fused rule is observably different from multiply-then-add


def test_dequant_to_i8_truncates_toward_zero():
    N, K = 4, 128
    q = np.zeros((N, K), np.uint8)
    q[0, :4] = [1, 2, 3, 15]
    s = np.full((8, N), 0, np.float16)
    z = np.full((8, N), 0, np.float16)
    s[0, :] = 1.5
    z[0, :] = -4.0            # values: -4, -2.5, -1, 0.5, 18.5
    w8 = O.dequant_to_i8(O.pack_int_awq(q), s, z)
    assert w8[0, :5].tolist() == [-2, -1, 0, 18, -4]   # -2.5->-2, -1, 0.5->0, 18.5->18, q=0 -> -4
    # saturation (cannot arise from prepare_weights, defined as clipping)
    s[0, :] = 100
    assert O.dequant_to_i8(O.pack_int_awq(q), s, z).max() == 127


def test_prepared_weights_roundtrip_error():
    w = O.synth_weights(32, 512, seed=4)
    p = O.prepare_weights(w)
    assert p["qweight"].shape == (8, 512) and p["qweight"].dtype == np.int16
    assert p["scales"].shape == (8, 32) and p["scales_1"].shape == (32,)
    w16 = O.dequant_to_f16(p["qweight"], p["scales"], p["scaled_zeros"])
    s1 = p["scales_1"].astype(np.float32)[:, None]
    # 4-bit step in the int8 domain is <= 254/15; half a step plus int8 rounding, scaled back
    bound = (254 / 15 / 2 + 0.5) * s1 * 1.02
    assert (np.abs(w16.astype(np.float32) - w.astype(np.float32)) <= bound).all()
    w8 = O.dequant_to_i8(p["qweight"], p["scales_to8"], p["scaled_zeros_to8"])
    assert np.abs(w8.astype(np.int32)).max() <= 127
    assert np.abs(w8.astype(np.int32) - p["w8_step1"]).max() <= 254 / 15 / 2 + 1.01
    assert not np.array_equal(w8, p["w8_step1"])   # C8 output is NOT the step-1 int8 tensor


# ---------------------------------------------------------------- A (quant_f16_to_i8.cu:45-81)
def test_quant_act_hand_cases():
    x = np.zeros((4, 8), np.float16)
    x[1] = [127, -127, 63.5, 62.5, 0.5, -0.5, 1.5, 2.5]      # t == 1 exactly -> ties to even
    x[2] = [2, -1, 0.5, 0, 0, 0, 0, 0]
    x[3, 0] = -65504
    q, s = O.quant_act_i8(x)
    assert q[0].tolist() == [0] * 8 and s[0] == 0             # 0*inf = NaN -> 0
    assert q[1].tolist() == [127, -127, 64, 62, 0, 0, 2, 2] and s[1] == np.float16(1.0)
    t = np.float32(127) / np.float32(2)
    assert q[2, :3].tolist() == [127, int(np.rint(np.float32(-1) * t)), int(np.rint(np.float32(0.5) * t))]
    assert q[2, 1] == -64 and q[2, 2] == 32                   # -63.5 -> -64, 31.75 -> 32
    assert s[2] == np.float16(np.float32(2) / np.float32(127))
    assert q[3, 0] == -127 and s[3] == np.float16(np.float32(65504) / np.float32(127))


def test_quant_act_invariants():
    x = O.synth_acts(32, 1024, seed=9)
    q, s = O.quant_act_i8(x)
    assert (np.abs(q.astype(np.int32)).max(axis=1) == 127).all()
    amax = np.abs(x.astype(np.float32)).max(1)
    assert np.array_equal(s, (amax / np.float32(127)).astype(np.float16))
    recon = q.astype(np.float32) * (amax / 127)[:, None]
    assert np.abs(recon - x.astype(np.float32)).max() <= (amax / 127).max() * 0.5 * (1 + 1e-5)
    assert np.array_equal(np.sign(q), np.sign(np.where(np.abs(recon) > 0, x, 0)).astype(np.int8))


# ---------------------------------------------------------------- G8
def test_gemm_i8_exact_against_python_ints():
    rng = np.random.default_rng(3)
    a = rng.integers(-128, 128, size=(5, 256)).astype(np.int8)
    w = rng.integers(-128, 128, size=(7, 256)).astype(np.int8)
    acc = O.gemm_i8_acc(a, w)
    assert acc.dtype == np.int32
    for m in range(5):
        for n in range(7):
            assert int(acc[m, n]) == sum(int(x) * int(y) for x, y in zip(a[m], w[n]))
    # extreme: every product is (-128)*(-128), K = 14336 (largest K on the path)
    a = np.full((1, 14336), -128, np.int8)
    assert int(O.gemm_i8_acc(a, a)[0, 0]) == 128 * 128 * 14336


def test_w8a8_epilogue_order():
    acc = np.array([[(1 << 24) + 1, -3], [5, 100000]], dtype=np.int32)   # first needs int->float rounding
    ws = np.array([0.001, 0.5], np.float16)
    as_ = np.array([0.01, 0.002], np.float16)
    out = O.w8a8_epilogue(acc, ws, as_)
    for m in range(2):
        for n in range(2):
            s = np.float32(np.float32(ws[n]) * np.float32(as_[m]))
            want = np.float16(np.float32(np.float32(acc[m, n]) * s))
            assert out[m, n] == want
    # linearity check against fp64: relative error stays at fp16 epsilon
    ref = acc.astype(np.float64) * ws.astype(np.float64)[None, :] * as_.astype(np.float64)[:, None]
    assert np.abs(out.astype(np.float64) - ref).max() / np.abs(ref).max() < 1e-3


# ---------------------------------------------------------------- fp16-output lanes against an unquantised reference
def test_switched_forward_lanes_close_to_dense():
    N, K, M = 64, 512, 8
    w = O.synth_weights(N, K, seed=12)
    x = O.synth_acts(M, K, seed=13)
    p = O.prepare_weights(w)
    dense = x.astype(np.float64) @ w.astype(np.float64).T
    for name in ("w4a16_gemv", "w4a16_gemm", "fp16", "w8a8", "w8a16_gemm"):
        out = O.switched_forward(x, p, O.COMP_TYPE_NAME[name]).astype(np.float64)
        rel = np.abs(out - dense).mean() / np.abs(dense).mean()
        assert rel < 0.2, (name, rel)          # the reference's own acceptance bar (test/mpGEMM.py:48-54)
    a = O.switched_forward(x, p, O.COMP_TYPE_NAME["fp16"])
    b = O.switched_forward(x, p, O.COMP_TYPE_NAME["w4a16_gemv"])
    assert np.array_equal(a, b)
    c = O.switched_forward(x, p, O.COMP_TYPE_NAME["w8a16_gemm"])
    assert O.max_abs_rel(c, a) < 0.05
