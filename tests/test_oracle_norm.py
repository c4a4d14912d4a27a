"""Pins the oracle's RMSNorm restatement (oracle.kairos_oracle.rmsnorm_f16), which the reference itself does not pin:
its modules run the eager norm of the loaded checkpoint.  Three independent anchors: rows whose result has a closed
form (every step exact, so any order of summation and any correct root give the same bits), torch's own CPU ops
composed the way the eager decoder module composes them, and the float64 sum against the kernel-ordered fp32 sum."""
import numpy as np
import pytest

from oracle import kairos_oracle as O


def ulp_distance(a, b):
    """Distance in fp16 steps between two fp16 arrays (sign-magnitude bits mapped to a line)."""
    def line(v):
        u = v.view(np.uint16).astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u)
    return np.abs(line(a) - line(b))


@pytest.mark.parametrize("K", [128, 3584, 4096])
@pytest.mark.parametrize("exact_sum", [False, True])
def test_constant_magnitude_rows_have_a_closed_form(K, exact_sum):
    """|x| = 2^e on the whole row: sum = K * 4^e exactly, var = 4^e, and with eps = 0 the factor is 2^-e, with
    eps = 3 * 4^e it is 2^-(e+1): y = gamma * sign (or gamma * sign / 2), exactly.  A dropped eps, a sum instead of
    a mean, a missing root or gamma applied before the rounding to fp16 each change these bits."""
    rng = np.random.default_rng(K)
    M = 6
    e = np.array([-3, -1, 0, 1, 2, 5])[:, None]
    sign = rng.choice(np.array([-1.0, 1.0]), size=(M, K))
    x = (sign * 2.0 ** e).astype(np.float16)
    gamma = rng.standard_normal(K).astype(np.float16)
    y, h = O.rmsnorm_f16(x, gamma, 0.0, exact_sum=exact_sum)
    assert h is not None and np.array_equal(h, x)
    assert np.array_equal(y.view(np.uint16), (gamma[None, :].astype(np.float32) * sign).astype(np.float16).view(np.uint16))
    for m in range(M):                                         # eps is per call: one row at a time
        y1, _ = O.rmsnorm_f16(x[m:m + 1], gamma, 3.0 * 4.0 ** float(e[m, 0]), exact_sum=exact_sum)
        want = (gamma.astype(np.float32) * (sign[m] * 0.5).astype(np.float16).astype(np.float32)).astype(np.float16)
        assert np.array_equal(y1[0].view(np.uint16), want.view(np.uint16))


def test_against_torch_cpu_ops_composed_as_the_eager_module():
    """hidden.to(float32); variance = hidden.pow(2).mean(-1); hidden * rsqrt(variance + eps); weight * hidden.to(fp16):
    the library routine fixes everything but the order of the fp32 sum, which moves the result by at most a step of
    the intermediate rounding (two steps of the product on rare elements)."""
    torch = pytest.importorskip("torch")
    for K, seed in ((4096, 1), (3584, 2), (14336, 3)):
        x = O.synth_acts(33, K, seed=seed)
        gamma = (1.0 + 0.1 * np.random.default_rng(seed).standard_normal(K)).astype(np.float16)
        eps = 1e-5
        hs = torch.from_numpy(x).to(torch.float32)
        var = hs.pow(2).mean(-1, keepdim=True)
        ref = (torch.from_numpy(gamma) * (hs * torch.rsqrt(var + eps)).to(torch.float16)).numpy()
        for exact_sum in (False, True):
            y, _ = O.rmsnorm_f16(x, gamma, eps, exact_sum=exact_sum)
            d = ulp_distance(y, ref)
            assert d.max() <= 2 and (d == 0).mean() > 0.995, (K, exact_sum, d.max(), (d == 0).mean())


def test_kernel_ordered_sum_against_float64_sum():
    for K in (128, 1024, 4096, 32768):
        x = O.synth_acts(17, K, seed=K)
        gamma = np.random.default_rng(K).standard_normal(K).astype(np.float16)
        a, _ = O.rmsnorm_f16(x, gamma, 1e-6)
        b, _ = O.rmsnorm_f16(x, gamma, 1e-6, exact_sum=True)
        d = ulp_distance(a, b)
        assert d.max() <= 2 and (d == 0).mean() > 0.995


def test_residual_is_added_in_fp16_with_one_rounding():
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((9, 256)) * 10).astype(np.float16)
    res = (rng.standard_normal((9, 256)) * 0.01).astype(np.float16)
    gamma = np.ones(256, dtype=np.float16)
    y, h = O.rmsnorm_f16(x, gamma, 1e-5, residual=res)
    want = (x.astype(np.float64) + res.astype(np.float64)).astype(np.float16)     # the float64 sum of two fp16 is exact
    assert np.array_equal(h.view(np.uint16), want.view(np.uint16))
    y2, _ = O.rmsnorm_f16(h, gamma, 1e-5)
    assert np.array_equal(y.view(np.uint16), y2.view(np.uint16))


def test_quantised_form_is_the_quantiser_on_the_norm_output():
    x = O.synth_acts(12, 512, seed=3)
    gamma = np.random.default_rng(3).standard_normal(512).astype(np.float16)
    q, s, y, _ = O.rmsnorm_quant_act(x, gamma, 1e-5)
    q2, s2 = O.quant_act_i8(y)
    assert np.array_equal(q, q2) and np.array_equal(s.view(np.uint16), s2.view(np.uint16))
    assert np.abs(q).max(axis=1).min() == 127                  # every row reaches full scale
    zero = np.zeros((2, 512), dtype=np.float16)                # an all-zero token: zeros and scale 0
    q0, s0, y0, _ = O.rmsnorm_quant_act(zero, gamma, 1e-5)
    assert not q0.any() and not s0.any() and not y0.any()


def test_silu_mul_against_torch_cpu_and_exact_points():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(7)
    gu = (rng.standard_normal((64, 2 * 512)) * 3).astype(np.float16)
    y = O.silu_mul_f16(gu)
    t = torch.from_numpy(gu)
    ref = (torch.nn.functional.silu(t[:, :512]) * t[:, 512:]).numpy()
    d = ulp_distance(y, ref)                                  # one step of s can become two of the product
    assert d.max() <= 2 and (d == 0).mean() > 0.99
    # exact points: silu(0) = 0; for g >= 20, exp(-g) < 2^-28 so silu(g) = g in fp32; for g <= -20 the result is
    # below the smallest fp16 subnormal times ... and rounds to -0
    g = np.array([[0.0, 20.0, 64.0, 1000.0, -30.0, -1000.0]], dtype=np.float16)
    u = np.array([[3.0, 0.5, -2.0, 1.0, 1.0, 1.0]], dtype=np.float16)
    out = O.silu_mul_f16(np.concatenate([g, u], axis=1))
    assert np.array_equal(out[0, :4], np.array([0.0, 10.0, -128.0, 1000.0], dtype=np.float16))
    assert abs(float(out[0, 4])) < 1e-6 and out[0, 5] == 0
    # silu(g) - silu(-g) = g: with u = 1 the two halves of a symmetric input differ by g up to the two roundings
    g = (rng.standard_normal((4, 256)) * 4).astype(np.float16)
    one = np.ones_like(g)
    a = O.silu_mul_f16(np.concatenate([g, one], axis=1)).astype(np.float64)
    b = O.silu_mul_f16(np.concatenate([-g, one], axis=1)).astype(np.float64)
    assert np.all(np.abs((a - b) - g.astype(np.float64)) <= 2.0 ** -10 * np.maximum(np.abs(g.astype(np.float64)), 2.0 ** -4))
