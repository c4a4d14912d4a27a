"""GPU parity of the fused RMSNorm + activation quantiser (kmi_rmsnorm_quant_act) and of the activation-matching
host layer: bit-exact against the oracle in the kernel's order of summation, closed-form rows, the size-independent
property "int8 output == stand-alone quantiser applied to the fp16 output" at full size, and DynamicLinear consuming
activations that arrive in the format of its lane."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")
from oracle import kairos_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from kairos_amd import ops as _ops
    return _ops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def bits(t):
    return t.cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("K", [128, 1000, 3584, 4096, 8192, 8200, 14336, 18944, 32768])
@pytest.mark.parametrize("M", [1, 5, 300])
def test_norm_quant_matches_oracle_bit_for_bit(ops, M, K):
    x = O.synth_acts(M, K, seed=M + K)
    rng = np.random.default_rng(K)
    gamma = (1.0 + 0.2 * rng.standard_normal(K)).astype(np.float16)
    res = (rng.standard_normal((M, K)) * 0.5).astype(np.float16)
    for residual in (None, res):
        q, s, y, h = O.rmsnorm_quant_act(x, gamma, 1e-5, residual)
        gy, gq, gs, gh = ops.rmsnorm_quant(dev(x), dev(gamma), 1e-5, None if residual is None else dev(residual))
        assert np.array_equal(bits(gy), y.view(np.uint16))
        assert np.array_equal(gq.cpu().numpy(), q) and np.array_equal(bits(gs), s.view(np.uint16))
        if residual is None:
            assert gh is None
        else:
            assert np.array_equal(bits(gh), h.view(np.uint16))
    # one format only: the other output is not produced, the produced one is unchanged
    y_only = ops.rmsnorm_quant(dev(x), dev(gamma), 1e-5, want_i8=False)
    assert y_only[1] is None and y_only[2] is None
    assert np.array_equal(bits(y_only[0]), O.rmsnorm_f16(x, gamma, 1e-5)[0].view(np.uint16))
    q_only = ops.rmsnorm_quant(dev(x), dev(gamma), 1e-5, dev(res), want_f16=False)
    assert q_only[0] is None and np.array_equal(q_only[1].cpu().numpy(), q) and np.array_equal(bits(q_only[3]), h.view(np.uint16))


def test_constant_magnitude_rows_closed_form(ops):
    """|x| = 2^e per row: y = gamma * sign exactly with eps = 0 (see tests/test_oracle_norm.py), and the int8 row is
    the quantiser applied to that."""
    K, M = 4096, 6
    rng = np.random.default_rng(0)
    e = np.array([-3, -1, 0, 1, 2, 5])[:, None]
    sign = rng.choice(np.array([-1.0, 1.0]), size=(M, K))
    x = (sign * 2.0 ** e).astype(np.float16)
    gamma = rng.standard_normal(K).astype(np.float16)
    want = (gamma[None, :].astype(np.float32) * sign).astype(np.float16)
    y, q, s, _ = ops.rmsnorm_quant(dev(x), dev(gamma), 0.0)
    assert np.array_equal(bits(y), want.view(np.uint16))
    q_ref, s_ref = O.quant_act_i8(want)
    assert np.array_equal(q.cpu().numpy(), q_ref) and np.array_equal(bits(s), s_ref.view(np.uint16))
    y3, _, _, _ = ops.rmsnorm_quant(dev(x[2:3]), dev(gamma), 3.0, want_i8=False)          # e = 0: var + eps = 4
    assert np.array_equal(bits(y3)[0], (gamma.astype(np.float32) * (sign[2] * 0.5)).astype(np.float16).view(np.uint16))


def test_zero_tokens_and_empty_batch(ops):
    gamma = torch.ones(256, dtype=torch.float16, device="cuda")
    y, q, s, _ = ops.rmsnorm_quant(torch.zeros(3, 256, dtype=torch.float16, device="cuda"), gamma, 1e-5)
    assert not y.any() and not q.any() and not s.any()
    y, q, s, _ = ops.rmsnorm_quant(torch.zeros(0, 256, dtype=torch.float16, device="cuda"), gamma, 1e-5)
    assert y.shape == (0, 256) and q.shape == (0, 256) and s.shape == (0,)
    with pytest.raises(ValueError):
        ops.rmsnorm_quant(torch.zeros(2, 256, dtype=torch.float16, device="cuda"), gamma[:128].contiguous(), 1e-5)


@pytest.mark.parametrize("M,K", [(4096, 4096), (30720, 4096), (2048, 14336)])
def test_full_size_int8_equals_quantiser_of_fp16_output(ops, M, K):
    """At the benchmark's sizes: the int8 / scale outputs must equal the stand-alone quantiser run on the kernel's own
    fp16 output (composition), the fp16 output must not depend on which formats were asked for, sampled rows must match
    the oracle, and h must be the fp16 sum."""
    g = torch.Generator(device="cuda").manual_seed(M + K)
    x = torch.randn((M, K), generator=g, device="cuda", dtype=torch.float16)
    res = torch.randn((M, K), generator=g, device="cuda", dtype=torch.float16)
    gamma = (1.0 + 0.1 * torch.randn((K,), generator=g, device="cuda")).to(torch.float16)
    y, q, s, h = ops.rmsnorm_quant(x, gamma, 1e-5, res)
    assert torch.equal(h, x + res)
    q2 = torch.empty_like(q)
    s2 = torch.empty_like(s)
    ops.quant_fp16_to_int8(q2, y, s2)
    assert torch.equal(q, q2) and torch.equal(s.view(torch.int16), s2.view(torch.int16))
    y_only = ops.rmsnorm_quant(h, gamma, 1e-5, want_i8=False)[0]
    assert torch.equal(y_only.view(torch.int16), y.view(torch.int16))
    rows = np.unique(np.concatenate([[0, M - 1], np.random.default_rng(K).integers(0, M, 14)]))
    ridx = torch.from_numpy(rows).cuda()
    yo, _ = O.rmsnorm_f16(h[ridx].cpu().numpy(), gamma.cpu().numpy(), 1e-5)
    assert np.array_equal(bits(y[ridx]), yo.view(np.uint16))


def test_dynamic_linear_consumes_matched_activations(ops):
    """MatchedRMSNorm asks its consumers for their lane: int8 + scales where it is W8A8, fp16 elsewhere, both when the
    consumers disagree.  The linear's output must equal, bit for bit, its output on the fp16 norm result."""
    from kairos.act_matching import MatchedRMSNorm
    from kairos.dynamic_linear import DynamicLinear
    from kairos.perf_profiler import Profiler
    K = 512
    shapes = [(256, K), (384, K)]
    prof = Profiler(shapes)
    for r, name in [(8, 'w4a16_gemv'), (64, 'w4a16_gemm'), (4096, 'w8a8')]:
        prof.record_best_comp(shapes[0], r, name)
    for r, name in [(8, 'w4a16_gemv'), (256, 'w4a16_gemm'), (4096, 'w8a8')]:
        prof.record_best_comp(shapes[1], r, name)
    old = DynamicLinear.prof
    DynamicLinear.prof = prof
    try:
        lins = []
        for i, (N, _) in enumerate(shapes):
            lin = torch.nn.Linear(K, N, bias=False, dtype=torch.float16)
            with torch.no_grad():
                lin.weight.copy_(torch.from_numpy(O.synth_weights(N, K, seed=20 + i)))
            lins.append(DynamicLinear.from_module(lin.cuda(), 'cuda'))
        gamma = (1.0 + 0.1 * torch.randn(K)).to(torch.float16).cuda()
        norm = MatchedRMSNorm(gamma, 1e-5, lins)
        for B, S, formats in [(1, 4, (True, False)), (2, 50, (True, True)), (3, 100, (False, True))]:
            assert norm.formats_for(B * S) == formats
            x = torch.from_numpy(O.synth_acts(B * S, K, seed=S)).cuda().reshape(B, S, K)
            act, h = norm(x)
            assert h is None and (act.f16 is not None, act.int_x is not None) == formats and act.shape == x.shape
            y = ops.rmsnorm_quant(x, gamma, 1e-5, want_i8=False)[0]
            for lin in lins:
                got = lin(act)
                assert got.shape == (B, S, lin.out_features)
                assert torch.equal(got.view(torch.int16), lin(y).view(torch.int16))
        only_i8, _ = norm(torch.from_numpy(O.synth_acts(300, K, seed=1)).cuda())
        with pytest.raises(ValueError):                       # forcing an fp16 lane on int8-only activations
            lins[0].pre_m, lins[0].comp_type = 300, 0
            lins[0](only_i8)
    finally:
        DynamicLinear.prof = old


@pytest.mark.parametrize("M,I", [(1, 128), (7, 1000), (33, 14336), (3, 18944), (2, 32768)])
def test_silu_mul_quant_against_oracle(ops, M, I):
    """SiLU within one fp16 step of the oracle (the exponential is an approximation on both sides), hence y within
    two, equal on > 99 % of the elements; the int8 / scale outputs are exactly the quantiser applied to the y the kernel produced, whichever
    outputs were asked for."""
    rng = np.random.default_rng(M + I)
    gu = (rng.standard_normal((M, 2 * I)) * 2.5).astype(np.float16)
    gu[:, ::97] *= 8
    y, q, s = ops.silu_mul_quant(dev(gu))
    want = O.silu_mul_f16(gu)
    a, b = y.cpu().numpy().view(np.uint16).astype(np.int32), want.view(np.uint16).astype(np.int32)
    line = lambda u: np.where(u & 0x8000, -(u & 0x7FFF), u)
    d = np.abs(line(a) - line(b))
    assert d.max() <= 2 and (d == 0).mean() > 0.99, (d.max(), (d == 0).mean())
    q_ref, s_ref = O.quant_act_i8(y.cpu().numpy())
    assert np.array_equal(q.cpu().numpy(), q_ref) and np.array_equal(bits(s), s_ref.view(np.uint16))
    y2, none_q, none_s = ops.silu_mul_quant(dev(gu), want_i8=False)
    assert none_q is None and none_s is None and torch.equal(y2.view(torch.int16), y.view(torch.int16))
    none_y, q2, s2 = ops.silu_mul_quant(dev(gu), want_f16=False)
    assert none_y is None and torch.equal(q2, q) and torch.equal(s2.view(torch.int16), s.view(torch.int16))


def test_silu_mul_quant_full_size_and_exact_points(ops):
    M, I = 4096, 14336
    g = torch.Generator(device="cuda").manual_seed(3)
    gu = torch.randn((M, 2 * I), generator=g, device="cuda", dtype=torch.float16) * 2
    y, q, s = ops.silu_mul_quant(gu)
    q2, s2 = torch.empty_like(q), torch.empty_like(s)
    ops.quant_fp16_to_int8(q2, y, s2)
    assert torch.equal(q, q2) and torch.equal(s.view(torch.int16), s2.view(torch.int16))
    ref = torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]              # the eager module on the same device
    assert float((y.float() - ref.float()).abs().max()) <= float(ref.abs().max()) * 2.0 ** -10
    rows = torch.tensor([0, 1, M // 2, M - 1], device="cuda")
    want = O.silu_mul_f16(gu[rows].cpu().numpy())
    got = y[rows].cpu().numpy()
    assert (got.view(np.uint16) == want.view(np.uint16)).mean() > 0.99
    # exact points: silu(0) * u = 0, silu(g) = g for g >= 20, an all-zero token quantises to zeros with scale 0
    pts = torch.tensor([[0.0, 20.0, 64.0, 1000.0] + [0.0] * 4 + [3.0, 0.5, -2.0, 1.0] + [0.0] * 4,
                        [0.0] * 16], dtype=torch.float16, device="cuda")
    y, q, s = ops.silu_mul_quant(pts)
    assert y[0, :4].tolist() == [0.0, 10.0, -128.0, 1000.0] and not y[1].any() and not q[1].any() and float(s[1]) == 0.0
    with pytest.raises(ValueError):
        ops.silu_mul_quant(torch.zeros(2, 129, dtype=torch.float16, device="cuda"))


def test_matched_silu_mul_feeds_the_down_projection(ops):
    from kairos.act_matching import MatchedSiluMul
    from kairos.dynamic_linear import DynamicLinear
    from kairos.perf_profiler import Profiler
    I, N = 1024, 256
    prof = Profiler([(N, I)])
    for r, name in [(8, 'w4a16_gemv'), (64, 'w4a16_gemm'), (4096, 'w8a8')]:
        prof.record_best_comp((N, I), r, name)
    old = DynamicLinear.prof
    DynamicLinear.prof = prof
    try:
        lin = torch.nn.Linear(I, N, bias=False, dtype=torch.float16)
        with torch.no_grad():
            lin.weight.copy_(torch.from_numpy(O.synth_weights(N, I, seed=31)))
        down = DynamicLinear.from_module(lin.cuda(), 'cuda')
        act_fn = MatchedSiluMul([down])
        for M, formats in [(4, (True, False)), (40, (True, False)), (200, (False, True))]:
            assert act_fn.formats_for(M) == formats
            gu = torch.randn((1, M, 2 * I), dtype=torch.float16, device="cuda")
            act = act_fn(gu)
            assert act.shape == (1, M, I) and (act.f16 is not None, act.int_x is not None) == formats
            y = ops.silu_mul_quant(gu, want_i8=False)[0]
            assert torch.equal(down(act).view(torch.int16), down(y).view(torch.int16))
    finally:
        DynamicLinear.prof = old
