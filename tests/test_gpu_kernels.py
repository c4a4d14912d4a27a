"""GPU parity tests proper: every HIP kernel, called through the C ABI, against the CPU oracle on the
same seeded inputs.  Bit-exact for conversion, activation quantisation and int32 accumulators;
max-abs-rel <= 1e-2 (in practice ~1e-3) for fp16 outputs."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")
from oracle import kairos_oracle as O

pytestmark = pytest.mark.gpu
TOL = 1e-2          # fp16-output tolerance (max|out-ref| / max|ref|)


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from kairos_amd import ops as _ops
    return _ops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def assert_same_bits(got, want):
    got = np.ascontiguousarray(got)
    want = np.ascontiguousarray(want)
    assert got.shape == want.shape and got.dtype == want.dtype
    bits = {1: np.uint8, 2: np.uint16, 4: np.uint32}[got.dtype.itemsize]
    bad = np.argwhere(got.view(bits) != want.view(bits))
    if len(bad):
        lines = [f"{tuple(i)}: got {got[tuple(i)]!r} want {want[tuple(i)]!r}" for i in bad[:8]]
        raise AssertionError(f"{len(bad)} of {got.size} elements differ\n" + "\n".join(lines))


_PREP = {}


def prep(N, K, seed=10):
    key = (N, K, seed)
    if key not in _PREP:
        p = O.prepare_weights(O.synth_weights(N, K, seed))
        p["w16"] = O.dequant_to_f16(p["qweight"], p["scales"], p["scaled_zeros"])
        p["w8"] = O.dequant_to_i8(p["qweight"], p["scales_to8"], p["scaled_zeros_to8"])
        _PREP[key] = p
    return _PREP[key]


# ------------------------------------------------------------------ conversion (C16 / C8), bit-exact
@pytest.mark.parametrize("N,K", [(4, 128), (64, 256), (128, 512), (256, 3584), (512, 4096)])
def test_cvt_prepared_weights_bit_exact(ops, N, K):
    p = prep(N, K)
    qw = dev(p["qweight"])
    out16 = torch.empty((N, K), dtype=torch.float16, device="cuda")
    ops.dequant_interleaved_int4_to_fp16(out16, qw, dev(p["scales"]), dev(p["scaled_zeros"]), 128)
    assert_same_bits(host(out16), p["w16"])
    out8 = torch.empty((N, K), dtype=torch.int8, device="cuda")
    ops.dequant_interleaved_int4_to_int8(out8, qw, dev(p["scales_to8"]), dev(p["scaled_zeros_to8"]), 128)
    assert_same_bits(host(out8), p["w8"])


def test_cvt_random_tables_bit_exact(ops):
    """Arbitrary (not prepare_weights) tables: subnormal products, negative scales, saturation."""
    N, K = 64, 512
    rng = np.random.default_rng(21)
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    qw = O.pack_int_awq(q)
    Gp = O.padded_groups(K)
    s = np.zeros((Gp, N), np.float16)
    z = np.zeros((Gp, N), np.float16)
    s[: K // 128] = rng.choice([1e-7, 3e-5, 1e-3, 0.3, 7.0, -2.5, 40.0], size=(K // 128, N)).astype(np.float16)
    z[: K // 128] = (rng.standard_normal((K // 128, N)) * 30).astype(np.float16)
    out16 = torch.empty((N, K), dtype=torch.float16, device="cuda")
    ops.dequant_interleaved_int4_to_fp16(out16, dev(qw), dev(s), dev(z), 128)
    assert_same_bits(host(out16), O.dequant_to_f16(qw, s, z))
    out8 = torch.empty((N, K), dtype=torch.int8, device="cuda")
    ops.dequant_interleaved_int4_to_int8(out8, dev(qw), dev(s), dev(z), 128)
    assert_same_bits(host(out8), O.dequant_to_i8(qw, s, z))


def test_cvt_identity_is_pure_unpack(ops):
    N, K = 128, 256
    rng = np.random.default_rng(22)
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    Gp = O.padded_groups(K)
    out8 = torch.empty((N, K), dtype=torch.int8, device="cuda")
    ops.dequant_interleaved_int4_to_int8(out8, dev(O.pack_int_awq(q)), dev(np.ones((Gp, N), np.float16)),
                                         dev(np.zeros((Gp, N), np.float16)), 128)
    assert np.array_equal(host(out8), q.astype(np.int8))


@pytest.mark.parametrize("N,K", [(128, 128), (256, 512), (384, 3584)])
def test_cvt_tiled_roundtrip(ops, N, K):
    p = prep(N, K)
    qw = dev(p["qweight"])
    t16 = torch.empty((N, K), dtype=torch.float16, device="cuda")
    ops.dequant_interleaved_int4_to_fp16(t16, qw, dev(p["scales"]), dev(p["scaled_zeros"]), 128, tiled=True)
    assert np.array_equal(host(ops.untile(t16, N, K)).view(np.uint16), p["w16"].view(np.uint16))
    t8 = torch.empty((N, K), dtype=torch.int8, device="cuda")
    ops.dequant_interleaved_int4_to_int8(t8, qw, dev(p["scales_to8"]), dev(p["scaled_zeros_to8"]), 128, tiled=True)
    assert np.array_equal(host(ops.untile(t8, N, K)), p["w8"])
    if N * K > 128 * 128:
        assert not np.array_equal(host(t8).reshape(N, K), p["w8"])     # the layout really is permuted


# ------------------------------------------------------------------ activation quantiser (A), bit-exact
@pytest.mark.parametrize("M,K", [(1, 128), (3, 4096), (16, 4096), (33, 14336), (257, 1024), (5, 28672)])
def test_quant_act_bit_exact(ops, M, K):
    x = O.synth_acts(M, K, seed=M + K)
    if M >= 3:
        x[1] = 0                                            # all-zero token
        x[2, : min(K, 512)] = np.linspace(-3, 3, min(K, 512)).astype(np.float16)
    q_ref, s_ref = O.quant_act_i8(x)
    xd = dev(x)
    q = torch.empty((M, K), dtype=torch.int8, device="cuda")
    s = torch.empty((M,), dtype=torch.float16, device="cuda")
    ops.quant_fp16_to_int8(q, xd, s)
    assert_same_bits(host(s), s_ref)
    assert_same_bits(host(q), q_ref)


def test_quant_act_ties_and_extremes(ops):
    K = 128
    x = np.zeros((4, K), np.float16)
    x[0, :8] = [127, -127, 63.5, 62.5, 0.5, -0.5, 1.5, 2.5]
    x[1, 0] = -65504
    x[1, 1] = 65504
    x[2, :3] = [6e-8, -6e-8, 0]                             # smallest subnormal
    x[3, :4] = [2, -1, 0.5, 1e-4]
    q_ref, s_ref = O.quant_act_i8(x)
    q = torch.empty((4, K), dtype=torch.int8, device="cuda")
    s = torch.empty((4,), dtype=torch.float16, device="cuda")
    ops.quant_fp16_to_int8(q, dev(x), s)
    assert np.array_equal(host(q), q_ref) and np.array_equal(host(s).view(np.uint16), s_ref.view(np.uint16))
    assert host(q)[0, :8].tolist() == [127, -127, 64, 62, 0, 0, 2, 2]


# ------------------------------------------------------------------ W4A16 small-M (Gv), 1e-2
@pytest.mark.parametrize("M", [1, 2, 5, 16, 17, 31, 32, 33, 48, 64])
@pytest.mark.parametrize("N,K", [(256, 512), (1024, 4096)])
def test_gemv_w4a16(ops, M, N, K):
    p = prep(N, K)
    x = O.synth_acts(M, K, seed=100 + M)
    ref = O.gemm_f16(x, p["w16"])
    out = ops.gemv_forward(dev(x)[None], dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), M, N, K, 128)
    assert out.shape == (1, M, N)
    assert O.max_abs_rel(host(out)[0], ref) < TOL


@pytest.mark.parametrize("nt,nw", [(1, 4), (1, 8), (1, 16), (2, 4), (2, 8), (4, 4), (4, 8)])
@pytest.mark.parametrize("M", [3, 20])
def test_gemv_every_split(ops, M, nt, nw):
    N, K = 512, 2048
    p = prep(N, K)
    x = O.synth_acts(M, K, seed=7)
    ref = O.gemm_f16(x, p["w16"])
    out = ops.gemv_forward(dev(x), dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), M, N, K, 128, cfg=(nt, nw))
    assert O.max_abs_rel(host(out), ref) < 2e-3
    again = ops.gemv_forward(dev(x), dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), M, N, K, 128, cfg=(nt, nw))
    assert torch.equal(out, again)                          # fixed reduction order


@pytest.mark.parametrize("nw", [4, 8])
@pytest.mark.parametrize("M,N", [(8, 512), (16, 272), (3, 2048)])
def test_gemv_eight_column_tiles(ops, M, N, nw):
    """The 128-column workgroup (one row tile only), also with a ragged last strip; more than 16 rows are refused."""
    K = 1024
    p = prep(N, K)
    x = O.synth_acts(M, K, seed=M)
    out = ops.gemv_forward(dev(x), dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), M, N, K, 128, cfg=(8, nw))
    assert O.max_abs_rel(host(out), O.gemm_f16(x, p["w16"])) < 2e-3
    from kairos_amd._lib import KairosMiError
    with pytest.raises(KairosMiError):
        ops.gemv_forward(dev(O.synth_acts(17, K, seed=1)), dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]),
                         17, N, K, 128, cfg=(8, nw))


@pytest.mark.parametrize("nt", [3, 5, 6, 7])
@pytest.mark.parametrize("nw", [4, 8])
def test_gemv_odd_column_tile_counts(ops, nt, nw):
    """Column tiles per wave that do not divide the strip count: the last workgroup is ragged (33 strips)."""
    N, K = 528, 1024
    p = prep(N, K)
    for M in (2, 16):
        x = O.synth_acts(M, K, seed=M + nt)
        out = ops.gemv_forward(dev(x), dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), M, N, K, 128, cfg=(nt, nw))
        assert O.max_abs_rel(host(out), O.gemm_f16(x, p["w16"])) < 2e-3


@pytest.mark.parametrize("N", [4608, 10240, 28672])
def test_gemv_default_split_on_unbalanced_widths(ops, N):
    """Widths whose default is 2, 3 or 7 column tiles per wave; every M range of the default rule."""
    K = 512
    p = prep(N, K)
    for M in (1, 8, 16, 32, 64):
        x = O.synth_acts(M, K, seed=M)
        out = ops.gemv_forward(dev(x), dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), M, N, K, 128)
        assert O.max_abs_rel(host(out), O.gemm_f16(x, p["w16"])) < 2e-3


@pytest.mark.parametrize("M,nt,nw,ks", [(1, 1, 16, 2), (3, 2, 8, 4), (8, 4, 8, 7), (16, 4, 8, 8), (20, 2, 8, 3), (40, 2, 4, 2), (64, 1, 8, 4)])
def test_gemv_split_over_workgroups(ops, M, nt, nw, ks):
    """K split over several workgroups per column strip (long, narrow weights): the workgroup that arrives last adds the
    partial sums in split order, so the result is the same on every call; the arrival counters are zero again afterwards
    and a second call on the same scratch works; bias applied once."""
    N, K = 320, 3584                                         # 28 groups: uneven over 3, 7 and 8 splits; ragged last strip
    p = prep(N, K)
    x = O.synth_acts(M, K, seed=40 + M)
    bias = np.random.default_rng(M).standard_normal(N).astype(np.float16)
    ref = (O.gemm_w4a16(x, p["qweight"], p["scales"], p["scaled_zeros"]).astype(np.float32) + bias.astype(np.float32)).astype(np.float16)
    args = (dev(x), dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), M, N, K, 128)
    outs = [ops.gemv_forward(*args, bias=dev(bias), cfg=(nt, nw, ks)) for _ in range(4)]
    torch.cuda.synchronize()
    assert O.max_abs_rel(host(outs[0]), ref) < 2e-3
    assert all(torch.equal(outs[0].view(torch.int16), o.view(torch.int16)) for o in outs[1:])
    ws = ops.gemv_workspace_for("cuda")
    assert int(ws[:65536].view(torch.int32).abs().sum().item()) == 0
    unsplit = ops.gemv_forward(*args, bias=dev(bias), cfg=(nt, nw, 1))
    assert O.max_abs_rel(host(outs[0]), host(unsplit)) < 1e-3


def test_gemv_bias_and_ragged_strip(ops):
    N, K, M = 48, 256, 4                                    # N is not a multiple of the 64-column strip
    p = prep(N, K)
    x = O.synth_acts(M, K, seed=3)
    bias = (np.random.default_rng(1).standard_normal(N)).astype(np.float16)
    ref = (O.gemm_f16(x, p["w16"]).astype(np.float32) + bias.astype(np.float32)).astype(np.float16)
    out = ops.gemv_forward(dev(x), dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), M, N, K, 128,
                           bias=dev(bias), cfg=(4, 4))
    assert O.max_abs_rel(host(out), ref) < 2e-3


# ---- ring form of the small-M kernel (operands travel global -> LDS, per-wave ring of slots)
@pytest.mark.parametrize("M,nt,nw,ks", [(1, 1, 8, 1), (3, 2, 4, 1), (4, 7, 8, 1), (5, 2, 8, 2), (8, 8, 4, 1), (9, 3, 8, 1),
                                          (16, 4, 8, 4), (17, 1, 8, 1), (32, 4, 8, 2), (33, 2, 4, 1), (48, 2, 8, 1), (64, 2, 4, 3)])
def test_gemv_ring_equals_register_form(ops, M, nt, nw, ks):
    """Same lanes, same arithmetic, same summation order as the register form with the same split: the two forms agree
    bit for bit at every ring depth (1 = load, wait, compute; 0 = as deep as fits), with bias and a ragged last strip."""
    N, K = 336, 3584                                         # 21 strips (ragged for nt = 2, 4, 8), 28 groups
    p = prep(N, K)
    x = O.synth_acts(M, K, seed=60 + M)
    bias = np.random.default_rng(M).standard_normal(N).astype(np.float16)
    ref = (O.gemm_w4a16(x, p["qweight"], p["scales"], p["scaled_zeros"]).astype(np.float32) + bias.astype(np.float32)).astype(np.float16)
    args = (dev(x), dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), M, N, K, 128)
    want = ops.gemv_forward(*args, bias=dev(bias), cfg=(nt, nw, ks))
    assert O.max_abs_rel(host(want), ref) < 2e-3
    for depth in (1, 2, 3, 0):
        got = ops.gemv_forward(*args, bias=dev(bias), ring=(nt, nw, ks, depth))
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), depth
    ws = ops.gemv_workspace_for("cuda")
    torch.cuda.synchronize()
    assert int(ws[:65536].view(torch.int32).abs().sum().item()) == 0          # arrival counters left at zero


@pytest.mark.parametrize("nw", [1, 2, 8])
@pytest.mark.parametrize("M", [1, 2, 4, 7, 8, 12, 16, 24, 32, 40, 48, 56, 64])
def test_gemv_ring_every_row_count(ops, M, nw):
    """Every activation-load count of the ring form (1, 2, 4, 8, 12, 16 loads per group) against the oracle, also with
    fewer K groups than ring slots and with waves that get no group at all (K = 512: four groups, eight waves)."""
    N = 256
    for K in (512, 2048):
        p = prep(N, K)
        x = O.synth_acts(M, K, seed=M)
        nt = 2 if M <= 32 else 1
        out = ops.gemv_forward(dev(x), dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), M, N, K, 128, ring=(nt, nw, 1, 0))
        assert O.max_abs_rel(host(out), O.gemm_f16(x, p["w16"])) < 2e-3, K


def test_gemv_ring_refuses_what_it_cannot_run(ops):
    from kairos_amd._lib import KairosMiError
    N, K, M = 256, 512, 20
    p = prep(N, K)
    args = (dev(O.synth_acts(M, K, seed=1)), dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), M, N, K, 128)
    with pytest.raises(KairosMiError):
        ops.gemv_forward(*args, ring=(5, 8, 1, 2))            # two row tiles x five column tiles: too many accumulators
    with pytest.raises(KairosMiError):
        ops.gemv_forward(*args, ring=(2, 3, 1, 2))            # waves per workgroup: 1, 2, 4 or 8
    with pytest.raises(ValueError):
        ops.gemv_forward(dev(O.synth_acts(M, 256, seed=1)), *args[1:])     # activation rows shorter than K


def test_gemv_workspace_reset(ops):
    """Counters of unknown history: the reset kernel zeroes the header and nothing else; a split call works afterwards."""
    N, K, M = 320, 3584, 8
    p = prep(N, K)
    x = O.synth_acts(M, K, seed=2)
    args = (dev(x), dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), M, N, K, 128)
    want = ops.gemv_forward(*args, cfg=(2, 8, 4))
    ws = ops.gemv_workspace_for("cuda")
    ws[:65536] = 7                                            # as a launch that died half-way might leave them
    ws[65536:65536 + 64] = 9
    ops.gemv_workspace_reset("cuda")
    torch.cuda.synchronize()
    assert int(ws[:65536].view(torch.int32).abs().sum().item()) == 0 and int(ws[65536:65536 + 64].min().item()) == 9
    assert torch.equal(ops.gemv_forward(*args, cfg=(2, 8, 4)).view(torch.int16), want.view(torch.int16))
    assert torch.equal(ops.gemv_forward(*args, ring=(2, 8, 4, 2)).view(torch.int16), want.view(torch.int16))


def test_read_probes_do_read(ops):
    """The floor probes must move their bytes (a reader whose result nothing observes compiles to an empty kernel): over
    copies of a 235 MB weight that exceed the last-level cache, neither probe can beat 12 TB/s, and both take several
    times an empty launch."""
    from kairos_amd import _lib
    lib = _lib.load()
    N, K = 57344, 8192
    nbytes = N * K // 2
    qw = [torch.randint(-32768, 32767, (N // 4, K), dtype=torch.int16, device="cuda") for _ in range(3)]
    st = ops._stream()

    def timed(fn, n=12):
        for i in range(3):
            assert fn(i) == 0
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(n):
            fn(i)
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e-3 / n                   # seconds per launch

    empty = timed(lambda i: lib.kmi_probe_empty(st))
    plain = timed(lambda i: lib.kmi_probe_stream_read(qw[i % 3].data_ptr(), nbytes, st))
    pattern = timed(lambda i: lib.kmi_probe_gemv_read(qw[i % 3].data_ptr(), N, K, 2, 8, st))
    for t in (plain, pattern):
        assert nbytes / t < 12e12 and t > 4 * empty, (empty, plain, pattern)


# ------------------------------------------------------------------ MFMA GEMMs
GEMM_M = [1, 7, 64, 65, 130, 300]


@pytest.mark.parametrize("tile", [64, 128, 256])
@pytest.mark.parametrize("M", GEMM_M)
def test_gemm_w8a8_int32_bit_exact(ops, M, tile):
    N, K = 384, 1024
    rng = np.random.default_rng(M)
    a8 = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    w8 = rng.integers(-128, 128, size=(N, K)).astype(np.int8)
    ops.force_gemm_tile(tile)
    try:
        acc = ops.w8a8_gemm_acc_i32(dev(a8), dev(w8), N)
    finally:
        ops.force_gemm_tile(0)
    assert np.array_equal(host(acc), O.gemm_i8_acc(a8, w8))


def test_gemm_w8a8_extreme_accumulator(ops):
    M, N, K = 2, 128, 14336
    a8 = np.full((M, K), -128, np.int8)
    w8 = np.full((N, K), -128, np.int8)
    acc = host(ops.w8a8_gemm_acc_i32(dev(a8), dev(w8), N))
    assert (acc == 128 * 128 * K).all()


@pytest.mark.parametrize("tile", [0, 64, 128, 256])
@pytest.mark.parametrize("M", GEMM_M)
def test_gemm_w8a8_path(ops, M, tile):
    """The whole w8a8 lane: C8 -> A -> G8, against the oracle lane; the fp16 result is compared bit for bit
    because the epilogue order is fixed."""
    N, K = 256, 512
    p = prep(N, K)
    x = O.synth_acts(M, K, seed=200 + M)
    ref = O.switched_forward(x, p, O.COMP_TYPE_NAME["w8a8"])
    w8 = torch.empty((N, K), dtype=torch.int8, device="cuda")
    ops.dequant_interleaved_int4_to_int8(w8, dev(p["qweight"]), dev(p["scales_to8"]), dev(p["scaled_zeros_to8"]), 128)
    xd = dev(x)
    a8 = torch.empty_like(xd, dtype=torch.int8)
    sx = torch.empty((M,), dtype=torch.float16, device="cuda")
    ops.quant_fp16_to_int8(a8, xd, sx)
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    ops.force_gemm_tile(tile)
    try:
        ops.w8a8_gemm_forward(a8, w8, dev(p["scales_1"]), sx, out)
    finally:
        ops.force_gemm_tile(0)
    assert_same_bits(host(out), ref)


@pytest.mark.parametrize("tile", [0, 64, 128, 256])
def test_gemm_w8a8_subnormal_token_scales(ops, tile):
    """Tokens whose largest value is below 127 * 2^-14 have a per-token scale that is subnormal in fp16 (down to the
    smallest one, 2^-24), and the epilogue forms scale products on the matrix pipe: they must come out as exactly as the
    oracle's fp32 products do (a pipe that flushed subnormal fp16 inputs would return zeros for these rows)."""
    M, N, K = 70, 256, 512
    p = prep(N, K)
    x = O.synth_acts(M, K, seed=77).astype(np.float32)
    x[::3] *= 1e-4                                            # scales around 3e-6
    x[1::7] *= 1e-6                                           # scales of one or two units of 2^-24
    x = x.astype(np.float16)
    a8_np, sx_np = O.quant_act_i8(x)
    sub = (sx_np.astype(np.float32) < 2.0 ** -14) & (sx_np.astype(np.float32) > 0)
    assert sub.sum() >= 20                                    # the case is what it says
    _, ref = O.gemm_w8a8(a8_np, p["w8"], p["scales_1"], sx_np)
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    ops.force_gemm_tile(tile)
    try:
        ops.w8a8_gemm_forward(dev(a8_np), dev(p["w8"]), dev(p["scales_1"]), dev(sx_np), out)
    finally:
        ops.force_gemm_tile(0)
    assert_same_bits(host(out), ref)
    assert np.abs(host(out)[sub].astype(np.float32)).max() > 0


@pytest.mark.parametrize("tile", [0, 128, 130, 192, 256, 512])  # 130: the 128 x 128 tile with two wave quartets; 512: 512 x 128
@pytest.mark.parametrize("M", GEMM_M)
def test_gemm_w4a8_bit_exact(ops, M, tile):
    """W4A8 (int4 weights decoded to the converter's int8 values inside the int8 MFMA GEMM): int32 accumulators and
    fp16 outputs against the oracle's W8A8 chain, bit for bit; N = 384 leaves both tiles ragged."""
    N, K = 384, 1024
    p = prep(N, K)
    x = O.synth_acts(M, K, seed=700 + M)
    a8, sx = O.quant_act_i8(x)
    acc_ref, out_ref = O.gemm_w8a8(a8, p["w8"], p["scales_1"], sx)
    bias = np.random.default_rng(M).standard_normal(N).astype(np.float16)
    out_b_ref = (out_ref.astype(np.float32) + bias.astype(np.float32)).astype(np.float16)
    qw, s8, z8 = dev(p["qweight"]), dev(p["scales_to8"]), dev(p["scaled_zeros_to8"])
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    out_b = torch.empty((M, N), dtype=torch.float16, device="cuda")
    ops.force_gemm_tile(tile)
    ops.force_gemm_splits(1)
    try:
        acc = ops.w4a8_gemm_acc_i32(dev(a8), qw, s8, z8)
        ops.w4a8_gemm_forward(dev(a8), qw, s8, z8, dev(p["scales_1"]), dev(sx), out)
        ops.w4a8_gemm_forward(dev(a8), qw, s8, z8, dev(p["scales_1"]), dev(sx), out_b, bias=dev(bias))
    finally:
        ops.force_gemm_tile(0)
        ops.force_gemm_splits(0)
    assert_same_bits(host(acc), acc_ref)
    assert_same_bits(host(out), out_ref)
    assert_same_bits(host(out_b), out_b_ref)


@pytest.mark.parametrize("tile", [128, 130, 192, 256, 512])
def test_gemm_w4a8_several_ragged_row_tiles(ops, tile):
    """M = 700 is two 512-row tiles (the second quartet of the second tile lies wholly beyond M), three 256-row tiles
    and six 128-row tiles, all ragged; N = 640 leaves the 256-column tiles ragged: accumulators and biased fp16
    outputs against the oracle's W8A8 chain, bit for bit."""
    M, N, K = 700, 640, 1024
    p = prep(N, K, seed=tile)
    x = O.synth_acts(M, K, seed=tile + 1)
    a8, sx = O.quant_act_i8(x)
    acc_ref, out_ref = O.gemm_w8a8(a8, p["w8"], p["scales_1"], sx)
    bias = np.random.default_rng(tile).standard_normal(N).astype(np.float16)
    out_b_ref = (out_ref.astype(np.float32) + bias.astype(np.float32)).astype(np.float16)
    qw, s8, z8 = dev(p["qweight"]), dev(p["scales_to8"]), dev(p["scaled_zeros_to8"])
    out_b = torch.full((M + 8, N), float("nan"), dtype=torch.float16, device="cuda")     # rows beyond M must stay untouched
    ops.force_gemm_tile(tile)
    ops.force_gemm_splits(1)
    try:
        acc = ops.w4a8_gemm_acc_i32(dev(a8), qw, s8, z8)
        ops.w4a8_gemm_forward(dev(a8), qw, s8, z8, dev(p["scales_1"]), dev(sx), out_b[:M], bias=dev(bias))
    finally:
        ops.force_gemm_tile(0)
        ops.force_gemm_splits(0)
    assert_same_bits(host(acc), acc_ref)
    assert_same_bits(host(out_b[:M]), out_b_ref)
    assert torch.isnan(out_b[M:]).all()


@pytest.mark.parametrize("sel,M,N", [(640, 520, 19200), (448, 300, 38400)])
def test_gemm_w4a8_whole_rounds_plus_a_tail_launch(ops, sel, M, N):
    """More tiles than compute units with a thin last round: the columns of the whole rounds run as one launch of the
    large tile (512 x 128: 2 x 150 = 300 tiles -> 128 column tiles; 256 x 256: 2 x 150 -> 128), the remaining columns as
    256 x 128 tiles in a second launch.  The seam must not show: outputs equal the 128 x 128 kernel's bit for bit, and
    the oracle's on sampled rows."""
    K = 256
    p = prep(N, K, seed=sel)
    x = O.synth_acts(M, K, seed=sel + 1)
    a8_np, sx_np = O.quant_act_i8(x)
    bias_np = np.random.default_rng(sel).standard_normal(N).astype(np.float16)
    a8, sx, bias = dev(a8_np), dev(sx_np), dev(bias_np)
    qw, s8, z8, s1 = dev(p["qweight"]), dev(p["scales_to8"]), dev(p["scaled_zeros_to8"]), dev(p["scales_1"])
    got = {}
    for tile in (sel, 128):
        ops.force_gemm_tile(tile)
        try:
            if tile == sel:
                assert ops.gemm_w4a8_tile_for(M, N, K) == sel          # the split applies to this shape
            acc = ops.w4a8_gemm_acc_i32(a8, qw, s8, z8)
            out = torch.empty((M, N), dtype=torch.float16, device="cuda")
            ops.w4a8_gemm_forward(a8, qw, s8, z8, s1, sx, out, bias=bias)
            got[tile] = (acc, out)
        finally:
            ops.force_gemm_tile(0)
    assert torch.equal(got[sel][0], got[128][0]) and torch.equal(got[sel][1], got[128][1])
    rows = np.array([0, 1, 255, 256, M - 1])
    acc_ref, out_ref = O.gemm_w8a8(a8_np[rows], p["w8"], p["scales_1"], sx_np[rows])
    assert_same_bits(host(got[sel][0])[rows], acc_ref)
    ref_b = (out_ref.astype(np.float32) + bias_np.astype(np.float32)).astype(np.float16)
    assert_same_bits(host(got[sel][1])[rows], ref_b)


@pytest.mark.parametrize("K", [128, 256, 384])
@pytest.mark.parametrize("tile", [128, 130, 192, 256, 512])
def test_gemm_w4a8_k_shorter_than_the_pipeline(ops, tile, K):
    """Two, four or six 64-byte stages: fewer than the four the load pipeline keeps in flight (the loads past the end
    re-read the last stage and are never used).  Selector 130 needs K % 256 == 0 and falls back to one quartet
    otherwise.  Accumulators against the oracle, bit for bit."""
    M, N = 520, 256
    p = prep(N, K, seed=K + tile)
    a8 = np.random.default_rng(K).integers(-128, 128, size=(M, K), dtype=np.int8)
    ops.force_gemm_tile(tile)
    ops.force_gemm_splits(1)
    try:
        acc = ops.w4a8_gemm_acc_i32(dev(a8), dev(p["qweight"]), dev(p["scales_to8"]), dev(p["scaled_zeros_to8"]))
    finally:
        ops.force_gemm_tile(0)
        ops.force_gemm_splits(0)
    assert_same_bits(host(acc), O.gemm_i8_acc(a8, p["w8"]))


@pytest.mark.parametrize("tile,splits", [(128, 1), (256, 1), (128, 3), (256, 2), (192, 1), (192, 4), (130, 1), (130, 2), (130, 3), (512, 1), (512, 2), (0, 0)])
def test_gemm_w4a8_random_tables_and_splits(ops, tile, splits):
    """Arbitrary tables (every table byte differs from row to row and group to group, values beyond the int8 range are
    clipped as the converter clips them), full-range activations, K split over workgroups: accumulators equal the
    oracle's and the W8A8 GEMM's on the converter's output."""
    rng = np.random.default_rng(tile + splits)
    N, K, M = 512, 2048, 200
    Gp = O.padded_groups(K)
    qw_np = rng.integers(-32768, 32768, size=(N // 4, K), dtype=np.int16)
    s_np = (rng.random((Gp, N), dtype=np.float32) * 17.5 + 0.01).astype(np.float16)
    z_np = (rng.standard_normal((Gp, N), dtype=np.float32) * 70.0).astype(np.float16)
    a8_np = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    w8_ref = O.dequant_to_i8(qw_np, s_np, z_np)
    assert w8_ref.min() == -128 and w8_ref.max() == 127           # the clip is exercised
    qw, s8, z8, a8 = dev(qw_np), dev(s_np), dev(z_np), dev(a8_np)
    w8 = torch.empty((N, K), dtype=torch.int8, device="cuda")
    ops.dequant_interleaved_int4_to_int8(w8, qw, s8, z8, 128)
    ops.force_gemm_tile(tile)
    ops.force_gemm_splits(splits)
    try:
        acc = ops.w4a8_gemm_acc_i32(a8, qw, s8, z8)
        again = ops.w4a8_gemm_acc_i32(a8, qw, s8, z8)
    finally:
        ops.force_gemm_tile(0)
        ops.force_gemm_splits(0)
    assert_same_bits(host(w8), w8_ref)
    assert_same_bits(host(acc), O.gemm_i8_acc(a8_np, w8_ref))
    assert torch.equal(acc, again) and torch.equal(acc, ops.w8a8_gemm_acc_i32(a8, w8, N))


def _int_factor_case(N, K, seed):
    """A weight through both quantisers of the version-2 layer: the resident nibbles (this layer's own) and the integer
    factors of the second quantiser (what its id 7 multiplies them with)."""
    w = O.synth_weights(N, K, seed)
    p = O.prepare_weights(w)
    w8, s1 = O.qserve_quantize_int8(w)
    _, si, zi = O.qserve_quantize_int4(w8)
    S, Z = O.qserve_tables(si, zi, N)
    return p["qweight"], S, Z, s1.reshape(-1)


@pytest.mark.parametrize("tile", [0, 128, 130, 192, 256, 512])
@pytest.mark.parametrize("M", [1, 33, 300])
def test_gemm_w4a8_int_factors_bit_exact(ops, M, tile):
    """W4A8 with integer per-group factors (the arithmetic of the version-2 candidate's own GEMM,
    thirdparty/Qserve/qserve_kernels/csrc/qgemm/w4a8_per_group/gemm_cuda.cu:299-329, 620-627): int32 accumulators and
    fp16 outputs, with and without a bias, against the oracle bit for bit; N = 384 leaves every tile ragged."""
    N, K = 384, 1024
    qw_np, S, Z, s1 = _int_factor_case(N, K, seed=tile + 1)
    x = O.synth_acts(M, K, seed=900 + M)
    a8, sx = O.quant_act_i8(x)
    acc_ref, out_ref = O.gemm_w4a8_int(a8, qw_np, S, Z, s1, sx)
    bias = np.random.default_rng(M).standard_normal(N).astype(np.float16)
    out_b_ref = (out_ref.astype(np.float32) + bias.astype(np.float32)).astype(np.float16)
    qw, s2, z2 = dev(qw_np), dev(S), dev(Z)
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    out_b = torch.empty((M, N), dtype=torch.float16, device="cuda")
    ops.force_gemm_tile(tile)
    ops.force_gemm_splits(1)
    try:
        acc = ops.w4a8_int_gemm_acc_i32(dev(a8), qw, s2, z2)
        ops.w4a8_int_gemm_forward(dev(a8), qw, s2, z2, dev(s1), dev(sx), out)
        ops.w4a8_int_gemm_forward(dev(a8), qw, s2, z2, dev(s1), dev(sx), out_b, bias=dev(bias))
    finally:
        ops.force_gemm_tile(0)
        ops.force_gemm_splits(0)
    assert_same_bits(host(acc), acc_ref)
    assert_same_bits(host(out), out_ref)
    assert_same_bits(host(out_b), out_b_ref)


@pytest.mark.parametrize("tile,splits", [(128, 1), (256, 2), (192, 1), (192, 4), (130, 2), (512, 1), (512, 2), (0, 0)])
def test_gemm_w4a8_int_factors_any_bytes_and_splits(ops, tile, splits):
    """Arbitrary nibbles and arbitrary factor bytes (scales up to 255, negative bytes): every weight byte wraps modulo
    256 on its own, as the oracle's does; full-range activations, K split over workgroups."""
    rng = np.random.default_rng(tile + splits)
    N, K, M = 512, 2048, 200
    qw_np = rng.integers(-32768, 32768, size=(N // 4, K), dtype=np.int16)
    S = rng.integers(-128, 128, size=(K // 128, N), dtype=np.int8)
    Z = rng.integers(-128, 128, size=(K // 128, N), dtype=np.int8)
    a8_np = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    w8_ref = O.dequant_w4a8_int(qw_np, S, Z)
    assert w8_ref.min() == -128 and w8_ref.max() == 127
    ops.force_gemm_tile(tile)
    ops.force_gemm_splits(splits)
    try:
        acc = ops.w4a8_int_gemm_acc_i32(dev(a8_np), dev(qw_np), dev(S), dev(Z))
        again = ops.w4a8_int_gemm_acc_i32(dev(a8_np), dev(qw_np), dev(S), dev(Z))
    finally:
        ops.force_gemm_tile(0)
        ops.force_gemm_splits(0)
    assert_same_bits(host(acc), O.gemm_i8_acc(a8_np, w8_ref))
    assert torch.equal(acc, again)
    assert torch.equal(acc, ops.w8a8_gemm_acc_i32(dev(a8_np), dev(w8_ref), N))


def test_gemm_w4a8_int_factors_reject_wrong_tables(ops):
    qw = torch.zeros((64, 256), dtype=torch.int16, device="cuda")
    a8 = torch.zeros((4, 256), dtype=torch.int8, device="cuda")
    good = torch.zeros((2, 256), dtype=torch.int8, device="cuda")
    with pytest.raises(TypeError):
        ops.w4a8_int_gemm_acc_i32(a8, qw, good.half(), good)
    with pytest.raises(ValueError):
        ops.w4a8_int_gemm_acc_i32(a8, qw, good[:1], good)
    with pytest.raises(ValueError):
        ops.w4a8_int_gemm_acc_i32(a8, qw, good, good[:, :128].contiguous())


@pytest.mark.parametrize("K,N,wide", [(128, 7808, 256), (384, 7808, 256), (384, 7680, 320), (128, 7808, 320)])
def test_gemm_256_tile_walking_several_tiles_per_workgroup(ops, K, N, wide):
    """More 256 x 256 tiles than compute units (9 x 31 = 279, ragged in M and N): the tiled-weight W8A8 and fp16 GEMMs
    then run one workgroup per CU that walks the tiles and starts a tile's first loads while the previous one is
    written out.  K = 128 is shorter than the load pipeline.  Outputs equal the 128-row-tile kernel's bit for bit
    (same accumulation order) and the oracle's on sampled rows, with and without a bias."""
    M = 2100                                                # N = 7680: 9 x 40 tiles of 256 x 192, tiles that start in the middle of a weight strip
    p = prep(N, K, seed=K)
    x = O.synth_acts(M, K, seed=K + 1)
    a8_np, sx_np = O.quant_act_i8(x)
    bias_np = np.random.default_rng(K).standard_normal(N).astype(np.float16)
    rows = np.array([0, 1, 255, 256, 2047, 2048, 2099])
    _, ref8 = O.gemm_w8a8(a8_np[rows], p["w8"], p["scales_1"], sx_np[rows])
    ref8_b = (ref8.astype(np.float32) + bias_np.astype(np.float32)).astype(np.float16)
    w8_t = torch.empty((N, K), dtype=torch.int8, device="cuda")
    ops.dequant_interleaved_int4_to_int8(w8_t, dev(p["qweight"]), dev(p["scales_to8"]), dev(p["scaled_zeros_to8"]), 128, tiled=True)
    w16_t = torch.empty((N, K), dtype=torch.float16, device="cuda")
    ops.dequant_interleaved_int4_to_fp16(w16_t, dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), 128, tiled=True)
    a8, sx, xd, bias, s1 = dev(a8_np), dev(sx_np), dev(x), dev(bias_np), dev(p["scales_1"])
    got = {}
    for tile in (wide, 128):
        ops.force_gemm_tile(tile)
        ops.force_gemm_splits(1)
        try:
            o8 = torch.empty((M, N), dtype=torch.float16, device="cuda")
            o8b = torch.empty((M, N), dtype=torch.float16, device="cuda")
            ops.w8a8_gemm_forward(a8, w8_t, s1, sx, o8, tiled=True)
            ops.w8a8_gemm_forward(a8, w8_t, s1, sx, o8b, bias=bias, tiled=True)
            got[tile] = (o8, o8b, ops.f16_gemm_forward(xd, w16_t, N, tiled=True),
                         ops.f16_gemm_forward(xd, w16_t, N, bias=bias, tiled=True))
        finally:
            ops.force_gemm_tile(0)
            ops.force_gemm_splits(0)
    for a, b in zip(got[wide], got[128]):
        assert torch.equal(a, b)
    assert_same_bits(host(got[wide][0])[rows], ref8)
    assert_same_bits(host(got[wide][1])[rows], ref8_b)
    assert O.max_abs_rel(host(got[wide][2])[rows], O.gemm_f16(x[rows], p["w16"])) < 2e-3


@pytest.mark.parametrize("tile", [64, 128, 256])
@pytest.mark.parametrize("M", GEMM_M)
def test_gemm_w4a16_f16_w8a16(ops, M, tile):
    N, K = 384, 1024
    p = prep(N, K)
    x = O.synth_acts(M, K, seed=300 + M)
    ref = O.gemm_f16(x, p["w16"])
    xd = dev(x)
    ops.force_gemm_tile(tile)
    ops.force_gemm_splits(1)                                # one workgroup per tile walks all of K
    try:
        out4 = ops.gemm_forward(xd, dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]))
        out16 = ops.f16_gemm_forward(xd, dev(p["w16"]), N)
        out816 = ops.w8a16_gemm_forward(xd, dev(p["w8"]), dev(p["scales_1"]), N)
    finally:
        ops.force_gemm_tile(0)
        ops.force_gemm_splits(0)
    assert O.max_abs_rel(host(out4), ref) < 2e-3
    assert O.max_abs_rel(host(out16), ref) < 2e-3
    assert torch.equal(out4, out16)                         # same fp16 weights, same accumulation order
    assert O.max_abs_rel(host(out816), O.gemm_w8a16(x, p["w8"], p["scales_1"])) < 2e-3


@pytest.mark.parametrize("tile", [64, 128, 192, 256, 320])     # 320: 256 x 192 tiles (tiled operands; row-major runs 256 x 256)
def test_gemm_tiled_operands_match_row_major(ops, tile):
    N, K, M = 384, 1024, 150
    p = prep(N, K)
    x = O.synth_acts(M, K, seed=5)
    xd = dev(x)
    qw = dev(p["qweight"])
    t16 = torch.empty((N, K), dtype=torch.float16, device="cuda")
    ops.dequant_interleaved_int4_to_fp16(t16, qw, dev(p["scales"]), dev(p["scaled_zeros"]), 128, tiled=True)
    t8 = torch.empty((N, K), dtype=torch.int8, device="cuda")
    ops.dequant_interleaved_int4_to_int8(t8, qw, dev(p["scales_to8"]), dev(p["scaled_zeros_to8"]), 128, tiled=True)
    a8 = torch.empty_like(xd, dtype=torch.int8)
    sx = torch.empty((M,), dtype=torch.float16, device="cuda")
    ops.quant_fp16_to_int8(a8, xd, sx)
    s1 = dev(p["scales_1"])
    ops.force_gemm_tile(tile)
    try:
        a = ops.f16_gemm_forward(xd, dev(p["w16"]), N)
        b = ops.f16_gemm_forward(xd, t16, N, tiled=True)
        e = torch.empty((M, N), dtype=torch.float16, device="cuda")
        f = torch.empty((M, N), dtype=torch.float16, device="cuda")
        ops.w8a8_gemm_forward(a8, dev(p["w8"]), s1, sx, e)
        ops.w8a8_gemm_forward(a8, t8, s1, sx, f, tiled=True)
    finally:
        ops.force_gemm_tile(0)
    assert torch.equal(a, b) and torch.equal(e, f)


@pytest.mark.parametrize("splits", [2, 3, 4])
@pytest.mark.parametrize("tile", [64, 128])
def test_gemm_split_k(ops, tile, splits):
    """K split over several workgroups with the partial sums reduced in a second kernel: the int8 lane
    stays bit-exact (integer partials), the fp16 lanes stay within tolerance and deterministic."""
    N, K, M = 256, 2048, 100
    p = prep(N, K)
    x = O.synth_acts(M, K, seed=9)
    xd = dev(x)
    ref = O.gemm_f16(x, p["w16"])
    a8_ref, sx_ref = O.quant_act_i8(x)
    ops.ensure_workspace()
    ops.force_gemm_tile(tile)
    ops.force_gemm_splits(splits)
    try:
        out4 = ops.gemm_forward(xd, dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]))
        again = ops.gemm_forward(xd, dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]))
        out16 = ops.f16_gemm_forward(xd, dev(p["w16"]), N)
        out816 = ops.w8a16_gemm_forward(xd, dev(p["w8"]), dev(p["scales_1"]), N)
        acc = ops.w8a8_gemm_acc_i32(dev(a8_ref), dev(p["w8"]), N)
        out88 = torch.empty((M, N), dtype=torch.float16, device="cuda")
        ops.w8a8_gemm_forward(dev(a8_ref), dev(p["w8"]), dev(p["scales_1"]), dev(sx_ref), out88)
    finally:
        ops.force_gemm_tile(0)
        ops.force_gemm_splits(0)
    assert O.max_abs_rel(host(out4), ref) < 2e-3 and torch.equal(out4, again)
    assert O.max_abs_rel(host(out16), ref) < 2e-3
    assert O.max_abs_rel(host(out816), O.gemm_w8a16(x, p["w8"], p["scales_1"])) < 2e-3
    acc_ref, out_ref = O.gemm_w8a8(a8_ref, p["w8"], p["scales_1"], sx_ref)
    assert np.array_equal(host(acc), acc_ref)
    assert_same_bits(host(out88), out_ref)


def test_gemm_bias(ops):
    N, K, M = 256, 512, 33
    p = prep(N, K)
    x = O.synth_acts(M, K, seed=8)
    bias = np.random.default_rng(2).standard_normal(N).astype(np.float16)
    ref = O.switched_forward(x, p, O.COMP_TYPE_NAME["fp16"], bias=bias)
    out = ops.gemm_forward(dev(x), dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), bias=dev(bias))
    assert O.max_abs_rel(host(out), ref) < 2e-3


# ------------------------------------------------------------------ error behaviour of the boundary
def test_argument_errors(ops):
    from kairos_amd import _lib
    N, K = 64, 256
    p = prep(N, K)
    x = dev(O.synth_acts(4, K))
    with pytest.raises(_lib.KairosMiError) as e:
        ops.gemv_forward(x, dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), 4, N, K, 64)
    assert e.value.code == -3
    big = dev(O.synth_acts(65, K))
    with pytest.raises(_lib.KairosMiError) as e:
        ops.gemv_forward(big, dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]), 65, N, K, 128)
    assert e.value.code == -4
    with pytest.raises(TypeError):
        ops.quant_fp16_to_int8(torch.empty((4, K), dtype=torch.int8, device="cuda"), x.float(), torch.empty(4, dtype=torch.float16, device="cuda"))


@pytest.mark.gpu
@pytest.mark.parametrize("tiled", [False, True])
@pytest.mark.parametrize("M,N,K", [(1, 128, 128), (7, 256, 512), (300, 384, 1024), (64, 128, 4096)])
def test_prep_w8a8_equals_separate_kernels(ops, tiled, M, N, K):
    """The fused launch (conversion + activation quantiser) gives the bits of the two stand-alone entry points."""
    import torch
    w = O.synth_weights(N, K, N + K)
    pw = O.prepare_weights(w, 128)
    dev = "cuda"
    qw = torch.from_numpy(pw["qweight"]).to(dev)
    s8 = torch.from_numpy(pw["scales_to8"]).to(dev)
    z8 = torch.from_numpy(pw["scaled_zeros_to8"]).to(dev)
    x = torch.from_numpy(O.synth_acts(M, K, M)).to(dev)
    x[0, :] = 0 if M > 3 else x[0, :]                       # an all-zero token among the rows
    w_ref = torch.empty((N, K), dtype=torch.int8, device=dev)
    ops.dequant_interleaved_int4_to_int8(w_ref, qw, s8, z8, 128, tiled=tiled)
    a_ref = torch.empty((M, K), dtype=torch.int8, device=dev)
    sc_ref = torch.empty((M,), dtype=torch.float16, device=dev)
    ops.quant_fp16_to_int8(a_ref, x, sc_ref)
    w_f = torch.full((N, K), 77, dtype=torch.int8, device=dev)
    a_f = torch.full((M, K), 77, dtype=torch.int8, device=dev)
    sc_f = torch.full((M,), 3.0, dtype=torch.float16, device=dev)
    ops.prep_w8a8(w_f, qw, s8, z8, a_f, x, sc_f, 128, tiled=tiled)
    assert torch.equal(w_f, w_ref)
    assert torch.equal(a_f, a_ref)
    assert torch.equal(sc_f.view(torch.int16), sc_ref.view(torch.int16))
    # and against the oracle directly
    a_o, sc_o = O.quant_act_i8(x.cpu().numpy())
    assert np.array_equal(a_f.cpu().numpy(), a_o)


@pytest.mark.gpu
def test_gemm_tail_round_split(ops):
    """More than 256 tiles of 256x256 with a thin last round: the automatic choice runs the tail columns with
    the 128x128 tile in a second launch.  Integer results must equal the single-tile runs bit for bit and the
    oracle on sampled rows; the fp16-output lanes must equal their single-tile runs too."""
    M, N, K = 4096, 6144, 256                      # 16 x 24 = 384 tiles -> head 16 column tiles, tail 8
    rng = np.random.default_rng(5)
    a8 = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    w8 = rng.integers(-128, 128, size=(N, K)).astype(np.int8)
    a8d, w8d = dev(a8), dev(w8)
    acc_auto = ops.w8a8_gemm_acc_i32(a8d, w8d, N)
    ops.force_gemm_tile(128)
    try:
        acc_128 = ops.w8a8_gemm_acc_i32(a8d, w8d, N)
    finally:
        ops.force_gemm_tile(0)
    assert torch.equal(acc_auto, acc_128)
    rows = np.r_[0:8, 2040:2056, M - 8:M]
    assert np.array_equal(host(acc_auto)[rows], O.gemm_i8_acc(a8[rows], w8))
    # scaled fp16 output with bias, and the fp16 GEMM, across the seam at column 4096
    ws = dev(rng.random(N).astype(np.float16)); as_ = dev(rng.random(M).astype(np.float16))
    bias = dev(rng.standard_normal(N).astype(np.float16))
    out_auto = torch.empty((M, N), dtype=torch.float16, device="cuda")
    out_256 = torch.empty_like(out_auto)
    ops.w8a8_gemm_forward(a8d, w8d, ws, as_, out_auto, bias=bias)
    x = dev(rng.standard_normal((M, K)).astype(np.float16)); w16 = dev((rng.standard_normal((N, K)) * 0.05).astype(np.float16))
    f_auto = ops.f16_gemm_forward(x, w16, N)
    ops.force_gemm_tile(256)
    try:
        ops.w8a8_gemm_forward(a8d, w8d, ws, as_, out_256, bias=bias)
        f_256 = ops.f16_gemm_forward(x, w16, N)
    finally:
        ops.force_gemm_tile(0)
    assert torch.equal(out_auto, out_256)
    assert torch.equal(f_auto, f_256)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,sel,splits", [
    (5, 128, 128, 1032, 0), (32, 256, 512, 1032, 0), (64, 256, 512, 1064, 0), (33, 384, 1024, 1064, 0),
    (64, 128, 4096, 1064, 2), (100, 256, 512, 1064, 0), (128, 256, 1024, 1128, 0), (48, 132, 256, 1064, 0),
    (17, 256, 2048, 1032, 3), (300, 384, 512, 1128, 0), (1, 128, 14336, 1032, 0),
    # every remainder of the four-deep software pipeline (k-tiles per quartet = 1..7), both quartet counts
    (64, 256, 384, 1064, 0), (64, 256, 640, 1064, 0), (96, 256, 768, 1128, 0), (64, 256, 896, 1064, 0),
    (64, 256, 128, 2064, 0), (128, 128, 384, 2128, 0), (32, 256, 640, 2032, 0), (200, 384, 896, 2128, 0),
    (130, 260, 256, 2128, 0), (64, 128, 1792, 2064, 2)])
def test_gemm_w4a16_wave_private(ops, M, N, K, sel, splits):
    """The small-M W4A16 variant (weights decoded in registers by the wave that owns their columns, quartets
    splitting K inside the workgroup, optional split over workgroups) against the oracle, with and without
    bias, ragged N included; repeated calls give the same bits."""
    p = prep(N, K, seed=N + K)
    x = O.synth_acts(M, K, seed=M)
    ref = O.gemm_w4a16(x, p["qweight"], p["scales"], p["scaled_zeros"])
    bias = np.random.default_rng(1).standard_normal(N).astype(np.float16)
    args = (dev(x), dev(p["qweight"]), dev(p["scales"]), dev(p["scaled_zeros"]))
    ops.force_gemm_tile(sel)
    ops.force_gemm_splits(splits)
    try:
        out = ops.gemm_forward(*args)
        again = ops.gemm_forward(*args)
        outb = ops.gemm_forward(*args, bias=dev(bias))
    finally:
        ops.force_gemm_tile(0)
        ops.force_gemm_splits(0)
    assert O.max_abs_rel(host(out), ref) < 2e-3
    assert torch.equal(out, again)
    refb = (host(out).astype(np.float32) + bias.astype(np.float32)).astype(np.float16)   # fp16 add after rounding
    assert_same_bits(host(outb), refb)


@pytest.mark.gpu
def test_gemm_w4a16_variant_choice(ops):
    assert ops.gemm_w4a16_wp_rows(1, 4096, 4096) == 32 and ops.gemm_w4a16_wp_rows(64, 28672, 4096) == 64
    assert ops.gemm_w4a16_wp_rows(256, 6144, 4096) == 64 and ops.gemm_w4a16_wp_rows(512, 6144, 4096) == 128
    assert ops.gemm_w4a16_wp_rows(256, 4096, 14336) == 128 and ops.gemm_w4a16_wp_rows(256, 28672, 4096) == 128
    assert ops.gemm_w4a16_wp_rows(512, 28672, 4096) == 0 and ops.gemm_w4a16_wp_rows(2048, 4096, 4096) == 0
    assert ops.gemm_w4a16_wp_rows(64, 4096, 4096) == 32 and ops.gemm_w4a16_wp_rows(384, 28672, 4096) == 128
    assert ops.gemm_w4a16_wp_rows(128, 10240, 8192) == 128 and ops.gemm_w4a16_wp_rows(128, 4096, 14336) == 64


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(48, 28672, 4096), (200, 4096, 14336)])
def test_gemm_w4a16_variants_agree_at_full_size(ops, M, N, K):
    """At the benchmark's full sizes the oracle is too slow; the two W4A16 GEMM variants (wave-private, register-staged) and
    the small-M kernel are independent implementations of the same product and must agree within the fp16
    tolerance on random packed weights."""
    g = torch.Generator(device="cuda").manual_seed(M + N)
    qw = torch.randint(-32768, 32767, (N // 4, K), device="cuda", dtype=torch.int16, generator=g)
    Gp = (K // 128 + 7) // 8 * 8
    s = (torch.rand((Gp, N), device="cuda", generator=g) * 0.01 + 0.002).to(torch.float16)
    z = (-(s.float() * 7.5)).to(torch.float16)
    x = torch.randn((M, K), device="cuda", generator=g).to(torch.float16)
    auto = ops.gemm_forward(x, qw, s, z)
    assert ops.gemm_w4a16_wp_rows(M, N, K) in (64, 128)
    ops.force_gemm_tile(64)
    try:
        staged = ops.gemm_forward(x, qw, s, z)
    finally:
        ops.force_gemm_tile(0)
    a, b = auto.float(), staged.float()
    scale = b.abs().max()
    assert ((a - b).abs().max() / scale).item() < 2e-3
    if M <= 64:
        v = ops.gemv_forward(x, qw, s, z, M, N, K, 128).float()
        assert ((a - v).abs().max() / scale).item() < 2e-3


# ------------------------------------------------------------------ offline weight preparation on the device, bit-exact
PREP_KEYS = ("qweight", "scales", "scaled_zeros", "scales_to8", "scaled_zeros_to8", "scales_1")


def check_prepare(ops, w):
    want = O.prepare_weights(w)
    got = ops.prepare_weight(dev(w))
    for key in PREP_KEYS:
        g, r = host(got[key]), want[key]
        if g.dtype == np.float16:          # 0 * inf in a degenerate group: NaN on both sides, sign and payload are not defined
            both_nan = np.isnan(g) & np.isnan(r)
            g, r = np.where(both_nan, np.float16(0), g), np.where(both_nan, np.float16(0), r)
        assert_same_bits(g, r)


@pytest.mark.parametrize("N,K", [(4, 128), (8, 256), (64, 512), (128, 3584), (64, 18944), (256, 4096), (36, 640)])
def test_prepare_weight_bit_exact(ops, N, K):
    check_prepare(ops, O.synth_weights(N, K, seed=N + K))


def test_prepare_weight_edge_rows(ops):
    """Rows and groups the arithmetic treats specially: all-zero rows (scale clamps, -0 zero-points), constant groups
    (zero-point overflows fp16 to -inf as on the host), outliers (most groups collapse to few levels), exact ties."""
    rng = np.random.default_rng(5)
    N, K = 32, 1024
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    w[0] = 0
    w[1, :128] = np.float16(0.0123)
    w[2] = np.float16(-0.5)
    w[3, 7] = np.float16(30.0)
    w[4] = (rng.integers(-127, 128, K) * 0.5).astype(np.float16)          # x/s lands on .5 ties after step 1
    w[4, 0] = np.float16(63.5)
    w[5, :] = np.float16(6e-8)                                            # fp16 subnormals
    w[6, ::2] = np.float16(65504.0)
    w[7] = np.where(np.arange(K) % 128 < 64, np.float16(1.0), np.float16(-1.0))
    with np.errstate(over="ignore", invalid="ignore"):
        check_prepare(ops, w)


def test_prepare_weight_feeds_the_kernels(ops):
    """End to end: device-prepared tensors through the converter equal the oracle's conversion of its own preparation."""
    N, K = 256, 1024
    w = O.synth_weights(N, K, seed=3)
    got = ops.prepare_weight(dev(w))
    p = prep(N, K, 3)
    out = torch.empty((N, K), dtype=torch.int8, device="cuda")
    ops.dequant_interleaved_int4_to_int8(out, got["qweight"], got["scales_to8"], got["scaled_zeros_to8"], 128)
    assert_same_bits(host(out), p["w8"])


def test_prepare_weight_rejects_bad_arguments(ops):
    with pytest.raises(TypeError):
        ops.prepare_weight(torch.zeros((8, 128), device="cuda"))
    with pytest.raises(Exception):
        ops.prepare_weight(torch.zeros((6, 128), dtype=torch.float16, device="cuda"))
    with pytest.raises(Exception):
        ops.prepare_weight(torch.zeros((8, 192), dtype=torch.float16, device="cuda"))


def test_prepare_weight_every_group_range(ops):
    """Step 2 exhaustively: every reachable (lo, hi, x) of a group of int8 values.  Rows hold integers and a +-127, so
    step 1 is the identity (s1 = 1); each later group spans one (lo, hi) pair and carries every value between."""
    groups = []
    for lo in range(-127, 128):
        groups.append([lo] * 128)                                             # constant group
        for hi in range(lo + 1, 128):
            inner = list(range(lo + 1, hi))
            for at in range(0, max(len(inner), 1), 126):
                piece = inner[at:at + 126]
                groups.append([lo, hi] + piece + [lo] * (126 - len(piece)))
    per_row = 31
    rows = -(-len(groups) // per_row)
    rows += -rows % 4
    groups += [groups[-1]] * (rows * per_row - len(groups))
    body = np.asarray(groups, dtype=np.float16).reshape(rows, per_row * 128)
    first = np.zeros((rows, 128), dtype=np.float16)
    first[:, 0], first[:, 1] = 127, -127
    w = np.concatenate([first, body], axis=1)
    assert w.shape[1] == 4096
    with np.errstate(over="ignore", invalid="ignore"):
        check_prepare(ops, w)


def test_prepare_weight_every_numerator(ops):
    """Step 1 for 64 divisors (row maxima, drawn over the whole fp16 range, edge values included): every positive
    finite fp16 value up to the maximum appears in the row, so each division w / s1 the row can need is checked."""
    rng = np.random.default_rng(9)
    allpos = np.arange(1, 0x7C00, dtype=np.uint16).view(np.float16)           # every positive finite fp16, ascending
    tops = list(rng.integers(1, 0x7C00, 58).astype(np.uint16).view(np.float16))
    tops += [np.float16(65504), np.float16(1.0), np.float16(127.0), np.float16(6e-8), np.float16(6.1e-5), np.float16(0.02)]
    K = 32768
    w = np.zeros((64, K), dtype=np.float16)
    for i, top in enumerate(tops):
        vals = allpos[allpos <= top]
        w[i, :len(vals)] = vals
        w[i, len(vals):] = -np.resize(vals, K - len(vals))                    # the same values, negative, repeated
    with np.errstate(over="ignore", invalid="ignore"):
        check_prepare(ops, w)


# ------------------------------------------------------------------ re-pack into the W4A8 operand layout, bit-exact
@pytest.mark.parametrize("N,K", [(32, 64), (64, 192), (96, 3584), (1024, 4096), (4096, 4096), (4096, 14336), (14336, 4096)])
def test_trans_layout_w4a8_known_answer(ops, N, K):
    """The reference's own test (test/test_trans_layout.py:46-52, same four large shapes): re-packing the resident
    format of a random uint4 matrix must equal packing that matrix directly."""
    q = np.random.default_rng(N ^ K).integers(0, 16, size=(N, K), dtype=np.uint8)
    got = ops.trans_layout_c16_to_c8_awq(dev(O.pack_int_awq(q)), N, K)
    assert got.dtype == torch.int8 and tuple(got.shape) == (N, K // 2)
    assert_same_bits(host(got), O.pack_int_w4a8(q))


def test_trans_layout_w4a8_rejects_bad_shapes(ops):
    t = torch.zeros((8, 64), dtype=torch.int16, device="cuda")
    with pytest.raises(Exception):
        ops.trans_layout_c16_to_c8_awq(t, 16, 128)          # N % 32
    with pytest.raises(ValueError):
        ops.trans_layout_c16_to_c8_awq(t, 64, 64)           # size mismatch


# ------------------------------------------------------------------ random shapes: every variant of a lane agrees
def test_random_shapes_every_variant_agrees(ops):
    """Sixty random (M, N, K) with ragged N, odd M and optional bias.  W8A8: every tile, row-major and tiled weights,
    separate and fused preparation give the same bits, and the int32 accumulators equal an exact matmul.  W4A16: every
    kernel variant (three staged tiles, six wave-private ones, the small-M kernel) and the fp16 GEMM on converted
    weights stay within the fp16 tolerance of an fp32 product of the converted weights."""
    import random
    rnd = random.Random(7)

    def same(a, b):
        return torch.equal(a.view(torch.int16) if a.dtype == torch.float16 else a,
                           b.view(torch.int16) if b.dtype == torch.float16 else b)

    for it in range(60):
        M = rnd.choice([1, 3, 17, 33, 64, 65, 100, 128, 129, 200, 256, 257, 300, 511, 512, 700, 1024])
        N = 4 * rnd.randint(1, 500) if rnd.random() < 0.5 else 128 * rnd.randint(1, 24)
        K = 128 * rnd.randint(1, 20)
        tag = f"case {it}: M={M} N={N} K={K}"
        g = torch.Generator(device="cuda").manual_seed(it)
        qw = torch.randint(-32768, 32767, (N // 4, K), device="cuda", dtype=torch.int16, generator=g)
        gp = O.padded_groups(K)
        s = (torch.rand((gp, N), device="cuda", generator=g) * 0.01 + 0.002).to(torch.float16)
        z = (-(s.float() * 7.5)).to(torch.float16)
        s8 = (torch.rand((gp, N), device="cuda", generator=g) * 6 + 2).to(torch.float16)
        z8 = (-(s8.float() * 7.5)).to(torch.float16)
        x = torch.randn((M, K), device="cuda", generator=g).to(torch.float16)
        bias = torch.randn((N,), device="cuda", generator=g).to(torch.float16) if rnd.random() < 0.5 else None
        w8 = torch.empty((N, K), device="cuda", dtype=torch.int8)
        ops.dequant_interleaved_int4_to_int8(w8, qw, s8, z8, 128)
        a8 = torch.empty((M, K), device="cuda", dtype=torch.int8)
        sx = torch.empty((M,), device="cuda", dtype=torch.float16)
        ops.quant_fp16_to_int8(a8, x, sx)
        ws = torch.rand((N,), device="cuda", generator=g).to(torch.float16)
        outs = []
        try:
            for tile in (0, 64, 128, 192, 256):
                ops.force_gemm_tile(tile)
                o = torch.empty((M, N), device="cuda", dtype=torch.float16)
                ops.w8a8_gemm_forward(a8, w8, ws, sx, o, bias=bias)
                outs.append(o)
                if N % 128 == 0:
                    w8t, a8b, sxb = torch.empty_like(w8), torch.empty_like(a8), torch.empty_like(sx)
                    ops.prep_w8a8(w8t, qw, s8, z8, a8b, x, sxb, 128, tiled=True)
                    ot = torch.empty((M, N), device="cuda", dtype=torch.float16)
                    ops.w8a8_gemm_forward(a8b, w8t, ws, sxb, ot, bias=bias, tiled=True)
                    outs.append(ot)
                    assert same(a8, a8b) and same(sx, sxb) and same(ops.untile(w8t, N, K), w8), tag
        finally:
            ops.force_gemm_tile(0)
        assert all(same(outs[0], o) for o in outs[1:]), tag
        assert same(ops.w8a8_gemm_acc_i32(a8, w8, N), (a8.double() @ w8.double().T).to(torch.int32)), tag
        w16 = torch.empty((N, K), device="cuda", dtype=torch.float16)
        ops.dequant_interleaved_int4_to_fp16(w16, qw, s, z, 128)
        want = x.float() @ w16.float().T
        if bias is not None:
            want = want + bias.float()
        scale = want.abs().max().item() + 1e-6
        for sel in (0, 64, 128, 256, 1032, 1064, 1128, 2032, 2064, 2128):
            ops.force_gemm_tile(sel)
            try:
                o = ops.gemm_forward(x, qw, s, z, bias=bias)
            finally:
                ops.force_gemm_tile(0)
            assert (o.float() - want).abs().max().item() / scale < 4e-3, (tag, sel)
        if M <= 64 and N % 16 == 0:
            o = ops.gemv_forward(x, qw, s, z, M, N, K, 128, bias=bias)
            assert (o.float() - want).abs().max().item() / scale < 4e-3, (tag, "small-M kernel")
        o = ops.f16_gemm_forward(x, w16, N, bias=bias)
        assert (o.float() - want).abs().max().item() / scale < 4e-3, (tag, "fp16 GEMM")


def test_pipe_probes_measure_what_they_say():
    """The register-only probes behind the pipe figures: a lone wave's int8 32 x 32 x 32 MFMA holds the matrix pipe 32
    cycles (8 passes of 4), a few vector instructions behind each MFMA are free and many are not, a vector-only wave
    runs beside an MFMA-only wave of the same SIMD in far less than the sum of their times, and the chip-wide loop
    reports a plausible clock."""
    import kairos_amd._lib as L
    lib = L.load()
    cyc = torch.zeros(8, dtype=torch.int64, device="cuda")

    def run(mode):
        for _ in range(2):
            L.check(lib.kmi_probe_pipe_overlap(mode, cyc.data_ptr(), None))
            torch.cuda.synchronize()
        return cyc.tolist()
    alone = run(1)[0]
    valu = run(2)[4]
    both = run(3)
    assert 30.0 < alone / 2048 < 40.0
    assert 3.5 < valu / 16384 < 8.0
    assert both[0] < 1.15 * alone and both[4] < 0.85 * (alone + valu)
    assert run(5)[0] < 1.15 * alone and run(8)[0] > 1.8 * alone          # + 4 hidden, + 16 not
    with pytest.raises(RuntimeError):
        L.check(lib.kmi_probe_pipe_overlap(13, cyc.data_ptr(), None))
    clk = torch.zeros(2, dtype=torch.int64, device="cuda")
    buf = torch.full((8192,), 0x01010101, dtype=torch.int32, device="cuda")
    L.check(lib.kmi_probe_mfma_stream(0, buf.data_ptr(), buf.numel() * 4, 256, 2000, clk.data_ptr(), None))
    torch.cuda.synchronize()
    c = clk.tolist()
    assert 30.0 < c[0] / (2000 * 16) < 40.0                              # one wave per SIMD: back-to-back MFMAs
    assert 800 < c[0] / c[1] * 100 < 2600                                 # MHz
