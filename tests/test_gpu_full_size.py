"""GPU parity at the benchmark's full sizes, where the oracle is too slow to produce every element.

Each test combines (a) whole-matrix properties that any wrong element breaks -- row and column checksums of exact
integer results against the same sums computed from the inputs (a checksum of checksums), periodicity of the output
under replicated weights, agreement of independent layouts -- with (b) the oracle on a sample of rows, which are
independent of each other in every kernel of the path.  Inputs are chosen so that the compared quantities are exactly
computable (also through the fp16 epilogue), hence the comparisons are bit-exact.
"""
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


def sample_rows(M, n, seed):
    rows = np.unique(np.concatenate([[0, M - 1, M // 2, 255, 256], np.random.default_rng(seed).integers(0, M, n)]))
    return rows[rows < M]


@pytest.mark.parametrize("M,N,K", [(4096, 28672, 4096), (4096, 4096, 14336), (4096, 6144, 4096)])
def test_w8a8_accumulators_full_size(ops, M, N, K):
    """int32 accumulators over full-range int8 operands: both checksums of the whole M x N result and sampled rows."""
    rng = np.random.default_rng(M + N + K)
    a8 = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    w8 = rng.integers(-128, 128, size=(N, K), dtype=np.int8)
    acc = ops.w8a8_gemm_acc_i32(dev(a8), dev(w8), N)
    torch.cuda.synchronize()
    a64, w64 = a8.astype(np.float64), w8.astype(np.float64)                   # all sums below stay under 2^53: exact
    row_sum = a64 @ w64.sum(axis=0)                                           # sum_n acc[m, n]
    col_sum = w64 @ a64.sum(axis=0)                                           # sum_m acc[m, n]
    assert np.array_equal(acc.sum(dim=1, dtype=torch.int64).cpu().numpy(), row_sum.astype(np.int64))
    assert np.array_equal(acc.sum(dim=0, dtype=torch.int64).cpu().numpy(), col_sum.astype(np.int64))
    rows = sample_rows(M, 24, N)
    assert np.array_equal(acc[torch.from_numpy(rows).cuda()].cpu().numpy(), O.gemm_i8_acc(a8[rows], w8))


@pytest.mark.parametrize("M,N,K", [(4096, 28672, 4096), (2048, 4096, 14336), (1024, 6144, 4096), (512, 28672, 4096),
                                   (30720, 4096, 4096)])            # last: the largest M of the shipped lookup tables
def test_w8a8_lane_full_size_through_tiled_weights(ops, M, N, K):
    """The production order of the W8A8 lane at full size: fused preparation launch (int4 -> tiled int8 + activation
    quantiser), tiled int8 MFMA GEMM (256-row tiles, tail launch where the shape has one), fp16 epilogue.  Tables
    s = 1, z = -8 make the converted weight the integer q - 8; activations are sparse +-127, so their scale is exactly
    1 and the quantised row is the row itself; with the channel scale 1/128 the epilogue's fp32 value is exact, so the
    fp16 output is one known rounding of an exactly computable number: compared bit for bit over the whole matrix."""
    rng = np.random.default_rng(N + K)
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    w8 = q.astype(np.int8) - 8
    Gp = O.padded_groups(K)
    ones = torch.ones((Gp, N), dtype=torch.float16, device="cuda")
    a = np.zeros((M, K), dtype=np.int8)                                        # 16 entries of +-1 per row, scaled to +-127 below
    idx = np.argsort(rng.random((M, K), dtype=np.float32), axis=1)[:, :16]    # 16 distinct columns per row
    np.put_along_axis(a, idx, rng.choice(np.array([-1, 1], dtype=np.int8), size=(M, 16)), axis=1)
    x = dev((a.astype(np.float16) * np.float16(127.0)))                       # amax = 127 -> scale 1, a8 = +-127
    w8_t = torch.empty((N, K), dtype=torch.int8, device="cuda")
    a8 = torch.empty((M, K), dtype=torch.int8, device="cuda")
    sx = torch.empty((M,), dtype=torch.float16, device="cuda")
    ops.prep_w8a8(w8_t, dev(O.pack_int_awq(q)), ones, ones * -8.0, a8, x, sx, 128, tiled=True)
    assert torch.equal(a8.cpu(), torch.from_numpy(a) * 127) and bool((sx == 1.0).all())
    assert torch.equal(ops.untile(w8_t, N, K).cpu(), torch.from_numpy(w8))    # the tiled converter at full size
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    ws = torch.full((N,), 1.0 / 128.0, dtype=torch.float16, device="cuda")    # a power of two: the scaling is exact
    ops.w8a8_gemm_forward(a8, w8_t, ws, sx, out, tiled=True)
    torch.cuda.synchronize()
    # acc = 127 * (a . w8) with |a . w8| <= 16 * 8; out = fp16(fp32(acc) * (1/128 * 1))
    exact = (a.astype(np.float32) @ w8.astype(np.float32).T) * np.float32(127.0 / 128.0)   # every step exact in fp32
    want = exact.astype(np.float16)                                           # the one rounding of the epilogue
    rows = sample_rows(M, 24, K)
    assert np.array_equal(out[torch.from_numpy(rows).cuda()].cpu().numpy().view(np.uint16), want[rows].view(np.uint16))
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("N,K", [(57344, 8192), (8192, 28672), (10240, 8192)])
def test_gemv_periodic_weights_70b_shapes(ops, N, K):
    """Small-M W4A16 at the Llama-3-70B shapes: the weight is a prepared 1024-row slice repeated along N, so every
    output column must equal, bit for bit, the column 1024 to its left, and the first 1024 columns must match the oracle."""
    base = 1024
    p = O.prepare_weights(O.synth_weights(base, K, seed=K))
    reps = N // base
    qw = dev(p["qweight"]).repeat(reps, 1)
    s, z = dev(p["scales"]).repeat(1, reps), dev(p["scaled_zeros"]).repeat(1, reps)
    for M in (1, 8, 32):
        x = O.synth_acts(M, K, seed=M)
        out = ops.gemv_forward(dev(x), qw, s, z, M, N, K, 128)
        torch.cuda.synchronize()
        first = out[:, :base]
        assert torch.equal(out.view(M, reps, base).view(torch.int16), first.view(torch.int16)[:, None, :].expand(M, reps, base))
        ref = O.gemm_w4a16(x, p["qweight"], p["scales"], p["scaled_zeros"])
        assert O.max_abs_rel(first.cpu().numpy(), ref) < 1e-2


@pytest.mark.parametrize("N,K", [(6144, 4096), (28672, 4096), (4096, 14336), (4096, 4096)])
def test_gemv_automatic_choice_8b_shapes_against_oracle(ops, N, K):
    """The small-M entry point as the benchmark calls it (no tuning arguments) at the true Llama-3-8B shapes, on the
    benchmark's kind of data, against the oracle on 1024 sampled columns (columns are independent of each other); the
    plan query must report the launch that ran: a K split over workgroups on the long, narrow down projection, the ring
    form wherever the library's rule says so."""
    w = O.synth_weights(N, K, seed=10)
    p = ops.prepare_weight(dev(w))
    blocks = np.sort(np.random.default_rng(N + K).choice(N // 16, size=64, replace=False))     # 64 strips of 16 columns
    cols = (blocks[:, None] * 16 + np.arange(16)[None, :]).reshape(-1)
    q_rows = (blocks[:, None] * 4 + np.arange(4)[None, :]).reshape(-1)                          # packed rows of those strips
    cidx = torch.from_numpy(cols).cuda()
    qs = p["qweight"][torch.from_numpy(q_rows).cuda()].cpu().numpy()
    sc, sz = p["scales"][:, cidx].cpu().numpy(), p["scaled_zeros"][:, cidx].cpu().numpy()
    w16_ref = O.dequant_to_f16(qs, sc, sz)
    seen = set()
    for M in (1, 8, 16, 32):
        plan = ops.gemv_plan(M, N, K)
        seen.add((plan["form"], plan["ks"] > 1))
        x = O.synth_acts(M, K, seed=M)
        out = ops.gemv_forward(dev(x), p["qweight"], p["scales"], p["scaled_zeros"], M, N, K, 128)
        torch.cuda.synchronize()
        assert O.max_abs_rel(out[:, cidx].cpu().numpy(), O.gemm_f16(x, w16_ref)) < 2e-3, (M, plan)
        if plan["form"] == "register":      # the tuning entry point with the planned split is the same launch
            same = ops.gemv_forward(dev(x), p["qweight"], p["scales"], p["scaled_zeros"], M, N, K, 128, cfg=(plan["nt"], plan["nw"], plan["ks"]))
        else:
            same = ops.gemv_forward(dev(x), p["qweight"], p["scales"], p["scaled_zeros"], M, N, K, 128,
                                    ring=(plan["nt"], plan["nw"], plan["ks"], plan["depth"]))
        assert torch.equal(same.view(torch.int16), out.view(torch.int16)), (M, plan)
    if (N, K) == (4096, 14336):
        assert any(split for _, split in seen), seen           # the split over workgroups engaged on this shape
    if (N, K) == (28672, 4096):
        assert ("register", False) in seen and any(form == "ring" for form, _ in seen), seen
    ws = ops.gemv_workspace_for("cuda")
    assert int(ws[:65536].view(torch.int32).abs().sum().item()) == 0


@pytest.mark.parametrize("N,K", [(28672, 4096), (4096, 14336), (37888, 3584)])
def test_conversion_layouts_agree_full_size(ops, N, K):
    """Conversion at full size: with s = 1, z = 0 the fp16 result is the unpacked nibble itself (pure layout), the int8
    result likewise; row-major and tiled outputs must hold the same matrix."""
    q = np.random.default_rng(N).integers(0, 16, size=(N, K), dtype=np.uint8)
    qw = dev(O.pack_int_awq(q))
    Gp = O.padded_groups(K)
    one = torch.ones((Gp, N), dtype=torch.float16, device="cuda")
    zero = torch.zeros((Gp, N), dtype=torch.float16, device="cuda")
    want = torch.from_numpy(q).cuda()
    for dtype, fn in ((torch.float16, ops.dequant_interleaved_int4_to_fp16), (torch.int8, ops.dequant_interleaved_int4_to_int8)):
        rows = torch.empty((N, K), dtype=dtype, device="cuda")
        fn(rows, qw, one, zero, 128)
        assert torch.equal(rows.to(torch.uint8), want) and bool((rows >= 0).all())
        if N % 128 == 0:
            tiled = torch.empty((N, K), dtype=dtype, device="cuda")
            fn(tiled, qw, one, zero, 128, tiled=True)
            assert torch.equal(ops.untile(tiled, N, K), rows)


def test_module_forward_full_size_rows(ops):
    """DynamicLinear.forward at M = 4096 on a 4096 x 4096 layer through the W8A8 lane (bit-exact on sampled tokens:
    every token is quantised and scaled on its own) and at M = 16 through the small-M lane (1e-2)."""
    from kairos.dynamic_linear import COMP_TYPE_NAME, DynamicLinear
    N = K = 4096
    w = O.synth_weights(N, K, seed=10)
    lin = torch.nn.Linear(K, N, bias=False, dtype=torch.float16)
    with torch.no_grad():
        lin.weight.copy_(torch.from_numpy(w))
    dl = DynamicLinear.from_module(lin.cuda(), 'cuda')
    p = O.prepare_weights(w)
    for key in ("qweight", "scales", "scaled_zeros", "scales_to8", "scaled_zeros_to8", "scales_1"):
        assert np.array_equal(getattr(dl, key).cpu().numpy().view(np.uint16), p[key].view(np.uint16)), key
    M = 4096
    x = O.synth_acts(M, K, seed=11)
    out = dl._forward(dev(x)[None], M, COMP_TYPE_NAME['w8a8'])[0]
    rows = sample_rows(M, 12, 3)
    ref = O.switched_forward(x[rows], p, COMP_TYPE_NAME['w8a8'])
    assert np.array_equal(out[torch.from_numpy(rows).cuda()].cpu().numpy().view(np.uint16), ref.view(np.uint16))
    x16 = O.synth_acts(16, K, seed=12)
    out16 = dl._forward(dev(x16)[None], 16, COMP_TYPE_NAME['w4a16_gemv'])[0]
    assert O.max_abs_rel(out16.cpu().numpy(), O.switched_forward(x16, p, COMP_TYPE_NAME['w4a16_gemv'])) < 1e-2


def _exact_case(M, N, K, seed):
    """Inputs whose product is exactly computable through every fp16 lane: integer weights q - 8 (tables s = 1,
    z = -8), activations with sixteen entries of +-1, +-2, +-3 per row.  Every product and every partial sum is a
    small integer (|sum| <= 16 * 3 * 8 = 384), exact in fp16 operands, fp32 accumulators and the fp16 output, in any
    summation order.  Returns (q uint8 [N, K], a int8 [M, K], want fp16 [M, N])."""
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    a = np.zeros((M, K), dtype=np.int8)
    # sixteen distinct columns per row: base + j * step, step < K / 16
    idx = (rng.integers(0, K, size=(M, 1)) + rng.integers(1, K // 16, size=(M, 1)) * np.arange(16)[None, :]) % K
    np.put_along_axis(a, idx, rng.choice(np.array([-3, -2, -1, 1, 2, 3], dtype=np.int8), size=(M, 16)), axis=1)
    want = (a.astype(np.float32) @ (q.astype(np.float32) - 8.0).T).astype(np.float16)   # exact at every step
    return q, a, want


# every M x shape of the benchmark's large-M region; (lane, tile selector) pairs to run for each
_FULL_F16 = [(M, N, K) for (N, K) in [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)] for M in (1024, 2048, 4096)]


@pytest.mark.parametrize("M,N,K", _FULL_F16)
def test_f16_lanes_full_size_exact(ops, M, N, K):
    """The fp16-output GEMM lanes at the benchmark's sizes, every kernel variant that can run them, bit for bit
    against an exactly computable product: the register-staged kernel (W4A16 and W8A16; tiles 128 and 256 and the
    automatic choice, which at 6144 columns and M = 4096 splits the launch into a 256-tile head and a 128-tile
    tail), the wave-private W4A16 kernel (128-row tiles, one and two wave quartets, at the M it is selected for),
    the direct-to-LDS fp16 kernel on row-major and on tiled weights (tiles 128, 192, 256, automatic), with a bias."""
    q, a, want = _exact_case(M, N, K, seed=M + N + K)
    qw = dev(O.pack_int_awq(q))
    Gp = O.padded_groups(K)
    ones = torch.ones((Gp, N), dtype=torch.float16, device="cuda")
    x = dev(a.astype(np.float16))
    bias_np = np.random.default_rng(N).integers(-64, 65, size=N).astype(np.float16)      # integer bias: still exact
    bias = dev(bias_np)
    want_b = (want.astype(np.float32) + bias_np.astype(np.float32)[None, :]).astype(np.float16)
    want_t, want_bt = dev(want), dev(want_b)
    w16 = torch.empty((N, K), dtype=torch.float16, device="cuda")
    ops.dequant_interleaved_int4_to_fp16(w16, qw, ones, ones * -8.0, 128)
    w16t = torch.empty((N, K), dtype=torch.float16, device="cuda")
    ops.dequant_interleaved_int4_to_fp16(w16t, qw, ones, ones * -8.0, 128, tiled=True)
    w8 = torch.empty((N, K), dtype=torch.int8, device="cuda")
    ops.dequant_interleaved_int4_to_int8(w8, qw, ones, ones * -8.0, 128)
    half = torch.full((N,), 0.5, dtype=torch.float16, device="cuda")                     # W8A16 channel scale, exact
    want_half = dev((want.astype(np.float32) * 0.5).astype(np.float16))

    def same(got, ref, what):
        torch.cuda.synchronize()
        bad = (got.view(torch.int16) != ref.view(torch.int16)).sum().item()
        assert bad == 0, f"{what}: {bad} of {got.numel()} elements differ (M={M} N={N} K={K})"

    w4_tiles = [0, 128, 256] + ([1128, 2128] if M <= 1024 else [])
    try:
        for tile in w4_tiles:
            ops.force_gemm_tile(tile)
            same(ops.gemm_forward(x, qw, ones, ones * -8.0), want_t, f"w4a16 tile {tile}")
        ops.force_gemm_tile(0)
        same(ops.gemm_forward(x, qw, ones, ones * -8.0, bias=bias), want_bt, "w4a16 with bias")
        for tile in (0, 128, 256):
            ops.force_gemm_tile(tile)
            same(ops.w8a16_gemm_forward(x, w8, half, N), want_half, f"w8a16 tile {tile}")
        for tile in (0, 128, 192, 256):
            ops.force_gemm_tile(tile)
            same(ops.f16_gemm_forward(x, w16, N), want_t, f"f16 row-major tile {tile}")
            same(ops.f16_gemm_forward(x, w16t, N, tiled=True), want_t, f"f16 tiled tile {tile}")
        ops.force_gemm_tile(0)
        same(ops.f16_gemm_forward(x, w16t, N, bias=bias, tiled=True), want_bt, "f16 tiled with bias")
    finally:
        ops.force_gemm_tile(0)


@pytest.mark.parametrize("M,N,K", [(1024, 28672, 4096), (2048, 4096, 14336), (4096, 6144, 4096)])
def test_f16_lanes_full_size_oracle_rows(ops, M, N, K):
    """The same lanes on the benchmark's own data (prepared N(0, 0.02) weights, N(0, 1) activations with outlier
    channels) against the oracle on sampled rows and a slice of columns: 2e-3 (bar 1e-2)."""
    w = O.synth_weights(N, K, seed=10)
    p = ops.prepare_weight(dev(w))
    x = O.synth_acts(M, K, seed=11)
    xd = dev(x)
    rows = sample_rows(M, 6, N)
    cols = slice(0, 1024)                                                      # 256 packed rows: the oracle's slice
    qs = p["qweight"][: 1024 // 4].cpu().numpy()
    sc, sz = p["scales"][:, cols].cpu().numpy(), p["scaled_zeros"][:, cols].cpu().numpy()
    w16_ref = O.dequant_to_f16(qs, sc, sz)
    ref = O.gemm_f16(x[rows], w16_ref)
    ridx = torch.from_numpy(rows).cuda()
    out4 = ops.gemm_forward(xd, p["qweight"], p["scales"], p["scaled_zeros"])
    w16t = torch.empty((N, K), dtype=torch.float16, device="cuda")
    ops.dequant_interleaved_int4_to_fp16(w16t, p["qweight"], p["scales"], p["scaled_zeros"], 128, tiled=True)
    out16 = ops.f16_gemm_forward(xd, w16t, N, tiled=True)
    w8 = torch.empty((N, K), dtype=torch.int8, device="cuda")
    ops.dequant_interleaved_int4_to_int8(w8, p["qweight"], p["scales_to8"], p["scaled_zeros_to8"], 128)
    out816 = ops.w8a16_gemm_forward(xd, w8, p["scales_1"], N)
    torch.cuda.synchronize()
    assert O.max_abs_rel(out4[ridx][:, cols].cpu().numpy(), ref) < 2e-3
    assert O.max_abs_rel(out16[ridx][:, cols].cpu().numpy(), ref) < 2e-3
    w8_ref = O.dequant_to_i8(qs, p["scales_to8"][:, cols].cpu().numpy(), p["scaled_zeros_to8"][:, cols].cpu().numpy())
    ref816 = O.gemm_w8a16(x[rows], w8_ref, p["scales_1"][cols].cpu().numpy())
    assert O.max_abs_rel(out816[ridx][:, cols].cpu().numpy(), ref816) < 2e-3


@pytest.mark.parametrize("N,K", [(3584, 18944), (4608, 3584)])
def test_conversion_qwen_shapes_against_oracle(ops, N, K):
    """int4 -> int8 / fp16, row-major and tiled, on the two Qwen2.5-7B shapes with padded table rows (K = 18944:
    152 rows, 148 used; K = 3584: 32 rows, 28 used) and with N = 4608 = 36 strips of 128: every element against the
    oracle, on prepared weights (whose tables the device preparation kernel wrote, zeros in the padded rows)."""
    p = ops.prepare_weight(dev(O.synth_weights(N, K, seed=K)))
    h = {k: v.cpu().numpy() for k, v in p.items()}
    assert h["scales"].shape[0] == O.padded_groups(K) and not h["scales"][K // 128:].any()
    want16 = O.dequant_to_f16(h["qweight"], h["scales"], h["scaled_zeros"])
    want8 = O.dequant_to_i8(h["qweight"], h["scales_to8"], h["scaled_zeros_to8"])
    for dtype, fn, tabs, want in ((torch.float16, ops.dequant_interleaved_int4_to_fp16, ("scales", "scaled_zeros"), want16),
                                  (torch.int8, ops.dequant_interleaved_int4_to_int8, ("scales_to8", "scaled_zeros_to8"), want8)):
        rows = torch.empty((N, K), dtype=dtype, device="cuda")
        fn(rows, p["qweight"], p[tabs[0]], p[tabs[1]], 128)
        tiled = torch.empty((N, K), dtype=dtype, device="cuda")
        fn(tiled, p["qweight"], p[tabs[0]], p[tabs[1]], 128, tiled=True)
        torch.cuda.synchronize()
        bits = np.uint16 if dtype is torch.float16 else np.uint8
        assert np.array_equal(rows.cpu().numpy().view(bits), want.view(bits))
        assert np.array_equal(ops.untile(tiled, N, K).cpu().numpy().view(bits), want.view(bits))
    # the fused preparation launch writes the same int8 weight (and quantises a few tokens beside it)
    x = dev(O.synth_acts(5, K, seed=3))
    w8 = torch.empty((N, K), dtype=torch.int8, device="cuda")
    a8 = torch.empty((5, K), dtype=torch.int8, device="cuda")
    sx = torch.empty((5,), dtype=torch.float16, device="cuda")
    ops.prep_w8a8(w8, p["qweight"], p["scales_to8"], p["scaled_zeros_to8"], a8, x, sx, 128, tiled=True)
    assert np.array_equal(ops.untile(w8, N, K).cpu().numpy(), want8)


@pytest.mark.parametrize("M,N,K", [(4096, 28672, 4096), (2048, 4096, 14336), (1024, 6144, 4096), (512, 28672, 4096),
                                   (256, 4096, 4096), (2048, 28672, 4096), (4096, 6144, 4096),    # these two: two launches
                                   (128, 28672, 4096), (1024, 4096, 14336), (128, 4096, 14336),   # two wave quartets per workgroup
                                   (1024, 28672, 4096), (4096, 4096, 14336)])                      # 512 x 128 tiles
def test_w4a8_lane_full_size(ops, M, N, K):
    """The W4A8 lane at the benchmark's sizes.  (a) On the exactly computable inputs of the W8A8 full-size test (tables
    s = 1, z = -8, sparse +-127 activations, channel scale 1/128) the whole fp16 output is one known rounding of an
    exact number.  (b) On the benchmark's own data (prepared N(0, 0.02) weights, outlier activations) the output equals
    the W8A8 lane's (converter + int8 GEMM on tiled weights) bit for bit, and sampled rows equal the oracle's."""
    rng = np.random.default_rng(N + K + M)
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    w8 = q.astype(np.int8) - 8
    Gp = O.padded_groups(K)
    ones = torch.ones((Gp, N), dtype=torch.float16, device="cuda")
    a = np.zeros((M, K), dtype=np.int8)
    idx = (rng.integers(0, K, size=(M, 1)) + rng.integers(1, K // 16, size=(M, 1)) * np.arange(16)[None, :]) % K
    np.put_along_axis(a, idx, rng.choice(np.array([-127, 127], dtype=np.int8), size=(M, 16)), axis=1)
    sx = torch.ones((M,), dtype=torch.float16, device="cuda")
    ws = torch.full((N,), 1.0 / 128.0, dtype=torch.float16, device="cuda")
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    ops.w4a8_gemm_forward(dev(a), dev(O.pack_int_awq(q)), ones, ones * -8.0, ws, sx, out)
    torch.cuda.synchronize()
    exact = ((a.astype(np.float32) / np.float32(127.0)) @ w8.astype(np.float32).T) * np.float32(127.0 / 128.0)
    assert np.array_equal(out.cpu().numpy().view(np.uint16), exact.astype(np.float16).view(np.uint16))
    # (b) benchmark data
    p = ops.prepare_weight(dev(O.synth_weights(N, K, seed=10)))
    x_np = O.synth_acts(M, K, seed=11)
    x = dev(x_np)
    a8 = torch.empty((M, K), dtype=torch.int8, device="cuda")
    sxx = torch.empty((M,), dtype=torch.float16, device="cuda")
    w8_t = torch.empty((N, K), dtype=torch.int8, device="cuda")
    ops.prep_w8a8(w8_t, p["qweight"], p["scales_to8"], p["scaled_zeros_to8"], a8, x, sxx, 128, tiled=True)
    want = torch.empty((M, N), dtype=torch.float16, device="cuda")
    ops.w8a8_gemm_forward(a8, w8_t, p["scales_1"], sxx, want, tiled=True)
    got = torch.empty((M, N), dtype=torch.float16, device="cuda")
    ops.w4a8_gemm_forward(a8, p["qweight"], p["scales_to8"], p["scaled_zeros_to8"], p["scales_1"], sxx, got)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    rows = sample_rows(M, 4, N)
    cols = slice(0, 512)
    hp = {k: v.cpu().numpy() for k, v in p.items()}
    w8_ref = O.dequant_to_i8(hp["qweight"][: 512 // 4], hp["scales_to8"][:, cols], hp["scaled_zeros_to8"][:, cols])
    a8_ref, sx_ref = O.quant_act_i8(x_np[rows])
    ref = O.gemm_w8a8(a8_ref, w8_ref, hp["scales_1"][cols], sx_ref)[1]
    assert np.array_equal(got[torch.from_numpy(rows).cuda()][:, cols].cpu().numpy().view(np.uint16), ref.view(np.uint16))
