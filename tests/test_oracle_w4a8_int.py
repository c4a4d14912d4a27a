"""What pins the oracle's restatement of the version-2 `w4a8_qserve` operands and arithmetic (integer per-group
factors): hand cases of the two quantisers (thirdparty/Qserve/quantization.py:4-36), the protective range that keeps
the kernel's byte-wise arithmetic from wrapping, the textbook (q - zero) * scale form, wrap-around cases against
Python integers, and the host-side mirror in kairos_amd.weight_prep."""
import numpy as np
import pytest

from oracle import kairos_oracle as O

torch = pytest.importorskip("torch")


def test_int8_level_hand_cases():
    w = np.array([[119.0, 1.5, -2.5, 0.4], [0.0, 0.0, 0.0, 0.0], [238.0, -238.0, 119.0, 3.0]], dtype=np.float32)
    q, s = O.qserve_quantize_int8(w)
    assert q[0].tolist() == [119, 2, -2, 0] and float(s[0, 0]) == 1.0           # step 1: halves go to the even neighbour
    assert q[1].tolist() == [0, 0, 0, 0] and float(s[1, 0]) == 0.0              # 1e-7 / 119 is below the fp16 subnormals
    assert q[2].tolist() == [119, -119, 60, 2] and float(s[2, 0]) == 2.0        # 59.5 -> 60, 1.5 -> 2
    assert s.dtype == np.float16 and q.dtype == np.int8


def test_int4_level_hand_cases():
    g = np.zeros((3, 128), dtype=np.int8)
    g[0, :2] = (-119, 119)           # range 238 -> scale round(15.87) = 16, zero round(119 / 16) = 7
    g[1, :] = 5                      # constant: scale round(~0) = 0 -> 1, zero = -5, q = 0
    g[2, :3] = (-8, 7, 0)            # range 15 -> scale 1, zero 8
    q, s, z = O.qserve_quantize_int4(g)
    assert s.reshape(-1).tolist() == [16, 1, 1] and z.reshape(-1).tolist() == [7, -5, 8]
    assert q[0, :3].tolist() == [0, 14, 7]                    # -119/16 + 7 = -0.44 -> 0; 119/16 + 7 = 14.44; 0 -> 7
    assert q[1].tolist() == [0] * 128 and q[2, :3].tolist() == [0, 15, 8]
    S, Z = O.qserve_tables(s, z, 3)
    assert S.reshape(-1).tolist() == [16, 1, 1] and Z.reshape(-1).tolist() == [-112, 5, -8]
    w8 = O.dequant_w4a8_int(O.pack_int_awq(np.tile(q, (4, 1))[:4]), np.tile(S, (1, 4))[:, :4], np.tile(Z, (1, 4))[:, :4])
    assert w8.shape == (4, 128)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_protective_range_means_no_wrap_and_textbook_dequant(seed):
    """|w8| <= 119 and whole-number factors: q * scale - zero * scale stays inside int8 for every nibble value the
    quantiser can emit, so the kernel's modulo-256 bytes ARE (q - zero) * scale, and away from the clamp they are
    within scale / 2 of the int8 weight."""
    rng = np.random.default_rng(seed)
    N, K = 64, 512
    w = (rng.standard_normal((N, K)) * rng.uniform(0.01, 3.0, size=(N, 1))).astype(np.float16)
    w[3] = 0
    w[5, :128] = 0.25                                         # a constant group
    w8, s1 = O.qserve_quantize_int8(w)
    assert np.abs(w8.astype(np.int32)).max() <= 119
    q, si, zi = O.qserve_quantize_int4(w8)
    assert q.min() >= 0 and q.max() <= 15 and si.min() >= 1 and si.max() <= 16
    S, Z = O.qserve_tables(si, zi, N)
    got = O.dequant_w4a8_int(O.pack_int_awq(q), S, Z).astype(np.int32)
    text = ((q.reshape(N, -1, 128).astype(np.int32) - zi.reshape(N, -1, 1)) * si.reshape(N, -1, 1)).reshape(N, K)
    assert np.array_equal(got, text) and text.min() >= -128 and text.max() <= 127
    f = w8.reshape(N, -1, 128).astype(np.float32) / si.reshape(N, -1, 1) + zi.reshape(N, -1, 1)
    free = ((f > -0.5) & (f < 15.5)).reshape(N, K)            # not clamped
    assert (np.abs(got - w8)[free] * 2 <= np.broadcast_to(si.reshape(N, -1, 1), (N, K // 128, 128)).reshape(N, K)[free]).all()


def test_bytes_wrap_one_by_one():
    """Factors no quantiser emits: every byte is (q * scale + zero) mod 256 on its own, scale read as unsigned."""
    rng = np.random.default_rng(7)
    N, K = 8, 256
    q = rng.integers(0, 16, size=(N, K), dtype=np.int8)
    S = rng.integers(-128, 128, size=(2, N), dtype=np.int8)
    Z = rng.integers(-128, 128, size=(2, N), dtype=np.int8)
    got = O.dequant_w4a8_int(O.pack_int_awq(q), S, Z)
    for n in range(N):
        for k in range(0, K, 37):
            v = (int(q[n, k]) * (int(S[k // 128, n]) & 0xFF) + (int(Z[k // 128, n]) & 0xFF)) % 256
            assert int(got[n, k]) == (v - 256 if v > 127 else v)


def test_product_is_the_integer_matmul_with_the_w8a8_epilogue():
    rng = np.random.default_rng(11)
    M, N, K = 5, 8, 128
    q = rng.integers(0, 16, size=(N, K), dtype=np.int8)
    S = rng.integers(1, 17, size=(1, N), dtype=np.int8)
    Z = (-(rng.integers(0, 8, size=(1, N)) * S.astype(np.int32))).astype(np.int8)
    a8 = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    ws = rng.random(N).astype(np.float16)
    as_ = rng.random(M).astype(np.float16)
    acc, out = O.gemm_w4a8_int(a8, O.pack_int_awq(q), S, Z, ws, as_)
    w8 = O.dequant_w4a8_int(O.pack_int_awq(q), S, Z)
    for m in range(M):
        for n in range(N):
            exact = sum(int(a8[m, k]) * int(w8[n, k]) for k in range(K))
            assert int(acc[m, n]) == exact
            assert out[m, n] == np.float16(np.float32(exact) * (np.float32(ws[n]) * np.float32(as_[m])))


def test_host_mirror_equals_oracle():
    from kairos_amd import weight_prep as W
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((96, 512)) * 0.05).astype(np.float16)
    w[7] = 0
    t = W.qserve_factor_tables(torch.from_numpy(w))
    w8, s1 = O.qserve_quantize_int8(w)
    q, si, zi = O.qserve_quantize_int4(w8)
    S, Z = O.qserve_tables(si, zi, 96)
    assert np.array_equal(t["s1_scales"].numpy().view(np.uint16), s1.reshape(-1).view(np.uint16))
    assert np.array_equal(t["s2_scales"].numpy(), S) and np.array_equal(t["s2_zeros"].numpy(), Z)
    q8, c1 = W.qserve_quantize_tensor_int8(torch.from_numpy(w))
    q4, c2 = W.qserve_quantize_tensor_int4(q8, group_size=128)
    assert np.array_equal(q8.numpy(), w8) and np.array_equal(q4.numpy(), q)
    assert c2["scale"].dtype == torch.int8 and c2["zero_pt"].dtype == torch.int8


def test_version2_layer_keeps_the_integer_factors_on_the_host():
    """Host logic of from_module(..., qserve_factors=True): three more buffers beside the six resident ones, carried by
    the state dict into a module built with the plain constructor; without a GPU the lane itself refuses loudly."""
    from kairos.dynamic_linear_v2 import COMP_TYPE_NAME, DynamicLinear
    lin = torch.nn.Linear(256, 64, bias=True, dtype=torch.float16)
    plain = DynamicLinear.from_module(lin, 'cpu')
    q = DynamicLinear.from_module(lin, 'cpu', qserve_factors=True)
    extra = {"qserve_s1_scales", "qserve_s2_scales", "qserve_s2_zeros"}
    assert set(q.state_dict()) - set(plain.state_dict()) == extra and plain.qserve_s2_scales is None
    w8, s1 = O.qserve_quantize_int8(lin.weight.detach().numpy())
    _, si, zi = O.qserve_quantize_int4(w8)
    S, Z = O.qserve_tables(si, zi, 64)
    assert np.array_equal(q.qserve_s2_scales.numpy(), S) and np.array_equal(q.qserve_s2_zeros.numpy(), Z)
    fresh = DynamicLinear(256, 64, True, 'cpu', 128)
    fresh.load_state_dict(q.state_dict())
    for key in extra:
        assert torch.equal(getattr(fresh, key), getattr(q, key))
    empty = DynamicLinear.from_module(lin, 'cpu', init_only=True, qserve_factors=True)
    assert empty.qserve_s2_zeros.shape == (2, 64) and empty.qserve_s1_scales.dtype == torch.float16
    with pytest.raises(ValueError, match="GPU tensor"):
        q._forward(torch.zeros(1, 3, 256, dtype=torch.float16), 3, COMP_TYPE_NAME['w4a8_qserve'])
