"""The shipped host-side weight preparation (torch) against the numpy oracle, bit for bit, on CPU."""
import numpy as np
import pytest
import torch

from kairos_amd import weight_prep as W
from oracle import kairos_oracle as O


@pytest.mark.parametrize("N,K", [(4, 64), (8, 128), (64, 3584), (128, 512)])
def test_pack_unpack(N, K):
    q = np.random.default_rng(N + K).integers(0, 16, size=(N, K), dtype=np.uint8)
    got = W.pack_int_awq(torch.from_numpy(q.astype(np.int8)))
    assert got.dtype == torch.int16 and tuple(got.shape) == (N // 4, K)
    assert np.array_equal(got.numpy(), O.pack_int_awq(q))
    assert np.array_equal(W.unpack_int_awq(got).numpy(), q.astype(np.int8))


def test_all_fifteens_is_minus_one():
    q = torch.full((4, 64), 15, dtype=torch.int8)
    assert (W.pack_int_awq(q) == -1).all()


@pytest.mark.parametrize("K", [128, 3584, 4096, 18944])
def test_zero_width(K):
    assert W.calculate_zeros_width(K) * 8 == O.padded_groups(K)


@pytest.mark.parametrize("N,K", [(16, 256), (64, 3584), (256, 1024)])
def test_prepare_matches_oracle(N, K):
    w = O.synth_weights(N, K, seed=N)
    ref = O.prepare_weights(w)
    got = W.prepare_linear_weight(torch.from_numpy(w))
    for key in ("qweight", "scales", "scaled_zeros", "scales_to8", "scaled_zeros_to8", "scales_1"):
        a, b = got[key].numpy(), ref[key]
        assert a.shape == b.shape and a.dtype == b.dtype, key
        assert np.array_equal(a.view(np.uint16), b.view(np.uint16)), key


def test_int8_and_int4_steps():
    w = O.synth_weights(32, 256, seed=77)
    q8, cfg = W.quantize_tensor_int8(torch.from_numpy(w), max_int=127)
    r8, rs = O.quantize_int8(w)
    assert np.array_equal(q8.numpy(), r8) and np.array_equal(cfg["scale"].numpy(), rs)
    q4, cfg4 = W.kairos_quantize_tensor_int4(q8, group_size=128)
    r4, s4, z4 = O.quantize_int4_kairos(r8)
    assert np.array_equal(q4.numpy(), r4)
    assert np.array_equal(cfg4["scale_f"].numpy(), s4) and np.array_equal(cfg4["zero_pt_f"].numpy(), z4)
    assert cfg4["zero_pt_i"].dtype == torch.int8 and cfg4["scale_i"].dtype == torch.int8
    with pytest.raises(ValueError):
        W.kairos_quantize_tensor_int4(q8[:, :100], group_size=128)


def test_integer_second_level_factors():
    """scale_i = floor(scale_f), zero_pt_i = round(zero_pt_f) of the version-2 quantiser (kairos/dynamic_linear_v2.py:36-41):
    the host mirror against the oracle, and the oracle against hand cases -- a group spanning -120..105 has scale 15 and
    zero-point 8 exactly; -128..127 gives scale floor(17) and zero round(7.529) = 8; a half-way zero-point rounds to even."""
    import numpy as np
    import torch
    from oracle import kairos_oracle as O
    from kairos_amd import weight_prep as W
    hand = np.zeros((3, 128), dtype=np.int8)
    hand[0, :2] = (-120, 105)              # range 225: scale 15, zero 120 / 15 = 8
    hand[1, :2] = (-128, 127)              # range 255: scale 17, zero 128 / 17 = 7.53
    hand[2, :2] = (-75, 75)                # range 150: scale 10, zero 7.5 -> 8 (half to even)
    si, zi, ok = O.quantize_int4_int_factors(hand)
    assert si.reshape(-1).tolist() == [15, 17, 10] and zi.reshape(-1).tolist() == [8, 8, 8] and ok.all()
    hand[2, :2] = (-65, 85)                # scale 10, zero 6.5 -> 6
    assert O.quantize_int4_int_factors(hand)[1].reshape(-1).tolist() == [8, 8, 6]
    w8 = np.random.default_rng(3).integers(-128, 128, size=(16, 512), dtype=np.int8)
    w8[5, 128:256] = 33                    # a constant group: its zero-point leaves the int8 range
    si, zi, ok = O.quantize_int4_int_factors(w8)
    _q, cfg = W.kairos_quantize_tensor_int4(torch.from_numpy(w8), group_size=128)
    assert np.array_equal(cfg["scale_i"].numpy(), si)
    assert not ok[5 * 4 + 1] and ok.sum() == ok.size - 1
    assert np.array_equal(cfg["zero_pt_i"].numpy()[ok], zi[ok])          # where the int8 value is defined
    # consistency with the float factors the lanes use: |scale_f - scale_i| < 1, |zero_pt_f - zero_pt_i| <= 0.5 (+ fp16 rounding)
    assert np.all(cfg["scale_f"].numpy().astype(np.float32)[ok] - si[ok] < 1.01)
    assert np.all(np.abs(cfg["zero_pt_f"].numpy().astype(np.float32)[ok] - zi[ok]) <= 0.51)
