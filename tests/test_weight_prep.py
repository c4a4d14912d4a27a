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
