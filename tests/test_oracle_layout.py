"""Pins the oracle's int4 layout (row F) and scale tables (row S) without running the reference.

The reference states the layout twice, independently: step by step
(thirdparty/AWQ/awq_method.py:5-38) and as one reshape/permute (test/depacking.py:8-19, inverse
:22-38).  Both are re-typed here in numpy and must agree with the oracle's index formula, with
each other, and with a brute-force enumeration of every nibble position.
"""
import numpy as np
import pytest

from oracle import kairos_oracle as O


def pack_stepwise(q):
    """awq_method.py:5-38, one numpy statement per torch statement."""
    N, K = q.shape
    p = q.reshape(N, K // 32, 32).astype(np.int16)
    p = p.reshape(N, K // 32, 4, 4, 2).transpose(0, 1, 3, 2, 4).reshape(N, K // 32, 32)
    p = p.reshape(N, K // 32, 4, 4, 2).transpose(0, 1, 2, 4, 3).reshape(N, K)
    p = p.reshape(N // 4, 4, K // 64, 64).transpose(0, 2, 1, 3)
    p = np.ascontiguousarray(p).reshape(N // 4, K // 64, 64, 4).astype(np.uint16)
    p = p[..., 0] | (p[..., 1] << 4) | (p[..., 2] << 8) | (p[..., 3] << 12)
    return p.reshape(N // 4, K).view(np.int16)


def pack_closed_form(q):
    """test/depacking.py:8-19."""
    N, K = q.shape
    p = q.reshape(N // 4, 4, K // 64, 2, 4, 4, 2).transpose(0, 2, 1, 3, 5, 6, 4)
    p = np.ascontiguousarray(p).astype(np.uint16)
    p = p[..., 0] | (p[..., 1] << 4) | (p[..., 2] << 8) | (p[..., 3] << 12)
    return p.reshape(N // 4, K).view(np.int16)


def unpack_closed_form(packed):
    """test/depacking.py:22-38."""
    N4, K = packed.shape
    u = packed.view(np.uint16)
    nib = np.stack([u & 0xF, (u >> 4) & 0xF, (u >> 8) & 0xF, (u >> 12) & 0xF], axis=-1)
    nib = nib.reshape(N4, K // 64, 4, 2, 4, 2, 4).transpose(0, 2, 1, 3, 6, 4, 5)
    return nib.reshape(N4 * 4, K).astype(np.uint8)


@pytest.mark.parametrize("N,K", [(4, 64), (8, 128), (32, 256), (64, 3584)])
def test_three_statements_agree(N, K):
    rng = np.random.default_rng(N * 1000 + K)
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    a = O.pack_int_awq(q)
    assert a.dtype == np.int16 and a.shape == (N // 4, K)
    assert np.array_equal(a, pack_stepwise(q))
    assert np.array_equal(a, O.pack_int_awq_by_index(q))
    assert np.array_equal(O.unpack_int_awq_by_index(a), q)
    assert np.array_equal(a, pack_closed_form(q))
    assert np.array_equal(O.unpack_int_awq(a), q)
    assert np.array_equal(unpack_closed_form(a), q)


def test_brute_force_every_position():
    """One-hot inputs: element (n, k) must set exactly the nibble the formula names."""
    N, K = 8, 128
    for n in range(N):
        for k in range(K):
            q = np.zeros((N, K), dtype=np.uint8)
            q[n, k] = 0xF
            ref = pack_stepwise(q).view(np.uint16).ravel()
            nz = np.nonzero(ref)[0]
            assert len(nz) == 1
            word, nib = O.awq_position(n, k, K)
            assert nz[0] == word
            assert ref[nz[0]] == 0xF << (4 * nib)


def test_position_is_a_bijection():
    N, K = 16, 256
    nn, kk = np.meshgrid(np.arange(N), np.arange(K), indexing="ij")
    word, nib = O.awq_position(nn, kk, K)
    slot = word * 4 + nib
    assert np.array_equal(np.sort(slot.ravel()), np.arange(N * K))


def test_consumer_view_128bit_chunk():
    """A 16-byte chunk holds 32 weights of ONE row: words j=0..7 carry k%8=j, nibble a carries
    k = 32h + 8a + j (the indexing a streaming consumer relies on;
    kernels/csrc/kairos_kernel/dequant_awq_format/dequant_i4_to_f16.cu:95-151)."""
    N, K = 8, 128
    q = np.arange(N * K, dtype=np.int64).reshape(N, K) % 16
    kmap = np.tile(np.arange(K), (N, 1))
    packed_k = {}
    for n in range(N):
        for k in range(K):
            w, a = O.awq_position(n, k, K)
            packed_k[(int(w), int(a))] = (n, k)
    for n in range(N):
        for kb in range(K // 64):
            for h in range(2):
                base = (n // 4) * K + kb * 64 + (n % 4) * 16 + h * 8
                for j in range(8):
                    for a in range(4):
                        assert packed_k[(base + j, a)] == (n, kb * 64 + 32 * h + 8 * a + j)


@pytest.mark.parametrize("K,Gp", [(4096, 32), (14336, 112), (3584, 32), (18944, 152), (8192, 64), (28672, 224), (128, 8)])
def test_padded_group_table(K, Gp):
    assert O.padded_groups(K) == Gp


def test_qfactor_layout_values():
    N, K = 8, 384
    rng = np.random.default_rng(0)
    s = rng.uniform(0.01, 2.0, size=(N, K // 128)).astype(np.float16)
    z = rng.uniform(0.0, 15.0, size=(N, K // 128)).astype(np.float16)
    st, szt = O.qfactor_layout(s, z)
    assert st.shape == (8, N) and szt.shape == (8, N) and st.dtype == np.float16
    assert np.array_equal(st[:3], s.T)
    assert not st[3:].any() and not szt[3:].any()
    for n in range(N):
        for g in range(3):
            want = -np.float16(np.float32(s[n, g]) * np.float32(z[n, g]))
            assert szt[g, n] == want
    # hand case: s=0.5, z=3 -> -1.5 exactly
    st, szt = O.qfactor_layout(np.full((4, 1), 0.5, np.float16), np.full((4, 1), 3, np.float16))
    assert (szt[0] == np.float16(-1.5)).all()


# ---------------------------------------------------------------------------------------------------------
# W4A8 operand layout (the v2 candidate's weight format) and the re-pack of the resident format into it.
# The reference states the layout twice and its own test fixes the re-pack bit for bit:
#   trans_layout_c16_to_c8_awq(pack_int_awq(A)) == pack_int_qserve(A)          (test/test_trans_layout.py:46-52)
# ---------------------------------------------------------------------------------------------------------
def w4a8_one_permutation(q):
    """test/test_trans_layout.py:8-14."""
    N, K = q.shape
    p = q.reshape(N // 32, 2, 2, 8, K // 32, 2, 4, 4).transpose(0, 4, 3, 6, 5, 2, 7, 1)
    p = np.ascontiguousarray(p).astype(np.int8)
    return ((p[..., 1] << 4) + p[..., 0]).reshape(N, K // 2)


def w4a8_two_permutations(q):
    """thirdparty/Qserve/w4a8_linear.py:187-205."""
    N, K = q.shape
    p = np.ascontiguousarray(q.reshape(N // 32, 2, 2, 8, K // 32, 2, 4, 4).transpose(0, 4, 3, 6, 1, 5, 2, 7))
    p = np.ascontiguousarray(p.transpose(0, 1, 2, 3, 5, 6, 7, 4)).astype(np.int8)
    p = (p[..., 1] << 4) + p[..., 0]
    return p.reshape(N // 32, K // 32, 32, 16).reshape(N, K // 2)


def trans_layout_reference_python(awq_packed, N, K):
    """trans_layout_pytorch, test/test_trans_layout.py:25-37 (the reference's own torch restatement of its kernel)."""
    a = awq_packed.view(np.uint16).reshape(N // 4, K // 64, 4, 2, 4, 2)
    u = np.stack([a & 0xF, (a >> 4) & 0xF, (a >> 8) & 0xF, (a >> 12) & 0xF], axis=-1).astype(np.int8)
    u = u.transpose(0, 2, 1, 3, 6, 4, 5).reshape(N // 32, 2, 2, 8, K // 32, 2, 4, 4)
    u = u.transpose(0, 4, 3, 6, 5, 2, 7, 1)
    return np.ascontiguousarray((u[..., 1] << 4) + u[..., 0]).reshape(N, K // 2)


@pytest.mark.parametrize("N,K", [(32, 64), (64, 128), (96, 320), (128, 3584)])
def test_w4a8_layout_statements_agree(N, K):
    rng = np.random.default_rng(N + K)
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    a = O.pack_int_w4a8(q)
    assert a.dtype == np.int8 and a.shape == (N, K // 2)
    assert np.array_equal(a, w4a8_one_permutation(q))
    assert np.array_equal(a, w4a8_two_permutations(q))
    assert np.array_equal(a, O.pack_int_w4a8_by_index(q))
    awq = O.pack_int_awq(q)
    assert np.array_equal(O.trans_layout_c16_to_c8(awq), a)                       # the reference test's contract
    assert np.array_equal(trans_layout_reference_python(awq, N, K), a)


def test_w4a8_layout_brute_force():
    N, K = 32, 64
    for n in range(N):
        for k in range(K):
            q = np.zeros((N, K), dtype=np.uint8)
            q[n, k] = 0xF
            out = O.pack_int_w4a8(q).view(np.uint8).ravel()
            byte, nib = O.w4a8_position(n, k, K)
            assert out[byte] == 0xF << (4 * int(nib)) and np.count_nonzero(out) == 1
