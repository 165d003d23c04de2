"""Pins the oracle's pack / unpack / table-index restatements (CPU only).

The reference ships no golden vectors for this path, so each function is pinned
by what the format fixes: hand-written known-answer words, a scalar brute-force
loop written here independently of both restatements, the reference's own
self-check identity (unpack(pack(B), a) == einsum(B, a),
zeroShot/models/kernel.py:96-120), and agreement of the numpy and C versions.
"""
import numpy as np
import pytest

import oracle as orc


def _signs(rng, shape):
    return (rng.integers(0, 2, size=shape, dtype=np.int8) * 2 - 1).astype(np.int8)


# ---- known answers ---------------------------------------------------------

@pytest.mark.parametrize("pack", [orc.pack_binary_weight_np, orc.pack_binary_weight_c])
def test_pack_known_answers(pack):
    ones = np.ones((1, 1, 32, 1), dtype=np.int8)
    assert pack(-ones)[0, 0, 0] == 0                      # all -1 -> no bit set
    assert pack(ones)[0, 0, 0] == -1                      # all +1 -> 0xFFFFFFFF as int32
    only31 = -ones.copy()
    only31[0, 0, 31, 0] = 1
    assert pack(only31)[0, 0, 0] == -2147483648           # bit 31 is the int32 sign
    only0 = -ones.copy()
    only0[0, 0, 0, 0] = 1
    assert pack(only0)[0, 0, 0] == 1                      # LSB first
    alt = -ones.copy()
    alt[0, 0, 0::2, 0] = 1                                # +1 at even positions
    assert pack(alt)[0, 0, 0] == 0x55555555
    assert np.uint32(pack(-alt)[0, 0, 0]) == np.uint32(0xAAAAAAAA)


@pytest.mark.parametrize("pack", [orc.pack_binary_weight_np, orc.pack_binary_weight_c])
def test_pack_shape_and_axis_order(pack):
    # [A, G, S, nb]: (G, S) flatten to one axis that is cut in words of 32;
    # word j covers flattened entries 32j .. 32j+31; the bit-plane axis stays last
    A, G, S, nb = 3, 2, 48, 2          # L = 96 -> 3 words, groups straddle words
    B = -np.ones((A, G, S, nb), dtype=np.int8)
    B[1, 1, 20, 1] = 1                 # flattened index 48 + 20 = 68 -> word 2, bit 4
    out = pack(B)
    assert out.shape == (A, 3, nb) and out.dtype == np.int32
    expect = np.zeros((A, 3, nb), dtype=np.int32)
    expect[1, 2, 1] = 1 << 4
    assert np.array_equal(out, expect)


@pytest.mark.parametrize("pack", [orc.pack_binary_weight_np, orc.pack_binary_weight_c])
def test_pack_rejects_non_binary(pack):
    B = np.ones((1, 1, 32, 1), dtype=np.int8)
    B[0, 0, 3, 0] = 0
    with pytest.raises(ValueError):
        pack(B)


def test_pack_rejects_wrong_rank_and_length():
    with pytest.raises(ValueError):
        orc.pack_binary_weight_np(np.ones((2, 32, 1), dtype=np.int8))
    with pytest.raises(ValueError):
        orc.pack_binary_weight_np(np.ones((1, 1, 33, 1), dtype=np.int8))


# ---- brute force -----------------------------------------------------------

def _brute_pack(B):
    A, G, S, nb = B.shape
    flat = B.reshape(A, G * S, nb)
    out = np.zeros((A, G * S // 32, nb), dtype=np.int64)
    for a in range(A):
        for l in range(G * S):
            for b in range(nb):
                if flat[a, l, b] == 1:
                    out[a, l // 32, b] += 1 << (l % 32)
    out[out >= 2 ** 31] -= 2 ** 32
    return out.astype(np.int32)


def _brute_unpack(bW, alpha):
    A, J, nb = bW.shape
    G = alpha.shape[1]
    L = J * 32
    W = np.zeros((A, L), dtype=np.float64)
    for a in range(A):
        for l in range(L):
            for b in range(nb):
                bit = (int(bW[a, l // 32, b]) >> (l % 32)) & 1
                W[a, l] += float(alpha[a, l // (L // G), b]) * (1.0 if bit else -1.0)
    return W


@pytest.mark.parametrize("seed,A,G,S,nb", [(0, 3, 2, 32, 1), (1, 2, 3, 64, 3), (2, 5, 1, 96, 4),
                                            (3, 1, 4, 16, 2)])
def test_pack_and_unpack_match_brute_force(seed, A, G, S, nb):
    rng = np.random.default_rng(seed)
    B = _signs(rng, (A, G, S, nb))
    alpha = np.abs(rng.standard_normal((A, G, nb))).astype(np.float32)
    want = _brute_pack(B)
    got_np, got_c = orc.pack_binary_weight_np(B), orc.pack_binary_weight_c(B)
    assert np.array_equal(got_np, want)
    assert np.array_equal(got_c, want)
    Wb = _brute_unpack(want, alpha)
    for W in (orc.unpack_weight_np(want, alpha), orc.unpack_weight_c(want, alpha)):
        assert W.shape == (A, G * S) and W.dtype == np.float32
        np.testing.assert_allclose(W, Wb, rtol=0, atol=2e-6)


def test_unpack_negative_words_use_bit31():
    # int32 sign bit is bit 31 of the word: entry 31 must come out +1
    bW = np.array([[[-2147483648]]], dtype=np.int32)
    alpha = np.array([[[2.0]]], dtype=np.float32)
    for W in (orc.unpack_weight_np(bW, alpha), orc.unpack_weight_c(bW, alpha)):
        assert W[0, 31] == 2.0 and np.all(W[0, :31] == -2.0)


# ---- the reference's own self-check identity --------------------------------

@pytest.mark.parametrize("seed", [0, 1])
def test_unpack_of_pack_equals_einsum(seed):
    # zeroShot/models/kernel.py:96-120 at its own sizes: N=128, K=768, g=128, 3 bits
    rng = np.random.default_rng(seed)
    N, G, S, nb = 128, 6, 128, 3
    B = _signs(rng, (N, G, S, nb))
    alpha = np.abs(rng.standard_normal((N, G, nb))).astype(np.float32)
    Q = np.einsum("nijl,nil->nij", B.astype(np.float64), alpha.astype(np.float64)).reshape(N, -1)
    packed = orc.pack_binary_weight_np(B)
    assert packed.shape == (N, G * S // 32, nb)
    for W in (orc.unpack_weight_np(packed, alpha), orc.unpack_weight_c(packed, alpha)):
        np.testing.assert_allclose(W, Q, rtol=0, atol=1e-5)
    # round trip of the bits
    assert np.array_equal(orc.unpack_bits_np(packed).reshape(B.shape), B)


def test_unpack_np_and_c_bit_identical():
    rng = np.random.default_rng(7)
    B = _signs(rng, (16, 2, 128, 4))
    alpha = np.abs(rng.standard_normal((16, 2, 4))).astype(np.float32)
    packed = orc.pack_binary_weight_np(B)
    a = orc.unpack_weight_np(packed, alpha)
    c = orc.unpack_weight_c(packed, alpha)
    assert np.array_equal(a.view(np.uint32), c.view(np.uint32))   # same fp32 order of adds


# ---- kernel layout: table indices and the look-up table ---------------------

def test_table_indices_are_the_word_bytes():
    rng = np.random.default_rng(3)
    N, K, nb = 8, 64, 2
    B = _signs(rng, (N, 1, K, nb))
    Wp, _ = orc.rowwise_to_kernel_layout(B, np.ones((N, 1, nb), dtype=np.float32))
    assert Wp.shape == (K // 32, nb, N)
    idx = orc.table_indices_c(Wp)
    assert idx.shape == (K // 8, nb, N)
    # independent derivation straight from the signs: bit i of the index is
    # (B[n, 8c+i, b] == +1), LSB = lowest input  (mv_fp16_bias.hpp:19-26,87-90)
    Bf = B.reshape(N, K, nb)
    for c in range(K // 8):
        for b in range(nb):
            for n in range(N):
                want = sum(int(Bf[n, 8 * c + i, b] == 1) << i for i in range(8))
                assert idx[c, b, n] == want
    # and byte j of the little-endian word is chunk 4w + j
    as_bytes = np.ascontiguousarray(Wp).view(np.uint8).reshape(K // 32, nb, N, 4)
    assert np.array_equal(as_bytes.transpose(0, 3, 1, 2).reshape(K // 8, nb, N), idx)


def test_lut_identities():
    rng = np.random.default_rng(11)
    x = rng.standard_normal(8).astype(np.float16)
    lut = orc.build_lut_c(x)
    xf = x.astype(np.float64)
    assert lut[255] == pytest.approx(xf.sum(), abs=0)            # all bits set -> +sum
    assert lut[0] == pytest.approx(-xf.sum(), abs=0)
    for i in (1, 2, 77, 128, 200):
        want = sum((1 if (i >> j) & 1 else -1) * xf[j] for j in range(8))
        assert lut[i] == pytest.approx(want, abs=1e-12)
        assert lut[255 - i] == pytest.approx(-lut[i], abs=1e-12)  # complement = negation
    # single-bit entries isolate one input: lut[1<<j] - lut[0] = 2 x[j]
    for j in range(8):
        assert lut[1 << j] - lut[0] == pytest.approx(2 * xf[j], abs=1e-12)


# ---- fp16 conversion helpers of the C file against numpy ---------------------

def test_half_conversions_match_numpy_exhaustively():
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16).astype(np.float32)
    for b in list(range(0, 65536, 97)) + [0, 1, 0x3ff, 0x400, 0x7bff, 0x7c00, 0x8000, 0x8001, 0xfbff, 0xfc00]:
        f = orc.half_to_float_c(b)
        if np.isnan(vals[b]):
            assert np.isnan(f)
        else:
            assert f == vals[b]
    rng = np.random.default_rng(5)
    samples = np.concatenate([
        rng.standard_normal(2000).astype(np.float32) * 10,
        (rng.standard_normal(500) * 1e-6).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, 2.0 ** -24, 2.0 ** -25,
                  1.5 * 2.0 ** -25, 2.0 ** -14, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11], dtype=np.float32)])
    for f in samples:
        want = np.float32(f).astype(np.float16).view(np.uint16)
        assert orc.float_to_half_c(float(f)) == int(want), f
