"""Pins the oracle's GEMV restatements (CPU only).

The C table-lookup emulation of each kernel variant is checked against:
  * the dense path (dequantise with the numpy closed form, then a double
    matmul) -- a different decomposition of the same sum, so a wrong byte
    order, group index, transposed alpha or dropped bit plane shows up;
  * special cases with a textbook answer: x = e_k returns column k of W_q,
    alpha = 1 with one bit plane returns B x, x = 0 leaves the bias;
  * hand-computed tiny cases for the alpha decoders.
"""
import numpy as np
import pytest

import oracle as orc


def _signs(rng, shape):
    return (rng.integers(0, 2, size=shape, dtype=np.int8) * 2 - 1).astype(np.int8)


def _rowwise(rng, N, K, nb, gs, pow2=True):
    B = _signs(rng, (N, K // gs, gs, nb))
    if pow2:
        alpha = np.exp2(rng.integers(-8, -3, size=(N, K // gs, nb))).astype(np.float32)
    else:
        alpha = np.abs(rng.standard_normal((N, K // gs, nb))).astype(np.float32)
    Wp, a16 = orc.rowwise_to_kernel_layout(B, alpha)
    return B, alpha, Wp, a16


@pytest.mark.parametrize("N,K,nb,gs,M", [(8, 64, 1, 32, 1), (12, 256, 3, 128, 1), (16, 384, 4, 64, 3),
                                          (4, 96, 2, 96, 2)])
def test_rowwise_lut_emulation_equals_dense(N, K, nb, gs, M):
    rng = np.random.default_rng(N * K + nb)
    B, alpha, Wp, a16 = _rowwise(rng, N, K, nb, gs, pow2=False)
    x = rng.standard_normal((M, K)).astype(np.float16)
    Wq = orc.dequant_rowwise_kernel_layout(Wp, a16)           # uses the fp16-rounded alphas
    y_dense = orc.dense_gemv_np(Wq, x)
    _, y_lut = orc.gemv_rowwise_c(Wp, a16, x, K // gs)
    np.testing.assert_allclose(y_lut, y_dense, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(orc.dense_gemv_c(Wq, x), y_dense, rtol=1e-6, atol=1e-6)
    # and W_q itself equals the einsum over the original signs
    a_r = a16.astype(np.float32).transpose(2, 0, 1)
    Q = np.einsum("nijl,nil->nij", B.astype(np.float64), a_r.astype(np.float64)).reshape(N, K)
    np.testing.assert_allclose(Wq, Q, rtol=0, atol=1e-6)


def test_rowwise_unit_vector_returns_a_column():
    rng = np.random.default_rng(1)
    N, K, nb, gs = 8, 128, 3, 64
    _, _, Wp, a16 = _rowwise(rng, N, K, nb, gs)
    Wq = orc.dequant_rowwise_kernel_layout(Wp, a16)
    for k in (0, 7, 8, 31, 32, 63, 64, 127):
        x = np.zeros((1, K), dtype=np.float16)
        x[0, k] = 1.0
        _, y = orc.gemv_rowwise_c(Wp, a16, x, K // gs)
        np.testing.assert_allclose(y[0], Wq[:, k], rtol=0, atol=1e-7)


def test_rowwise_alpha_one_single_plane_is_sign_matvec():
    rng = np.random.default_rng(2)
    N, K = 8, 64
    B = _signs(rng, (N, 1, K, 1))
    Wp, a16 = orc.rowwise_to_kernel_layout(B, np.ones((N, 1, 1), dtype=np.float32))
    x = rng.integers(-3, 4, size=(1, K)).astype(np.float16)
    _, y = orc.gemv_rowwise_c(Wp, a16, x, 1)
    want = B.reshape(N, K).astype(np.int64) @ x[0].astype(np.int64)
    assert np.array_equal(y[0], want.astype(np.float32))        # small integers: exact


def test_accumulates_into_prefilled_output():
    rng = np.random.default_rng(3)
    N, K, nb, gs = 8, 64, 2, 32
    _, _, Wp, a16 = _rowwise(rng, N, K, nb, gs)
    bias = rng.standard_normal((1, N)).astype(np.float16)
    out0, _ = orc.gemv_rowwise_c(Wp, a16, np.zeros((1, K), dtype=np.float16), K // gs, out=bias)
    assert np.array_equal(out0, bias)                            # x = 0 -> bias untouched
    x = rng.standard_normal((1, K)).astype(np.float16)
    out1, y = orc.gemv_rowwise_c(Wp, a16, x, K // gs, out=bias)
    assert np.array_equal(out1, orc.accumulate_into_fp16(bias, y))
    assert not np.array_equal(out1, bias)


def _block(rng, N, K, nb, R):
    B = _signs(rng, (N, 1, K, nb))
    Wp = np.ascontiguousarray(orc.pack_binary_weight_np(B).transpose(1, 2, 0))
    return B.reshape(N, K, nb), Wp


@pytest.mark.parametrize("N,K,nb,R,M", [(16, 64, 2, 4, 1), (32, 96, 3, 8, 2), (8, 32, 1, 1, 1)])
def test_block_f16_equals_dense(N, K, nb, R, M):
    rng = np.random.default_rng(N + K + R)
    B, Wp = _block(rng, N, K, nb, R)
    a = np.abs(rng.standard_normal((K // 8, nb, R))).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    Wq = orc.dequant_block_kernel_layout(Wp, a.astype(np.float32))
    # brute force W_q from the definition
    rows = N // R
    for n in (0, N // 2, N - 1):
        for k in (0, 9, K - 1):
            want = sum(float(a[k // 8, b, n // rows]) * B[n, k, b] for b in range(nb))
            assert Wq[n, k] == pytest.approx(want, abs=1e-6)
    _, y = orc.gemv_block_c(Wp, a, x, R, kind=orc.ALPHA_F16)
    np.testing.assert_allclose(y, orc.dense_gemv_np(Wq, x), rtol=1e-5, atol=1e-5)


def test_shift_u16_decoder_known_answers():
    # fields f0 = u&7, f1 = (u>>3)&7, f2 = (u>>6)&7 ; multiplier 2^f0 + 2^f1 + 2^f2
    assert orc.shift_u16_to_alpha(np.array([0]))[0] == 3.0                 # 1 + 1 + 1
    assert orc.shift_u16_to_alpha(np.array([0b111_111_111]))[0] == 384.0   # 3 * 128
    assert orc.shift_u16_to_alpha(np.array([0b010_001_011]))[0] == 8 + 2 + 4
    assert orc.shift_u16_to_alpha(np.array([0xFE00]))[0] == 3.0            # bits above 9 ignored


def test_apot_i8_decoder_known_answers():
    assert orc.apot_i8_to_alpha(np.array([[0, 0, 0]], dtype=np.int8))[0] == 3.0
    assert orc.apot_i8_to_alpha(np.array([[-3, -128, -128]], dtype=np.int8))[0] == 0.125
    assert orc.apot_i8_to_alpha(np.array([[-1, -2, -128]], dtype=np.int8))[0] == 0.75
    assert orc.apot_i8_to_alpha(np.array([[2, -4, -6]], dtype=np.int8))[0] == 4 + 1 / 16 + 1 / 64
    assert orc.apot_i8_to_alpha(np.array([[-128, -128, -128]], dtype=np.int8))[0] == 0.0


@pytest.mark.parametrize("kind", ["u16", "i8"])
def test_block_shift_variants_equal_dense(kind):
    rng = np.random.default_rng(17)
    N, K, nb, R, M = 16, 64, 3, 4, 2
    _, Wp = _block(rng, N, K, nb, R)
    x = rng.standard_normal((M, K)).astype(np.float16)
    if kind == "u16":
        code = rng.integers(0, 512, size=(K // 8, nb, R)).astype(np.uint16)
        a_eff = orc.shift_u16_to_alpha(code)
        _, y = orc.gemv_block_c(Wp, code.view(np.int16), x, R, kind=orc.ALPHA_SHIFT_U16)
    else:
        code = rng.integers(-12, -2, size=(K // 8, nb, R, 3)).astype(np.int8)
        code[rng.random(code.shape) < 0.3] = -128
        a_eff = orc.apot_i8_to_alpha(code)
        _, y = orc.gemv_block_c(Wp, code, x, R, kind=orc.ALPHA_APOT_I8)
    Wq = orc.dequant_block_kernel_layout(Wp, a_eff)
    np.testing.assert_allclose(y, orc.dense_gemv_np(Wq, x), rtol=1e-5, atol=1e-5)


def test_uniform_mode_equals_its_formula():
    # out = sum_g ( q[g,n] * sum_{k in g} x_k + sum_b alpha[g,n] / 2^(b+1) * sum_k B x )
    rng = np.random.default_rng(23)
    N, K, nb, gs, M = 8, 128, 3, 64, 2
    B = _signs(rng, (N, K // gs, gs, nb))
    Wp = np.ascontiguousarray(orc.pack_binary_weight_np(B).transpose(1, 2, 0))
    alpha = np.abs(rng.standard_normal((K // gs, N))).astype(np.float16)
    q = rng.standard_normal((K // gs, N)).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    _, y = orc.gemv_uniform_c(Wp, alpha, q, x, K // gs)
    xf = x.astype(np.float64)
    Bf = B.reshape(N, K, nb).astype(np.float64)
    want = np.zeros((M, N))
    for g in range(K // gs):
        sl = slice(g * gs, (g + 1) * gs)
        want += xf[:, sl].sum(axis=1, keepdims=True) * q[g].astype(np.float64)[None, :]
        for b in range(nb):
            want += (xf[:, sl] @ Bf[:, sl, b].T) * (alpha[g].astype(np.float64) / 2 ** (b + 1))[None, :]
    np.testing.assert_allclose(y, want, rtol=1e-5, atol=1e-5)


def test_lat_disk_layout_conversion_and_dequant():
    # on disk: bWeight [K, N/32, nb] packed along N, alpha [K/8, R, nb]
    rng = np.random.default_rng(29)
    N, K, nb, R = 64, 96, 2, 4
    Bk = _signs(rng, (K, R, N // R, nb))
    disk_bW = orc.pack_binary_weight_np(Bk)
    assert disk_bW.shape == (K, N // 32, nb)
    disk_alpha = np.exp2(rng.integers(-8, -3, size=(K // 8, R, nb))).astype(np.float32)
    W_dense = orc.dequant_lat_disk(disk_bW, disk_alpha)             # [N, K]
    assert W_dense.shape == (N, K)
    # definition: W[n, k] = sum_b alpha[k//8, n//(N/R), b] * B[k, n, b]
    Bflat = Bk.reshape(K, N, nb)
    for n in (0, 17, N - 1):
        for k in (0, 8, 50, K - 1):
            want = sum(float(disk_alpha[k // 8, n // (N // R), b]) * Bflat[k, n, b] for b in range(nb))
            assert W_dense[n, k] == pytest.approx(want, abs=1e-7)
    Wp, a = orc.lat_disk_to_kernel_layout(disk_bW, disk_alpha)
    assert Wp.shape == (K // 32, nb, N) and a.shape == (K // 8, nb, R)
    np.testing.assert_array_equal(orc.dequant_block_kernel_layout(Wp, a), W_dense)
    x = rng.standard_normal((1, K)).astype(np.float16)
    _, y = orc.gemv_block_c(Wp, a.astype(np.float16), x, R)
    np.testing.assert_allclose(y, orc.dense_gemv_np(W_dense, x), rtol=1e-5, atol=1e-6)


def test_pow2_round_known_answers():
    a = np.array([1.0, 0.3, 0.75, 0.7, -0.02, 3.0, 2.9, 0.17677], dtype=np.float32)
    #            2^0  2^-2 (log2 .75=-.415 -> 0 -> 1) 2^-1 (-.51->-1)  -2^-6 (log2 .02=-5.64)  4 (1.58->2)  2 (1.536->2: 4)  2^-2 (-2.5000.. )
    got = orc.pow2_round_np(a)
    assert got[0] == 1.0 and got[1] == 0.25 and got[2] == 1.0 and got[3] == 0.5
    assert got[4] == -2.0 ** -6 and got[5] == 4.0 and got[6] == 4.0
    assert np.all(np.log2(np.abs(got)) == np.rint(np.log2(np.abs(got))))


def test_shape_errors():
    Wp = np.zeros((2, 1, 8), dtype=np.int32)
    with pytest.raises(ValueError):
        orc.gemv_rowwise_c(Wp, np.zeros((3, 1, 8), dtype=np.float16), np.zeros((1, 64), dtype=np.float16), 3)
    with pytest.raises(ValueError):
        orc.gemv_block_c(Wp, np.zeros((8, 1, 3), dtype=np.float16), np.zeros((1, 64), dtype=np.float16), 3)
    with pytest.raises(TypeError):
        orc.gemv_rowwise_c(Wp, np.zeros((2, 1, 8), dtype=np.float16), np.zeros((1, 64), dtype=np.float32), 2)
