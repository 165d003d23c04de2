"""Committed golden fixtures (tests/golden/lutgemm_cases.npz, written by
tests/golden/make_fixtures.py): the oracle and the host-side packers must keep
reproducing them bit for bit (CPU), and the HIP kernels must match them (GPU)."""
import ctypes
import os

import numpy as np
import pytest
import torch

import oracle as orc

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "lutgemm_cases.npz")


@pytest.fixture(scope="module")
def fx():
    return dict(np.load(FIX))


def test_oracle_reproduces_fixtures(fx):
    assert np.array_equal(orc.pack_binary_weight_c(fx["row_B"]), fx["row_packed"])
    assert np.array_equal(np.ascontiguousarray(fx["row_packed"].transpose(1, 2, 0)), fx["row_bW"])
    y16, y32 = orc.gemv_rowwise_c(fx["row_bW"], fx["row_alpha"], fx["row_x"], 4, out=fx["row_bias"])
    assert np.array_equal(y16.view(np.uint16), fx["row_out"].view(np.uint16))
    assert np.array_equal(y32, fx["row_y32"])
    y16, _ = orc.gemv_block_c(fx["blk_bW"], fx["blk_alpha"], fx["blk_x"], 8, kind=orc.ALPHA_F16)
    assert np.array_equal(y16.view(np.uint16), fx["blk_out"].view(np.uint16))
    y16, _ = orc.gemv_block_c(fx["blk_bW"], fx["blk_apot"], fx["blk_x"], 8, kind=orc.ALPHA_APOT_I8)
    assert np.array_equal(y16.view(np.uint16), fx["blk_apot_out"].view(np.uint16))
    # power-of-two block alphas: the int8 exponent form is exact, same output
    assert np.array_equal(fx["blk_apot_out"].view(np.uint16), fx["blk_out"].view(np.uint16))
    y16, _ = orc.gemv_block_c(fx["misc_bW"], fx["u16_alpha"], fx["misc_xs"], 4, kind=orc.ALPHA_SHIFT_U16)
    assert np.array_equal(y16.view(np.uint16), fx["u16_out"].view(np.uint16))
    y16, _ = orc.gemv_uniform_c(fx["misc_bW"], fx["uni_alpha"], fx["uni_qbias"], fx["misc_x"], 4)
    assert np.array_equal(y16.view(np.uint16), fx["uni_out"].view(np.uint16))


def test_host_packers_reproduce_fixtures(fx):
    from shiftaddllm_amd.lut_gemm import kernel as K_
    from shiftaddllm_amd.lut_gemm.quant import encode_apot_int8
    assert np.array_equal(K_.pack_binaryWeight(torch.from_numpy(fx["row_B"])).numpy(), fx["row_packed"])
    bW, a = K_.convert_weight(torch.from_numpy(fx["blk_disk_bW"]), torch.from_numpy(fx["blk_disk_alpha"]))
    assert np.array_equal(bW.numpy(), fx["blk_bW"]) and np.array_equal(a.half().numpy(), fx["blk_alpha"])
    assert np.array_equal(encode_apot_int8(torch.from_numpy(fx["blk_alpha"]).float()).numpy(), fx["blk_apot"])
    # dense dequantisation of the on-disk tensors, then matmul, gives the fixture's fp32 result
    W = K_.dequantize_lat(torch.from_numpy(fx["blk_disk_bW"]), torch.from_numpy(fx["blk_disk_alpha"]))
    y = torch.from_numpy(fx["blk_x"]).double() @ W.double().t()
    np.testing.assert_allclose(y.numpy(), fx["blk_y32"], rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
def test_kernels_match_fixtures(fx, gpu_device):
    from shiftaddllm_amd import native
    lib = native.cabi()
    dev = gpu_device
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    p = lambda x: ctypes.c_void_p(x.data_ptr())
    sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def close(got, want):
        rel, mad = orc.error_metrics(got.float().cpu().numpy(), want.astype(np.float32))
        assert rel <= 2e-4 and mad <= 1e-3, (rel, mad)

    bW, al, x, out = t(fx["row_bW"]), t(fx["row_alpha"]), t(fx["row_x"]), t(fx["row_bias"])
    assert lib.lutgemm_gemv_rowwise_f16(p(bW), p(al), p(x), p(out), 96, 512, 3, 4, 2, sp) == 0
    torch.cuda.synchronize()
    close(out, fx["row_out"])

    bW, x = t(fx["blk_bW"]), t(fx["blk_x"])
    for alpha, fn, extra, want in ((fx["blk_alpha"], lib.lutgemm_gemv_block_f16, (), fx["blk_out"]),
                                   (fx["blk_apot"], lib.lutgemm_gemv_block_apot_i8, (3,), fx["blk_apot_out"])):
        al, out = t(alpha), torch.zeros((1, 64), dtype=torch.float16, device=dev)
        assert fn(p(bW), p(al), p(x), p(out), 64, 288, 2, 8, *extra, 1, sp) == 0
        torch.cuda.synchronize()
        close(out, want)

    bW = t(fx["misc_bW"])
    al, x, out = t(fx["u16_alpha"]), t(fx["misc_xs"]), torch.zeros((1, 64), dtype=torch.float16, device=dev)
    assert lib.lutgemm_gemv_block_shift_u16(p(bW), p(al), p(x), p(out), 64, 256, 3, 4, 3, 1, sp) == 0
    torch.cuda.synchronize()
    close(out, fx["u16_out"])
    al, q, x = t(fx["uni_alpha"]), t(fx["uni_qbias"]), t(fx["misc_x"])
    out = torch.zeros((1, 64), dtype=torch.float16, device=dev)
    assert lib.lutgemm_gemv_uniform_f16(p(bW), p(al), p(q), p(x), p(out), 64, 256, 3, 4, 1, sp) == 0
    torch.cuda.synchronize()
    close(out, fx["uni_out"])


def test_bcq_quantiser_reproduces_reference_output():
    """workload.bcq_shift_quantize against (B, alpha) written by the reference's own
    quantize_shift body (greedy + 5 refinement rounds, BST assignment, one power-of-two
    term) -- tests/golden/make_bcq_fixture.py made the file from the reference checkout."""
    import os
    import numpy as np
    import torch
    from shiftaddllm_amd import workload
    d = np.load(os.path.join(os.path.dirname(__file__), "golden", "bcq_shift_reference.npz"))
    assert int(d["cases"]) == 4
    for c in range(int(d["cases"])):
        w, nb = torch.from_numpy(d[f"w{c}"]), int(d[f"nb{c}"])
        B, alpha = workload.bcq_shift_quantize(w, nb, rounds=5)
        assert np.array_equal(alpha.numpy(), d[f"alpha{c}"]), c
        assert np.array_equal(B.numpy(), d[f"B{c}"]), c
        # what the fixture itself must satisfy: +-1 signs, descending power-of-two scales
        assert set(np.unique(d[f"B{c}"])) <= {-1, 1}
        e = np.log2(d[f"alpha{c}"])
        assert np.array_equal(e, np.round(e)) and np.all(np.diff(d[f"alpha{c}"], axis=1) <= 0)
