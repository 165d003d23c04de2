"""The reference module's test-data helpers (lut_gemm/lutgemm_cuda.cpp:104-223: makeRandom*
and parsing), rebuilt in the `lutgemm` module with the same signatures and in-place
contract: shapes, value ranges, packing consistency on the CPU; device-side generation and
a GEMV on what they produce on the GPU.  The BCQ quantiser restatement is also run on the
GPU against the fixture written from the reference's own quantiser."""
import os

import numpy as np
import pytest
import torch

import oracle as orc
from shiftaddllm_amd import native, workload
from shiftaddllm_amd.lut_gemm.kernel import pack_binaryWeight


@pytest.fixture(scope="module")
def ext():
    return native.lutgemm


def test_module_exports_the_reference_helper_names(ext):
    for name in ("makeRandomInput", "makeRandomAlpha", "makeRandomBias", "makeRandomScale",
                 "makeRandomWeight_int3", "makeRandomWeight", "parsing"):       # lutgemm_cuda.cpp:231-237
        assert callable(getattr(ext, name)), name


def _check_fills(ext, dev):
    K, nb, N, G = 256, 3, 64, 2
    torch.manual_seed(0)
    # makeRandomWeight: qW [K, nb, N] of +-1 and bW [K/32, nb, N], bit t of word w <=> qW[32w + t] = +1
    qW = torch.zeros((K, nb, N), device=dev)
    bW = torch.zeros((K // 32, nb, N), dtype=torch.int32, device=dev)
    ext.makeRandomWeight(qW, bW, N, nb, K)
    assert set(qW.unique().tolist()) == {-1.0, 1.0}
    assert 0.4 < (qW > 0).float().mean().item() < 0.6
    repacked = pack_binaryWeight(qW.cpu().permute(2, 0, 1).reshape(N, 1, K, nb)).permute(1, 2, 0)
    assert torch.equal(repacked, bW.cpu())
    assert np.array_equal(orc.pack_binary_weight_c(qW.cpu().permute(2, 0, 1).reshape(N, 1, K, nb).numpy()),
                          bW.cpu().permute(2, 0, 1).contiguous().numpy())
    # makeRandomInput: only [:M, :K] is written, values in (-1, 1), both signs
    inp = torch.full((3, K + 8), 7.0, dtype=torch.float16, device=dev)
    ext.makeRandomInput(inp, 2, K)
    assert inp[:2, :K].abs().max().item() <= 1.0 and (inp[:2, :K] < 0).any() and (inp[:2, :K] > 0).any()
    assert (inp[2] == 7).all() and (inp[:, K:] == 7).all()
    # E|u1 u2| = 1/4 for the product of two uniforms
    big = torch.zeros((64, 1024), device=dev)
    ext.makeRandomInput(big, 64, 1024)
    assert abs(big.abs().mean().item() - 0.25) < 0.01
    # makeRandomAlpha: alpha[g][b][n] in (-1, 1) / 2^b, q_bias in (-1, 1) / 2^nb
    alpha = torch.zeros((G, nb, N), dtype=torch.float16, device=dev)
    qb = torch.zeros((G, N), dtype=torch.float16, device=dev)
    ext.makeRandomAlpha(alpha, qb, G, nb, N)
    for b in range(nb):
        assert 0 < alpha[:, b].abs().max().item() <= 1.0 / (1 << b)
    assert 0 < qb.abs().max().item() <= 1.0 / (1 << nb)
    scale = torch.zeros(N, device=dev)
    bias = torch.zeros(N, device=dev)
    ext.makeRandomScale(scale, N)
    ext.makeRandomBias(bias, N)
    assert scale.abs().max() <= 1 and bias.abs().max() <= 1 and scale.abs().sum() > 0 and bias.abs().sum() > 0
    w3 = torch.full((5, 9), -1, dtype=torch.int32, device=dev)
    ext.makeRandomWeight_int3(w3, 8, 4)
    assert (w3[:4, :8] >= 0).all() and (w3[4] == -1).all() and (w3[:, 8] == -1).all()
    return qW, bW, alpha, qb


def test_helpers_fill_host_tensors(ext):
    _check_fills(ext, torch.device("cpu"))
    with pytest.raises(RuntimeError):
        ext.makeRandomInput(torch.zeros((2, 8)), 3, 8)                 # more rows than the tensor has
    with pytest.raises(RuntimeError):
        ext.makeRandomWeight(torch.zeros((32, 1, 4)), torch.zeros((1, 1, 4)), 4, 1, 32)     # bW not int32


@pytest.mark.gpu
def test_helpers_generate_on_the_device_and_feed_the_kernels(ext, gpu_device):
    """What the reference's own test flow does with these helpers: random weights, alphas and
    q_bias on the host, parsing() to flat device buffers, one uniform-mode GEMV on them."""
    _check_fills(ext, gpu_device)
    K, nb, N, G = 512, 3, 256, 4
    torch.manual_seed(1)
    qW = torch.zeros((K, nb, N))
    bW = torch.zeros((K // 32, nb, N), dtype=torch.int32)
    alpha3 = torch.zeros((G, nb, N))
    qb = torch.zeros((G, N))
    x = torch.zeros((1, K), dtype=torch.float16)
    ext.makeRandomWeight(qW, bW, N, nb, K)
    ext.makeRandomAlpha(alpha3, qb, G, nb, N)
    ext.makeRandomInput(x, 1, K)
    # uniform mode reads one alpha per (group, output): plane 0 of the generated alphas
    alpha = alpha3[:, 0, :].contiguous()
    d_bW, d_qb, d_alpha = ext.parsing(bW, alpha, N, K, 1, True, G, qb, gpu_device.index or 0)
    assert d_bW.is_cuda and d_bW.dtype == torch.int32 and d_bW.numel() == K * N * 1 // 32
    assert d_qb.dtype == torch.float16 and d_qb.numel() == G * N
    assert d_alpha.dtype == torch.float16 and d_alpha.numel() == G * N
    assert torch.equal(d_alpha.cpu(), alpha.reshape(-1).half())
    # the flat word buffer is the first plane-count's worth of bW: use the full tensor for the GEMV
    out = torch.zeros((1, N), dtype=torch.float16, device=gpu_device)
    ext.lutgemm_compute(out, bW.to(gpu_device), d_alpha.view(G, N), d_qb.view(G, N), x.to(gpu_device), N, K, nb, G)
    torch.cuda.synchronize()
    want, _ = orc.gemv_uniform_c(bW.numpy(), alpha.half().numpy(), qb.half().numpy(), x.numpy(), G)
    rel, mad = orc.error_metrics(out.float().cpu().numpy(), want.astype(np.float32))
    assert rel <= 2e-4 and mad <= 1e-3, (rel, mad)


@pytest.mark.gpu
def test_bcq_quantiser_on_the_device_matches_the_reference_fixture(gpu_device):
    """workload.bcq_shift_quantize run on the GPU against (B, alpha) written by the reference's
    own greedy + refinement code on the CPU (tests/golden/bcq_shift_reference.npz), bit for bit.
    (The GPU's fp32 row sums differ from the CPU's in the last bit, which the power-of-two
    rounding absorbs; what does matter is the order of equal code values in the sort of
    assign_signs, hence its stable=True.)"""
    d = np.load(os.path.join(os.path.dirname(__file__), "golden", "bcq_shift_reference.npz"))
    for c in range(int(d["cases"])):
        w, nb = torch.from_numpy(d[f"w{c}"]).to(gpu_device), int(d[f"nb{c}"])
        B, alpha = workload.bcq_shift_quantize(w, nb, rounds=5)
        assert B.is_cuda and alpha.is_cuda
        a_ok = np.array_equal(alpha.cpu().numpy(), d[f"alpha{c}"])
        b_ok = np.array_equal(B.cpu().numpy(), d[f"B{c}"])
        assert a_ok and b_ok, (f"case {c}: alpha equal={a_ok}, B equal={b_ok}, "
                              f"B mismatches={int((B.cpu().numpy() != d[f'B{c}']).sum())} of {B.numel()}")
