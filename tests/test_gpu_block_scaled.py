"""The block-scaled matrix-core path (lutgemm_gemv_rowwise_pow2_f16) on the GPU, through the C ABI:
power-of-two alphas as the matrix instruction's block scales, sign bits as 4-bit floats, activations
split into three 8-bit floats.  Against the CPU oracle, and against the fp16 matrix-core kernel that
lutgemm_gemv_rowwise_f16 takes for the same call."""
import ctypes

import numpy as np
import pytest
import torch

import oracle as orc
from shiftaddllm_amd import native

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _block_scaled_wherever_it_applies():
    """By default the entry point takes the block-scaled kernel only where it is the faster one (few
    rows, large matrices); these tests want it for every shape it can run."""
    lib = native.cabi()
    which = native.OPTIONS["BLOCK_SCALED"]
    lib.lutgemm_set_option(which, 2)
    yield
    lib.lutgemm_set_option(which, -1)
    lib.lutgemm_set_option(native.OPTIONS["POW2_CONVERT"], -1)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _sp():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _problem(N, K, nb, M, seed, group=128, spread=1.0):
    g = torch.Generator().manual_seed(seed)
    bW = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 32, nb, N), generator=g, dtype=torch.int32)
    e = torch.randint(-12, -4, (K // group, 1, N), generator=g).float() - torch.arange(nb).float().view(1, nb, 1)
    alpha = torch.exp2(e).to(torch.float16).contiguous()
    x = torch.randn((M, K), generator=g)
    if spread != 1.0:                       # a wide range of magnitudes inside the blocks of 32
        x = x * torch.exp2(torch.randint(-10, 4, (M, K), generator=g).float() * spread)
    bias = (torch.randn((M, N), generator=g) * 0.1).half()
    return bW, alpha, x.half(), bias


def _run(fn, dev, bW, alpha, x, bias, group=128):
    N, K, nb, M = bW.shape[2], bW.shape[0] * 32, bW.shape[1], x.shape[0]
    d = [t.to(dev) for t in (bW, alpha, x)]
    out = bias.clone().to(dev)
    rc = fn(_ptr(d[0]), _ptr(d[1]), _ptr(d[2]), _ptr(out), N, K, nb, K // group, M, _sp())
    assert rc == 0, native.cabi().lutgemm_strerror(rc).decode()
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("N,K,nb,M,group", [
    (256, 256, 1, 3, 128), (1024, 1024, 2, 4, 128), (4096, 4096, 3, 16, 128), (2048, 1024, 4, 17, 128),
    (528, 512, 3, 5, 256), (1040, 2048, 4, 33, 512), (11008, 4096, 3, 8, 128), (4096, 11008, 2, 32, 128),
    (64, 128, 4, 16, 128), (16, 1024, 2, 7, 128)])
def test_block_scaled_path_against_the_oracle(gpu_device, N, K, nb, M, group):
    lib = native.cabi()
    print(f"block-scaled N={N} K={K} nb={nb} M={M} group={group}", flush=True)
    bW, alpha, x, bias = _problem(N, K, nb, M, seed=N + K + nb + M, group=group)
    want, _ = orc.gemv_rowwise_c(bW.numpy(), alpha.numpy(), x.numpy(), K // group, out=bias.numpy())
    got = _run(lib.lutgemm_gemv_rowwise_pow2_f16, gpu_device, bW, alpha, x, bias, group)
    rel, mad = orc.error_metrics(got.float().cpu().numpy(), want.astype(np.float32))
    assert rel <= 2e-4 and mad <= 1e-3, (rel, mad)
    # the fp16 matrix-core kernel rounds the same exact sums: the two agree to an fp16 rounding
    other = _run(lib.lutgemm_gemv_rowwise_f16, gpu_device, bW, alpha, x, bias, group)
    assert torch.allclose(got.float(), other.float(), rtol=2e-3, atol=2e-3 * float(other.float().abs().max()))


def test_activations_of_mixed_magnitude_and_special_values(gpu_device):
    """Values of very different size inside one block of 32 (the split keeps everything within 2^14 of
    the block's largest value exactly), zeros, a block of zeros, and non-finite inputs."""
    lib = native.cabi()
    N, K, nb, M = 512, 1024, 3, 6
    bW, alpha, x, bias = _problem(N, K, nb, M, seed=5, spread=1.0)
    g = torch.Generator().manual_seed(9)
    x = (torch.randn((M, K), generator=g) * torch.exp2(torch.randint(-12, 3, (M, K), generator=g).float())).half()
    x[0, :64] = 0                          # two blocks of zeros
    x[1, 5] = 60000.0                      # near the top of fp16
    x[2, 7] = 6e-8                         # an fp16 subnormal beside ordinary values
    want, _ = orc.gemv_rowwise_c(bW.numpy(), alpha.numpy(), x.numpy(), K // 128, out=bias.numpy())
    got = _run(lib.lutgemm_gemv_rowwise_pow2_f16, gpu_device, bW, alpha, x, bias)
    finite = np.isfinite(want.astype(np.float32)).all(axis=1)
    rel, mad = orc.error_metrics(got.float().cpu().numpy()[finite], want.astype(np.float32)[finite])
    assert rel <= 2e-4 and mad <= 1e-3, (rel, mad)
    # non-finite activations poison their row, and only their row
    x2 = x.clone()
    x2[3, 100] = float("inf")
    x2[4, 900] = float("nan")
    got2 = _run(lib.lutgemm_gemv_rowwise_pow2_f16, gpu_device, bW, alpha, x2, bias).float().cpu()
    assert torch.isnan(got2[3]).all() and torch.isnan(got2[4]).all()
    assert torch.equal(got2[[0, 1, 2, 5]], got.float().cpu()[[0, 1, 2, 5]])


def test_pow2_entry_point_falls_back_where_the_block_scaled_kernel_does_not_apply(gpu_device):
    """One or two rows, K not a multiple of 128, groups of 32: the call runs as lutgemm_gemv_rowwise_f16
    does and gives its bits; with the option off likewise."""
    lib = native.cabi()
    for (N, K, nb, M, group) in [(1024, 1024, 3, 1, 128), (1024, 1024, 3, 2, 128), (512, 96, 2, 8, 32), (512, 2048, 2, 4, 32)]:
        bW, alpha, x, bias = _problem(N, K, nb, M, seed=N + M, group=group)
        a = _run(lib.lutgemm_gemv_rowwise_pow2_f16, gpu_device, bW, alpha, x, bias, group)
        b = _run(lib.lutgemm_gemv_rowwise_f16, gpu_device, bW, alpha, x, bias, group)
        assert torch.equal(a, b), (N, K, nb, M, group)
    which = native.OPTIONS["BLOCK_SCALED"]
    lib.lutgemm_set_option(which, 0)
    lib.lutgemm_set_option(native.OPTIONS["POW2_CONVERT"], 0)
    try:
        bW, alpha, x, bias = _problem(2048, 1024, 3, 8, seed=3)
        a = _run(lib.lutgemm_gemv_rowwise_pow2_f16, gpu_device, bW, alpha, x, bias)
        b = _run(lib.lutgemm_gemv_rowwise_f16, gpu_device, bW, alpha, x, bias)
        assert torch.equal(a, b)
    finally:
        lib.lutgemm_set_option(which, 2)
        lib.lutgemm_set_option(native.OPTIONS["POW2_CONVERT"], -1)


def test_default_rule_takes_the_block_scaled_kernel_for_few_rows_of_a_large_matrix(gpu_device):
    """Option value 1 (the default): 4 rows of an 8192 x 16384 x 3-bit matrix (48 MB of sign words) run
    block-scaled, 16 rows do not; the result is the oracle's either way."""
    lib = native.cabi()
    which = native.OPTIONS["BLOCK_SCALED"]
    lib.lutgemm_set_option(which, 1)
    N, K, nb = 8192, 16384, 3
    for M, kernel in ((4, 2), (16, 1)):
        plan = native.Plan()
        assert lib.lutgemm_describe_pow2_plan(N, K, nb, K // 128, M, ctypes.byref(plan)) == 0
        assert plan.kernel == kernel
        bW, alpha, x, bias = _problem(N, K, nb, M, seed=M)
        want, _ = orc.gemv_rowwise_c(bW.numpy(), alpha.numpy(), x.numpy(), K // 128, out=bias.numpy())
        got = _run(lib.lutgemm_gemv_rowwise_pow2_f16, gpu_device, bW, alpha, x, bias)
        rel, mad = orc.error_metrics(got.float().cpu().numpy(), want.astype(np.float32))
        assert rel <= 2e-4 and mad <= 1e-3, (M, rel, mad)


def test_lutlinear_takes_the_pow2_entry_for_a_few_rows(gpu_device):
    """LutLinear.forward looks at its alphas once: powers of two and 3 to 8 rows go through
    lutgemm_compute_shift_scale_pow2 (here, with the option at 2, onto the block-scaled kernel);
    an alpha that is no power of two, or other row counts, keep the ordinary entry."""
    from shiftaddllm_amd.lut_gemm.quant import LutLinear
    N, K, nb = 512, 1024, 3
    bW, alpha, x, _ = _problem(N, K, nb, 8, seed=5)
    lin = LutLinear(K, N, group_size=128, wbit=nb, bias=None, alpha_format="rowwise_fp16").to(gpu_device)
    lin.binaryWeight.data = bW.to(gpu_device)
    lin.alpha.data = alpha.to(gpu_device)
    lib = native.cabi()
    for M in (1, 4, 8):
        xm = x[:M].contiguous()
        want, _ = orc.gemv_rowwise_c(bW.numpy(), alpha.numpy(), xm.numpy(), K // 128)
        got = lin(xm.to(gpu_device))
        assert lin._alphas_are_powers_of_two()
        rel, mad = orc.error_metrics(got.float().cpu().numpy(), want.astype(np.float32))
        assert rel <= 2e-4 and mad <= 1e-3, (M, rel, mad)
        direct = _run(lib.lutgemm_gemv_rowwise_pow2_f16, gpu_device, bW, alpha, xm, torch.zeros((M, N)).half())
        assert torch.equal(got, direct)
    # one alpha with a mantissa bit: the module notices (the tensor's version changed) and keeps the fp16 entry
    lin.alpha.data[0, 0, 0] = 0.75 * lin.alpha.data[0, 0, 0]
    lin.alpha.data = lin.alpha.data.clone()
    assert not lin._alphas_are_powers_of_two()
    a2 = lin.alpha.data.cpu()
    xm = x[:4].contiguous()
    want, _ = orc.gemv_rowwise_c(bW.numpy(), a2.numpy(), xm.numpy(), K // 128)
    got = lin(xm.to(gpu_device))
    rel, mad = orc.error_metrics(got.float().cpu().numpy(), want.astype(np.float32))
    assert rel <= 2e-4 and mad <= 1e-3, (rel, mad)
    assert torch.equal(got, _run(lib.lutgemm_gemv_rowwise_f16, gpu_device, bW, a2, xm, torch.zeros((4, N)).half()))


@pytest.mark.parametrize("N,K,nb,M,group", [
    (256, 256, 1, 3, 128), (1024, 1024, 2, 4, 128), (4096, 4096, 3, 16, 128), (2048, 1024, 4, 17, 128),
    (528, 512, 3, 5, 256), (1040, 2048, 4, 33, 512), (11008, 4096, 3, 8, 128), (4096, 11008, 2, 32, 128),
    (64, 128, 4, 16, 128), (16, 1024, 2, 7, 128), (8192, 8192, 4, 16, 128)])
def test_fp16_matrix_core_kernel_with_converted_sign_operands(gpu_device, N, K, nb, M, group):
    """With the block-scaled kernel switched off, a pow2 call takes the fp16 matrix-core kernel whose sign
    operands come from the LDS table and the scaled fp4 -> fp16 conversion (option POW2_CONVERT, default
    1 = where it is faster, 2 = always): the same exact products as the shift-and-bit-operation form,
    summed in another order, so the two agree to a rounding of the fp32 sums; and the oracle's result.
    With the option at 0 the call is lutgemm_gemv_rowwise_f16 bit for bit."""
    lib = native.cabi()
    lib.lutgemm_set_option(native.OPTIONS["BLOCK_SCALED"], 0)
    lib.lutgemm_set_option(native.OPTIONS["POW2_CONVERT"], 2)
    print(f"converted signs N={N} K={K} nb={nb} M={M} group={group}", flush=True)
    bW, alpha, x, bias = _problem(N, K, nb, M, seed=N + K + nb + M, group=group)
    want, _ = orc.gemv_rowwise_c(bW.numpy(), alpha.numpy(), x.numpy(), K // group, out=bias.numpy())
    got = _run(lib.lutgemm_gemv_rowwise_pow2_f16, gpu_device, bW, alpha, x, bias, group)
    rel, mad = orc.error_metrics(got.float().cpu().numpy(), want.astype(np.float32))
    assert rel <= 2e-4 and mad <= 1e-3, (rel, mad)
    other = _run(lib.lutgemm_gemv_rowwise_f16, gpu_device, bW, alpha, x, bias, group)
    assert torch.allclose(got.float(), other.float(), rtol=2e-3, atol=2e-3 * float(other.float().abs().max()))
    which = native.OPTIONS["POW2_CONVERT"]
    lib.lutgemm_set_option(which, 0)
    try:
        assert torch.equal(_run(lib.lutgemm_gemv_rowwise_pow2_f16, gpu_device, bW, alpha, x, bias, group), other)
    finally:
        lib.lutgemm_set_option(which, -1)


@pytest.mark.parametrize("block_scaled,convert", [(2, 0), (0, 2), (1, 1)])
def test_random_shapes_of_the_pow2_entry_against_a_dense_product(gpu_device, block_scaled, convert):
    """90 seeded random problems per setting (K % 128, N % 16, group sizes from 128 up, 1-4 bit planes,
    3-40 rows, power-of-two alphas over nine binades, activations of mixed magnitude, a bias in `out`)
    through lutgemm_gemv_rowwise_pow2_f16 with the block-scaled kernel forced, with the converted
    sign operands forced, and under the default rules, against the dense fp64 product of the
    dequantised matrix formed on the GPU by framework operations."""
    import random
    dev = gpu_device
    lib = native.cabi()
    lib.lutgemm_set_option(native.OPTIONS["BLOCK_SCALED"], block_scaled)
    lib.lutgemm_set_option(native.OPTIONS["POW2_CONVERT"], convert)
    rng = random.Random(77 + 10 * block_scaled + convert)
    plan = native.Plan()
    kernels = set()
    for case in range(90):
        K = 128 * rng.randint(1, 72)
        N = 16 * rng.randint(1, 520)
        gs = rng.choice([g for g in (128, 256, 512, 1024, K) if K % g == 0])
        nb = rng.randint(1, 4)
        M = rng.choice((3, 4, 5, 6, 8, 9, 13, 16, 17, 24, 32, 33, 40))
        g = torch.Generator(device=dev).manual_seed(1000 + case)
        bW = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 32, nb, N), generator=g, device=dev, dtype=torch.int32)
        e = torch.randint(-13, -4, (K // gs, nb, N), generator=g, device=dev).float()
        alpha = torch.exp2(e).half()
        x = torch.randn((M, K), generator=g, device=dev)
        if case % 3 == 0:
            x = x * torch.exp2(torch.randint(-8, 3, (M, K), generator=g, device=dev).float())
        x = x.half()
        bias = torch.randn((M, N), generator=g, device=dev).half()
        out = bias.clone()
        rc = lib.lutgemm_gemv_rowwise_pow2_f16(_ptr(bW), _ptr(alpha), _ptr(x), _ptr(out), N, K, nb, K // gs, M, _sp())
        assert rc == 0, lib.lutgemm_strerror(rc).decode()
        torch.cuda.synchronize()
        signs = ((bW.unsqueeze(1) >> torch.arange(32, device=dev).view(1, 32, 1, 1)) & 1).double() * 2 - 1
        Wq = (signs.reshape(K, nb, N) * alpha.double().repeat_interleave(gs, dim=0)).sum(1)      # [K][N]
        want = bias.double() + x.double() @ Wq
        rel = ((out.double() - want).norm() / want.norm()).item()
        mad = ((out.double() - want).abs().max() / want.abs().max()).item()
        assert lib.lutgemm_describe_pow2_plan(N, K, nb, K // gs, M, ctypes.byref(plan)) == 0
        kernels.add(plan.kernel)
        assert rel <= 5e-4 and mad <= 2.5e-3, (N, K, nb, gs, M, rel, mad)
    assert kernels == ({2} if block_scaled == 2 else {1}), kernels
