"""Every tuning option of lutgemm_set_option selects code of its own (kernel instances, launch
plans); each setting is run here, in this process, on a row-wise, a two-row, a several-row and a
block-alpha problem against the CPU oracle."""
import ctypes

import numpy as np
import pytest
import torch

import oracle as orc
from shiftaddllm_amd import native

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _sp():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _rowwise_case(dev, N, K, nb, M, seed):
    g = torch.Generator().manual_seed(seed)
    bW = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 32, nb, N), generator=g, dtype=torch.int32)
    e = torch.randint(-9, -5, (K // 128, 1, N), generator=g).float() - torch.arange(nb).float().view(1, nb, 1)
    alpha = torch.exp2(e).to(torch.float16).contiguous()
    x = torch.randn((M, K), generator=g).half()
    bias = (torch.randn((M, N), generator=g) * 0.1).half()
    want, _ = orc.gemv_rowwise_c(bW.numpy(), alpha.numpy(), x.numpy(), K // 128, out=bias.numpy())
    return [t.to(dev) for t in (bW, alpha, x, bias)], want, (N, K, nb, M)


def _block_case(dev, N, K, nb, R, seed):
    g = torch.Generator().manual_seed(seed)
    bW = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 32, nb, N), generator=g, dtype=torch.int32)
    code = torch.randint(-12, -4, (K // 8, nb, R, 3), generator=g).to(torch.int8)
    code[..., 1:][torch.rand(code[..., 1:].shape, generator=g) < 0.5] = -128
    x = torch.randn((1, K), generator=g).half()
    want, _ = orc.gemv_block_c(bW.numpy(), code.numpy(), x.numpy(), R, kind=orc.ALPHA_APOT_I8)
    return [t.to(dev) for t in (bW, code, x)], want, (N, K, nb, R)


SETTINGS = [("PAIR_TABLES", 0), ("SINGLE_ITEM", 0), ("TARGET_BLOCKS", 512), ("TARGET_BLOCKS", 96), ("FIRST_SHARE", 50),
            ("FIRST_SHARE", 70), ("MFMA_MIN_M", 2), ("MFMA_MIN_M", 1000), ("MFMA_BLOCKS", 512)]


@pytest.fixture(scope="module")
def cases(gpu_device):
    dev = gpu_device
    row = [_rowwise_case(dev, 4096, 4096, 3, 1, 1),      # one item per range: the single-item instance
           _rowwise_case(dev, 3072, 768, 3, 1, 2),
           _rowwise_case(dev, 8192, 4096, 4, 2, 3),      # two rows, above 12 MB of signs: pair tables
           _rowwise_case(dev, 2048, 1024, 2, 2, 4),
           _rowwise_case(dev, 4096, 4096, 3, 4, 5),      # several rows: matrix cores unless switched off
           _rowwise_case(dev, 5120, 8192, 4, 1, 6)]      # 512 workgroups with unequal ranges
    blk = [_block_case(dev, 2048, 2048, 2, 8, 7), _block_case(dev, 1024, 512, 3, 16, 8)]
    return row, blk


@pytest.mark.parametrize("name,value", SETTINGS)
def test_every_option_setting_against_the_oracle(gpu_device, cases, name, value):
    lib = native.cabi()
    row, blk = cases
    which = native.OPTIONS[name]
    assert lib.lutgemm_set_option(which, value) == 0
    try:
        for (bW, alpha, x, bias), want, (N, K, nb, M) in row:
            print(f"option {name}={value}: row-wise N={N} K={K} nb={nb} M={M}", flush=True)
            out = bias.clone()
            rc = lib.lutgemm_gemv_rowwise_f16(_ptr(bW), _ptr(alpha), _ptr(x), _ptr(out), N, K, nb, K // 128, M, _sp())
            assert rc == 0, lib.lutgemm_strerror(rc).decode()
            torch.cuda.synchronize()
            rel, mad = orc.error_metrics(out.float().cpu().numpy(), want.astype(np.float32))
            assert rel <= 5e-4 and mad <= 2e-3, (name, value, N, K, nb, M, rel, mad)
        for (bW, code, x), want, (N, K, nb, R) in blk:
            print(f"option {name}={value}: block N={N} K={K} nb={nb} R={R}", flush=True)
            out = torch.zeros((1, N), dtype=torch.float16, device=gpu_device)
            rc = lib.lutgemm_gemv_block_apot_i8(_ptr(bW), _ptr(code), _ptr(x), _ptr(out), N, K, nb, R, 3, 1, _sp())
            assert rc == 0, lib.lutgemm_strerror(rc).decode()
            torch.cuda.synchronize()
            rel, mad = orc.error_metrics(out.float().cpu().numpy(), want.astype(np.float32))
            assert rel <= 2e-4 and mad <= 1e-3, (name, value, N, K, nb, R, rel, mad)
    finally:
        lib.lutgemm_set_option(which, -1)


def test_thirty_nine_contributions_per_output(gpu_device):
    """One item per workgroup on a tile whose K extent is 39 sets: every output's accumulator word
    takes 39 fixed-point contributions (the planner's limit is 40), all of one sign here so that the
    running sum is as large as the data allows."""
    lib = native.cabi()
    N, K, nb = 512, 39 * 256, 2
    g = torch.Generator().manual_seed(77)
    bW = torch.full((K // 32, nb, N), -1, dtype=torch.int32)              # every sign +1
    alpha = torch.full((K // 128, nb, N), 2.0 ** -6, dtype=torch.float16)
    x = (torch.randn((1, K), generator=g).abs() * 4).half()
    want, _ = orc.gemv_rowwise_c(bW.numpy(), alpha.numpy(), x.numpy(), K // 128)
    which = native.OPTIONS["TARGET_BLOCKS"]
    assert lib.lutgemm_set_option(which, 4096) == 0
    try:
        plan = native.Plan()
        assert lib.lutgemm_describe_plan(0, N, K, nb, K // 128, 1, ctypes.byref(plan)) == 0
        assert plan.items_per_long_range == 1 and plan.workgroups == 2 * 39 and plan.needs_workspace == 1
        d = [t.to(gpu_device) for t in (bW, alpha, x)]
        out = torch.zeros((1, N), dtype=torch.float16, device=gpu_device)
        for _ in range(2):                                                # twice: the words must be left at zero
            out.zero_()
            rc = lib.lutgemm_gemv_rowwise_f16(_ptr(d[0]), _ptr(d[1]), _ptr(d[2]), _ptr(out), N, K, nb, K // 128, 1, _sp())
            assert rc == 0, lib.lutgemm_strerror(rc).decode()
            torch.cuda.synchronize()
            rel, mad = orc.error_metrics(out.float().cpu().numpy(), want.astype(np.float32))
            assert rel <= 2e-4 and mad <= 1e-3, (rel, mad)
    finally:
        lib.lutgemm_set_option(which, -1)
