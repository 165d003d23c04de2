"""The entry point that allocates nothing, through the C ABI on the GPU.

lutgemm_gemv_rowwise_f16_noalloc takes its accumulator words from a fixed device
array inside the library instead of a per-stream workspace.  It must give the
bits lutgemm_gemv_rowwise_f16 gives (same kernels, same launch plan, integer
accumulation), on two calls in a row that share the array, the second with a
smaller input; it must refuse sizes beyond the array; and it must not change
the amount of device memory in use.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle as orc
from shiftaddllm_amd import native

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _operands(dev, N, K, nb, M, seed, group=128):
    g = torch.Generator().manual_seed(seed)
    bW = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 32, nb, N), generator=g, dtype=torch.int32)
    e = torch.randint(-9, -5, (K // group, 1, N), generator=g).float() - torch.arange(nb).float().view(1, nb, 1)
    alpha = torch.exp2(e).to(torch.float16).contiguous()
    x = torch.randn((M, K), generator=g).half()
    bias = (torch.randn((M, N), generator=g) * 0.1).half()
    return bW, alpha, x, bias


def _call(fn, d, out, stream):
    bW, alpha, x = d
    N, K, nb, M = bW.shape[2], bW.shape[0] * 32, bW.shape[1], x.shape[0]
    rc = fn(_ptr(bW), _ptr(alpha), _ptr(x), _ptr(out), N, K, nb, K // 128, M, ctypes.c_void_p(stream.cuda_stream))
    assert rc == 0, native.cabi().lutgemm_strerror(rc).decode()
    stream.synchronize()
    return out


def test_no_alloc_entry_matches_the_allocating_one_twice_in_a_row(gpu_device):
    dev = gpu_device
    lib = native.cabi()
    stream = torch.cuda.Stream()
    # Every case uses accumulator words (checked through the launch plan): K split over many
    # workgroups of the look-up kernel, then a smaller problem that reuses the first words of the
    # array, then two rows through the look-up kernel's pair tables, then several rows on the
    # matrix-core kernel with K cut into slices, then the first shape again: a call that left a
    # word dirty would show up in the next one.
    cases = [(4096, 4096, 3, 1, 11), (1024, 2048, 2, 1, 12), (8192, 4096, 4, 2, 14), (4096, 4096, 3, 8, 13),
             (4096, 4096, 3, 1, 15)]
    # set-up: the first call on a device resolves the array's address (the runtime places
    # the library's device variables in memory at that moment at the latest)
    w = _operands(dev, 256, 256, 1, 1, 1)
    _call(lib.lutgemm_gemv_rowwise_f16_noalloc, [t.to(dev) for t in w[:3]], w[3].clone().to(dev), stream)
    for (N, K, nb, M, seed) in cases:
        print(f"no-alloc case N={N} K={K} nb={nb} M={M} seed={seed}", flush=True)
        plan = native.Plan()
        assert lib.lutgemm_describe_plan(0, N, K, nb, K // 128, M, ctypes.byref(plan)) == 0
        assert plan.needs_workspace == 1, (N, K, nb, M)
        ops = _operands(dev, N, K, nb, M, seed)
        d = [t.to(dev) for t in ops[:3]]
        out_a, out_b = ops[3].clone().to(dev), ops[3].clone().to(dev)
        torch.cuda.synchronize()
        want = _call(lib.lutgemm_gemv_rowwise_f16, d, out_a, stream)
        free_before = torch.cuda.mem_get_info()[0]
        got = _call(lib.lutgemm_gemv_rowwise_f16_noalloc, d, out_b, stream)
        assert torch.cuda.mem_get_info()[0] >= free_before      # nothing was allocated by the call
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (N, K, nb, M)
        # and both agree with the oracle to the bar of the parity suite (pair tables: fp16 entries)
        ref, _ = orc.gemv_rowwise_c(ops[0].numpy(), ops[1].numpy(), ops[2].numpy(), K // 128, out=ops[3].numpy())
        rel, mad = orc.error_metrics(got.float().cpu().numpy(), ref.astype(np.float32))
        assert rel <= (5e-4 if M == 2 else 2e-4) and mad <= 2e-3, (rel, mad)


def test_no_alloc_entry_refuses_what_does_not_fit(gpu_device):
    dev = gpu_device
    lib = native.cabi()
    N = native.NOALLOC_MAX_WORDS + 256            # one row of outputs more than the array holds
    bW = torch.zeros((1, 1, N), dtype=torch.int32, device=dev)
    alpha = torch.ones((1, 1, N), dtype=torch.float16, device=dev)
    x = torch.zeros((1, 32), dtype=torch.float16, device=dev)
    out = torch.zeros((1, N), dtype=torch.float16, device=dev)
    rc = lib.lutgemm_gemv_rowwise_f16_noalloc(_ptr(bW), _ptr(alpha), _ptr(x), _ptr(out), N, 32, 1, 1, 1, None)
    assert rc == -7
    assert b"NOALLOC" in lib.lutgemm_strerror(rc)
    # the same call with rows: M * N counts
    rc = lib.lutgemm_gemv_rowwise_f16_noalloc(_ptr(bW), _ptr(alpha), _ptr(x), _ptr(out), N // 2, 32, 1, 1, 3, None)
    assert rc == -7
