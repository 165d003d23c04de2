"""Parity of the HIP kernels with the CPU oracle, on the GPU, through the C ABI.

Bars: packed words and table indices are bit-exact by construction of the
operands (checked on the CPU side); outputs are fp16 and must satisfy
rel-L2 <= 2e-3 and max|dy| <= 1e-2 * max|y_ref| against the oracle.  The
kernels accumulate in fp32 and round once, so the tests also hold them to a
ten times tighter bound.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle as orc
from shiftaddllm_amd import native, workload

pytestmark = pytest.mark.gpu

REL_L2_BAR = 2e-3          # relative L2 error bound on the fp16 output
MAX_ABS_BAR = 1e-2         # max |dy| / max |y_ref|
TIGHT = 0.1                # our own margin inside those bars
PAIR_TABLES = 0.25         # the same for rows that share fp16-pair tables (see _rows_margin)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _check(rc):
    assert rc == 0, native.cabi().lutgemm_strerror(rc).decode()


def _assert_close(y_gpu, y_ref, what="", margin=TIGHT):
    """y_ref is the oracle's fp16 output (same single rounding as the kernel):
    held to a tenth of the bars.  Against an un-rounded fp32 reference pass
    margin=0.25, fp16 rounding alone costs about 2e-4."""
    rel, mad = orc.error_metrics(y_gpu.float().cpu().numpy(), np.asarray(y_ref, dtype=np.float32))
    assert rel <= REL_L2_BAR * margin and mad <= MAX_ABS_BAR * margin, (what, rel, mad)
    return rel, mad


def run_rowwise(dev, bW, alpha, x, num_groups, out=None):
    N, K, nb = bW.shape[2], bW.shape[0] * 32, bW.shape[1]
    M = x.shape[0]
    d_out = (torch.zeros((M, N), dtype=torch.float16) if out is None else out.clone()).to(dev)
    d_bW, d_a, d_x = bW.to(dev), alpha.to(dev), x.to(dev).contiguous()
    _check(native.cabi().lutgemm_gemv_rowwise_f16(_ptr(d_bW), _ptr(d_a), _ptr(d_x), _ptr(d_out),
                                                  N, K, nb, num_groups, M, _stream()))
    torch.cuda.synchronize()
    return d_out


def run_block(dev, bW, alpha, x, R, kind, out=None):
    N, K, nb = bW.shape[2], bW.shape[0] * 32, bW.shape[1]
    M = x.shape[0]
    d_out = (torch.zeros((M, N), dtype=torch.float16) if out is None else out.clone()).to(dev)
    d_bW, d_a, d_x = bW.to(dev), alpha.to(dev), x.to(dev).contiguous()
    lib = native.cabi()
    if kind == orc.ALPHA_F16:
        rc = lib.lutgemm_gemv_block_f16(_ptr(d_bW), _ptr(d_a), _ptr(d_x), _ptr(d_out), N, K, nb, R, M, _stream())
    elif kind == orc.ALPHA_SHIFT_U16:
        rc = lib.lutgemm_gemv_block_shift_u16(_ptr(d_bW), _ptr(d_a), _ptr(d_x), _ptr(d_out), N, K, nb, R, 3, M,
                                              _stream())
    else:
        rc = lib.lutgemm_gemv_block_apot_i8(_ptr(d_bW), _ptr(d_a), _ptr(d_x), _ptr(d_out), N, K, nb, R, 3, M,
                                            _stream())
    _check(rc)
    torch.cuda.synchronize()
    return d_out


# ---- row-wise alpha (configs 1, 2, 4, 5) -------------------------------------

def test_config1_opt125m_fc1_real_bcq(gpu_device):
    N, K = workload.OPT125M_FC1
    p = workload.make_rowwise_problem(N, K, nb=3, group_size=128, seed=0)
    # operands are bit-exact restatements of the reference packing
    assert np.array_equal(p.bW.permute(2, 0, 1).contiguous().numpy(),
                          orc.pack_binary_weight_c(p.B.numpy()))
    want, y32 = orc.gemv_rowwise_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), p.num_groups)
    got = run_rowwise(gpu_device, p.bW, p.alpha, p.x, p.num_groups)
    _assert_close(got, want, "config1")
    # and against the dense dequantise-and-matmul path
    Wq = orc.dequant_rowwise_kernel_layout(p.bW.numpy(), p.alpha.numpy())
    _assert_close(got, orc.dense_gemv_np(Wq, p.x.numpy()), "config1 dense", margin=0.25)


@pytest.mark.parametrize("N,K,nb,gs,M", [
    (4, 32, 1, 32, 1),         # smallest legal problem
    (8, 64, 2, 32, 1),
    (132, 96, 3, 96, 1),       # N tail inside a step, K not a multiple of 256
    (260, 288, 4, 32, 2),      # partial table set, two rows
    (512, 512, 3, 128, 1),
    (1024, 768, 2, 256, 3),
    (3072, 768, 3, 128, 5),    # config-1 shape with a batch
    (384, 2048, 4, 2048, 1),   # a single group along K
    (128, 8192, 3, 128, 1),    # long K, one N tile
])
def test_rowwise_ragged_shapes(gpu_device, N, K, nb, gs, M):
    p = workload.make_rowwise_problem(N, K, nb=nb, group_size=gs, M=M, seed=N + K + nb, quantize=False)
    want, _ = orc.gemv_rowwise_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), p.num_groups)
    got = run_rowwise(gpu_device, p.bW, p.alpha, p.x, p.num_groups)
    _assert_close(got, want, (N, K, nb, gs, M), margin=_rows_margin(K, gs, M))


def _rows_margin(K, gs, M):
    """Two or more rows through the look-up kernel (shapes the matrix-core kernel does not take: K
    not a multiple of 128, groups not a multiple of 128 inputs) share one table set whose entries
    hold two rows as fp16 halves: one more fp16 rounding per table entry, about 3e-4 on the
    output.  Held to a quarter of the bars instead of a tenth."""
    on_matrix_cores = M >= 3 and K % 128 == 0 and gs % 128 == 0
    return TIGHT if M == 1 or on_matrix_cores else PAIR_TABLES


@pytest.mark.parametrize("N,K,nb,gs,M", [
    (512, 288, 3, 32, 2),        # look-up kernel, one pair of rows
    (512, 288, 4, 96, 3),        # two pairs, the fourth row a repeat of the third
    (300, 1056, 2, 32, 4),       # two pairs, K tail, N tail
    (11008, 4096, 3, 128, 2),    # two rows on a sign stream long enough for the look-up kernel
])
def test_rows_sharing_pair_tables(gpu_device, N, K, nb, gs, M):
    p = workload.make_rowwise_problem(N, K, nb=nb, group_size=gs, M=M, seed=N + M, quantize=False)
    want, _ = orc.gemv_rowwise_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), p.num_groups)
    got = run_rowwise(gpu_device, p.bW, p.alpha, p.x, p.num_groups)
    _assert_close(got, want, (N, K, nb, gs, M), margin=PAIR_TABLES)
    # the rows of a pair do not leak into each other: row 0 alone gives row 0 of the batch to
    # within the same bar (the single-row kernel uses fp32 tables)
    one = run_rowwise(gpu_device, p.bW, p.alpha, p.x[:1].contiguous(), p.num_groups)
    _assert_close(got[:1], one.cpu().numpy(), ("row 0 alone", N, K, nb, gs, M), margin=PAIR_TABLES)


def test_rowwise_general_alpha_values(gpu_device):
    # the binding accepts any fp16 alpha, not only powers of two
    g = torch.Generator().manual_seed(5)
    N, K, nb, gs = 256, 512, 3, 64
    p = workload.make_rowwise_problem(N, K, nb=nb, group_size=gs, seed=5, quantize=False)
    alpha = (torch.rand(p.alpha.shape, generator=g) * 0.05).half()
    want, _ = orc.gemv_rowwise_c(p.bW.numpy(), alpha.numpy(), p.x.numpy(), p.num_groups)
    _assert_close(run_rowwise(gpu_device, p.bW, alpha, p.x, p.num_groups), want)


def test_accumulates_into_bias_and_is_deterministic(gpu_device):
    N, K = 1024, 1024
    p = workload.make_rowwise_problem(N, K, nb=3, group_size=128, M=2, seed=9, quantize=False)
    bias = (torch.randn((2, N), generator=torch.Generator().manual_seed(1))).half()
    want, _ = orc.gemv_rowwise_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), p.num_groups, out=bias.numpy())
    got1 = run_rowwise(gpu_device, p.bW, p.alpha, p.x, p.num_groups, out=bias)
    got2 = run_rowwise(gpu_device, p.bW, p.alpha, p.x, p.num_groups, out=bias)
    _assert_close(got1, want)
    assert torch.equal(got1, got2)                      # fixed summation order
    # x = 0 leaves the pre-filled output untouched, bit for bit
    zero = torch.zeros_like(p.x)
    assert torch.equal(run_rowwise(gpu_device, p.bW, p.alpha, zero, p.num_groups, out=bias).cpu(), bias)


def test_unit_vectors_return_columns_of_wq(gpu_device):
    N, K, nb, gs = 256, 512, 3, 128
    p = workload.make_rowwise_problem(N, K, nb=nb, group_size=gs, seed=3, quantize=False)
    Wq = orc.dequant_rowwise_kernel_layout(p.bW.numpy(), p.alpha.numpy())
    ks = [0, 7, 8, 31, 32, 255, 256, 511]
    x = torch.zeros((len(ks), K), dtype=torch.float16)
    for i, k in enumerate(ks):
        x[i, k] = 1.0
    got = run_rowwise(gpu_device, p.bW, p.alpha, x, p.num_groups).float().cpu().numpy()
    for i, k in enumerate(ks):
        # W_q entries are sums of <= 3 powers of two: exactly representable in fp16 here
        assert np.array_equal(got[i], Wq[:, k].astype(np.float16).astype(np.float32)), k


@pytest.mark.parametrize("name,N,K", workload.LLAMA2_7B_LINEARS[3:])   # o_proj, gate, up, down
def test_config2_llama7b_shapes_real_bcq(gpu_device, name, N, K):
    # quantise on the GPU (pure torch), check against the CPU oracle at full size
    p = workload.make_rowwise_problem(N, K, nb=3, group_size=128, seed=0, device=gpu_device)
    bW, alpha, x = p.bW.cpu(), p.alpha.cpu(), p.x.cpu()
    want, _ = orc.gemv_rowwise_c(bW.numpy(), alpha.numpy(), x.numpy(), p.num_groups)
    got = run_rowwise(gpu_device, bW, alpha, x, p.num_groups)
    _assert_close(got, want, name)
    # linearity, a size-independent property: f(x1) + f(x2) == f(x1 + x2) up to fp16 rounding
    x2 = torch.randn((1, K), generator=torch.Generator().manual_seed(4)).half()
    y1 = got.float()
    y2 = run_rowwise(gpu_device, bW, alpha, x2, p.num_groups).float()
    y12 = run_rowwise(gpu_device, bW, alpha, (x.float() + x2.float()).half(), p.num_groups).float()
    rel, _ = orc.error_metrics((y1 + y2).cpu().numpy(), y12.cpu().numpy())
    assert rel < 3e-3


@pytest.mark.parametrize("N,K,nb", [(8192, 8192, 2), (1024, 8192, 4), (8192, 8192, 4)])
def test_config5_llama70b_shapes_m1(gpu_device, N, K, nb):
    p = workload.make_rowwise_problem(N, K, nb=nb, group_size=128, seed=1, sigma=0.015, quantize=False)
    want, _ = orc.gemv_rowwise_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), p.num_groups)
    _assert_close(run_rowwise(gpu_device, p.bW, p.alpha, p.x, p.num_groups), want)


@pytest.mark.parametrize("M", [4, 16, 32])
def test_config5_small_batches(gpu_device, M):
    N, K, nb = 1024, 8192, 2
    p = workload.make_rowwise_problem(N, K, nb=nb, group_size=128, M=M, seed=2, sigma=0.015, quantize=False)
    want, _ = orc.gemv_rowwise_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), p.num_groups)
    _assert_close(run_rowwise(gpu_device, p.bW, p.alpha, p.x, p.num_groups), want)


@pytest.mark.parametrize("N,K,nb,gs,M", [
    (16, 128, 1, 128, 3),        # smallest problem the matrix-core path takes
    (80, 256, 2, 128, 5),        # N not a multiple of the wave tile, odd row count
    (256, 1024, 3, 128, 16),
    (1024, 4096, 4, 128, 17),    # second row chunk almost empty
    (272, 384, 3, 128, 33),      # three row chunks, ragged N
    (4096, 4096, 3, 256, 8),     # group of 256 inputs (two K-steps per alpha)
    (11008, 4096, 2, 4096, 32),  # one group along K
    (22016, 4096, 3, 128, 4),    # 344 tiles: two K-slices each, more workgroups than are resident at once
    (5120, 13824, 3, 128, 4),    # 108 K-steps in three slices of unequal length
    (5120, 5120, 3, 128, 16),    # 40 K-steps, slices of 16, 16 and 8
])
def test_small_batch_matrix_core_path(gpu_device, N, K, nb, gs, M):
    p = workload.make_rowwise_problem(N, K, nb=nb, group_size=gs, M=M, seed=N + M, quantize=False)
    bias = torch.randn((M, N), generator=torch.Generator().manual_seed(M)).half()
    want, _ = orc.gemv_rowwise_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), p.num_groups, out=bias.numpy())
    got = run_rowwise(gpu_device, p.bW, p.alpha, p.x, p.num_groups, out=bias)
    _assert_close(got, want, (N, K, nb, gs, M))
    assert torch.equal(got, run_rowwise(gpu_device, p.bW, p.alpha, p.x, p.num_groups, out=bias))


def test_random_shapes_against_a_dense_product(gpu_device):
    """240 seeded random problems (any K % 32, N % 4, group size, 1-4 bit planes, 1-33 rows, general
    fp16 alphas, a bias in `out`) against the dense fp64 product of the dequantised matrix, formed on
    the GPU by framework operations: a reference that shares nothing with the oracle's look-up
    formulation.  Every launch plan the planner has is hit (checked through lutgemm_describe_plan)."""
    import random
    dev = gpu_device
    lib = native.cabi()
    rng = random.Random(2024)
    plan = native.Plan()
    seen = set()
    for case in range(240):
        if case % 3 == 0:     # shapes the matrix-core kernel takes from three rows on
            K = 128 * rng.randint(1, 64)
            N = 16 * rng.randint(1, 500)
            gs = rng.choice([g for g in (128, 256, 512, K) if K % g == 0])
        else:
            K = 32 * rng.randint(1, 200)
            N = 4 * rng.randint(1, 1800)
            gs = rng.choice([g for g in (32, 64, 96, 128, 256, K) if K % g == 0])
        nb = rng.randint(1, 4)
        M = rng.choice((1, 1, 1, 2, 2, 3, 4, 5, 8, 16, 17, 33))
        g = torch.Generator(device=dev).manual_seed(case)
        bW = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 32, nb, N), generator=g, device=dev, dtype=torch.int32)
        alpha = (torch.rand((K // gs, nb, N), generator=g, device=dev) * 0.02 + 0.001).half()
        x = torch.randn((M, K), generator=g, device=dev).half()
        bias = torch.randn((M, N), generator=g, device=dev).half()
        out = bias.clone()
        _check(lib.lutgemm_gemv_rowwise_f16(_ptr(bW), _ptr(alpha), _ptr(x), _ptr(out), N, K, nb, K // gs, M, _stream()))
        torch.cuda.synchronize()
        signs = ((bW.unsqueeze(1) >> torch.arange(32, device=dev).view(1, 32, 1, 1)) & 1).double() * 2 - 1
        Wq = (signs.reshape(K, nb, N) * alpha.double().repeat_interleave(gs, dim=0)).sum(1)      # [K][N]
        want = bias.double() + x.double() @ Wq
        rel = ((out.double() - want).norm() / want.norm()).item()
        mad = ((out.double() - want).abs().max() / want.abs().max()).item()
        _check(lib.lutgemm_describe_plan(0, N, K, nb, K // gs, M, ctypes.byref(plan)))
        seen.add((plan.kernel, plan.rows_per_pass))
        # against an un-rounded reference: a quarter of the bars (the final fp16 rounding alone is 2e-4)
        assert rel <= REL_L2_BAR * 0.25 and mad <= MAX_ABS_BAR * 0.25, (N, K, nb, gs, M, rel, mad)
    assert seen == {(0, 1), (0, 2), (0, 4), (1, 16), (1, 32)}, seen


def test_batch_rows_agree_with_single_row_calls(gpu_device):
    # every row of a batched call equals the batch-1 call on that row (different kernels)
    p = workload.make_rowwise_problem(2048, 2048, nb=3, group_size=128, M=8, seed=77, quantize=False)
    batched = run_rowwise(gpu_device, p.bW, p.alpha, p.x, p.num_groups).float().cpu()
    for m in (0, 3, 7):
        single = run_rowwise(gpu_device, p.bW, p.alpha, p.x[m:m + 1], p.num_groups).float().cpu()
        rel, _ = orc.error_metrics(batched[m:m + 1].numpy(), single.numpy())
        assert rel <= 2e-4, (m, rel)


# ---- block alpha (config 3 and the LutLinear default format) -----------------

def test_config3_llama13b_block_real_bcq(gpu_device):
    N, K = workload.LLAMA2_13B_SHAPES[0]
    p = workload.make_block_problem(N, K, nb=2, R=8, seed=0, device=gpu_device)
    bW, alpha, x = p.bW.cpu(), p.alpha.cpu(), p.x.cpu()
    want, _ = orc.gemv_block_c(bW.numpy(), alpha.numpy(), x.numpy(), 8, kind=orc.ALPHA_F16)
    _assert_close(run_block(gpu_device, bW, alpha, x, 8, orc.ALPHA_F16), want)
    # dense path from the ON-DISK tensors (dequantise, transpose, matmul)
    W = orc.dequant_lat_disk(p.disk_bWeight.cpu().numpy(), p.disk_alpha.cpu().numpy())
    _assert_close(run_block(gpu_device, bW, alpha, x, 8, orc.ALPHA_F16), orc.dense_gemv_np(W, x.numpy()),
                  margin=0.25)


@pytest.mark.parametrize("N,K", workload.LLAMA2_13B_SHAPES[1:])
def test_config3_non_square_shapes(gpu_device, N, K):
    p = workload.make_block_problem(N, K, nb=2, R=8, seed=1, quantize=False)
    want, _ = orc.gemv_block_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), 8, kind=orc.ALPHA_F16)
    _assert_close(run_block(gpu_device, p.bW, p.alpha, p.x, 8, orc.ALPHA_F16), want)


@pytest.mark.parametrize("N,K,nb,R,M", [(32, 32, 1, 1, 1), (64, 96, 3, 4, 2), (640, 288, 2, 8, 1),
                                         (256, 512, 4, 64, 3), (1024, 1024, 3, 8, 1),
                                         (2560, 544, 3, 4, 3),     # tiles straddle row groups, several rows
                                         (2048, 256, 4, 2, 5)])
def test_block_f16_ragged(gpu_device, N, K, nb, R, M):
    p = workload.make_block_problem(N, K, nb=nb, R=R, M=M, seed=N + R, quantize=False)
    want, _ = orc.gemv_block_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), R, kind=orc.ALPHA_F16)
    _assert_close(run_block(gpu_device, p.bW, p.alpha, p.x, R, orc.ALPHA_F16), want)


@pytest.mark.parametrize("N,K,nb,R,M", [(64, 64, 2, 8, 1), (768, 768, 3, 8, 1), (512, 1024, 3, 16, 2)])
def test_block_shift_u16(gpu_device, N, K, nb, R, M):
    p = workload.make_block_problem(N, K, nb=nb, R=R, M=M, seed=3, quantize=False)
    g = torch.Generator().manual_seed(N)
    code = torch.randint(0, 512, (K // 8, nb, R), generator=g).to(torch.int16)
    x = (p.x.float() * 0.01).half()          # multipliers reach 384: keep outputs inside fp16
    want, _ = orc.gemv_block_c(p.bW.numpy(), code.numpy(), x.numpy(), R, kind=orc.ALPHA_SHIFT_U16)
    _assert_close(run_block(gpu_device, p.bW, code, x, R, orc.ALPHA_SHIFT_U16), want)


@pytest.mark.parametrize("N,K,nb,R,M", [(64, 64, 2, 8, 1), (768, 768, 3, 8, 1), (3072, 768, 3, 8, 1),
                                         (512, 1024, 3, 16, 2)])
def test_block_apot_i8(gpu_device, N, K, nb, R, M):
    p = workload.make_block_problem(N, K, nb=nb, R=R, M=M, seed=4, quantize=False)
    g = torch.Generator().manual_seed(K)
    code = torch.randint(-12, -3, (K // 8, nb, R, 3), generator=g).to(torch.int8)
    code[torch.rand(code.shape, generator=g) < 0.4] = -128       # absent terms
    want, _ = orc.gemv_block_c(p.bW.numpy(), code.numpy(), p.x.numpy(), R, kind=orc.ALPHA_APOT_I8)
    _assert_close(run_block(gpu_device, p.bW, code, p.x, R, orc.ALPHA_APOT_I8), want)


# ---- uniform mode -------------------------------------------------------------

@pytest.mark.parametrize("N,K,nb,gs,M", [(64, 128, 3, 64, 1), (1024, 1024, 4, 128, 1), (260, 288, 2, 32, 2)])
def test_uniform_mode(gpu_device, N, K, nb, gs, M):
    p = workload.make_rowwise_problem(N, K, nb=nb, group_size=gs, M=M, seed=6, quantize=False)
    g = torch.Generator().manual_seed(7)
    alpha = (torch.rand((K // gs, N), generator=g) * 0.05).half()
    q = (torch.randn((K // gs, N), generator=g) * 0.01).half()
    want, _ = orc.gemv_uniform_c(p.bW.numpy(), alpha.numpy(), q.numpy(), p.x.numpy(), K // gs)
    dev = gpu_device
    d_out = torch.zeros((M, N), dtype=torch.float16, device=dev)
    d = [t.to(dev) for t in (p.bW, alpha, q, p.x)]
    _check(native.cabi().lutgemm_gemv_uniform_f16(_ptr(d[0]), _ptr(d[1]), _ptr(d[2]), _ptr(d[3]), _ptr(d_out),
                                                  N, K, nb, K // gs, M, _stream()))
    torch.cuda.synchronize()
    _assert_close(d_out, want, margin=TIGHT if M == 1 else PAIR_TABLES)   # (uniform mode has no matrix-core path)


# ---- the Python operator surface ----------------------------------------------

def test_python_module_and_lutlinear(gpu_device):
    from shiftaddllm_amd.lut_gemm.quant import LutLinear, encode_apot_int8
    dev = gpu_device
    ext = native.lutgemm
    N, K, R, nb = 768, 768, 8, 3
    p = workload.make_block_problem(N, K, nb=nb, R=R, seed=0)
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(2)) * 0.1).half()

    # reference call pattern: output = bias.clone(); ext(output, ...) (lut_gemm/quant.py:46-51)
    code = encode_apot_int8(p.alpha.float())                      # exact: alphas are powers of two
    out = bias.clone().to(dev).reshape(1, N)
    ext.lutgemm_compute_block_shiftInt8(out, p.bW.to(dev), code.to(dev), p.x.to(dev), N, K, nb, R, 3)
    torch.cuda.synchronize()
    want, _ = orc.gemv_block_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), R, kind=orc.ALPHA_F16,
                               out=bias.numpy().reshape(1, N))
    _assert_close(out, want)

    lin = LutLinear(K, N, group_size=K // R, wbit=nb, bias=bias.to(dev)).to(dev)
    lin.binaryWeight.data = p.bW.to(dev)
    lin.alpha.data = lin.quantize_to_apot(p.alpha.float()).to(dev)
    y = lin(p.x.to(dev).reshape(1, 1, K))                          # [batch, token, K] like a decoder
    assert tuple(y.shape) == (1, 1, N) and y.dtype == torch.float16
    _assert_close(y.reshape(1, N), want)

    # no bias (Llama) and several tokens: supersets of the reference behaviour
    lin2 = LutLinear(K, N, group_size=K // R, wbit=nb, bias=None, alpha_format="block_fp16").to(dev)
    lin2.binaryWeight.data = p.bW.to(dev)
    lin2.alpha.data = p.alpha.to(dev)
    x4 = torch.randn((2, 2, K), generator=torch.Generator().manual_seed(3)).half()
    y4 = lin2(x4.to(dev))
    want4, _ = orc.gemv_block_c(p.bW.numpy(), p.alpha.numpy(), x4.reshape(4, K).numpy(), R, kind=orc.ALPHA_F16)
    assert tuple(y4.shape) == (2, 2, N)
    _assert_close(y4.reshape(4, N), want4)

    # wrong dtype / shape raise instead of corrupting memory
    with pytest.raises(RuntimeError):
        ext.lutgemm_compute_block(out, p.bW.to(dev), p.alpha.float().to(dev), p.x.to(dev), N, K, nb, R)
    with pytest.raises(RuntimeError):
        ext.lutgemm_compute_block(out, p.bW.to(dev)[:, :, :-4].contiguous(), p.alpha.to(dev), p.x.to(dev),
                                  N, K, nb, R)
    with pytest.raises(RuntimeError):
        ext.lutgemm_compute_block_shiftInt8(out, p.bW.to(dev), code.to(dev), p.x.to(dev), N, K, nb, R, 2)


def test_runs_on_a_side_stream(gpu_device):
    p = workload.make_rowwise_problem(512, 1024, nb=3, group_size=128, seed=8, quantize=False)
    want, _ = orc.gemv_rowwise_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), p.num_groups)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        got = run_rowwise(gpu_device, p.bW, p.alpha, p.x, p.num_groups)
    s.synchronize()
    _assert_close(got, want)


# ---- several GEMVs in one launch ------------------------------------------------

def _grouped(dev, problems, outs=None):
    """problems: list of RowwiseProblem (CPU). Returns the list of device outputs."""
    lib = native.cabi()
    arr = (native.RowwiseProblem * len(problems))()
    keep = []
    d_outs = []
    for i, p in enumerate(problems):
        M = p.x.shape[0]
        d = [p.bW.to(dev), p.alpha.to(dev), p.x.to(dev).contiguous(),
             (torch.zeros((M, p.N), dtype=torch.float16) if outs is None else outs[i].clone()).to(dev)]
        keep.append(d)
        d_outs.append(d[3])
        arr[i] = native.RowwiseProblem(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(),
                                       p.N, p.K, p.nb, p.num_groups, M)
    _check(lib.lutgemm_gemv_rowwise_f16_grouped(len(problems), arr, _stream()))
    torch.cuda.synchronize()
    return d_outs


def test_grouped_launch_mixed_shapes_and_bits(gpu_device):
    specs = [(512, 1024, 3, 128, 1), (1024, 1024, 2, 128, 1), (260, 288, 4, 32, 2), (4096, 512, 3, 128, 1),
             (128, 2048, 1, 64, 1)]
    probs = [workload.make_rowwise_problem(N, K, nb=nb, group_size=gs, M=M, seed=40 + i, quantize=False)
             for i, (N, K, nb, gs, M) in enumerate(specs)]
    bias = [torch.randn((p.x.shape[0], p.N), generator=torch.Generator().manual_seed(i)).half()
            for i, p in enumerate(probs)]
    got = _grouped(gpu_device, probs, outs=bias)
    for p, b, g in zip(probs, bias, got):
        want, _ = orc.gemv_rowwise_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), p.num_groups, out=b.numpy())
        _assert_close(g, want, (p.N, p.K, p.nb))
        # agrees with the single-problem entry point to fp16 rounding (K may be cut
        # differently, so the fp32 partial sums are not bit-identical)
        single = run_rowwise(gpu_device, p.bW, p.alpha, p.x, p.num_groups, out=b)
        rel, _ = orc.error_metrics(g.float().cpu().numpy(), single.float().cpu().numpy())
        assert rel <= 2e-4


def test_grouped_llama7b_block(gpu_device):
    # the seven linears of one decoder block in a single launch
    probs = [workload.make_rowwise_problem(N, K, nb=3, group_size=128, seed=60 + i, quantize=False)
             for i, (_, N, K) in enumerate(workload.LLAMA2_7B_LINEARS)]
    got = _grouped(gpu_device, probs)
    for p, g in zip(probs, got):
        want, _ = orc.gemv_rowwise_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), p.num_groups)
        _assert_close(g, want, (p.N, p.K))


def test_grouped_rejects_bad_counts(gpu_device):
    lib = native.cabi()
    arr = (native.RowwiseProblem * 1)()
    assert lib.lutgemm_gemv_rowwise_f16_grouped(0, arr, None) == -1
    assert lib.lutgemm_gemv_rowwise_f16_grouped(native.MAX_GROUP + 1, arr, None) == -1
    assert lib.lutgemm_gemv_rowwise_f16_grouped(1, arr, None) == -1      # null operands inside


def test_repeated_calls_leave_the_workspace_clean(gpu_device):
    # K-split accumulators are cleared by whoever completes a sum: many calls in a
    # row, of different shapes on one stream, must keep giving the same answer
    a = workload.make_rowwise_problem(1024, 4096, nb=3, group_size=128, seed=70, quantize=False)
    b = workload.make_rowwise_problem(2048, 2048, nb=2, group_size=128, seed=71, quantize=False)
    wa, _ = orc.gemv_rowwise_c(a.bW.numpy(), a.alpha.numpy(), a.x.numpy(), a.num_groups)
    wb, _ = orc.gemv_rowwise_c(b.bW.numpy(), b.alpha.numpy(), b.x.numpy(), b.num_groups)
    first = run_rowwise(gpu_device, a.bW, a.alpha, a.x, a.num_groups)
    for _ in range(5):
        _assert_close(run_rowwise(gpu_device, b.bW, b.alpha, b.x, b.num_groups), wb)
        again = run_rowwise(gpu_device, a.bW, a.alpha, a.x, a.num_groups)
        _assert_close(again, wa)
        assert torch.equal(again, first)


def test_saturation_of_non_finite_partial_sums(gpu_device):
    # a NaN / inf activation must not poison the K-split accumulators for later calls
    p = workload.make_rowwise_problem(512, 4096, nb=3, group_size=128, seed=72, quantize=False)
    want, _ = orc.gemv_rowwise_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), p.num_groups)
    bad = p.x.clone()
    bad[0, 5] = float("inf")
    y_bad = run_rowwise(gpu_device, p.bW, p.alpha, bad, p.num_groups)
    assert not torch.isfinite(y_bad).all()
    _assert_close(run_rowwise(gpu_device, p.bW, p.alpha, p.x, p.num_groups), want)


# ---- decode harness (config 4) ---------------------------------------------------

def test_decoder_matches_dense_dequantised_model(gpu_device):
    """A small mixed-bit decoder through LutLinear (eager, fused, and graph replay)
    against the same network with every linear replaced by a dense fp32 matmul on
    oracle-dequantised weights."""
    from shiftaddllm_amd import decode
    cfg = decode.DecoderConfig(vocab_size=512, hidden=256, intermediate=512, layers=2, heads=4, kv_heads=2,
                               max_positions=32, group_size=128)
    qc = workload.mixed_bit_config(cfg.layers, seed=3)
    torch.manual_seed(0)
    ids = torch.randint(0, cfg.vocab_size, (2, 6))

    def run(model, capture):
        if capture:
            model.capture()
        model.reset()
        outs = []
        for t in range(ids.shape[1]):
            outs.append(model.forward_token(ids[:, t].to(gpu_device), t).float().cpu().clone())
        torch.cuda.synchronize()
        return torch.stack(outs)

    lut = decode.LutDecoder(cfg, qc, batch=2, seed=5, device=gpu_device, fuse_launches=True)
    bits = sorted({l.wbit for b in lut.blocks for l in (b.q_proj, b.k_proj, b.down_proj, b.gate_proj)})
    assert len(bits) >= 2                                   # the draw really mixes bit widths

    dense = decode.LutDecoder(cfg, qc, batch=2, seed=5, device=gpu_device, fuse_launches=False, glue="torch")
    table = {}
    for blk in dense.blocks:
        for lin in (blk.q_proj, blk.k_proj, blk.v_proj, blk.o_proj, blk.gate_proj, blk.up_proj, blk.down_proj):
            Wq = orc.dequant_rowwise_kernel_layout(lin.binaryWeight.cpu().numpy(), lin.alpha.cpu().numpy())
            table[id(lin)] = torch.from_numpy(Wq).to(gpu_device)
    dense._linears = lambda lins, x: [(x.float() @ table[id(l)].t()).half() for l in lins]

    want = run(dense, capture=False)
    got_fused = run(lut, capture=False)
    got_graph = run(lut, capture=True)
    lut.fuse = False
    lut._graph = None
    got_plain = run(lut, capture=False)
    # the same LutLinear layers between framework operations instead of the fused glue kernels
    lut.glue, lut.fuse = "torch", True
    got_torch_glue = run(lut, capture=False)
    lut.glue = "hip"
    # RMSNorm: folded into the q,k,v and gate,up launches is the default at this batch size; the
    # other fused form splits it over the launch that completes the residual row and its readers
    assert lut.fold_norm and lut.split_norm
    lut.fold_norm = False
    got_split_norm = run(lut, capture=False)
    lut.fold_norm = True
    for name, got in (("fused", got_fused), ("graph", got_graph), ("plain", got_plain),
                      ("torch glue", got_torch_glue), ("split norm", got_split_norm)):
        rel, mad = orc.error_metrics(got.numpy(), want.numpy())
        assert rel <= REL_L2_BAR and mad <= MAX_ABS_BAR, (name, rel, mad)
    # replaying the graph gives what the eager fused path gave
    assert torch.allclose(got_graph, got_fused, atol=2e-3, rtol=2e-3)
    # greedy continuation runs and is reproducible
    r1 = decode.benchmark(lut, ids, generate=4, warmup=1)
    r2 = decode.benchmark(lut, ids, generate=4, warmup=1)
    assert r1["generated"].shape == (2, 4) and torch.equal(r1["generated"], r2["generated"])
    assert r1["median_s_per_token"] > 0


def test_captured_graph_survives_workspace_growth(gpu_device):
    """A graph captured on a stream keeps working after a larger problem on the same
    stream made the library outgrow the K-split workspace the graph points at."""
    lib = native.cabi()
    small = workload.make_rowwise_problem(512, 1024, nb=3, M=1, seed=21, device=gpu_device, quantize=False)
    big = workload.make_rowwise_problem(8192, 1024, nb=2, M=40, seed=22, device=gpu_device, quantize=False)
    want, _ = orc.gemv_rowwise_c(small.bW.cpu().numpy(), small.alpha.cpu().numpy(), small.x.cpu().numpy(),
                                 small.num_groups)
    stream = torch.cuda.Stream()
    sp = ctypes.c_void_p(stream.cuda_stream)
    out = torch.zeros((1, 512), dtype=torch.float16, device=gpu_device)
    p = lambda t: ctypes.c_void_p(t.data_ptr())

    def call(pr, o):
        rc = lib.lutgemm_gemv_rowwise_f16(p(pr.bW), p(pr.alpha), p(pr.x), p(o), pr.N, pr.K, pr.nb, pr.num_groups,
                                          pr.x.shape[0], sp)
        assert rc == 0, lib.lutgemm_strerror(rc).decode()

    with torch.cuda.stream(stream):
        call(small, out)                                  # sizes the stream's workspace
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        call(small, out)
    big_out = torch.zeros((40, 8192), dtype=torch.float16, device=gpu_device)
    with torch.cuda.stream(stream):
        call(big, big_out)                                # 40 x 8192 words: larger than the first allocation
    stream.synchronize()
    for _ in range(3):
        with torch.cuda.stream(stream):
            out.zero_()
            graph.replay()
        stream.synchronize()
        _assert_close(out, want, "replay after growth")


def test_grouped_launch_rejects_overlapping_outputs(gpu_device):
    lib = native.cabi()
    a = workload.make_rowwise_problem(256, 256, nb=2, seed=1, device=gpu_device, quantize=False)
    out = torch.zeros((1, 512), dtype=torch.float16, device=gpu_device)
    arr = (native.RowwiseProblem * 2)()
    for i, off in enumerate((0, 128)):                      # second output starts inside the first
        arr[i] = native.RowwiseProblem(a.bW.data_ptr(), a.alpha.data_ptr(), a.x.data_ptr(), out.data_ptr() + 2 * off,
                                       256, 256, 2, a.num_groups, 1)
    assert lib.lutgemm_gemv_rowwise_f16_grouped(2, arr, _stream()) == -1
    arr[1].out_f16 = out.data_ptr() + 2 * 256               # adjacent is fine
    assert lib.lutgemm_gemv_rowwise_f16_grouped(2, arr, _stream()) == 0
    torch.cuda.synchronize()
    assert torch.equal(out[:, :256], out[:, 256:])


@pytest.mark.parametrize("N,K,nb", [(28672, 8192, 4), (8192, 28672, 2)])
def test_config5_largest_shapes_by_size_independent_properties(gpu_device, N, K, nb):
    """The two largest 70B shapes, too big for the scalar oracle within the suite's
    budget: exact columns for unit vectors (the dequantised entry is computed from the
    sign bit and the alphas directly), for the look-up kernel (1 row) and the
    matrix-core kernel (6 and 20 rows); linearity; rows of a batch against single rows."""
    g = torch.Generator(device=gpu_device).manual_seed(N + nb)
    bW = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 32, nb, N), generator=g, device=gpu_device, dtype=torch.int32)
    e = torch.randint(-9, -5, (K // 128, 1, N), generator=g, device=gpu_device).float()
    alpha = torch.exp2(e - torch.arange(nb, device=gpu_device).float().view(1, nb, 1)).half().contiguous()
    lib = native.cabi()
    vp = lambda t: ctypes.c_void_p(t.data_ptr())

    def call(x):
        out = torch.zeros((x.shape[0], N), dtype=torch.float16, device=gpu_device)
        rc = lib.lutgemm_gemv_rowwise_f16(vp(bW), vp(alpha), vp(x), vp(out), N, K, nb, K // 128, x.shape[0], _stream())
        assert rc == 0, lib.lutgemm_strerror(rc).decode()
        torch.cuda.synchronize()
        return out

    def column(k):          # W_q[:, k] = sum_b alpha[k // 128][b] * (2 * bit - 1), exact in fp16 here
        bits = (bW[k // 32] >> (k % 32)) & 1                          # [nb, N]
        return ((2 * bits - 1).float() * alpha[k // 128].float()).sum(dim=0)

    ks = [0, 31, 32, 127, 128, K // 2 + 5, K - 33, K - 1]
    for rows in (1, 6, 20):
        pick = (ks * 3)[:rows]
        x = torch.zeros((rows, K), dtype=torch.float16, device=gpu_device)
        for i, k in enumerate(pick):
            x[i, k] = 1.0
        got = call(x).float()
        for i, k in enumerate(pick):
            assert torch.equal(got[i], column(k)), (rows, i, k)
    # linearity and batch/single agreement on random activations
    x1 = torch.randn((1, K), generator=g, device=gpu_device).half()
    x2 = torch.randn((1, K), generator=g, device=gpu_device).half()
    y1, y2 = call(x1).float(), call(x2).float()
    y12 = call((x1.float() + x2.float()).half()).float()
    rel, _ = orc.error_metrics((y1 + y2).cpu().numpy(), y12.cpu().numpy())
    assert rel < 3e-3
    both = call(torch.cat([x1, x2, x1, x2, x1])).float()               # 5 rows: matrix-core kernel
    for i, y in enumerate((y1, y2, y1, y2, y1)):
        rel, _ = orc.error_metrics(both[i:i + 1].cpu().numpy(), y.cpu().numpy())
        assert rel <= 2e-4, (i, rel)


@pytest.mark.parametrize("batch", [1, 8])
def test_decoder_full_width_hip_glue_matches_framework_glue(gpu_device, batch):
    """Two Llama-2-7B-sized blocks (hidden 4096, intermediate 11008, 32 heads of 128):
    the fused decode step (graph replay) against the same step spelt in framework
    operations over the same LutLinear layers, at the real shapes."""
    from shiftaddllm_amd import decode
    cfg = decode.DecoderConfig(vocab_size=2048, layers=2, max_positions=64)
    qc = workload.mixed_bit_config(cfg.layers, seed=1)
    ids = torch.randint(0, cfg.vocab_size, (batch, 5), generator=torch.Generator().manual_seed(2))
    outs = {}
    for glue in ("hip", "torch"):
        model = decode.LutDecoder(cfg, qc, batch=batch, seed=7, device=gpu_device, glue=glue)
        if glue == "hip":
            model.capture()
        model.reset()
        seq = [model.forward_token(ids[:, t].to(gpu_device), t).float().cpu().clone() for t in range(ids.shape[1])]
        torch.cuda.synchronize()
        outs[glue] = torch.stack(seq)
        del model
    rel, mad = orc.error_metrics(outs["hip"].numpy().reshape(-1, cfg.vocab_size),
                                 outs["torch"].numpy().reshape(-1, cfg.vocab_size))
    assert rel <= 5e-3 and mad <= 2e-2, (rel, mad)       # two fp16 networks with differently rounded glue
