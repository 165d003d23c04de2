"""Parity with the CPU oracle at the full BASELINE sizes, through the C ABI on the GPU.

Operands are built as packed sign words directly (random words, power-of-two alphas
halving per bit plane): the oracle consumes packed words, so nothing of size
N x K x nb has to be materialised, and its scalar C loop does the largest batch-1
case (28672 x 8192, 4 bits: 117 M look-ups) in a fraction of a second.  Same bars as
tests/test_gpu_parity.py: rel-L2 <= 2e-3 and max|dy| <= 1e-2 max|y_ref| on the fp16
output, held to a tenth of that.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle as orc
from shiftaddllm_amd import native, workload

pytestmark = pytest.mark.gpu

REL_L2_BAR, MAX_ABS_BAR, TIGHT = 2e-3, 1e-2, 0.1


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _assert_close(y_gpu, y_ref, what, margin=TIGHT):
    rel, mad = orc.error_metrics(y_gpu.float().cpu().numpy(), np.asarray(y_ref, dtype=np.float32))
    assert rel <= REL_L2_BAR * margin and mad <= MAX_ABS_BAR * margin, (what, rel, mad)


def packed_rowwise(N, K, nb, M, seed, group=128):
    g = torch.Generator().manual_seed(seed)
    bW = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 32, nb, N), generator=g, dtype=torch.int32)
    e = torch.randint(-9, -5, (K // group, 1, N), generator=g).float() - torch.arange(nb).float().view(1, nb, 1)
    alpha = torch.exp2(e).to(torch.float16).contiguous()
    x = torch.randn((M, K), generator=g).half()
    return bW, alpha, x


def run_rowwise(dev, bW, alpha, x, group=128):
    N, K, nb, M = bW.shape[2], bW.shape[0] * 32, bW.shape[1], x.shape[0]
    d = [t.to(dev) for t in (bW, alpha, x)]
    out = torch.zeros((M, N), dtype=torch.float16, device=dev)
    rc = native.cabi().lutgemm_gemv_rowwise_f16(_ptr(d[0]), _ptr(d[1]), _ptr(d[2]), _ptr(out), N, K, nb, K // group, M,
                                                _stream())
    assert rc == 0, native.cabi().lutgemm_strerror(rc).decode()
    torch.cuda.synchronize()
    return out


# ---- config 5: Llama-2-70B shapes, 2 and 4 bits -------------------------------------

LLAMA70B = [(8192, 8192), (28672, 8192), (8192, 28672), (1024, 8192)]


@pytest.mark.parametrize("nb", [2, 4])
@pytest.mark.parametrize("N,K", LLAMA70B)
def test_config5_every_shape_one_row(gpu_device, N, K, nb):
    print(f"config5 N={N} K={K} nb={nb} M=1", flush=True)
    bW, alpha, x = packed_rowwise(N, K, nb, 1, seed=N + K + nb)
    want, _ = orc.gemv_rowwise_c(bW.numpy(), alpha.numpy(), x.numpy(), K // 128)
    _assert_close(run_rowwise(gpu_device, bW, alpha, x), want, (N, K, nb))


@pytest.mark.parametrize("M", [4, 16, 32])
@pytest.mark.parametrize("N,K,nb", [(8192, 8192, 2), (8192, 8192, 4), (28672, 8192, 4)])
def test_config5_small_batches_full_size(gpu_device, N, K, nb, M):
    print(f"config5 N={N} K={K} nb={nb} M={M}", flush=True)
    bW, alpha, x = packed_rowwise(N, K, nb, M, seed=N + nb + M)
    want, _ = orc.gemv_rowwise_c(bW.numpy(), alpha.numpy(), x.numpy(), K // 128)
    _assert_close(run_rowwise(gpu_device, bW, alpha, x), want, (N, K, nb, M))


@pytest.mark.parametrize("N,K,nb,M", [(28672, 8192, 2, 32), (8192, 28672, 2, 32), (8192, 28672, 4, 16),
                                      (8192, 28672, 4, 32)])
def test_config5_long_k_and_wide_cells_at_16_and_32_rows(gpu_device, N, K, nb, M):
    """The matrix-core plans of the two largest shapes at 16 and 32 rows (224 K-steps per tile on
    8192 x 28672): a few seconds of scalar oracle each."""
    print(f"config5 N={N} K={K} nb={nb} M={M}", flush=True)
    bW, alpha, x = packed_rowwise(N, K, nb, M, seed=N + nb + M)
    want, _ = orc.gemv_rowwise_c(bW.numpy(), alpha.numpy(), x.numpy(), K // 128)
    _assert_close(run_rowwise(gpu_device, bW, alpha, x), want, (N, K, nb, M))


@pytest.mark.parametrize("N,K,nb,group", [(9000, 8224, 4, 32), (13824, 5120, 4, 128), (25604, 4128, 3, 32)])
def test_ragged_shapes_on_unequal_ranges(gpu_device, N, K, nb, group):
    """More than 24 MB of signs: 512 workgroups whose ranges come in two sizes (the
    workgroup dispatched first on a CU takes the larger share), here with a last tile
    and a last set that are only partly filled."""
    print(f"ragged N={N} K={K} nb={nb}", flush=True)
    bW, alpha, x = packed_rowwise(N, K, nb, 1, seed=N + K, group=group)
    want, _ = orc.gemv_rowwise_c(bW.numpy(), alpha.numpy(), x.numpy(), K // group)
    _assert_close(run_rowwise(gpu_device, bW, alpha, x, group=group), want, (N, K, nb))


# ---- config 3: Llama-2-13B shapes in the integer alpha formats -----------------------

@pytest.mark.parametrize("kind", ["apot_i8", "shift_u16"])
@pytest.mark.parametrize("N,K", workload.LLAMA2_13B_SHAPES)
def test_config3_integer_alpha_formats_full_size(gpu_device, N, K, kind):
    print(f"config3 N={N} K={K} kind={kind}", flush=True)
    nb, R = 2, 8
    g = torch.Generator().manual_seed(N + K)
    bW = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 32, nb, N), generator=g, dtype=torch.int32)
    x = torch.randn((1, K), generator=g).half()
    lib = native.cabi()
    if kind == "apot_i8":
        # what LutLinear.forward passes: three signed exponents per multiplier, -128 = absent
        code = torch.randint(-12, -4, (K // 8, nb, R, 3), generator=g).to(torch.int8)
        code[..., 1:][torch.rand(code[..., 1:].shape, generator=g) < 0.5] = -128
        okind, fn, extra = orc.ALPHA_APOT_I8, lib.lutgemm_gemv_block_apot_i8, (3,)
    else:
        code = torch.randint(0, 512, (K // 8, nb, R), generator=g).to(torch.int16)
        x = (x.float() * 0.002).half()          # multipliers reach 384: keep outputs inside fp16
        okind, fn, extra = orc.ALPHA_SHIFT_U16, lib.lutgemm_gemv_block_shift_u16, (3,)
    want, _ = orc.gemv_block_c(bW.numpy(), code.numpy(), x.numpy(), R, kind=okind)
    d = [t.to(gpu_device) for t in (bW, code, x)]
    out = torch.zeros((1, N), dtype=torch.float16, device=gpu_device)
    rc = fn(_ptr(d[0]), _ptr(d[1]), _ptr(d[2]), _ptr(out), N, K, nb, R, *extra, 1, _stream())
    assert rc == 0, lib.lutgemm_strerror(rc).decode()
    torch.cuda.synchronize()
    _assert_close(out, want, (N, K, kind))


# ---- non-finite inputs ----------------------------------------------------------------

@pytest.mark.parametrize("N,K", [(256, 256), (512, 4096)])      # one workgroup per tile / K split over workgroups
def test_non_finite_activations_never_give_finite_outputs(gpu_device, N, K):
    """NaN stays NaN and an infinite input gives inf or NaN whatever the launch plan: the
    split-K accumulator carries sticky flags instead of saturating."""
    bW, alpha, x = packed_rowwise(N, K, 3, 4, seed=5)
    bW[:] = -1                                      # every sign +1: y[n] = sum_k alpha * x[k] > 0 for x > 0
    x = x.abs()
    x[1, 7] = float("nan")
    x[2, K - 3] = float("inf")
    x[3, 5] = float("inf")
    x[3, K - 9] = float("-inf")
    for rows in ([0, 1, 2, 3], [1], [2], [3]):      # matrix-core kernel, then the look-up kernel row by row
        got = run_rowwise(gpu_device, bW, alpha, x[rows]).float().cpu()
        for i, r in enumerate(rows):
            if r == 0:
                assert torch.isfinite(got[i]).all()
            elif r == 1:
                assert torch.isnan(got[i]).all(), (rows, r)
            else:
                # an infinite input makes its table entries inf or NaN (the entries are formed
                # by adding and subtracting the inputs): never a finite output
                assert (~torch.isfinite(got[i])).all(), (rows, r)


# ---- workspace contract ---------------------------------------------------------------

def test_reserve_then_capture_without_a_warm_up_call(gpu_device):
    """A fresh stream whose workspace was reserved can be captured straight away; without
    the reservation the call is refused with LUTGEMM_ECAPTURE and the capture survives."""
    lib = native.cabi()
    N, K, nb = 2048, 2048, 3
    bW, alpha, x = packed_rowwise(N, K, nb, 1, seed=21)
    want, _ = orc.gemv_rowwise_c(bW.numpy(), alpha.numpy(), x.numpy(), K // 128)
    d = [t.to(gpu_device) for t in (bW, alpha, x)]
    out = torch.zeros((1, N), dtype=torch.float16, device=gpu_device)
    torch.cuda.synchronize()

    def call(stream):
        return lib.lutgemm_gemv_rowwise_f16(_ptr(d[0]), _ptr(d[1]), _ptr(d[2]), _ptr(out), N, K, nb, K // 128, 1,
                                            ctypes.c_void_p(stream.cuda_stream))

    # no reservation: refused, nothing launched, the capture goes on
    s1 = torch.cuda.Stream()
    g1 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g1, stream=s1):
        rc = call(s1)
        out.add_(0)                      # something capturable, so that the graph is not empty
    assert rc == -6, rc
    assert b"reserve" in lib.lutgemm_strerror(rc)

    # reservation on a second fresh stream, then capture without any warm-up call
    s2 = torch.cuda.Stream()
    words = lib.lutgemm_workspace_words(N, 1)
    assert words == N
    assert lib.lutgemm_reserve_workspace(ctypes.c_void_p(s2.cuda_stream), words) == 0
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g2, stream=s2):
        rc = call(s2)
    assert rc == 0, lib.lutgemm_strerror(rc).decode()
    for _ in range(3):                   # the call accumulates: replay it three times from zero
        out.zero_()
        torch.cuda.synchronize()
        g2.replay()
        torch.cuda.synchronize()
        _assert_close(out, want, "replay")


# ---- two full-width decoder blocks against dense fp16 weights --------------------------

@pytest.mark.parametrize("batch", [1, 8])
def test_decoder_full_width_matches_dense_dequantised_blocks(gpu_device, batch):
    """Two Llama-2-7B-sized blocks (hidden 4096, intermediate 11008, 32 heads of 128),
    mixed 2/3/4 bits: the fused decode step (HIP glue, graph replay) against the same
    blocks with every linear a dense matmul on oracle-dequantised weights."""
    from shiftaddllm_amd import decode
    cfg = decode.DecoderConfig(vocab_size=2048, layers=2, max_positions=64)
    qc = workload.mixed_bit_config(cfg.layers, seed=1)
    ids = torch.randint(0, cfg.vocab_size, (batch, 5), generator=torch.Generator().manual_seed(2))

    def run(model):
        model.reset()
        seq = [model.forward_token(ids[:, t].to(gpu_device), t).float().cpu().clone() for t in range(ids.shape[1])]
        torch.cuda.synchronize()
        return torch.stack(seq)

    lut = decode.LutDecoder(cfg, qc, batch=batch, seed=7, device=gpu_device)
    lut.capture()
    got = run(lut)

    dense = decode.LutDecoder(cfg, qc, batch=batch, seed=7, device=gpu_device, fuse_launches=False, glue="torch")
    table = {}
    for blk in dense.blocks:
        for lin in (blk.q_proj, blk.k_proj, blk.v_proj, blk.o_proj, blk.gate_proj, blk.up_proj, blk.down_proj):
            Wq = orc.dequant_rowwise_kernel_layout(lin.binaryWeight.cpu().numpy(), lin.alpha.cpu().numpy())
            table[id(lin)] = torch.from_numpy(Wq).to(gpu_device)
    dense._linears = lambda lins, x: [(x.float() @ table[id(l)].t()).half() for l in lins]
    want = run(dense)
    rel, mad = orc.error_metrics(got.numpy().reshape(-1, cfg.vocab_size), want.numpy().reshape(-1, cfg.vocab_size))
    assert rel <= 5e-3 and mad <= 2e-2, (rel, mad)       # two fp16 networks, differently rounded glue and linears
