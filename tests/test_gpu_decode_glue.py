"""GPU tests of the decode-step glue kernels, called through the C ABI and checked
against plain fp32 torch restatements of the same operations."""
import ctypes
import math

import pytest
import torch

from shiftaddllm_amd import native

pytestmark = pytest.mark.gpu


def _sp():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ok(rc):
    assert rc == 0, native.cabi().lutgemm_strerror(rc).decode()


@pytest.mark.parametrize("rows,hidden", [(1, 4096), (8, 4096), (3, 264), (2, 11008)])
def test_rmsnorm_and_clear(gpu_device, rows, hidden):
    lib = native.cabi()
    g = torch.Generator(device=gpu_device).manual_seed(rows * 131 + hidden)
    x = (torch.randn((rows, hidden), generator=g, device=gpu_device) * 3).half()
    w = (1 + 0.1 * torch.randn((hidden,), generator=g, device=gpu_device)).half()
    y = torch.empty_like(x)
    junk = torch.full((rows * 3 * hidden + 8,), 7.0, dtype=torch.float16, device=gpu_device)
    clear_bytes = (junk.numel() - 8) * 2
    _ok(lib.lutgemm_decode_rmsnorm_f16(x.data_ptr(), w.data_ptr(), y.data_ptr(), rows, hidden, 1e-5,
                                       junk.data_ptr(), clear_bytes, _sp()))
    torch.cuda.synchronize()
    xf = x.float()
    want = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).half().float() * w.float()
    assert torch.allclose(y.float(), want, rtol=2e-3, atol=2e-3)
    assert torch.count_nonzero(junk[:-8]) == 0 and torch.all(junk[-8:] == 7.0)   # cleared exactly the range


def test_rmsnorm_rejects_bad_arguments(gpu_device):
    lib = native.cabi()
    x = torch.zeros((1, 64), dtype=torch.float16, device=gpu_device)
    assert lib.lutgemm_decode_rmsnorm_f16(x.data_ptr(), x.data_ptr(), x.data_ptr(), 1, 60, 1e-5, None, 0, _sp()) == -1
    assert lib.lutgemm_decode_rmsnorm_f16(x.data_ptr(), x.data_ptr(), x.data_ptr(), 1, 64, 1e-5, None, 16, _sp()) == -1
    assert lib.lutgemm_decode_rmsnorm_f16(x.data_ptr() + 2, x.data_ptr(), x.data_ptr(), 1, 32, 1e-5, None, 0,
                                          _sp()) == -2


def _rope(t, cos, sin):
    half = t.shape[-1] // 2
    rot = torch.cat([-t[..., half:], t[..., :half]], dim=-1)
    return t * cos + rot * sin


@pytest.mark.parametrize("B,H,KV,hd,max_pos,positions", [
    (1, 32, 32, 128, 256, (0, 1, 100, 255)),
    (2, 4, 2, 64, 32, (0, 5, 31)),
    (2, 8, 2, 128, 700, (0, 300, 699)),        # more keys than threads in a workgroup
    (1, 4, 4, 96, 40, (0, 17, 39)),            # the generic head-dim path
    (3, 6, 3, 64, 520, (519,)),
    (1, 2, 2, 128, 1100, (256, 257, 512, 1099)),   # either side of the 256-position blocks the kernel walks in
    (1, 2, 1, 64, 1030, (511, 512, 513, 1029)),    # (512 positions a block at this head size)
])
def test_attention_step(gpu_device, B, H, KV, hd, max_pos, positions):
    lib = native.cabi()
    g = torch.Generator(device=gpu_device).manual_seed(B * 1000 + H * 10 + hd)
    inv = 1.0 / (10000.0 ** (torch.arange(0, hd, 2, device=gpu_device).float() / hd))
    ang = torch.arange(max_pos, device=gpu_device).float()[:, None] * inv[None, :]
    cos = torch.cat([ang.cos(), ang.cos()], -1).half()
    sin = torch.cat([ang.sin(), ang.sin()], -1).half()
    for pos in positions:
        kc = torch.randn((B, KV, max_pos, hd), generator=g, device=gpu_device).half()
        vc = torch.randn((B, KV, max_pos, hd), generator=g, device=gpu_device).half()
        kc0, vc0 = kc.clone(), vc.clone()
        q = torch.randn((B, H * hd), generator=g, device=gpu_device).half()
        k = torch.randn((B, KV * hd), generator=g, device=gpu_device).half()
        v = torch.randn((B, KV * hd), generator=g, device=gpu_device).half()
        out = torch.zeros((B, H * hd), dtype=torch.float16, device=gpu_device)
        p = torch.tensor([pos], dtype=torch.long, device=gpu_device)
        _ok(lib.lutgemm_decode_attention_f16(q.data_ptr(), k.data_ptr(), v.data_ptr(), cos.data_ptr(),
                                             sin.data_ptr(), kc.data_ptr(), vc.data_ptr(), p.data_ptr(),
                                             out.data_ptr(), B, H, KV, hd, max_pos, _sp()))
        torch.cuda.synchronize()
        # fp32 restatement
        c, s = cos[pos].float(), sin[pos].float()
        qr = _rope(q.float().view(B, H, hd), c, s).half().float()
        kr = _rope(k.float().view(B, KV, hd), c, s).half()
        want_k, want_v = kc0.clone(), vc0.clone()
        want_k[:, :, pos] = kr
        want_v[:, :, pos] = v.view(B, KV, hd)
        assert torch.equal(vc, want_v)
        assert torch.allclose(kc.float(), want_k.float(), rtol=2e-3, atol=2e-3)
        assert torch.equal(kc[:, :, pos + 1:], kc0[:, :, pos + 1:]) and torch.equal(kc[:, :, :pos], kc0[:, :, :pos])
        keys = want_k[:, :, :pos + 1].float().repeat_interleave(H // KV, dim=1)       # [B, H, T, hd]
        vals = want_v[:, :, :pos + 1].float().repeat_interleave(H // KV, dim=1)
        att = torch.softmax(torch.einsum("bhd,bhtd->bht", qr, keys) / math.sqrt(hd), dim=-1)
        want = torch.einsum("bht,bhtd->bhd", att, vals).reshape(B, H * hd)
        assert torch.allclose(out.float(), want, rtol=5e-3, atol=5e-3), (pos, (out.float() - want).abs().max())


def test_attention_rejects_bad_arguments(gpu_device):
    lib = native.cabi()
    t = torch.zeros((4096,), dtype=torch.float16, device=gpu_device)
    p = torch.zeros((1,), dtype=torch.long, device=gpu_device)
    a = t.data_ptr()
    call = lambda B, H, KV, hd, mp: lib.lutgemm_decode_attention_f16(a, a, a, a, a, a, a, p.data_ptr(), a, B, H, KV,
                                                                     hd, mp, _sp())
    assert call(1, 4, 3, 64, 16) == -1        # heads not a multiple of kv heads
    assert call(1, 4, 4, 60, 16) == -1        # head dim not a multiple of 8
    assert call(1, 4, 4, 512, 16) == -1       # head dim too large
    assert call(1, 4, 4, 64, 10000) == -1     # more positions than the kernel's LDS budget


@pytest.mark.parametrize("count", [8, 11008, 8 * 11008, 4104])
def test_silu_mul(gpu_device, count):
    lib = native.cabi()
    g = torch.Generator(device=gpu_device).manual_seed(count)
    gate = (torch.randn((count,), generator=g, device=gpu_device) * 4).half()
    up = torch.randn((count,), generator=g, device=gpu_device).half()
    out = torch.empty_like(gate)
    _ok(lib.lutgemm_decode_silu_mul_f16(gate.data_ptr(), up.data_ptr(), out.data_ptr(), count, _sp()))
    torch.cuda.synchronize()
    want = torch.nn.functional.silu(gate.float()).half().float() * up.float()
    assert torch.allclose(out.float(), want, rtol=2e-3, atol=1e-3)
    assert lib.lutgemm_decode_silu_mul_f16(gate.data_ptr(), up.data_ptr(), out.data_ptr(), count + 1, _sp()) == -1


# ---- element-wise work folded into the row-wise GEMV ------------------------------------

def _fused_call(lib, lins, x, outs, norm=None, gate=None, overwrite=False, eps=1e-5):
    arr = (native.FusedProblem * len(lins))()
    for i, ((bW, alpha, N, K, nb), o) in enumerate(zip(lins, outs)):
        arr[i] = native.FusedProblem(bW.data_ptr(), alpha.data_ptr(), x.data_ptr(), o.data_ptr(), N, K, nb, K // 128,
                                     x.shape[0], int(overwrite), norm.data_ptr() if norm is not None else None,
                                     gate.data_ptr() if gate is not None else None, eps)
    return lib.lutgemm_gemv_rowwise_f16_fused(len(lins), arr, _sp())


def _random_lin(gpu_device, N, K, nb, seed):
    g = torch.Generator(device=gpu_device).manual_seed(seed)
    bW = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 32, nb, N), generator=g, device=gpu_device, dtype=torch.int32)
    e = torch.randint(-8, -5, (K // 128, 1, N), generator=g, device=gpu_device).float()
    alpha = torch.exp2(e - torch.arange(nb, device=gpu_device).float().view(1, nb, 1)).half().contiguous()
    return bW, alpha, N, K, nb


def _plain(lib, lin, x, out):
    bW, alpha, N, K, nb = lin
    _ok(lib.lutgemm_gemv_rowwise_f16(bW.data_ptr(), alpha.data_ptr(), x.data_ptr(), out.data_ptr(), N, K, nb,
                                     K // 128, x.shape[0], _sp()))


@pytest.mark.parametrize("M,K,Ns,nbs", [(1, 4096, (4096, 1024, 1024), (3, 2, 4)), (2, 1024, (512, 2752), (3, 3)),
                                          (5, 512, (256,), (2,))])
def test_fused_rmsnorm_gemv_equals_separate_kernels(gpu_device, M, K, Ns, nbs):
    """norm folded into the GEMV == rmsnorm kernel followed by the plain GEMV, and both
    agree with the oracle on the normalised input."""
    import numpy as np
    import oracle as orc
    lib = native.cabi()
    g = torch.Generator(device=gpu_device).manual_seed(M * 7 + K)
    x = (torch.randn((M, K), generator=g, device=gpu_device) * 2.5).half()
    w = (1 + 0.2 * torch.randn((K,), generator=g, device=gpu_device)).half()
    lins = [_random_lin(gpu_device, N, K, nb, 11 * i + N) for i, (N, nb) in enumerate(zip(Ns, nbs))]
    h = torch.empty_like(x)
    _ok(lib.lutgemm_decode_rmsnorm_f16(x.data_ptr(), w.data_ptr(), h.data_ptr(), M, K, 1e-5, None, 0, _sp()))
    want = [torch.zeros((M, N), dtype=torch.float16, device=gpu_device) for N in Ns]
    for lin, o in zip(lins, want):
        _plain(lib, lin, h, o)
    got = [torch.full((M, N), 9.0, dtype=torch.float16, device=gpu_device) for N in Ns]     # overwritten
    _ok(_fused_call(lib, lins, x, got, norm=w, overwrite=True))
    torch.cuda.synchronize()
    for lin, a, b in zip(lins, got, want):
        assert torch.allclose(a.float(), b.float(), rtol=2e-3, atol=2e-3 * float(b.float().abs().max()))
        ref, _ = orc.gemv_rowwise_c(lin[0].cpu().numpy(), lin[1].cpu().numpy(), h.cpu().numpy(), K // 128)
        rel, mad = orc.error_metrics(a.float().cpu().numpy(), ref.astype(np.float32))
        assert rel <= 2e-3 and mad <= 1e-2, (rel, mad)


@pytest.mark.parametrize("M,K,N,nb", [(1, 11008, 4096, 3), (2, 1408, 512, 4), (4, 512, 256, 2),
                                        (8, 11008, 4096, 3), (33, 1024, 528, 4)])    # several rows: matrix-core kernel
def test_fused_swiglu_gemv_equals_separate_kernels(gpu_device, M, K, N, nb):
    lib = native.cabi()
    g = torch.Generator(device=gpu_device).manual_seed(M * 13 + K)
    gate = (torch.randn((M, K), generator=g, device=gpu_device) * 2).half()
    up = torch.randn((M, K), generator=g, device=gpu_device).half()
    res = torch.randn((M, N), generator=g, device=gpu_device).half()
    lin = _random_lin(gpu_device, N, K, nb, 5)
    act = torch.empty_like(up)
    _ok(lib.lutgemm_decode_silu_mul_f16(gate.data_ptr(), up.data_ptr(), act.data_ptr(), M * K, _sp()))
    want = res.clone()
    _plain(lib, lin, act, want)
    got = res.clone()
    _ok(_fused_call(lib, [lin], up, [got], gate=gate))                 # accumulates into the residual
    torch.cuda.synchronize()
    if M == 1:
        assert torch.equal(got, want)                                  # same inputs, same plan: same bits
    else:                                                              # the plain call took the matrix-core kernel
        assert torch.allclose(got.float(), want.float(), rtol=2e-3, atol=2e-3 * float(want.float().abs().max()))


def test_fused_entry_point_rejects_bad_problems(gpu_device):
    lib = native.cabi()
    lin = _random_lin(gpu_device, 256, 512, 2, 1)
    x = torch.zeros((1, 512), dtype=torch.float16, device=gpu_device)
    o = torch.zeros((1, 256), dtype=torch.float16, device=gpu_device)
    assert _fused_call(lib, [lin], x, [o], norm=x, gate=x) == -1       # both transforms
    assert _fused_call(lib, [lin], x, [o], norm=x, eps=-1.0) == -1
    arr = (native.FusedProblem * 1)()
    assert lib.lutgemm_gemv_rowwise_f16_fused(0, arr, _sp()) == -1
    assert lib.lutgemm_gemv_rowwise_f16_fused(native.MAX_GROUP + 1, arr, _sp()) == -1


@pytest.mark.parametrize("M", [1, 2, 8, 20])
def test_overwrite_mode_ignores_previous_output(gpu_device, M):
    lib = native.cabi()
    g = torch.Generator(device=gpu_device).manual_seed(M)
    x = torch.randn((M, 1024), generator=g, device=gpu_device).half()
    lins = [_random_lin(gpu_device, N, 1024, nb, 3 * N) for N, nb in ((512, 3), (1024, 2))]
    want = [torch.zeros((M, l[2]), dtype=torch.float16, device=gpu_device) for l in lins]
    for l, o in zip(lins, want):
        _plain(lib, l, x, o)
    got = [torch.full((M, l[2]), float("nan"), dtype=torch.float16, device=gpu_device) for l in lins]
    _ok(_fused_call(lib, lins, x, got, overwrite=True))
    torch.cuda.synchronize()
    for a, b in zip(got, want):
        assert torch.allclose(a.float(), b.float(), rtol=2e-3, atol=2e-3 * float(b.float().abs().max()))


# ---- RMSNorm split over the completing and the consuming GEMV ---------------------------

def _split_call(lib, lin, x, out, M, **kw):
    bW, alpha, N, K, nb = lin
    ptr = lambda t: t.data_ptr() if t is not None else None
    arr = (native.FusedProblem * 1)()
    arr[0] = native.FusedProblem(bW.data_ptr(), alpha.data_ptr(), x.data_ptr(), out.data_ptr(), N, K, nb, K // 128, M,
                                 int(kw.get("overwrite", False)), None, ptr(kw.get("gate")), 1e-5,
                                 ptr(kw.get("next_norm")), ptr(kw.get("next_in")), ptr(kw.get("sumsq_out")),
                                 ptr(kw.get("sumsq_in")), kw["sumsq_in"].shape[-1] if kw.get("sumsq_in") is not None else 0)
    return lib.lutgemm_gemv_rowwise_f16_fused(1, arr, _sp())


@pytest.mark.parametrize("M", [1, 2, 8, 20])                 # look-up kernel (1, 2 rows), matrix cores (16- and 32-row tiles)
@pytest.mark.parametrize("N,K,N2,nb", [(1024, 2048, 768, 3), (4096, 1408 - 1408 % 128, 512, 4)])
def test_split_rmsnorm_equals_separate_kernels(gpu_device, M, N, K, N2, nb):
    """GEMV 1 completes a residual row and leaves (row * weight, sums of squares); GEMV 2
    reads those: together they equal GEMV, rmsnorm kernel, GEMV."""
    lib = native.cabi()
    g = torch.Generator(device=gpu_device).manual_seed(M * 31 + N)
    a = torch.randn((M, K), generator=g, device=gpu_device).half()
    res = (torch.randn((M, N), generator=g, device=gpu_device) * 3).half()
    w = (1 + 0.2 * torch.randn((N,), generator=g, device=gpu_device)).half()
    lin1, lin2 = _random_lin(gpu_device, N, K, nb, 3), _random_lin(gpu_device, N2, N, 3, 4)

    # separate kernels
    x_ref = res.clone()
    _plain(lib, lin1, a, x_ref)
    h_ref = torch.empty_like(x_ref)
    _ok(lib.lutgemm_decode_rmsnorm_f16(x_ref.data_ptr(), w.data_ptr(), h_ref.data_ptr(), M, N, 1e-5, None, 0, _sp()))
    y_ref = torch.zeros((M, N2), dtype=torch.float16, device=gpu_device)
    _plain(lib, lin2, h_ref, y_ref)

    # split norm
    x = res.clone()
    nxt = torch.full((M, N), 7.0, dtype=torch.float16, device=gpu_device)
    sumsq = torch.zeros((M, N // 32), dtype=torch.float32, device=gpu_device)
    _ok(_split_call(lib, lin1, a, x, M, next_norm=w, next_in=nxt, sumsq_out=sumsq))
    y = torch.full((M, N2), 9.0, dtype=torch.float16, device=gpu_device)
    _ok(_split_call(lib, lin2, nxt, y, M, overwrite=True, sumsq_in=sumsq))
    torch.cuda.synchronize()

    assert torch.allclose(x.float(), x_ref.float(), rtol=2e-3, atol=2e-3 * float(x_ref.float().abs().max()))
    assert torch.equal(nxt, (x.float() * w.float()).half())                    # one rounding of an exact product
    want_sq = x.float().pow(2).sum(-1)
    assert torch.allclose(sumsq.sum(-1), want_sq, rtol=1e-5)
    assert torch.allclose(y.float(), y_ref.float(), rtol=4e-3, atol=4e-3 * float(y_ref.float().abs().max()))


def test_split_rmsnorm_with_swiglu_input_and_bad_arguments(gpu_device):
    lib = native.cabi()
    g = torch.Generator(device=gpu_device).manual_seed(77)
    M, N, K = 1, 512, 1408 - 1408 % 128
    gate = torch.randn((M, K), generator=g, device=gpu_device).half()
    up = torch.randn((M, K), generator=g, device=gpu_device).half()
    res = torch.randn((M, N), generator=g, device=gpu_device).half()
    w = (1 + 0.2 * torch.randn((N,), generator=g, device=gpu_device)).half()
    lin = _random_lin(gpu_device, N, K, 2, 9)
    want = res.clone()
    _ok(_fused_call(lib, [lin], up, [want], gate=gate))
    x, nxt = res.clone(), torch.empty((M, N), dtype=torch.float16, device=gpu_device)
    sumsq = torch.zeros((M, N // 32), dtype=torch.float32, device=gpu_device)
    _ok(_split_call(lib, lin, up, x, M, gate=gate, next_norm=w, next_in=nxt, sumsq_out=sumsq))
    torch.cuda.synchronize()
    assert torch.equal(x, want)
    assert torch.equal(nxt, (x.float() * w.float()).half())
    assert torch.allclose(sumsq.sum(-1), x.float().pow(2).sum(-1), rtol=1e-5)
    # the weight and the destination of the weighted copy come together
    assert _split_call(lib, lin, up, x, M, next_in=nxt) == -1
    assert _split_call(lib, lin, up, x, M, next_norm=w) == -1
    # slots of 32 columns
    lin_odd = _random_lin(gpu_device, 528, K, 2, 9)
    x_odd = torch.zeros((M, 528), dtype=torch.float16, device=gpu_device)
    assert _split_call(lib, lin_odd, up, x_odd, M, sumsq_out=sumsq) == -1


# ---- the fused entry point directly against the oracle on numpy-transformed inputs ------

def _np_lin(lin):
    return lin[0].cpu().numpy(), lin[1].cpu().numpy()


@pytest.mark.parametrize("M", [1, 2])
def test_fused_norm_gate_and_overwrite_against_the_oracle(gpu_device, M):
    """RMSNorm input, SiLU(gate) * x input and overwrite, each checked against the scalar oracle fed
    with inputs transformed in numpy (nothing of the library on the reference side)."""
    import numpy as np
    import oracle as orc
    lib = native.cabi()
    K, N, eps = 2048, 768, 1e-5
    g = torch.Generator(device=gpu_device).manual_seed(900 + M)
    x = (torch.randn((M, K), generator=g, device=gpu_device) * 2.5).half()
    w = (1 + 0.2 * torch.randn((K,), generator=g, device=gpu_device)).half()
    gate = (torch.randn((M, K), generator=g, device=gpu_device) * 2).half()
    lin = _random_lin(gpu_device, N, K, 3, 17)
    bW, alpha = _np_lin(lin)
    xn, wn, gn = x.cpu().numpy().astype(np.float32), w.cpu().numpy().astype(np.float32), gate.cpu().numpy().astype(np.float32)

    # RMSNorm folded in: tables of fp16(x * weight), sums scaled by the row's reciprocal RMS; overwrite
    got = torch.full((M, N), float("nan"), dtype=torch.float16, device=gpu_device)
    _ok(_fused_call(lib, [lin], x, [got], norm=w, overwrite=True, eps=eps))
    torch.cuda.synchronize()
    h = (xn * wn).astype(np.float16)
    _, y32 = orc.gemv_rowwise_c(bW, alpha, h, K // 128)
    scale = 1.0 / np.sqrt((xn.astype(np.float64) ** 2).mean(-1, keepdims=True) + eps)
    rel, mad = orc.error_metrics(got.float().cpu().numpy(), (y32 * scale).astype(np.float32))
    assert rel <= 2e-3 and mad <= 1e-2, ("norm", rel, mad)

    # SiLU(gate) * x with the roundings of the separate fp16 operations; accumulates into a residual
    res = torch.randn((M, N), generator=g, device=gpu_device).half()
    got = res.clone()
    _ok(_fused_call(lib, [lin], x, [got], gate=gate))
    torch.cuda.synchronize()
    silu = (gn / (1.0 + np.exp(-gn))).astype(np.float16).astype(np.float32)
    act = (silu * xn).astype(np.float16)
    want, _ = orc.gemv_rowwise_c(bW, alpha, act, K // 128, out=res.cpu().numpy())
    rel, mad = orc.error_metrics(got.float().cpu().numpy(), want.astype(np.float32))
    assert rel <= 2e-3 and mad <= 1e-2, ("gate", rel, mad)


@pytest.mark.parametrize("M", [1, 8])                        # look-up kernel, matrix-core kernel
def test_split_norm_fields_against_the_oracle(gpu_device, M):
    """Completing side: out += W a, next_input = fp16(out * weight), sums of squares of out.
    Consuming side: y = rsqrt(sum / K + eps) * W next_input.  Both against the scalar oracle."""
    import numpy as np
    import oracle as orc
    lib = native.cabi()
    K, N, N2, eps = 1024, 2048, 512, 1e-5
    g = torch.Generator(device=gpu_device).manual_seed(950 + M)
    a = torch.randn((M, K), generator=g, device=gpu_device).half()
    res = (torch.randn((M, N), generator=g, device=gpu_device) * 3).half()
    w = (1 + 0.2 * torch.randn((N,), generator=g, device=gpu_device)).half()
    lin1, lin2 = _random_lin(gpu_device, N, K, 3, 23), _random_lin(gpu_device, N2, N, 2, 29)

    x = res.clone()
    nxt = torch.full((M, N), 7.0, dtype=torch.float16, device=gpu_device)
    sumsq = torch.zeros((M, N // 32), dtype=torch.float32, device=gpu_device)
    _ok(_split_call(lib, lin1, a, x, M, next_norm=w, next_in=nxt, sumsq_out=sumsq))
    y = torch.full((M, N2), float("nan"), dtype=torch.float16, device=gpu_device)
    _ok(_split_call(lib, lin2, nxt, y, M, overwrite=True, sumsq_in=sumsq))
    torch.cuda.synchronize()

    want_x, _ = orc.gemv_rowwise_c(*_np_lin(lin1), a.cpu().numpy(), K // 128, out=res.cpu().numpy())
    rel, mad = orc.error_metrics(x.float().cpu().numpy(), want_x.astype(np.float32))
    assert rel <= 2e-3 and mad <= 1e-2, ("completing", rel, mad)
    # derived from the outputs the GPU rounded: exact
    xg = x.cpu().numpy().astype(np.float32)
    assert np.array_equal(nxt.cpu().numpy(), (xg * w.cpu().numpy().astype(np.float32)).astype(np.float16))
    np.testing.assert_allclose(sumsq.sum(-1).cpu().numpy(), (xg.astype(np.float64) ** 2).sum(-1), rtol=1e-5)
    _, y32 = orc.gemv_rowwise_c(*_np_lin(lin2), nxt.cpu().numpy(), N // 128)
    scale = 1.0 / np.sqrt((xg.astype(np.float64) ** 2).sum(-1, keepdims=True) / N + eps)
    rel, mad = orc.error_metrics(y.float().cpu().numpy(), (y32 * scale).astype(np.float32))
    assert rel <= 2e-3 and mad <= 1e-2, ("consuming", rel, mad)
