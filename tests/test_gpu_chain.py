"""Chained launches on the GPU, through the C ABI: row-wise GEMVs that read each other's outputs
inside ONE kernel launch, handing activations over through tagged rows.

Checked against the same GEMVs as separate launches of the fused entry point (which have their
own oracle tests), against the scalar oracle directly, over graph replays with an advancing epoch,
and on the path where a wait gives up because nothing ever writes the row it waits for.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle as orc
from shiftaddllm_amd import native

pytestmark = pytest.mark.gpu

EPS = 1e-5


def _sp():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ok(rc):
    assert rc == 0, native.cabi().lutgemm_strerror(rc).decode()


def _lin(dev, N, K, nb, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    bW = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 32, nb, N), generator=g, device=dev, dtype=torch.int32)
    e = torch.randint(-8, -5, (K // 128, 1, N), generator=g, device=dev).float()
    alpha = torch.exp2(e - torch.arange(nb, device=dev).float().view(1, nb, 1)).half().contiguous()
    return bW, alpha, N, K, nb


def _fused(lin, x, out, M, norm=None, gate=None, overwrite=False):
    bW, alpha, N, K, nb = lin
    ptr = lambda t: t.data_ptr() if t is not None else None
    return native.FusedProblem(bW.data_ptr(), alpha.data_ptr(), x.data_ptr(), out.data_ptr(), N, K, nb, K // 128, M,
                               int(overwrite), ptr(norm), ptr(gate), EPS)


def _chain_problem(lin, x, out, M, x_tag=0, gate_tag=0, out_tag=0, **kw):
    return native.ChainProblem(_fused(lin, x, out, M, **kw), x_tag, gate_tag, out_tag)


class Sync:
    """Epoch and status words of a chain in device memory."""

    def __init__(self, dev, spin_us=0):
        self.words = torch.zeros(2, dtype=torch.int32, device=dev)
        self.ctl = native.ChainControl(self.words.data_ptr(), self.words.data_ptr() + 4, spin_us)

    def status(self):
        return native.cabi().lutgemm_chain_status(self.words.data_ptr() + 4, _sp())

    def advance(self, by):
        _ok(native.cabi().lutgemm_chain_advance_epoch(self.words.data_ptr(), by, _sp()))


def _chain(problems, sync):
    arr = (native.ChainProblem * len(problems))(*problems)
    return native.cabi().lutgemm_gemv_rowwise_f16_chain(len(problems), arr, ctypes.byref(sync.ctl), _sp())


def _tag(dst, src, tag, sync):
    _ok(native.cabi().lutgemm_chain_tag_rows(dst.data_ptr(), src.data_ptr(), src.numel(), tag, sync.words.data_ptr(), _sp()))


def _untag(src):
    out = torch.empty(src.shape, dtype=torch.float16, device=src.device)
    _ok(native.cabi().lutgemm_chain_untag_rows(out.data_ptr(), src.data_ptr(), src.numel(), _sp()))
    return out


def _separate(lib, problems):
    """The same GEMVs one launch each, in order, through the fused entry point."""
    for f in problems:
        arr = (native.FusedProblem * 1)(f)
        _ok(lib.lutgemm_gemv_rowwise_f16_fused(1, arr, _sp()))


def _close(a, b, what, tol=2e-3):
    a, b = a.float(), b.float()
    assert torch.allclose(a, b, rtol=tol, atol=tol * float(b.abs().max())), (what, float((a - b).abs().max()))


def test_tag_and_untag_round_trip(gpu_device):
    sync = Sync(gpu_device)
    src = torch.randn((3, 1000), device=gpu_device).half()
    tagged = torch.zeros((3, 1000), dtype=torch.int32, device=gpu_device)
    _tag(tagged, src, 7, sync)
    torch.cuda.synchronize()
    assert torch.equal(_untag(tagged), src)
    assert torch.all((tagged >> 16) & 0xffff == 8)          # effective tag = 1 + (7 + epoch 0) % 65535
    sync.advance(65535 - 7)                                 # wraps: base 7 + epoch 65528 = 65535 -> 0 -> tag 1
    _tag(tagged, src, 7, sync)
    torch.cuda.synchronize()
    assert torch.all((tagged >> 16) & 0xffff == 1)


@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("hidden,inter,nbs", [(1024, 2752 - 2752 % 128, (3, 2, 4, 3, 2, 3, 4)), (4096, 11008, (3, 3, 3, 3, 3, 3, 3))])
def test_decoder_block_as_one_chain(gpu_device, M, hidden, inter, nbs):
    """o_proj -> (gate, up) -> down_proj -> (q, k, v of the next block) as ONE launch: the residual row
    is a tagged row that o_proj and down_proj complete one after the other; gate/up and q/k/v form
    their RMSNorm from it; down_proj reads the tagged gate and up rows."""
    lib, dev = native.cabi(), gpu_device
    g = torch.Generator(device=dev).manual_seed(hidden + M)
    H, I = hidden, inter
    att = torch.randn((M, H), generator=g, device=dev).half()
    res = torch.randn((M, H), generator=g, device=dev).half()
    w_post = (1 + 0.2 * torch.randn((H,), generator=g, device=dev)).half()
    w_in = (1 + 0.2 * torch.randn((H,), generator=g, device=dev)).half()
    o, gate, up, down = _lin(dev, H, H, nbs[0], 1), _lin(dev, I, H, nbs[1], 2), _lin(dev, I, H, nbs[2], 3), _lin(dev, H, I, nbs[3], 4)
    q, k, v = _lin(dev, H, H, nbs[4], 5), _lin(dev, H // 4, H, nbs[5], 6), _lin(dev, H // 4, H, nbs[6], 7)

    # separate launches on plain rows
    x = res.clone()
    gbuf, ubuf = torch.empty((M, I), dtype=torch.float16, device=dev), torch.empty((M, I), dtype=torch.float16, device=dev)
    qo, ko, vo = (torch.empty((M, n), dtype=torch.float16, device=dev) for n in (H, H // 4, H // 4))
    _separate(lib, [_fused(o, att, x, M)])
    x_mid = x.clone()
    _separate(lib, [_fused(gate, x, gbuf, M, norm=w_post, overwrite=True), _fused(up, x, ubuf, M, norm=w_post, overwrite=True),
                    _fused(down, ubuf, x, M, gate=gbuf),
                    _fused(q, x, qo, M, norm=w_in, overwrite=True), _fused(k, x, ko, M, norm=w_in, overwrite=True),
                    _fused(v, x, vo, M, norm=w_in, overwrite=True)])
    torch.cuda.synchronize()

    # one chained launch on tagged rows
    sync = Sync(dev)
    xt = torch.zeros((M, H), dtype=torch.int32, device=dev)
    gt, ut = torch.zeros((M, I), dtype=torch.int32, device=dev), torch.zeros((M, I), dtype=torch.int32, device=dev)
    q2, k2, v2 = (torch.full((M, n), float("nan"), dtype=torch.float16, device=dev) for n in (H, H // 4, H // 4))
    _tag(xt, res, 100, sync)
    problems = [_chain_problem(o, att, xt, M, out_tag=1),
                _chain_problem(gate, xt, gt, M, x_tag=1, out_tag=2, norm=w_post, overwrite=True),
                _chain_problem(up, xt, ut, M, x_tag=1, out_tag=3, norm=w_post, overwrite=True),
                _chain_problem(down, ut, xt, M, x_tag=3, gate_tag=2, out_tag=4, gate=gt),
                _chain_problem(q, xt, q2, M, x_tag=4, norm=w_in, overwrite=True),
                _chain_problem(k, xt, k2, M, x_tag=4, norm=w_in, overwrite=True),
                _chain_problem(v, xt, v2, M, x_tag=4, norm=w_in, overwrite=True)]
    print(f"chain block hidden={hidden} inter={inter} M={M}", flush=True)
    _ok(_chain(problems, sync))
    assert sync.status() == 0
    x2 = _untag(xt)
    torch.cuda.synchronize()
    assert torch.all((xt >> 16) & 0xffff == 5)               # every residual value carries down_proj's tag
    _close(_untag(gt), gbuf, "gate")
    _close(_untag(ut), ubuf, "up")
    _close(x2, x, "residual")
    _close(q2, qo, "q")
    _close(k2, ko, "k")
    _close(v2, vo, "v")

    # the first GEMV of the chain against the scalar oracle
    want, _ = orc.gemv_rowwise_c(o[0].cpu().numpy(), o[1].cpu().numpy(), att.cpu().numpy(), H // 128, out=res.cpu().numpy())
    rel, mad = orc.error_metrics(x_mid.float().cpu().numpy(), want.astype(np.float32))
    assert rel <= 2e-3 and mad <= 1e-2
    # and the last ones on the chain's own residual row, normalised in numpy
    xn = x2.float().cpu().numpy()
    h = (xn * w_in.float().cpu().numpy()).astype(np.float16)
    scale = 1.0 / np.sqrt((xn.astype(np.float64) ** 2).mean(-1, keepdims=True) + EPS)
    for lin, got in ((q, q2), (k, k2)):
        _, y32 = orc.gemv_rowwise_c(lin[0].cpu().numpy(), lin[1].cpu().numpy(), h, H // 128)
        rel, mad = orc.error_metrics(got.float().cpu().numpy(), (y32 * scale).astype(np.float32))
        assert rel <= 2e-3 and mad <= 1e-2, (rel, mad)


def test_chain_replays_from_a_graph_with_an_advancing_epoch(gpu_device):
    """A captured chain is replayed with new inputs; the epoch word advances between replays so that
    the rows of the previous replay do not satisfy this replay's waits.  Every replay is checked."""
    lib, dev = native.cabi(), gpu_device
    M, H, I = 1, 1024, 2048
    g = torch.Generator(device=dev).manual_seed(5)
    a, b, c = _lin(dev, H, H, 3, 11), _lin(dev, I, H, 2, 12), _lin(dev, H, I, 4, 13)
    w = (1 + 0.2 * torch.randn((H,), generator=g, device=dev)).half()
    x_in = torch.zeros((M, H), dtype=torch.float16, device=dev)
    res = torch.zeros((M, H), dtype=torch.float16, device=dev)
    sync = Sync(dev)
    xt = torch.zeros((M, H), dtype=torch.int32, device=dev)
    mt = torch.zeros((M, I), dtype=torch.int32, device=dev)
    out = torch.zeros((M, H), dtype=torch.float16, device=dev)
    problems = [_chain_problem(a, x_in, xt, M, out_tag=1),
                _chain_problem(b, xt, mt, M, x_tag=1, out_tag=2, norm=w, overwrite=True),
                _chain_problem(c, mt, out, M, x_tag=2, overwrite=True)]
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())

    def step():
        _tag(xt, res, 50, sync)
        _ok(_chain(problems, sync))
        sync.advance(64)

    with torch.cuda.stream(stream):
        step()                                   # sizes the workspace of the capture stream
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        step()
    for it in range(6):
        x_in.copy_(torch.randn((M, H), generator=g, device=dev).half())
        res.copy_(torch.randn((M, H), generator=g, device=dev).half())
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert sync.status() == 0
        got = out.clone()
        # the same three GEMVs as separate launches
        x1 = res.clone()
        m1 = torch.empty((M, I), dtype=torch.float16, device=dev)
        y1 = torch.empty((M, H), dtype=torch.float16, device=dev)
        _separate(lib, [_fused(a, x_in, x1, M), _fused(b, x1, m1, M, norm=w, overwrite=True), _fused(c, m1, y1, M, overwrite=True)])
        torch.cuda.synchronize()
        _close(got, y1, f"replay {it}")
    assert int(sync.words[0].item()) == 64 * 7


def test_a_wait_that_nothing_satisfies_gives_up_and_is_reported(gpu_device):
    """The second problem waits for a tag that nobody writes (its row comes from outside the call):
    every workgroup gives up after the limit, the kernel ends, the status word says so, and the
    problem that waited has written nothing.  The next call, with a clean status word, works."""
    lib, dev = native.cabi(), gpu_device
    M, H = 1, 1024
    g = torch.Generator(device=dev).manual_seed(9)
    a, b = _lin(dev, H, H, 3, 21), _lin(dev, 512, H, 3, 22)
    x_in = torch.randn((M, H), generator=g, device=dev).half()
    xt = torch.zeros((M, H), dtype=torch.int32, device=dev)
    never = torch.zeros((M, H), dtype=torch.int32, device=dev)
    out = torch.full((M, 512), 3.0, dtype=torch.float16, device=dev)
    sync = Sync(dev, spin_us=300)
    problems = [_chain_problem(a, x_in, xt, M, out_tag=1, overwrite=True),
                _chain_problem(b, never, out, M, x_tag=9, overwrite=True)]
    print("chain give-up path", flush=True)
    _ok(_chain(problems, sync))
    assert sync.status() == -8
    assert b"gave up" in lib.lutgemm_strerror(-8)
    torch.cuda.synchronize()
    assert torch.all(out == 3.0)                              # the waiting problem wrote nothing
    want = torch.zeros((M, H), dtype=torch.float16, device=dev)
    _separate(lib, [_fused(a, x_in, want, M)])
    torch.cuda.synchronize()
    assert torch.equal(_untag(xt), want)                      # the independent problem finished normally
    # status word cleared, row provided: the same call succeeds
    sync.words[1] = 0
    _tag(never, x_in, 9, sync)
    _ok(_chain(problems, sync))
    assert sync.status() == 0
    want2 = torch.zeros((M, 512), dtype=torch.float16, device=dev)
    _separate(lib, [_fused(b, x_in, want2, M)])
    torch.cuda.synchronize()
    assert torch.equal(out, want2)


def test_chain_rejects_bad_calls(gpu_device):
    lib, dev = native.cabi(), gpu_device
    M, H = 1, 512
    a, b = _lin(dev, H, H, 3, 1), _lin(dev, H, H, 3, 2)
    x = torch.zeros((M, H), dtype=torch.float16, device=dev)
    t1 = torch.zeros((M, H), dtype=torch.int32, device=dev)
    t2 = torch.zeros((M, H), dtype=torch.int32, device=dev)
    o = torch.zeros((M, H), dtype=torch.float16, device=dev)
    sync = Sync(dev)
    # the consumer listed before its producer
    assert _chain([_chain_problem(b, t1, o, M, x_tag=1), _chain_problem(a, x, t1, M, out_tag=1)], sync) == -1
    # two writers of one plain row
    assert _chain([_chain_problem(a, x, o, M), _chain_problem(b, x, o, M)], sync) == -1
    # two writers of one tagged row that do not wait for each other
    assert _chain([_chain_problem(a, x, t1, M, out_tag=1), _chain_problem(b, x, t1, M, out_tag=2)], sync) == -1
    # accumulating into a row right behind its writer (no problem in between that guarantees it is complete)
    assert _chain([_chain_problem(a, x, t1, M, out_tag=1), _chain_problem(b, t1, t1, M, x_tag=1, out_tag=2)], sync) == -1
    # tags out of range, split-norm fields, too many rows, no status word
    assert _chain([_chain_problem(a, x, t1, M, out_tag=70000)], sync) == -1
    xs = torch.zeros((8, H), dtype=torch.float16, device=dev)
    os_ = torch.zeros((8, H), dtype=torch.float16, device=dev)
    assert _chain([_chain_problem(a, xs, os_, 8)], sync) == -3
    arr = (native.ChainProblem * 1)(_chain_problem(a, x, o, M))
    assert lib.lutgemm_gemv_rowwise_f16_chain(1, arr, None, _sp()) == -1
    bad = native.ChainControl(None, None, 0)
    assert lib.lutgemm_gemv_rowwise_f16_chain(1, arr, ctypes.byref(bad), _sp()) == -1
    # a well-formed pair still runs
    _ok(_chain([_chain_problem(a, x, t1, M, out_tag=1, overwrite=True), _chain_problem(b, t1, t2, M, x_tag=1, out_tag=2, overwrite=True)], sync))
    assert sync.status() == 0


@pytest.mark.parametrize("batch", [1, 2])
def test_chained_decoder_matches_the_dense_model(gpu_device, batch):
    """The decoder harness with one chained launch per block (attention kernel + chain) against the
    same network with every linear a dense fp32 matmul on oracle-dequantised weights, eager and from
    a captured graph, over several tokens (the epoch advances every step)."""
    from shiftaddllm_amd import decode, workload
    cfg = decode.DecoderConfig(vocab_size=512, hidden=256, intermediate=512, layers=3, heads=4, kv_heads=2,
                               max_positions=32, group_size=128)
    qc = workload.mixed_bit_config(cfg.layers, seed=3)
    ids = torch.randint(0, cfg.vocab_size, (batch, 7), generator=torch.Generator().manual_seed(0))

    def run(model, capture):
        if capture:
            model.capture()
        model.reset()
        outs = []
        for t in range(ids.shape[1]):
            outs.append(model.forward_token(ids[:, t].to(gpu_device), t).float().cpu().clone())
        torch.cuda.synchronize()
        return torch.stack(outs)

    lut = decode.LutDecoder(cfg, qc, batch=batch, seed=5, device=gpu_device, chain=True)
    assert lut.chain
    dense = decode.LutDecoder(cfg, qc, batch=batch, seed=5, device=gpu_device, fuse_launches=False, glue="torch")
    table = {}
    for blk in dense.blocks:
        for lin in (blk.q_proj, blk.k_proj, blk.v_proj, blk.o_proj, blk.gate_proj, blk.up_proj, blk.down_proj):
            Wq = orc.dequant_rowwise_kernel_layout(lin.binaryWeight.cpu().numpy(), lin.alpha.cpu().numpy())
            table[id(lin)] = torch.from_numpy(Wq).to(gpu_device)
    dense._linears = lambda lins, x: [(x.float() @ table[id(l)].t()).half() for l in lins]
    want = run(dense, capture=False)
    print(f"chained decoder batch={batch} eager", flush=True)
    got = run(lut, capture=False)
    assert lut.chain_status() == 0
    print(f"chained decoder batch={batch} graph", flush=True)
    got_graph = run(lut, capture=True)
    assert lut.chain_status() == 0
    for name, g in (("eager", got), ("graph", got_graph)):
        rel, mad = orc.error_metrics(g.numpy(), want.numpy())
        assert rel <= 2e-3 and mad <= 1e-2, (name, rel, mad)
    assert torch.allclose(got_graph, got, atol=2e-3, rtol=2e-3)
