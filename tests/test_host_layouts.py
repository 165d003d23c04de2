"""Host-side (torch) layout code of the package against the oracle (CPU only):
pack_binaryWeight, unpack_weight, convert_weight, the APoT encoder, the
synthetic BCQ generator's invariants and the LutLinear module surface."""
import numpy as np
import pytest
import torch
import torch.nn as nn

import oracle as orc
from shiftaddllm_amd import workload
from shiftaddllm_amd.lut_gemm import kernel as K_
from shiftaddllm_amd.lut_gemm import quant as Q_


def _signs(gen, shape):
    return (torch.randint(0, 2, shape, generator=gen, dtype=torch.int8) * 2 - 1)


@pytest.mark.parametrize("shape", [(4, 2, 64, 3), (3, 1, 32, 1), (5, 3, 96, 4)])
def test_pack_matches_oracle_bit_exact(shape):
    g = torch.Generator().manual_seed(sum(shape))
    B = _signs(g, shape)
    got = K_.pack_binaryWeight(B)
    assert got.dtype == torch.int32 and got.is_contiguous()
    assert np.array_equal(got.numpy(), orc.pack_binary_weight_np(B.numpy()))
    assert np.array_equal(got.numpy(), orc.pack_binary_weight_c(B.numpy()))
    # float inputs (what the quantiser hands over) pack the same
    assert torch.equal(K_.pack_binaryWeight(B.float()), got)


def test_pack_rejects_bad_input():
    with pytest.raises(AssertionError):
        K_.pack_binaryWeight(torch.ones(2, 32, 1))
    bad = torch.ones(1, 1, 32, 1)
    bad[0, 0, 5, 0] = 0
    with pytest.raises(AssertionError):
        K_.pack_binaryWeight(bad)


@pytest.mark.parametrize("shape,G", [((4, 8, 3), 2), ((6, 4, 2), 4), ((2, 3, 4), 1)])
def test_unpack_weight_matches_oracle_bit_exact(shape, G):
    g = torch.Generator().manual_seed(shape[1])
    bW = torch.randint(-2 ** 31, 2 ** 31 - 1, shape, generator=g, dtype=torch.int64).to(torch.int32)
    alpha = torch.rand((shape[0], G, shape[2]), generator=g)
    W = K_.unpack_weight(bW, alpha)
    ref = orc.unpack_weight_c(bW.numpy(), alpha.numpy())
    assert W.dtype == torch.float32 and tuple(W.shape) == (shape[0], shape[1] * 32)
    assert np.array_equal(W.numpy().view(np.uint32), ref.view(np.uint32))


def test_unpack_to_fake_binary_weight_round_trip():
    g = torch.Generator().manual_seed(3)
    B = _signs(g, (6, 2, 64, 3))
    back = K_.unpack_to_fake_binaryWeight(K_.pack_binaryWeight(B), n_groups=2)
    assert back.dtype == torch.int8 and torch.equal(back, B)


@pytest.mark.parametrize("N,K,nb,R", [(64, 64, 2, 8), (128, 96, 3, 4), (96, 160, 2, 1)])
def test_convert_weight_square_and_non_square(N, K, nb, R):
    g = torch.Generator().manual_seed(N + K)
    Bk = _signs(g, (K, R, N // R, nb))
    disk_bW = K_.pack_binaryWeight(Bk)
    disk_alpha = torch.exp2(torch.randint(-8, -3, (K // 8, R, nb), generator=g).float())
    want_bW, want_a = orc.lat_disk_to_kernel_layout(disk_bW.numpy(), disk_alpha.numpy())
    got_bW, got_a = K_.convert_weight(disk_bW, disk_alpha)
    assert got_bW.dtype == torch.int32 and tuple(got_bW.shape) == (K // 32, nb, N)
    assert np.array_equal(got_bW.numpy(), want_bW)
    assert got_a.dtype == torch.float32 and np.array_equal(got_a.numpy(), want_a)
    # the reference loader hands in alpha repeated 8x along dim 0: same result
    got_bW2, got_a2 = K_.convert_weight(disk_bW, disk_alpha.repeat_interleave(8, dim=0))
    assert torch.equal(got_bW2, got_bW) and torch.equal(got_a2, got_a)
    # dense dequantisation of the on-disk tensors agrees with the oracle
    W = K_.dequantize_lat(disk_bW, disk_alpha)
    assert np.array_equal(W.numpy(), orc.dequant_lat_disk(disk_bW.numpy(), disk_alpha.numpy()))


def test_apot_encoder_exact_cases_and_sentinel():
    a = torch.tensor([1.0, 0.125, 0.75, 0.6875, 2.0 ** -14, 5.0, 0.0, 7.0, 1.1875])
    code = Q_.encode_apot_int8(a)
    assert code.dtype == torch.int8 and tuple(code.shape) == (9, 3)
    assert code[0].tolist() == [0, -128, -128]
    assert code[1].tolist() == [-3, -128, -128]
    assert code[2].tolist() == [-1, -2, -128]
    assert code[3].tolist() == [-1, -3, -4]
    assert code[4].tolist() == [-14, -128, -128]
    assert code[5].tolist() == [2, 0, -128]
    assert code[6].tolist() == [-128, -128, -128]
    assert code[7].tolist() == [2, 1, 0]
    dec = Q_.decode_apot_int8(code)
    assert torch.equal(dec, a)
    assert np.array_equal(orc.apot_i8_to_alpha(code.numpy()), a.numpy())


def test_apot_encoder_error_bound():
    g = torch.Generator().manual_seed(0)
    a = torch.rand(4096, generator=g) * 0.1 + 1e-4
    dec = Q_.decode_apot_int8(Q_.encode_apot_int8(a))
    # three positive powers of two keep the top three mantissa bits (last one rounded)
    assert float(((dec - a).abs() / a).max()) <= 2.0 ** -3 + 1e-6
    assert float(((dec - a).abs() / a).mean()) < 0.04


def test_bcq_generator_invariants():
    g = torch.Generator().manual_seed(1)
    w = torch.randn((64, 128), generator=g) * 0.02
    B, alpha = workload.bcq_shift_quantize(w, 3, rounds=5)
    assert B.dtype == torch.int8 and bool(((B == 1) | (B == -1)).all())
    assert bool((alpha >= 0).all())
    assert torch.equal(alpha.sort(dim=1, descending=True).values, alpha)     # quantizer.py:78
    e = torch.log2(alpha)
    assert torch.equal(e, e.round())                                          # powers of two
    # signs are the element-wise nearest codeword: brute force over all 2^3
    book = torch.tensor([[1 if (c >> b) & 1 else -1 for b in range(3)] for c in range(8)]).float()
    vals = alpha @ book.t()                                                   # [64, 8]
    best = (w.unsqueeze(-1) - vals.unsqueeze(1)).abs().min(dim=-1).values
    recon = torch.einsum("rgb,rb->rg", B.float(), alpha)
    assert torch.allclose((w - recon).abs(), best, atol=1e-7)
    # quantisation is useful: error well below the weights' own scale
    assert float((w - recon).pow(2).mean().sqrt()) < 0.5 * float(w.pow(2).mean().sqrt())


def test_bcq_greedy_round0_closed_form():
    # rounds = 0: alpha_0 = mean |w|, B_0 = sign(w); alpha_1 = mean |w - alpha_0 B_0| (bcq_shift.py:131-161)
    g = torch.Generator().manual_seed(2)
    w = torch.randn((8, 64), generator=g)
    B, alpha = workload.bcq_shift_quantize(w, 2, rounds=0)
    a0 = w.abs().mean(dim=1)
    assert torch.allclose(alpha[:, 0], a0)
    assert torch.equal(B[:, :, 0].float(), torch.sign(w))
    r = w - torch.sign(w) * a0.unsqueeze(1)
    assert torch.allclose(alpha[:, 1], r.abs().mean(dim=1))


def test_rowwise_problem_matches_oracle_dequant():
    p = workload.make_rowwise_problem(32, 256, nb=3, group_size=128, seed=0)
    assert tuple(p.bW.shape) == (8, 3, 32) and p.bW.dtype == torch.int32
    assert tuple(p.alpha.shape) == (2, 3, 32) and p.alpha.dtype == torch.float16
    Wq = orc.dequant_rowwise_kernel_layout(p.bW.numpy(), p.alpha.numpy())
    # same thing through the package's own oracle-shaped function
    a_r = p.alpha.float().permute(2, 0, 1).contiguous()
    W2 = K_.unpack_weight(p.bW.permute(2, 0, 1).contiguous(), a_r)
    assert np.array_equal(Wq, W2.numpy())
    # 3-bit BCQ of N(0, 0.02) weights: relative error well under 50 %
    rel = np.linalg.norm(Wq - p.W.numpy()) / np.linalg.norm(p.W.numpy())
    assert rel < 0.35
    # seeded: same call, same bits
    p2 = workload.make_rowwise_problem(32, 256, nb=3, group_size=128, seed=0)
    assert torch.equal(p.bW, p2.bW) and torch.equal(p.alpha, p2.alpha) and torch.equal(p.x, p2.x)


def test_block_problem_matches_disk_format():
    p = workload.make_block_problem(64, 96, nb=2, R=8, seed=0)
    assert tuple(p.disk_bWeight.shape) == (96, 2, 2) and tuple(p.disk_alpha.shape) == (12, 8, 2)
    bW, a = K_.convert_weight(p.disk_bWeight, p.disk_alpha)
    assert torch.equal(bW, p.bW) and torch.equal(a.half(), p.alpha)
    W_disk = orc.dequant_lat_disk(p.disk_bWeight.numpy(), p.disk_alpha.numpy())
    W_kern = orc.dequant_block_kernel_layout(p.bW.numpy(), p.alpha.float().numpy())
    assert np.array_equal(W_disk, W_kern)


def test_mixed_bit_config_schema_and_ratio():
    cfg = workload.mixed_bit_config(32, seed=0)
    assert len(cfg) == 32 * 7
    assert all(set(v) == {"bits", "columnwise"} and v["bits"] in (2, 3, 4) for v in cfg.values())
    counts = {b: sum(v["bits"] == b for v in cfg.values()) for b in (2, 3, 4)}
    assert counts[3] > counts[2] and counts[3] > counts[4]
    assert cfg == workload.mixed_bit_config(32, seed=0)


def test_lutlinear_surface_and_make_lut():
    lin = Q_.LutLinear(256, 64, group_size=32, wbit=3, bias=None)
    sd = lin.state_dict()
    assert set(sd) == {"binaryWeight", "alpha"}
    assert tuple(sd["binaryWeight"].shape) == (8, 3, 64) and sd["binaryWeight"].dtype == torch.int32
    assert tuple(sd["alpha"].shape) == (32, 3, 8, 3) and sd["alpha"].dtype == torch.int8
    assert lin.num_groups == 8 and lin.K == 256 and lin.N == 64 and lin.wbit == 3

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj = nn.Linear(64, 64)
            self.fc1 = nn.Linear(64, 128, bias=False)
            self.norm = nn.LayerNorm(64)

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.layers = nn.ModuleList([Block(), Block()])
            self.head = nn.Linear(64, 10)

    net = Net()
    found = K_.find_layers(net.layers)
    assert set(found) == {"0.q_proj", "0.fc1", "1.q_proj", "1.fc1"}
    Q_.make_lut(net.layers, found, wbit=2, group_size=8)
    assert isinstance(net.layers[0].q_proj, Q_.LutLinear) and isinstance(net.layers[1].fc1, Q_.LutLinear)
    assert isinstance(net.head, nn.Linear) and isinstance(net.layers[0].norm, nn.LayerNorm)
    assert net.layers[0].q_proj.bias is not None and net.layers[0].fc1.bias is None
    assert net.layers[0].fc1.num_groups == 8 and net.layers[0].fc1.wbit == 2
    # reference-style state_dict with alpha repeated 8x along dim 0 loads
    l = net.layers[0].q_proj
    assert set(l.state_dict()) == {"binaryWeight", "alpha", "bias"}   # a Parameter bias registers itself
    sd = {"binaryWeight": torch.ones_like(l.binaryWeight), "bias": torch.zeros(64),
          "alpha": torch.arange(64, dtype=torch.int8).view(64, 1, 1, 1).expand(64, 2, 8, 3).contiguous()}
    l.load_state_dict(sd)
    assert tuple(l.alpha.shape) == (8, 2, 8, 3) and l.alpha[:, 0, 0, 0].tolist() == list(range(0, 64, 8))


def test_forward_without_native_library_fails_loudly(monkeypatch):
    # no silent CPU path: if the compiled module cannot be loaded, forward raises
    from shiftaddllm_amd import native

    def boom():
        raise native.NativeLibraryMissing("not built")

    monkeypatch.setattr(native, "_load_extension", boom)
    monkeypatch.delitem(native.__dict__, "lutgemm", raising=False)
    lin = Q_.LutLinear(64, 8, group_size=8, wbit=2)
    with pytest.raises(ImportError):
        lin(torch.zeros(1, 64, dtype=torch.float16))
