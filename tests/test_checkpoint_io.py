"""On-disk Lat. checkpoint format: writer, dense loader, kernel loader (CPU part),
and on the GPU the loaded LutLinear layers against the dense model."""
import numpy as np
import pytest
import torch
import torch.nn as nn

import oracle as orc
from shiftaddllm_amd import workload
from shiftaddllm_amd.lut_gemm import kernel as K
from shiftaddllm_amd.lut_gemm.quant import LutLinear


class _Attn(nn.Module):
    def __init__(self, h):
        super().__init__()
        self.q_proj = nn.Linear(h, h, bias=False)
        self.o_proj = nn.Linear(h, h, bias=False)


class _Mlp(nn.Module):
    def __init__(self, h, i):
        super().__init__()
        self.up_proj = nn.Linear(h, i, bias=False)
        self.down_proj = nn.Linear(i, h, bias=False)


class _Block(nn.Module):
    def __init__(self, h, i):
        super().__init__()
        self.self_attn = _Attn(h)
        self.mlp = _Mlp(h, i)


class _Inner(nn.Module):
    def __init__(self, n, h, i):
        super().__init__()
        self.layers = nn.ModuleList(_Block(h, i) for _ in range(n))


class TinyLlamaTree(nn.Module):
    """`model.model.layers[i].{self_attn,mlp}.*_proj`, the module paths of a Llama checkpoint."""
    def __init__(self, n=2, h=64, i=96):
        super().__init__()
        self.model = _Inner(n, h, i)


def _write_checkpoint(tmp_path, model, wbits, R, seed=0):
    want = {}
    layers = model.model.layers
    for i in range(len(layers)):
        for name, lin in K.find_layers(layers[i], layers=(nn.Linear,)).items():
            p = workload.make_block_problem(lin.out_features, lin.in_features, nb=wbits, R=R, seed=seed + 7 * i + len(name))
            path = K.save_shiftaddllm_weight(str(tmp_path), "tiny", f"{i}.{name}", wbits, p.disk_bWeight, p.disk_alpha)
            assert path.endswith(f"tiny_{i}.{name}_{wbits}bit.pt")
            want[(i, name)] = orc.dequant_lat_disk(p.disk_bWeight.numpy(), p.disk_alpha.numpy())     # [N, K]
    return want


def test_writer_rejects_malformed_tensors(tmp_path):
    bw = torch.zeros((64, 2, 3), dtype=torch.int32)
    al = torch.ones((8, 4, 3))
    with pytest.raises(ValueError):
        K.save_shiftaddllm_weight(str(tmp_path), "m", "0.x", 2, bw, al)          # bit count mismatch
    with pytest.raises(ValueError):
        K.save_shiftaddllm_weight(str(tmp_path), "m", "0.x", 3, bw, al[:4])      # alpha rows != K/8
    with pytest.raises(ValueError):
        K.save_shiftaddllm_weight(str(tmp_path), "m", "0.x", 3, bw.long(), al)


def test_dense_loader_round_trip(tmp_path):
    model = TinyLlamaTree()
    want = _write_checkpoint(tmp_path, model, wbits=3, R=4)
    missing = K.load_shiftaddllm_weight(model, str(tmp_path), "tiny", 3, is_lat=True)
    assert missing == []
    for (i, name), W in want.items():
        lin = K.find_layers(model.model.layers[i], layers=(nn.Linear,))[name]
        assert np.array_equal(lin.weight.detach().numpy(), W.astype(np.float32))


def test_dense_loader_reports_missing_files(tmp_path, capsys):
    model = TinyLlamaTree(n=1)
    missing = K.load_shiftaddllm_weight(model, str(tmp_path), "tiny", 3, is_lat=True)
    assert len(missing) == 4 and "WARNING: no such file" in capsys.readouterr().out


@pytest.mark.parametrize("alpha_format", ["apot_int8", "block_fp16"])
def test_kernel_loader_fills_lutlinear_buffers(tmp_path, alpha_format):
    model = TinyLlamaTree()
    want = _write_checkpoint(tmp_path, model, wbits=2, R=4, seed=3)
    missing = K.load_shiftaddllm_weight_with_kernel(model, str(tmp_path), "tiny", 2, is_lat=True,
                                                    alpha_format=alpha_format)
    assert missing == []
    luts = K.find_layers(model.model.layers[0], layers=(LutLinear,))
    assert set(luts) == {"self_attn.q_proj", "self_attn.o_proj", "mlp.up_proj", "mlp.down_proj"}
    for (i, name), W in want.items():
        lut = K.find_layers(model.model.layers[i], layers=(LutLinear,))[name]
        assert lut.num_groups == 4 and lut.wbit == 2
        bW = lut.binaryWeight.numpy()
        if alpha_format == "apot_int8":
            alpha = orc.apot_i8_to_alpha(lut.alpha.numpy())
        else:
            alpha = lut.alpha.numpy().astype(np.float32)
        got = orc.dequant_block_kernel_layout(bW, alpha)
        assert np.array_equal(got, W.astype(np.float32)), (i, name)


@pytest.mark.gpu
def test_loaded_layers_match_dense_layers_on_gpu(tmp_path, gpu_device):
    dense, lut = TinyLlamaTree(h=128, i=256), TinyLlamaTree(h=128, i=256)
    _write_checkpoint(tmp_path, dense, wbits=3, R=4, seed=5)
    K.load_shiftaddllm_weight(dense, str(tmp_path), "tiny", 3, is_lat=True)
    K.load_shiftaddllm_weight_with_kernel(lut, str(tmp_path), "tiny", 3, is_lat=True)
    dense, lut = dense.to(gpu_device), lut.to(gpu_device)
    x = torch.randn((1, 128), generator=torch.Generator().manual_seed(1)).half().to(gpu_device)
    for i in range(2):
        for name in ("self_attn.q_proj", "self_attn.o_proj", "mlp.up_proj"):
            d = K.find_layers(dense.model.layers[i], layers=(nn.Linear,))[name]
            l = K.find_layers(lut.model.layers[i], layers=(LutLinear,))[name]
            want = (x.float() @ d.weight.detach().float().t()).cpu().numpy()
            got = l(x).detach().float().cpu().numpy()
            rel, mad = orc.error_metrics(got, want)
            assert rel <= 2e-3 and mad <= 1e-2, (i, name, rel, mad)


# ---- the reference's own model family: an OPT tree (model.model.decoder.layers) -------

def _tiny_opt_config():
    transformers = pytest.importorskip("transformers")
    return transformers.OPTConfig(vocab_size=256, hidden_size=64, ffn_dim=128, num_hidden_layers=2,
                                  num_attention_heads=2, max_position_embeddings=32, word_embed_proj_dim=64,
                                  do_layer_norm_before=True, dropout=0.0)


def _write_opt_checkpoint(tmp_path, model, wbits, R, seed=0):
    want = {}
    layers = model.model.decoder.layers
    for i in range(len(layers)):
        for name, lin in K.find_layers(layers[i], layers=(nn.Linear,)).items():
            p = workload.make_block_problem(lin.out_features, lin.in_features, nb=wbits, R=R,
                                            seed=seed + 11 * i + len(name))
            K.save_shiftaddllm_weight(str(tmp_path), "opt-tiny", f"{i}.{name}", wbits, p.disk_bWeight, p.disk_alpha)
            want[(i, name)] = orc.dequant_lat_disk(p.disk_bWeight.numpy(), p.disk_alpha.numpy())
    return want


def test_kernel_loader_on_an_opt_tree(tmp_path):
    """The module tree the reference's loader is written for (lut_gemm/kernel.py:141):
    q/k/v/out_proj and fc1/fc2 (non-square, with bias) of every decoder layer."""
    import transformers
    torch.manual_seed(0)
    model = transformers.OPTForCausalLM(_tiny_opt_config()).eval()
    want = _write_opt_checkpoint(tmp_path, model, wbits=3, R=4)
    biases = {(i, n): l.bias.detach().clone() for i in range(2)
              for n, l in K.find_layers(model.model.decoder.layers[i], layers=(nn.Linear,)).items()}
    missing = K.load_shiftaddllm_weight_with_kernel(model, str(tmp_path), "opt-tiny", 3, is_lat=True)
    assert missing == []
    for i in range(2):
        luts = K.find_layers(model.model.decoder.layers[i], layers=(LutLinear,))
        assert set(luts) == {"self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.out_proj",
                             "fc1", "fc2"}
        for name, lut in luts.items():
            assert lut.num_groups == 4 and lut.wbit == 3
            assert torch.equal(lut.bias, biases[(i, name)])                       # the layer's bias is kept
            got = orc.dequant_block_kernel_layout(lut.binaryWeight.numpy(), orc.apot_i8_to_alpha(lut.alpha.numpy()))
            assert np.array_equal(got, want[(i, name)].astype(np.float32)), (i, name)


def test_load_lut_builds_the_skeleton_and_round_trips_a_state_dict(tmp_path):
    """load_lut (lut_gemm/quant.py:74-114) from an OPTConfig object: decoder linears become
    LutLinear with the reference's buffer names, lm_head stays dense, and a state_dict
    saved from one skeleton loads into another through `checkpoint=`."""
    from shiftaddllm_amd.lut_gemm.quant import load_lut
    cfg = _tiny_opt_config()
    a = load_lut(cfg, wbit=3, group_size=16)
    assert a.seqlen == cfg.max_position_embeddings
    assert isinstance(a.lm_head, nn.Linear)
    luts = K.find_layers(a, layers=(LutLinear,))
    assert len(luts) == 2 * 6
    keys = a.state_dict().keys()
    assert "model.decoder.layers.0.self_attn.q_proj.binaryWeight" in keys
    assert "model.decoder.layers.1.fc2.alpha" in keys
    # fill every tensor with something recognisable (to_empty leaves memory uninitialised)
    g = torch.Generator().manual_seed(0)
    state = {}
    for k, v in a.state_dict().items():
        if v.dtype in (torch.int32, torch.int8):
            state[k] = torch.randint(-100, 100, v.shape, generator=g).to(v.dtype)
        else:
            state[k] = torch.randn(v.shape, generator=g).to(v.dtype)
    path = str(tmp_path / "lut_state.pt")
    torch.save(state, path)
    b = load_lut(cfg, checkpoint=path, wbit=3, group_size=16)
    for k, v in b.state_dict().items():
        assert torch.equal(v, state[k]), k
    lut = K.find_layers(b, layers=(LutLinear,))["model.decoder.layers.0.fc1"]
    assert (lut.K, lut.N, lut.wbit, lut.num_groups) == (64, 128, 3, 4)
    assert tuple(lut.binaryWeight.shape) == (64 // 32, 3, 128)


@pytest.mark.gpu
def test_opt_model_from_files_matches_dense_model_on_gpu(tmp_path, gpu_device):
    """Whole OPT model, one token: linears loaded by the kernel loader against the same
    model with the dense loader's dequantised weights."""
    import transformers
    torch.manual_seed(0)
    dense = transformers.OPTForCausalLM(_tiny_opt_config()).half().eval()
    lut = transformers.OPTForCausalLM(_tiny_opt_config()).half().eval()
    lut.load_state_dict(dense.state_dict())
    _write_opt_checkpoint(tmp_path, dense, wbits=3, R=4, seed=2)
    assert K.load_shiftaddllm_weight(dense, str(tmp_path), "opt-tiny", 3, is_lat=True) == []
    assert K.load_shiftaddllm_weight_with_kernel(lut, str(tmp_path), "opt-tiny", 3, is_lat=True) == []
    dense, lut = dense.to(gpu_device), lut.to(gpu_device)
    ids = torch.randint(0, 256, (1, 1), generator=torch.Generator().manual_seed(3)).to(gpu_device)
    with torch.no_grad():
        want = dense(ids).logits.float().cpu().numpy().reshape(1, -1)
        got = lut(ids).logits.float().cpu().numpy().reshape(1, -1)
    rel, mad = orc.error_metrics(got, want)
    assert rel <= 5e-3 and mad <= 2e-2, (rel, mad)
