"""The reference's own call stack on the GPU: a HuggingFace OPT decoder whose linears are
swapped for LutLinear by make_lut (what load_shiftaddllm_weight_with_kernel does for a real
checkpoint), against the same network with dense dequantised weights."""
import numpy as np
import pytest
import torch
import torch.nn as nn

import oracle as orc
from shiftaddllm_amd import workload
from shiftaddllm_amd.lut_gemm.kernel import find_layers
from shiftaddllm_amd.lut_gemm.quant import LutLinear, make_lut

pytestmark = pytest.mark.gpu


def _tiny_opt():
    transformers = pytest.importorskip("transformers")
    cfg = transformers.OPTConfig(vocab_size=512, hidden_size=128, ffn_dim=256, num_hidden_layers=2,
                                 num_attention_heads=4, max_position_embeddings=64, word_embed_proj_dim=128,
                                 do_layer_norm_before=True, dropout=0.0)
    torch.manual_seed(0)
    return transformers.OPTForCausalLM(cfg).half().eval()


@pytest.mark.parametrize("alpha_format", ["rowwise_fp16", "apot_int8"])
def test_hf_opt_with_lutlinear_matches_dense_model(gpu_device, alpha_format):
    dense = _tiny_opt()
    lut = _tiny_opt()
    lut.load_state_dict(dense.state_dict())
    nb = 3
    for i, layer in enumerate(dense.model.decoder.layers):
        names = find_layers(layer, layers=(nn.Linear,))
        twin = lut.model.decoder.layers[i]
        for name, lin in names.items():
            N, K = lin.out_features, lin.in_features
            if alpha_format == "rowwise_fp16":
                p = workload.make_rowwise_problem(N, K, nb=nb, group_size=128, seed=31 * i + len(name))
                Wq = orc.dequant_rowwise_kernel_layout(p.bW.numpy(), p.alpha.numpy())
                group_size, alpha = 128, p.alpha
            else:
                p = workload.make_block_problem(N, K, nb=nb, R=4, seed=31 * i + len(name))
                Wq = orc.dequant_block_kernel_layout(p.bW.numpy(), p.alpha.numpy().astype(np.float32))
                group_size, alpha = K // 4, None
            lin.weight.data = torch.from_numpy(Wq).half()
            make_lut(twin, {name: None}, wbit=nb, group_size=group_size, alpha_format=alpha_format)
            mod = find_layers(twin, layers=(LutLinear,))[name]
            mod.binaryWeight.data = p.bW.clone()
            mod.alpha.data = alpha.clone() if alpha is not None else mod.quantize_to_apot(p.alpha.float())
    dense, lut = dense.to(gpu_device), lut.to(gpu_device)
    ids = torch.randint(0, 512, (1, 7), generator=torch.Generator().manual_seed(1)).to(gpu_device)
    with torch.no_grad():
        want = dense(ids).logits.float().cpu().numpy()
        got = lut(ids).logits.float().cpu().numpy()                  # 7 rows through every LutLinear
        got1 = lut(ids[:, :1]).logits.float().cpu().numpy()          # the reference's single-token case
        want1 = dense(ids[:, :1]).logits.float().cpu().numpy()
    for g, w in ((got, want), (got1, want1)):
        rel, mad = orc.error_metrics(g.reshape(-1, 512), w.reshape(-1, 512))
        assert rel <= 5e-3 and mad <= 2e-2, (rel, mad)    # fp16 network, two differently rounded linear paths


def test_lutlinear_output_and_bias_handling(gpu_device):
    """forward pre-fills its output from the bias as the reference does (lut_gemm/quant.py:46):
    a new tensor per call by default, one reused buffer with `reuse_output`; an in-place change
    of the bias is honoured; fp32 input comes back as fp32; a strided input is accepted."""
    N, K = 256, 512
    p = workload.make_rowwise_problem(N, K, nb=3, group_size=128, seed=3)
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(1)) * 0.5).half().to(gpu_device)
    lin = LutLinear(K, N, group_size=128, wbit=3, bias=bias, alpha_format="rowwise_fp16").to(gpu_device)
    lin.binaryWeight.data = p.bW.to(gpu_device)
    lin.alpha.data = p.alpha.to(gpu_device)
    x = p.x.to(gpu_device)
    want, _ = orc.gemv_rowwise_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), p.num_groups,
                                 out=bias.cpu().numpy().reshape(1, N))

    def close(y, ref):
        rel, mad = orc.error_metrics(y.float().cpu().numpy().reshape(1, N), np.asarray(ref, dtype=np.float32))
        return rel <= 2e-3 and mad <= 1e-2

    y1, y2 = lin(x), lin(x)
    assert y1.data_ptr() != y2.data_ptr() and torch.equal(y1, y2) and close(y1, want)
    assert lin(x.float()).dtype == torch.float32 and close(lin(x.float()), want)
    wide = torch.zeros((1, 2 * K), dtype=torch.float16, device=gpu_device)
    wide[:, ::2] = x
    assert close(lin(wide[:, ::2]), want)                          # non-contiguous input
    assert lin(x.view(1, 1, K)).shape == (1, 1, N)
    bias.add_(1.0)                                                 # in place: the cached rows are stale now
    want2, _ = orc.gemv_rowwise_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), p.num_groups,
                                  out=bias.cpu().numpy().reshape(1, N))
    assert close(lin(x), want2)
    lin.reuse_output = True
    z1 = lin(x)
    first = z1.clone()
    z2 = lin(x)
    assert z1.data_ptr() == z2.data_ptr() and torch.equal(first, z2) and close(z2, want2)
    lin.bias = None
    assert close(lin(x), want2 - bias.float().cpu().numpy().reshape(1, N))


def test_reference_benchmark_protocol_on_an_hf_model(gpu_device):
    """benchmark_hf (model/opt.py:367-423): one forward per token with the growing cache; its
    perplexity equals the one of a single forward over the whole sequence."""
    from shiftaddllm_amd import decode
    model = _tiny_opt().to(gpu_device)
    ids = torch.randint(0, 512, (1, 12), generator=torch.Generator().manual_seed(2))
    r = decode.benchmark_hf(model, ids, check=True, warmup=2)
    assert r["tokens"] == 12 and r["median_s_per_token"] > 0
    with torch.no_grad():
        logits = model(ids.to(gpu_device)).logits[0].float()
    want = torch.exp(torch.nn.functional.cross_entropy(logits[:-1], ids[0, 1:].to(gpu_device))).item()
    assert abs(r["ppl"] - want) <= 2e-2 * want, (r["ppl"], want)


def test_decoder_benchmark_reports_perplexity(gpu_device):
    from shiftaddllm_amd import decode
    cfg = decode.DecoderConfig(vocab_size=256, hidden=256, intermediate=512, layers=2, heads=4, kv_heads=4,
                               max_positions=32)
    model = decode.LutDecoder(cfg, None, batch=2, seed=0, device=gpu_device)
    prompt = torch.randint(0, 256, (2, 6), generator=torch.Generator().manual_seed(0))
    r = decode.benchmark(model, prompt, generate=4, warmup=1, check=True)
    # the same quantity from the logits of separate steps
    model.reset()
    tot = 0.0
    for i in range(5):
        logits = model.forward_token(prompt[:, i].to(gpu_device), i).float()
        tot += torch.nn.functional.cross_entropy(logits, prompt[:, i + 1].to(gpu_device)).item()
    import math
    assert abs(r["ppl"] - math.exp(tot / 5)) <= 1e-3 * r["ppl"]
    assert "ppl" not in decode.benchmark(model, prompt, generate=2, warmup=0)
