"""Bit-packing, dequantisation, layout conversion and per-layer checkpoint
loading for BCQ linear layers.

Function names and signatures are those of lut_gemm/kernel.py in the
ShiftAddLLM checkout (:9-179) so callers written against it keep working; the
bodies are independent, vectorised, device-agnostic torch.

Tensor formats
  pack input      +-1 [A, n_groups, group_size, wbit]
  packed          int32 [A, n_groups*group_size/32, wbit]; bit t of word j is
                  entry 32j+t of the flattened (n_groups, group_size) axis
  kernel signs    int32 [K/32, wbit, N]   (= packed row-wise BCQ .permute(1,2,0))
  Lat. on disk    bWeight int32 [K, N/32, wbit] (packed along the OUTPUT axis),
                  alpha fp32 [K/8, R, wbit]  (quant_methods/shiftaddllm.py:193-211)
"""
from __future__ import annotations

import os

import torch
import torch.nn as nn

from .quant import LutLinear, make_lut


def _bit_positions(device):
    return torch.arange(32, device=device, dtype=torch.int64)


def pack_binaryWeight(bWeight: torch.Tensor):
    """+-1 [A, n_groups, group_size, wbit] -> int32 [A, n_groups*group_size/32, wbit]
    (lut_gemm/kernel.py:9-23).  Bit t (LSB first) of a word is 1 where the entry
    is +1; bit 31 lands in the int32 sign."""
    if bWeight.dim() != 4:
        raise AssertionError(
            "BinaryWeight shape should be [N, n_groups, group_size, wbit], but got {}".format(bWeight.size()))
    A, n_groups, group_size, wbit = bWeight.shape
    L = n_groups * group_size
    if L % 32:
        raise AssertionError("n_groups * group_size must be a multiple of 32")
    positive = bWeight == 1
    if not bool((positive | (bWeight == -1)).all()):
        raise AssertionError("BinaryWeight should be 1 or -1, but got other values")
    bits = positive.reshape(A, L // 32, 32, wbit).to(torch.int64)
    shifts = _bit_positions(bWeight.device).view(1, 1, 32, 1)
    words = (bits << shifts).sum(dim=2)                      # 0 .. 2^32-1 in int64
    words = torch.where(words >= 2 ** 31, words - 2 ** 32, words)
    return words.to(torch.int32).contiguous()


def _unpack_signs(packed: torch.Tensor) -> torch.Tensor:
    """int32 [A, J, wbit] -> +-1 int8 [A, 32*J, wbit]."""
    A, J, wbit = packed.shape
    shifts = _bit_positions(packed.device).view(1, 1, 32, 1)
    bits = (packed.to(torch.int64).unsqueeze(2) >> shifts) & 1
    return (bits * 2 - 1).to(torch.int8).reshape(A, J * 32, wbit)


def unpack_weight(bW: torch.Tensor, alpha: torch.Tensor):
    """Dequantise (lut_gemm/kernel.py:26-56): bW int32 [A, L/32, wbit], alpha
    [A, G, wbit] -> fp32 [A, L] with W[a, l] = sum_b alpha[a, l // (L/G), b] * sign,
    accumulated in fp32 in bit-plane order."""
    if bW.dim() != 3 or alpha.dim() != 3:
        raise AssertionError("expected bW [A, L/32, wbit] and alpha [A, G, wbit]")
    if bW.size(2) != alpha.size(2):
        raise AssertionError("BinaryWeight and Alpha should have the same number of bits, but got {} and {}"
                             .format(bW.size(2), alpha.size(2)))
    if bW.size(0) != alpha.size(0):
        raise AssertionError("BinaryWeight and Alpha should have the same number of rows, but got {} and {}"
                             .format(bW.size(0), alpha.size(0)))
    A, J, wbit = bW.shape
    L, G = 32 * J, alpha.size(1)
    if L % G:
        raise AssertionError("number of alpha groups must divide the unpacked length")
    signs = _unpack_signs(bW).view(A, G, L // G, wbit)
    a = alpha.to(torch.float32)
    W = torch.zeros((A, G, L // G), dtype=torch.float32, device=bW.device)
    for b in range(wbit):
        W += a[:, :, b].unsqueeze(-1) * signs[..., b].to(torch.float32)
    return W.reshape(A, L)


def unpack_to_fake_binaryWeight(packed_bweight, n_groups=1):
    """int32 [A, L/32, wbit] -> +-1 int8 [A, n_groups, L/n_groups, wbit]
    (lut_gemm/kernel.py:58-75; there the uint8 arithmetic wraps -1 to 255)."""
    signs = _unpack_signs(packed_bweight)
    A, L, wbit = signs.shape
    return signs.view(A, n_groups, L // n_groups, wbit)


def find_layers(module, layers=(nn.Conv2d, nn.Linear, LutLinear), name=""):
    """{qualified name: module} of every leaf of the given types
    (lut_gemm/kernel.py:77-85; LutLinear is included so that an already swapped
    tree can be walked again)."""
    if type(module) in tuple(layers):
        return {name: module}
    found = {}
    for child_name, child in module.named_children():
        found.update(find_layers(child, layers=layers,
                                 name=name + "." + child_name if name != "" else child_name))
    return found


def _decoder_layers(model):
    """The list of transformer blocks: OPT (`model.model.decoder.layers`, the
    only family lut_gemm/kernel.py:141 knows), Llama/Mistral/Gemma
    (`model.model.layers`) or BLOOM (`model.transformer.h`)."""
    for path in ("model.decoder.layers", "model.layers", "transformer.h"):
        obj = model
        try:
            for part in path.split("."):
                obj = getattr(obj, part)
        except AttributeError:
            continue
        return obj
    raise AttributeError("cannot find the decoder layer list on this model")


def _layer_file(weights_dir, model_name, layer_name, wbits):
    return os.path.join(weights_dir, f"{model_name}_{layer_name}_{wbits}bit.pt")


def _read_layer_file(path):
    ckpt = torch.load(path, map_location="cpu", weights_only=True)
    return ckpt["bWeight"], ckpt["alpha"]


def save_shiftaddllm_weight(weights_dir, model_name, layer_name, wbits, bWeight, alpha):
    """Write one layer in the on-disk Lat. format the loaders read: a torch file
    `{model_name}_{layer_name}_{wbits}bit.pt` holding `bWeight` int32 [K, N/32, wbits]
    (signs packed along the OUTPUT axis) and `alpha` fp32 [K/8, R, wbits]
    (quant_methods/shiftaddllm.py:193-211 writes these keys and this name;
    `layer_name` is "<block index>.<module path>", e.g. "0.self_attn.q_proj").
    Returns the path."""
    if bWeight.dtype != torch.int32 or bWeight.dim() != 3 or bWeight.size(2) != wbits:
        raise ValueError("bWeight must be int32 [K, N/32, wbits]")
    if alpha.dim() != 3 or alpha.size(2) != wbits or alpha.size(0) * 8 != bWeight.size(0):
        raise ValueError("alpha must be [K/8, R, wbits]")
    os.makedirs(weights_dir, exist_ok=True)
    path = _layer_file(weights_dir, model_name, layer_name, wbits)
    torch.save({"bWeight": bWeight.cpu().contiguous(), "alpha": alpha.float().cpu().contiguous()}, path)
    return path


def dequantize_lat(BinaryWeight: torch.Tensor, alpha: torch.Tensor) -> torch.Tensor:
    """On-disk Lat. tensors -> dense W_q [N, K] fp32 (lut_gemm/kernel.py:101-106)."""
    return unpack_weight(BinaryWeight, alpha.repeat_interleave(8, dim=0)).transpose(0, 1).contiguous()


def load_shiftaddllm_weight(model, weights_dir, model_name, wbits, is_lat=False):
    """Dense path: dequantise every per-layer file into the ordinary nn.Linear
    weights (lut_gemm/kernel.py:87-109)."""
    assert is_lat, "Packed quantization weight only support lat method now"
    layers = _decoder_layers(model)
    missing = []
    for i in range(len(layers)):
        subset = find_layers(layers[i], layers=(nn.Conv2d, nn.Linear))
        for name, lin in subset.items():
            path = _layer_file(weights_dir, model_name, f"{i}.{name}", wbits)
            if not os.path.exists(path):
                missing.append(path)
                continue
            bW, alpha = _read_layer_file(path)
            W = dequantize_lat(bW, alpha)
            lin.weight.data = W.to(device=lin.weight.device, dtype=lin.weight.dtype)
    for path in missing:
        print(f"WARNING: no such file {path}")
    return missing


def convert_weight(BinaryWeight, Alpha):
    """On-disk Lat. layout -> kernel layout (lut_gemm/kernel.py:112-133).

    BinaryWeight int32 [K, N/32, wbit] packed along the output axis
    Alpha        [K/8, R, wbit], or the 8-fold row-repeated [K, R, wbit] that
                 the reference loader passes (kernel.py:172-173)
    returns      (int32 [K/32, wbit, N] packed along the input axis,
                  fp32 [K/8, wbit, R])
    Works for non-square layers, which the reference's view() rejects.
    """
    K, Nw, wbit = BinaryWeight.shape
    N = 32 * Nw
    if K % 32:
        raise ValueError("in_features must be a multiple of 32")
    signs = _unpack_signs(BinaryWeight)                         # [K, N, wbit]
    by_row = signs.permute(1, 0, 2).reshape(N, 1, K, wbit)      # [N, 1, K, wbit]
    compressed = pack_binaryWeight(by_row).permute(1, 2, 0).contiguous()   # [K/32, wbit, N]
    if Alpha.size(0) == K:
        Alpha = Alpha[::8]
    if Alpha.size(0) != K // 8:
        raise ValueError(f"alpha must have K/8 = {K // 8} rows (or K = {K} repeated rows)")
    alpha = Alpha.transpose(1, 2).float().contiguous()
    return compressed, alpha


def load_shiftaddllm_weight_with_kernel(model, weights_dir, model_name, wbits, is_lat=False,
                                        alpha_format="apot_int8"):
    """Kernel path: swap the decoder linears for LutLinear and fill them from the
    per-layer files (lut_gemm/kernel.py:135-179).  `alpha_format` chooses how
    alpha is stored: the reference's int8 exponent triples (default) or
    "block_fp16"."""
    assert is_lat, "Packed quantization weight only support lat method now"
    if alpha_format not in ("apot_int8", "block_fp16"):
        raise ValueError("alpha_format must be 'apot_int8' or 'block_fp16'")
    layers = _decoder_layers(model)

    first = find_layers(layers[0], layers=(nn.Conv2d, nn.Linear))
    probe = _layer_file(weights_dir, model_name, f"0.{next(iter(first))}", wbits)
    bW0, a0 = _read_layer_file(probe)
    if bW0.size(2) != wbits:
        raise AssertionError(f"Weight bit mismatch, expect {wbits} bits, but got {bW0.size(2)} bits")
    R = a0.size(1)

    missing = []
    for i in range(len(layers)):
        subset = find_layers(layers[i], layers=(nn.Conv2d, nn.Linear))
        # group_size = K / R per layer so that LutLinear.num_groups == R
        for name, lin in subset.items():
            make_lut(layers[i], {name: lin}, wbit=wbits, group_size=lin.in_features // R,
                     alpha_format=alpha_format)
        swapped = find_layers(layers[i], layers=(LutLinear,))
        for name, lut in swapped.items():
            path = _layer_file(weights_dir, model_name, f"{i}.{name}", wbits)
            if not os.path.exists(path):
                missing.append(path)
                continue
            bW, alpha = _read_layer_file(path)
            compressed, a = convert_weight(bW, alpha)
            lut.binaryWeight.data = compressed.to(lut.binaryWeight.dtype)
            if alpha_format == "apot_int8":
                lut.alpha.data = lut.quantize_to_apot(a)
            else:
                lut.alpha.data = a.to(torch.float16)
    for path in missing:
        print(f"WARNING: no such file {path}")
    return missing
