"""Quantised linear operator over the gfx950 LUT-GEMM engine.

Keeps the operator API of lut_gemm/quant.py in the ShiftAddLLM checkout
(`LutLinear` :8-61, `make_lut` :63-72, `load_lut` :74-114): constructor
arguments, buffer names (`binaryWeight`, `alpha` -- the state_dict keys) and
call semantics, so module trees and checkpoints written for the reference load
unchanged.  What differs is behind the call: `forward` launches the HIP kernels
of this package.  Where the reference crashes or reads out of bounds (no bias,
more than one token, fp32 input) this module does the evident thing instead.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import native

APOT_ABSENT = -128  # int8 exponent of an absent additive term

ALPHA_FORMATS = ("apot_int8", "block_fp16", "block_shift_u16", "rowwise_fp16")


def encode_apot_int8(alpha: torch.Tensor, num_apot: int = 3) -> torch.Tensor:
    """|alpha| -> int8 [..., num_apot] exponents with sum_a 2^s_a ~= |alpha|.

    The kernel adds the terms, all positive (mv_fp16_bias.hpp:473-482), so the
    encoder only emits positive terms: every term but the last is the largest
    power of two not above the remainder, the last is the power of two nearest
    to the remainder, and an exhausted remainder is written as -128 ("absent").
    A value with at most `num_apot` set mantissa bits -- any single power of two
    in particular -- is therefore encoded exactly.  (lut_gemm/quant.py:30-39
    keeps `round(log2|r|)` of a signed remainder and then drops the sign, which
    mis-encodes e.g. 0.75 as 1 + 0.25, and turns a zero remainder into
    int8(-inf).)
    """
    rem = alpha.detach().abs().to(torch.float64)
    terms = []
    for a in range(num_apot):
        live = rem > 0
        safe = torch.where(live, rem, torch.ones_like(rem))
        if a < num_apot - 1:
            e = torch.floor(torch.log2(safe))
            # guard the floor against log2 rounding at exact powers of two
            e = torch.where(torch.ldexp(torch.ones_like(safe), (e + 1).to(torch.int32)) <= safe, e + 1, e)
            e = torch.where(torch.ldexp(torch.ones_like(safe), e.to(torch.int32)) > safe, e - 1, e)
        else:
            lo = torch.floor(torch.log2(safe))
            lo_v = torch.ldexp(torch.ones_like(safe), lo.to(torch.int32))
            e = torch.where(safe - lo_v > 2 * lo_v - safe, lo + 1, lo)
        e = e.clamp(-127, 127)
        terms.append(torch.where(live, e, torch.full_like(e, APOT_ABSENT)).to(torch.int8))
        rem = torch.where(live, (rem - torch.ldexp(torch.ones_like(rem), e.to(torch.int32))).clamp_min(0), rem)
    return torch.stack(terms, dim=-1)


def decode_apot_int8(code: torch.Tensor) -> torch.Tensor:
    """int8 [..., 3] exponents -> fp32 multiplier, -128 contributing nothing."""
    e = code.to(torch.int32)
    val = torch.ldexp(torch.ones(e.shape, dtype=torch.float32, device=e.device), e.clamp_min(-127))
    return torch.where(e == APOT_ABSENT, torch.zeros_like(val), val).sum(dim=-1)


class LutLinear(nn.Module):
    """Drop-in for lut_gemm/quant.py:8-61.

    Buffers
      binaryWeight  int32 [K/32, wbit, N]  (bit t of word w <-> input 32w+t)
      alpha         depends on `alpha_format`:
        "apot_int8"       int8  [K/8, wbit, R, 3]  (what the reference forward uses)
        "block_fp16"      fp16  [K/8, wbit, R]
        "block_shift_u16" int16 [K/8, wbit, R]
        "rowwise_fp16"    fp16  [K/group_size, wbit, N]
    `num_groups = K // group_size` is passed to the kernel as in the reference:
    for the block formats callers choose group_size = K/R so that it equals the
    number R of row groups (lut_gemm/kernel.py:151,155); for "rowwise_fp16" it
    is the number of groups along K.
    """

    def __init__(self, infeatures: int, outfeatures: int, group_size: int = 128, wbit: int = 3,
                 bias=None, alpha_format: str = "apot_int8"):
        super().__init__()
        if alpha_format not in ALPHA_FORMATS:
            raise ValueError(f"alpha_format must be one of {ALPHA_FORMATS}")
        if infeatures % 32:
            raise ValueError("infeatures must be a multiple of 32")
        if infeatures % group_size:
            raise ValueError("group_size must divide infeatures")
        self.M = 1
        self.K = infeatures
        self.N = outfeatures
        self.group_size = group_size
        self.wbit = wbit
        self.num_groups = self.K // group_size
        self.num_apot = 3
        self.alpha_format = alpha_format

        self.register_buffer("binaryWeight",
                             torch.zeros((self.K // 32, wbit, self.N), dtype=torch.int32))
        if alpha_format == "apot_int8":
            a = torch.zeros((self.K // 8, wbit, self.num_groups, self.num_apot), dtype=torch.int8)
        elif alpha_format == "block_fp16":
            a = torch.zeros((self.K // 8, wbit, self.num_groups), dtype=torch.float16)
        elif alpha_format == "block_shift_u16":
            a = torch.zeros((self.K // 8, wbit, self.num_groups), dtype=torch.int16)
        else:
            a = torch.zeros((self.num_groups, wbit, self.N), dtype=torch.float16)
        self.register_buffer("alpha", a)
        # kept as a plain attribute like the reference (quant.py:28)
        self.bias = bias
        self.reuse_output = False      # see _output
        self._pow2_cache = None        # see _alphas_are_powers_of_two
        self._bias_cache = None
        self._out_cache = {}

    def quantize_to_apot(self, x):
        return encode_apot_int8(x, self.num_apot)

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        # The reference loader repeats every alpha row 8 times before storing it
        # (lut_gemm/kernel.py:172-176), giving K rows where the kernel indexes
        # K/8.  Accept such a tensor by keeping one row per 8-input chunk.
        key = prefix + "alpha"
        a = state_dict.get(key)
        if (a is not None and self.alpha_format != "rowwise_fp16" and a.dim() == self.alpha.dim()
                and a.shape[0] == self.K and tuple(a.shape[1:]) == tuple(self.alpha.shape[1:])):
            state_dict[key] = a[::8].contiguous()
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    def _bias_rows(self, rows, device):
        """The bias as `rows` contiguous fp16 rows on `device`, formed once per (rows, device)
        and per state of the bias tensor: what every call copies its output from."""
        b = self.bias
        key = (rows, device, b.data_ptr(), b._version)
        if self._bias_cache is None or self._bias_cache[0] != key:
            t = b.detach().to(device=device, dtype=torch.float16).reshape(1, self.N).expand(rows, self.N).contiguous()
            self._bias_cache = (key, t)
        return self._bias_cache[1]

    def _alphas_are_powers_of_two(self):
        """Whether every row-wise alpha is a positive normal fp16 power of two (what the reference's
        quantiser produces, quantizers/bcq_quant/bcq_shift.py:15-24): looked at once per state of the
        alpha tensor (one device synchronisation), and only by calls of three or more rows, which
        can then take the block-scaled matrix-core kernel."""
        a = self.alpha
        key = (a.data_ptr(), a._version, a.device)
        if self._pow2_cache is None or self._pow2_cache[0] != key:
            bits = a.view(torch.int16).to(torch.int32) & 0xffff
            field = (bits >> 10) & 0x1f
            ok = ((bits & 0x83ff) == 0) & (field >= 1) & (field <= 30)
            self._pow2_cache = (key, bool(ok.all().item()))
        return self._pow2_cache[1]

    def _output(self, rows, device):
        """The tensor the kernel accumulates into, pre-filled with the bias (or zeros): a new
        one per call like the reference's `bias.clone()` (lut_gemm/quant.py:46), or, with
        `reuse_output`, one buffer per (rows, device) that every call overwrites (no allocation
        on the call path, e.g. under HIP graph capture; the caller must be done with the previous
        result)."""
        if self.reuse_output:
            buf = self._out_cache.get((rows, device))
            if buf is None:
                buf = self._out_cache[(rows, device)] = torch.empty((rows, self.N), dtype=torch.float16, device=device)
            if self.bias is None:
                buf.zero_()
            else:
                buf.copy_(self._bias_rows(rows, device))
            return buf
        if self.bias is None:
            return torch.zeros((rows, self.N), dtype=torch.float16, device=device)
        return self._bias_rows(rows, device).clone()

    def forward(self, x):
        if x.shape[-1] != self.K:
            raise ValueError(f"expected last dimension {self.K}, got {tuple(x.shape)}")
        dtype = x.dtype
        # an fp16, contiguous input (what a half-precision decoder passes) goes to the kernel as it is
        x2 = x.reshape(-1, self.K)
        if dtype != torch.float16:
            x2 = x2.to(torch.float16)
        if not x2.is_contiguous():
            x2 = x2.contiguous()
        output = self._output(x2.shape[0], x2.device)

        ext = native.lutgemm
        fmt = self.alpha_format
        if fmt == "apot_int8":
            ext.lutgemm_compute_block_shiftInt8(output, self.binaryWeight, self.alpha, x2, self.N,
                                                self.K, self.wbit, self.num_groups, 3)
        elif fmt == "block_fp16":
            ext.lutgemm_compute_block(output, self.binaryWeight, self.alpha, x2, self.N, self.K,
                                      self.wbit, self.num_groups)
        elif fmt == "block_shift_u16":
            ext.lutgemm_compute_block_shift(output, self.binaryWeight, self.alpha, x2, self.N,
                                            self.K, self.wbit, self.num_groups, 3)
        elif 3 <= x2.shape[0] <= 8 and self._alphas_are_powers_of_two():
            ext.lutgemm_compute_shift_scale_pow2(output, self.binaryWeight, self.alpha, x2, self.N,
                                                 self.K, self.wbit, self.num_groups)
        else:
            ext.lutgemm_compute_shift_scale(output, self.binaryWeight, self.alpha, x2, self.N,
                                            self.K, self.wbit, self.num_groups)
        if dtype != torch.float16:
            output = output.to(dtype)
        return output.view(*x.shape[:-1], self.N)

    def extra_repr(self):
        return "in_features={}, out_features={}, bias={}, wbit={}, group_size={}, alpha_format={}".format(
            self.K, self.N, self.bias is not None, self.wbit, self.group_size, self.alpha_format)


def make_lut(module, names, name="", wbit=3, group_size=128, alpha_format="apot_int8"):
    """Swap every nn.Linear whose qualified name is in `names` for a LutLinear
    (lut_gemm/quant.py:63-72).  `names` may be any container of names, e.g. the
    dict returned by find_layers."""
    if isinstance(module, LutLinear):
        return
    for child_name, child in list(module.named_children()):
        full = name + "." + child_name if name != "" else child_name
        if full in names and isinstance(child, nn.Linear):
            setattr(module, child_name,
                    LutLinear(child.in_features, child.out_features, group_size, wbit,
                              bias=child.bias, alpha_format=alpha_format))
        else:
            make_lut(child, names, full, wbit, group_size, alpha_format)


def load_lut(model, checkpoint="", wbit=3, group_size=128):
    """Build an OPT skeleton whose decoder linears are LutLinear and optionally
    load a state_dict into it (lut_gemm/quant.py:74-114).  `model` is a hub name
    or local directory understood by OPTConfig.from_pretrained, or an OPTConfig."""
    from transformers import OPTConfig, OPTForCausalLM
    from .kernel import find_layers

    config = model if isinstance(model, OPTConfig) else OPTConfig.from_pretrained(model)
    previous = torch.get_default_dtype()
    torch.set_default_dtype(torch.half)
    try:
        with torch.device("meta"):
            skeleton = OPTForCausalLM(config)
        skeleton = skeleton.to_empty(device="cpu")
    finally:
        torch.set_default_dtype(previous)
    skeleton = skeleton.eval()
    layers = find_layers(skeleton)
    for skip in ("model.decoder.project_out", "model.decoder.project_in", "lm_head"):
        layers.pop(skip, None)
    make_lut(skeleton, layers, wbit=wbit, group_size=group_size)
    if checkpoint != "":
        skeleton.load_state_dict(torch.load(checkpoint, weights_only=True))
    skeleton.seqlen = skeleton.config.max_position_embeddings
    return skeleton
