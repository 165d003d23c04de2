"""Token-by-token decode harness over LutLinear layers.

Counterpart of the reference's kernel benchmark (`benchmark`, model/opt.py:367-423
in the ShiftAddLLM checkout): warm-up single-token forwards, then every token --
prompt tokens one at a time, then greedy continuations -- is one forward pass with
a KV cache, followed by a device synchronisation and a wall-clock reading; the
median seconds per token is reported.

The reference drives a HuggingFace OPT with its linears swapped for LutLinear and
needs the hub for the checkpoint.  This harness brings its own minimal
Llama-architecture decoder (RMSNorm, rotary embeddings, grouped-query-capable
attention over a static KV cache, SwiGLU MLP, fp16), random-initialised, whose
seven linears per block are LutLinear modules with a per-linear bit width taken
from a `{"<module>": {"bits": b, ...}}` map (the schema of the reference's
--quant_config files, model/opt.py:83-88).  One decode step can be captured in a
HIP graph; q/k/v and gate/up can be issued as one fused launch each.

Two implementations of everything between the linears exist: glue="hip" (the
default) runs this library's fused kernels -- RMSNorm, rotary + KV append +
attention, SiLU*up -- and lets o_proj / down_proj accumulate straight into the
residual stream, eight launches per block; glue="torch" spells the same step in
framework operations and is what the parity test's dense model is built from.
"""
from __future__ import annotations

import ctypes
import math
import statistics
import time
from dataclasses import dataclass

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import native
from .lut_gemm.quant import LutLinear


@dataclass
class DecoderConfig:
    vocab_size: int = 32000
    hidden: int = 4096
    intermediate: int = 11008
    layers: int = 32
    heads: int = 32
    kv_heads: int = 32
    max_positions: int = 256
    group_size: int = 128
    rope_theta: float = 10000.0
    rms_eps: float = 1e-5

    @property
    def head_dim(self):
        return self.hidden // self.heads


LLAMA2_7B = DecoderConfig()


def random_lut_linear(in_f, out_f, bits, group_size, gen, device):
    """LutLinear ("rowwise_fp16") with random sign planes and power-of-two scales
    shaped like BCQ output of N(0, 0.02) weights: per (group, row) a base exponent,
    one octave lower per further bit plane."""
    lin = LutLinear(in_f, out_f, group_size=group_size, wbit=bits, bias=None, alpha_format="rowwise_fp16")
    lin = lin.to(device)
    lin.binaryWeight.data = torch.randint(-2 ** 31, 2 ** 31 - 1, (in_f // 32, bits, out_f), generator=gen,
                                          device=device, dtype=torch.int32)
    e = torch.randint(-8, -5, (in_f // group_size, 1, out_f), generator=gen, device=device).float()
    e = e - torch.arange(bits, device=device).float().view(1, bits, 1)
    lin.alpha.data = torch.exp2(e).to(torch.float16).contiguous()
    return lin


class Block(nn.Module):
    def __init__(self, cfg: DecoderConfig, bits: dict, gen, device):
        super().__init__()
        h, kvd = cfg.hidden, cfg.kv_heads * cfg.head_dim
        mk = lambda name, i, o: random_lut_linear(i, o, bits[name], cfg.group_size, gen, device)
        self.q_proj = mk("self_attn.q_proj", h, h)
        self.k_proj = mk("self_attn.k_proj", h, kvd)
        self.v_proj = mk("self_attn.v_proj", h, kvd)
        self.o_proj = mk("self_attn.o_proj", h, h)
        self.gate_proj = mk("mlp.gate_proj", h, cfg.intermediate)
        self.up_proj = mk("mlp.up_proj", h, cfg.intermediate)
        self.down_proj = mk("mlp.down_proj", cfg.intermediate, h)
        self.input_norm = nn.Parameter(torch.ones(h, dtype=torch.float16, device=device))
        self.post_norm = nn.Parameter(torch.ones(h, dtype=torch.float16, device=device))


def rms_norm(x, w, eps):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype) * w


class LutDecoder(nn.Module):
    """Single-token-per-step decoder with a static KV cache of cfg.max_positions."""

    def __init__(self, cfg: DecoderConfig, quant_config: dict | None = None, batch: int = 1, seed: int = 0,
                 device="cuda:0", default_bits: int = 3, fuse_launches: bool = True,
                 module_prefix: str = "model.layers", glue: str = "hip", chain: bool = False):
        super().__init__()
        if glue not in ("hip", "torch"):
            raise ValueError(f"glue must be 'hip' or 'torch', got {glue!r}")
        self.cfg, self.batch, self.fuse, self.glue = cfg, batch, fuse_launches, glue
        # o_proj, gate/up, down_proj and the next block's q,k,v as ONE chained launch per block (tagged
        # rows hand the activations over inside the launch): two launches per block with the attention
        # kernel.  One or two sequences (the chained launch runs on the look-up kernel), hidden <= 8192.
        self.chain = bool(chain) and fuse_launches and glue == "hip" and batch <= 2 and cfg.hidden <= 8192
        # One or two sequences: RMSNorm inside the q,k,v and gate,up GEMVs (every workgroup re-reads
        # the row to form its RMS and scales its finished sums; the look-up kernel only).  Measured
        # against the split below on the 7B decoder at one sequence: 1.535 vs 1.572 ms per token.
        self.fold_norm = fuse_launches and batch <= 2
        # RMSNorm split over the GEMV that completes the residual row (it leaves x * norm weight and
        # the row's sums of squares) and the GEMVs that read it (they scale their sums): no norm
        # launches inside the stack, for any batch size
        self.split_norm = fuse_launches and cfg.hidden % 32 == 0
        dev = torch.device(device)
        gen = torch.Generator(device=dev).manual_seed(seed)
        names = ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
                 "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj")
        self.blocks = nn.ModuleList()
        for i in range(cfg.layers):
            bits = {n: (quant_config or {}).get(f"{module_prefix}.{i}.{n}", {}).get("bits", default_bits)
                    for n in names}
            self.blocks.append(Block(cfg, bits, gen, dev))
        scale = 0.02
        self.embed = nn.Parameter((torch.randn((cfg.vocab_size, cfg.hidden), generator=gen, device=dev) * scale).half())
        self.lm_head = nn.Parameter((torch.randn((cfg.vocab_size, cfg.hidden), generator=gen, device=dev) * scale).half())
        self.final_norm = nn.Parameter(torch.ones(cfg.hidden, dtype=torch.float16, device=dev))
        hd = cfg.head_dim
        inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, hd, 2, device=dev).float() / hd))
        ang = torch.arange(cfg.max_positions, device=dev).float()[:, None] * inv[None, :]
        self.register_buffer("cos", torch.cat([ang.cos(), ang.cos()], dim=-1).half(), persistent=False)
        self.register_buffer("sin", torch.cat([ang.sin(), ang.sin()], dim=-1).half(), persistent=False)
        shape = (cfg.layers, batch, cfg.kv_heads, cfg.max_positions, hd)
        self.register_buffer("k_cache", torch.zeros(shape, dtype=torch.float16, device=dev), persistent=False)
        self.register_buffer("v_cache", torch.zeros(shape, dtype=torch.float16, device=dev), persistent=False)
        self.register_buffer("positions", torch.arange(cfg.max_positions, device=dev), persistent=False)
        # static step inputs/outputs (graph replay reads and writes these)
        self.register_buffer("ids", torch.zeros((batch,), dtype=torch.long, device=dev), persistent=False)
        self.register_buffer("pos", torch.zeros((1,), dtype=torch.long, device=dev), persistent=False)
        self.register_buffer("logits", torch.zeros((batch, cfg.vocab_size), dtype=torch.float16, device=dev),
                             persistent=False)
        # static activations of the glue="hip" step
        H, KV, I = cfg.heads * hd, cfg.kv_heads * hd, cfg.intermediate
        f16 = dict(dtype=torch.float16, device=dev)
        self.register_buffer("x_res", torch.zeros((batch, cfg.hidden), **f16), persistent=False)
        self.register_buffer("h_norm", torch.zeros((batch, cfg.hidden), **f16), persistent=False)
        self.register_buffer("qkv", torch.zeros((batch * (H + 2 * KV),), **f16), persistent=False)
        self.register_buffer("att", torch.zeros((batch, H), **f16), persistent=False)
        self.register_buffer("gate_up", torch.zeros((2 * batch * I,), **f16), persistent=False)
        self.register_buffer("act", torch.zeros((batch, I), **f16), persistent=False)
        self.register_buffer("sumsq", torch.zeros((2 * cfg.layers, batch, max(cfg.hidden // 32, 1)),
                                                  dtype=torch.float32, device=dev), persistent=False)
        if self.chain:
            i32 = dict(dtype=torch.int32, device=dev)
            self.register_buffer("x_tagged", torch.zeros((batch, cfg.hidden), **i32), persistent=False)
            self.register_buffer("gate_tagged", torch.zeros((batch, I), **i32), persistent=False)
            self.register_buffer("up_tagged", torch.zeros((batch, I), **i32), persistent=False)
            self.register_buffer("chain_words", torch.zeros((2,), **i32), persistent=False)   # epoch, status
        self._graph = None
        self._stream = None

    def chain_status(self):
        """0, or -8 when a wait inside a chained launch gave up since the status word was last cleared
        (synchronises the current stream)."""
        if not self.chain:
            return 0
        return native.cabi().lutgemm_chain_status(self.chain_words.data_ptr() + 4,
                                                  ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))

    # ---- linear layers -----------------------------------------------------------------
    def _fused(self, lins, x):
        """Several LutLinears sharing the input x [B, K] in one launch."""
        outs = [torch.zeros((x.shape[0], l.N), dtype=torch.float16, device=x.device) for l in lins]
        arr = (native.RowwiseProblem * len(lins))()
        for i, (l, o) in enumerate(zip(lins, outs)):
            arr[i] = native.RowwiseProblem(l.binaryWeight.data_ptr(), l.alpha.data_ptr(), x.data_ptr(),
                                           o.data_ptr(), l.N, l.K, l.wbit, l.num_groups, x.shape[0])
        rc = native.cabi().lutgemm_gemv_rowwise_f16_grouped(
            len(lins), arr, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        if rc:
            raise RuntimeError(native.cabi().lutgemm_strerror(rc).decode())
        return outs

    def _linears(self, lins, x):
        if self.fuse and len(lins) > 1:
            return self._fused(lins, x)
        return [l(x) for l in lins]

    def _rope(self, t, cos, sin):
        half = t.shape[-1] // 2
        rot = torch.cat([-t[..., half:], t[..., :half]], dim=-1)
        return t * cos + rot * sin

    # ---- one token ---------------------------------------------------------------------------
    @torch.no_grad()
    def step(self):
        """Consumes self.ids [B] at position self.pos [1]; writes self.logits [B, V]."""
        if self.glue == "hip":
            return self._step_hip()
        return self._step_torch()

    def _gemv_into(self, lins, x, outs, sp):
        """outs[i] += lins[i](x); one grouped launch when fusing."""
        lib, B = native.cabi(), x.shape[0]
        if self.fuse and len(lins) > 1:
            arr = (native.RowwiseProblem * len(lins))()
            for i, (l, o) in enumerate(zip(lins, outs)):
                arr[i] = native.RowwiseProblem(l.binaryWeight.data_ptr(), l.alpha.data_ptr(), x.data_ptr(),
                                               o.data_ptr(), l.N, l.K, l.wbit, l.num_groups, B)
            rc = lib.lutgemm_gemv_rowwise_f16_grouped(len(lins), arr, sp)
            if rc:
                raise RuntimeError(lib.lutgemm_strerror(rc).decode())
            return
        for l, o in zip(lins, outs):
            rc = lib.lutgemm_gemv_rowwise_f16(l.binaryWeight.data_ptr(), l.alpha.data_ptr(), x.data_ptr(),
                                              o.data_ptr(), l.N, l.K, l.wbit, l.num_groups, B, sp)
            if rc:
                raise RuntimeError(lib.lutgemm_strerror(rc).decode())

    def _fused_gemv(self, lins, x, outs, sp, norm=None, gate=None, overwrite=False, next_norm=None, next_in=None,
                    sumsq_out=None, sumsq_in=None):
        """One launch: outs[i] (+)= lins[i](t(x)), t = RMSNorm with weight `norm`, or
        silu(gate) * x, or identity.  next_norm / next_in / sumsq_out: the outputs complete
        a residual row whose norm-weighted copy and sums of squares are left for the next
        GEMV; sumsq_in: x is such a copy and the sums are scaled by its reciprocal RMS."""
        lib, B = native.cabi(), x.shape[0]
        ptr = lambda t: t.data_ptr() if t is not None else None
        arr = (native.FusedProblem * len(lins))()
        for i, (l, o) in enumerate(zip(lins, outs)):
            arr[i] = native.FusedProblem(l.binaryWeight.data_ptr(), l.alpha.data_ptr(), x.data_ptr(), o.data_ptr(),
                                         l.N, l.K, l.wbit, l.num_groups, B, int(overwrite), ptr(norm), ptr(gate),
                                         self.cfg.rms_eps, ptr(next_norm), ptr(next_in), ptr(sumsq_out),
                                         ptr(sumsq_in), sumsq_in.shape[-1] if sumsq_in is not None else 0)
        rc = lib.lutgemm_gemv_rowwise_f16_fused(len(lins), arr, sp)
        if rc:
            raise RuntimeError(lib.lutgemm_strerror(rc).decode())

    def _step_chained(self):
        """glue="hip" with chain=True: per block the attention kernel and ONE chained launch."""
        cfg, B = self.cfg, self.batch
        hd, H, KV, I = cfg.head_dim, cfg.heads, cfg.kv_heads, cfg.intermediate
        lib = native.cabi()
        sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

        def check(rc):
            if rc:
                raise RuntimeError(lib.lutgemm_strerror(rc).decode())

        nq, nkv = B * H * hd, B * KV * hd
        q, k, v = self.qkv[:nq], self.qkv[nq:nq + nkv], self.qkv[nq + nkv:]
        x, h, xt, gt, ut = self.x_res, self.h_norm, self.x_tagged, self.gate_tagged, self.up_tagged
        epoch = self.chain_words.data_ptr()
        ctl = native.ChainControl(epoch, epoch + 4, 0)

        def problem(lin, src, dst, x_tag=0, gate_tag=0, out_tag=0, norm=None, gate=None, overwrite=False):
            return native.ChainProblem(
                native.FusedProblem(lin.binaryWeight.data_ptr(), lin.alpha.data_ptr(), src.data_ptr(), dst.data_ptr(), lin.N,
                                    lin.K, lin.wbit, lin.num_groups, B, int(overwrite),
                                    norm.data_ptr() if norm is not None else None,
                                    gate.data_ptr() if gate is not None else None, cfg.rms_eps),
                x_tag, gate_tag, out_tag)

        torch.index_select(self.embed, 0, self.ids, out=x)
        check(lib.lutgemm_chain_tag_rows(xt.data_ptr(), x.data_ptr(), x.numel(), 255, epoch, sp))
        first = self.blocks[0]
        self._fused_gemv([first.q_proj, first.k_proj, first.v_proj], x, [q, k, v], sp, norm=first.input_norm, overwrite=True)
        for li, blk in enumerate(self.blocks):
            check(lib.lutgemm_decode_attention_f16(q.data_ptr(), k.data_ptr(), v.data_ptr(), self.cos.data_ptr(),
                                                   self.sin.data_ptr(), self.k_cache[li].data_ptr(),
                                                   self.v_cache[li].data_ptr(), self.pos.data_ptr(),
                                                   self.att.data_ptr(), B, H, KV, hd, cfg.max_positions, sp))
            t = 4 * li                                     # tag bases of this block: t+1 .. t+4
            ps = [problem(blk.o_proj, self.att, xt, out_tag=t + 1),                                     # x += o_proj(att)
                  problem(blk.gate_proj, xt, gt, x_tag=t + 1, out_tag=t + 2, norm=blk.post_norm, overwrite=True),
                  problem(blk.up_proj, xt, ut, x_tag=t + 1, out_tag=t + 3, norm=blk.post_norm, overwrite=True),
                  problem(blk.down_proj, ut, xt, x_tag=t + 3, gate_tag=t + 2, out_tag=t + 4, gate=gt)]  # x += down(silu(g) * u)
            if li + 1 < len(self.blocks):
                nxt = self.blocks[li + 1]
                ps += [problem(lin, xt, dst, x_tag=t + 4, norm=nxt.input_norm, overwrite=True)
                       for lin, dst in ((nxt.q_proj, q), (nxt.k_proj, k), (nxt.v_proj, v))]
            arr = (native.ChainProblem * len(ps))(*ps)
            check(lib.lutgemm_gemv_rowwise_f16_chain(len(ps), arr, ctypes.byref(ctl), sp))
        check(lib.lutgemm_chain_untag_rows(x.data_ptr(), xt.data_ptr(), x.numel(), sp))
        check(lib.lutgemm_chain_advance_epoch(epoch, 4 * len(self.blocks) + 256, sp))
        check(lib.lutgemm_decode_rmsnorm_f16(x.data_ptr(), self.final_norm.data_ptr(), h.data_ptr(), B, cfg.hidden,
                                             cfg.rms_eps, None, 0, sp))
        torch.matmul(h, self.lm_head.t(), out=self.logits)

    def _step_hip(self):
        if self.chain:
            return self._step_chained()
        cfg, B = self.cfg, self.batch
        hd, H, KV, I = cfg.head_dim, cfg.heads, cfg.kv_heads, cfg.intermediate
        lib = native.cabi()
        sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

        def check(rc):
            if rc:
                raise RuntimeError(lib.lutgemm_strerror(rc).decode())

        nq, nkv = B * H * hd, B * KV * hd
        q, k, v = self.qkv[:nq], self.qkv[nq:nq + nkv], self.qkv[nq + nkv:]
        g, u = self.gate_up[:B * I].view(B, I), self.gate_up[B * I:].view(B, I)
        x, h = self.x_res, self.h_norm
        # With grouped launches on, q,k,v and gate,up overwrite their outputs and, with one
        # or two rows (look-up kernel), SiLU*up rides inside the down_proj kernel: seven
        # launches per block, eight with more rows.  Without grouped launches the glue
        # kernels also clear the accumulate-into outputs.
        fold = self.fuse
        fold_gate = fold and B <= 2                         # input transforms live in the look-up kernel
        fold_norm = fold_gate and self.fold_norm
        split = fold and self.split_norm and not fold_norm
        rmsnorm = lambda w, clear=None: check(lib.lutgemm_decode_rmsnorm_f16(
            x.data_ptr(), w.data_ptr(), h.data_ptr(), B, cfg.hidden, cfg.rms_eps,
            clear.data_ptr() if clear is not None else None, clear.numel() * 2 if clear is not None else 0, sp))
        torch.index_select(self.embed, 0, self.ids, out=x)
        if split:
            self.sumsq.zero_()
        for li, blk in enumerate(self.blocks):
            qkv_lins = [blk.q_proj, blk.k_proj, blk.v_proj]
            if split and li > 0:                                        # h, sums: left by the last down_proj
                self._fused_gemv(qkv_lins, h, [q, k, v], sp, overwrite=True, sumsq_in=self.sumsq[2 * li - 1])
            elif fold_norm:
                self._fused_gemv(qkv_lins, x, [q, k, v], sp, norm=blk.input_norm, overwrite=True)
            elif fold:
                rmsnorm(blk.input_norm)
                self._fused_gemv(qkv_lins, h, [q, k, v], sp, overwrite=True)
            else:
                rmsnorm(blk.input_norm, self.qkv)
                self._gemv_into(qkv_lins, h, [q, k, v], sp)
            check(lib.lutgemm_decode_attention_f16(q.data_ptr(), k.data_ptr(), v.data_ptr(), self.cos.data_ptr(),
                                                   self.sin.data_ptr(), self.k_cache[li].data_ptr(),
                                                   self.v_cache[li].data_ptr(), self.pos.data_ptr(),
                                                   self.att.data_ptr(), B, H, KV, hd, cfg.max_positions, sp))
            gate_up = [blk.gate_proj, blk.up_proj]
            if split:                                                   # x += o_proj(att); h = x * post_norm
                self._fused_gemv([blk.o_proj], self.att, [x], sp, next_norm=blk.post_norm, next_in=h,
                                 sumsq_out=self.sumsq[2 * li])
                self._fused_gemv(gate_up, h, [g, u], sp, overwrite=True, sumsq_in=self.sumsq[2 * li])
            else:
                self._gemv_into([blk.o_proj], self.att, [x], sp)        # x += o_proj(att)
                if fold_norm:
                    self._fused_gemv(gate_up, x, [g, u], sp, norm=blk.post_norm, overwrite=True)
                elif fold:
                    rmsnorm(blk.post_norm)
                    self._fused_gemv(gate_up, h, [g, u], sp, overwrite=True)
                else:
                    rmsnorm(blk.post_norm, self.gate_up)
                    self._gemv_into(gate_up, h, [g, u], sp)
            # x += down_proj(silu(g) * u), leaving the next block's normalised input behind
            nxt = dict(next_norm=self.blocks[li + 1].input_norm, next_in=h, sumsq_out=self.sumsq[2 * li + 1]) \
                if split and li + 1 < len(self.blocks) else {}
            if fold_gate:
                self._fused_gemv([blk.down_proj], u, [x], sp, gate=g, **nxt)
            else:
                check(lib.lutgemm_decode_silu_mul_f16(g.data_ptr(), u.data_ptr(), self.act.data_ptr(), B * I, sp))
                if nxt:
                    self._fused_gemv([blk.down_proj], self.act, [x], sp, **nxt)
                else:
                    self._gemv_into([blk.down_proj], self.act, [x], sp)
        rmsnorm(self.final_norm)
        torch.matmul(h, self.lm_head.t(), out=self.logits)

    def _step_torch(self):
        cfg, B = self.cfg, self.batch
        hd, H, KV = cfg.head_dim, cfg.heads, cfg.kv_heads
        x = self.embed[self.ids]                                    # [B, hidden]
        cos = self.cos.index_select(0, self.pos).view(1, 1, hd)
        sin = self.sin.index_select(0, self.pos).view(1, 1, hd)
        # keys at positions > pos are masked out
        mask = (self.positions <= self.pos).view(1, 1, 1, cfg.max_positions)
        for li, blk in enumerate(self.blocks):
            h = rms_norm(x, blk.input_norm, cfg.rms_eps).contiguous()
            q, k, v = self._linears([blk.q_proj, blk.k_proj, blk.v_proj], h)
            q = self._rope(q.view(B, H, hd), cos, sin)
            k = self._rope(k.view(B, KV, hd), cos, sin)
            self.k_cache[li].index_copy_(2, self.pos, k.unsqueeze(2))
            self.v_cache[li].index_copy_(2, self.pos, v.view(B, KV, 1, hd))
            kk, vv = self.k_cache[li], self.v_cache[li]
            if KV != H:
                kk = kk.repeat_interleave(H // KV, dim=1)
                vv = vv.repeat_interleave(H // KV, dim=1)
            att = F.scaled_dot_product_attention(q.unsqueeze(2), kk, vv, attn_mask=mask)   # [B, H, 1, hd]
            (o,) = self._linears([blk.o_proj], att.reshape(B, H * hd).contiguous())
            x = x + o
            h = rms_norm(x, blk.post_norm, cfg.rms_eps).contiguous()
            g, u = self._linears([blk.gate_proj, blk.up_proj], h)
            (d,) = self._linears([blk.down_proj], (F.silu(g) * u).contiguous())
            x = x + d
        x = rms_norm(x, self.final_norm, cfg.rms_eps)
        self.logits.copy_(x @ self.lm_head.t())

    @torch.no_grad()
    def capture(self):
        """Capture step() in a HIP graph (after one eager run on the capture stream,
        which also sizes the LUT-GEMM workspace of that stream)."""
        self._stream = torch.cuda.Stream()
        # weights, caches and the step's input buffers were filled on the creating stream:
        # without this wait the first step may read them (the token ids among them, which
        # index the embedding table) before they have been written
        self._stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(self._stream):
            self.step()
        self._stream.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=self._stream):
            self.step()
        self._graph = g

    @torch.no_grad()
    def forward_token(self, ids: torch.Tensor, position: int):
        # the attention kernel clamps the position into the cache: past its end it would
        # overwrite the last slot and return plausible but wrong logits
        if not 0 <= position < self.cfg.max_positions:
            raise ValueError(f"position {position} outside the KV cache of {self.cfg.max_positions} positions")
        self.ids.copy_(ids)
        self.pos.fill_(position)
        if self._graph is not None:
            self._graph.replay()
        else:
            self.step()
        return self.logits

    def reset(self):
        self.k_cache.zero_()
        self.v_cache.zero_()

    def linear_bytes_per_token(self):
        """Algorithmic HBM bytes of the LUT-GEMM calls of one step (signs + alphas
        + activations + outputs), for throughput accounting."""
        lib = native.cabi()
        total = 0
        for blk in self.blocks:
            for l in (blk.q_proj, blk.k_proj, blk.v_proj, blk.o_proj, blk.gate_proj, blk.up_proj, blk.down_proj):
                total += lib.lutgemm_algorithmic_bytes(l.N, l.K, l.wbit, self.batch, l.num_groups * l.wbit * l.N, 2)
        return total


@torch.no_grad()
def benchmark(model: LutDecoder, input_ids: torch.Tensor, generate: int = 128, warmup: int = 10, check: bool = False):
    """input_ids [B, T] prompt.  Every prompt token, then `generate` greedy tokens,
    is one synchronised single-token step.  Returns a dict with the median seconds
    per token over the generated tokens (and over the prompt tokens), tokens/s
    (batch * 1/median) and the generated ids.  With `check` the cross-entropy of every
    prompt position's logits against the next prompt token is accumulated as well and
    `ppl` = exp(mean loss) is returned, as model/opt.py:382-384,414-423 does (outside
    the timed region of a token)."""
    B, T = input_ids.shape
    assert B == model.batch and T + generate <= model.cfg.max_positions
    dev = model.ids.device
    input_ids = input_ids.to(dev)
    for _ in range(warmup):
        model.forward_token(input_ids[:, 0], 0)
        torch.cuda.synchronize()
    model.reset()
    times_prompt, times_gen, out_ids = [], [], []
    nxt = None
    tot = torch.zeros((), dtype=torch.float32, device=dev)
    for i in range(T + generate):
        ids = input_ids[:, i] if i < T else nxt
        torch.cuda.synchronize()
        tick = time.perf_counter()
        logits = model.forward_token(ids, i)
        torch.cuda.synchronize()
        (times_prompt if i < T else times_gen).append(time.perf_counter() - tick)
        if check and i < T - 1:
            tot += F.cross_entropy(logits.float(), input_ids[:, i + 1])
        nxt = logits.argmax(dim=-1)
        if i >= T - 1:
            out_ids.append(nxt.clone())
    med = statistics.median(times_gen) if times_gen else float("nan")
    res = {
        "batch": B, "prompt_tokens": T, "generated_tokens": generate,
        "median_s_per_token": med,
        "median_s_per_prompt_token": statistics.median(times_prompt),
        "tokens_per_s": B / med if med == med else float("nan"),
        "generated": torch.stack(out_ids[:-1], dim=1).cpu() if len(out_ids) > 1 else None,
    }
    if check:
        res["ppl"] = float(torch.exp(tot / max(T - 1, 1)).item())
    return res


@torch.no_grad()
def benchmark_hf(model, input_ids: torch.Tensor, check: bool = False, warmup: int = 100):
    """The reference's kernel benchmark itself (model/opt.py:367-423) for a HuggingFace
    causal LM whose linears may be LutLinear: `warmup` single-token forwards of the first
    token, then every token of input_ids [1, T] is one forward with the growing key/value
    cache, a device synchronisation and a wall-clock reading; returns the median seconds per
    token, tokens/s and, with `check`, the perplexity of the sequence under the model."""
    dev = next(model.parameters()).device
    input_ids = input_ids.to(dev)
    T = input_ids.numel()
    attention_mask = torch.ones((1, T), device=dev)
    torch.cuda.synchronize()
    for _ in range(warmup):
        model(input_ids[:, 0].reshape(1, -1), past_key_values=None, attention_mask=attention_mask[:, :1])
        torch.cuda.synchronize()
    past, times = None, []
    tot = torch.zeros((), dtype=torch.float32, device=dev)
    for i in range(T):
        tick = time.perf_counter()
        out = model(input_ids[:, i].reshape(1, -1), past_key_values=past, attention_mask=attention_mask[:, :i + 1],
                    use_cache=True)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - tick)
        if check and i != T - 1:
            tot += F.cross_entropy(out.logits[0].float(), input_ids[:, i + 1])
        past = out.past_key_values
        del out
    med = statistics.median(times)
    res = {"tokens": T, "median_s_per_token": med, "tokens_per_s": 1.0 / med}
    if check:
        res["ppl"] = float(torch.exp(tot / max(T - 1, 1)).item())
    return res
