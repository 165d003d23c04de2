"""Seeded synthetic BCQ problems for the parity tests and the benchmark.

Nothing here is on the inference path.  It restates, device-agnostically, how
ShiftAddLLM produces the operands the LUT-GEMM kernels consume:

  * `bcq_shift_quantize`  -- binary-coding quantisation with power-of-two
    scales: greedy initialisation plus alternating refinement, the algorithm of
    quantizers/bcq_quant/bcq_shift.py:82-245 in the ShiftAddLLM checkout
    (`quantize_shift`, apot_nums = 1), restated operation for operation so that
    it emits the reference's bits (checked against a committed fixture of the
    reference's own output, tests/golden/bcq_shift_reference.npz).
  * `assign_signs`        -- signs for given scales, quantizers/bcq_quant/quantizer.py:9-37.
  * row-wise problems (groups along K) and "Lat." block problems (8 input
    columns x N/R rows share one scale per bit plane,
    quant_methods/shiftaddllm.py:95-100,146-159).
"""
from __future__ import annotations

import math
import random
from dataclasses import dataclass

import torch

from .lut_gemm.kernel import pack_binaryWeight


def pow2_round(a: torch.Tensor) -> torch.Tensor:
    """sign(a) * 2^round(ln|a| / ln 2) (bcq_shift.py:15-39: natural log divided by
    np.log(2), round-half-to-even); zero stays zero."""
    mag = a.abs()
    e = torch.round(torch.log(torch.where(mag > 0, mag, torch.ones_like(mag))) / math.log(2.0))
    return torch.where(mag > 0, torch.sign(a) * (2.0 ** e), torch.zeros_like(a))


def _codebook(nb: int, device, dtype) -> torch.Tensor:
    """[2^nb, nb] of +-1 in the reference's enumeration order (list_binary_vecs,
    bcq_shift.py:194-198): plane 0 varies slowest, +1 before -1."""
    c = torch.arange(2 ** nb, device=device)
    bits = (c.unsqueeze(1) >> torch.arange(nb - 1, -1, -1, device=device)) & 1
    return (1 - 2 * bits).to(dtype)


def assign_signs(w: torch.Tensor, alpha: torch.Tensor, chunk_rows: int = 1 << 15) -> torch.Tensor:
    """Nearest codeword: w [rows, gs], alpha [rows, nb] -> B int8 [rows, gs, nb] of +-1
    minimising |w - sum_b alpha_b B_b| element-wise.  Same result as the reference's
    binary search tree (find_B_torch, bcq_shift.py:200-224): the 2^nb code values of
    a row are sorted, a weight goes to the interval of the midpoints it falls in (a
    weight exactly on a midpoint goes up), equal code values keep the sort's order."""
    rows, gs = w.shape
    nb = alpha.shape[1]
    book = _codebook(nb, w.device, torch.float32)            # [C, nb]
    out = torch.empty((rows, gs, nb), dtype=torch.int8, device=w.device)
    book8 = book.to(torch.int8)
    for r0 in range(0, rows, chunk_rows):
        r1 = min(rows, r0 + chunk_rows)
        values = alpha[r0:r1].float().mm(book.t())           # [r, C]
        # Equal code values are common (two planes with the same power-of-two scale): the
        # CPU sort the reference runs on keeps their order; asked for explicitly so that a
        # GPU breaks those ties the same way (otherwise it picks other, equivalent signs
        # and the next refinement round drifts off the reference's bits).
        vs, order = torch.sort(values, stable=True)
        mids = (vs[:, :-1] + vs[:, 1:]) / 2                  # non-decreasing
        slot = torch.searchsorted(mids, w[r0:r1].float().contiguous(), right=True)   # mids <= w
        out[r0:r1] = book8[torch.gather(order, 1, slot)]
    return out


def _least_squares_cg(gram: torch.Tensor, rhs: torch.Tensor, start: torch.Tensor) -> torch.Tensor:
    """nb steps of batched conjugate gradient on gram x = rhs from `start`, with the
    reference's 1e-6 guards in both quotients (batch_cg_torch, bcq_shift.py:226-245).
    gram [rows, nb, nb], rhs [rows, nb], start [rows, nb]."""
    rows, nb, _ = gram.shape
    x = start.clone().view(rows, nb, 1)
    res = rhs.view(rows, nb, 1) - gram.bmm(x)
    rr_new = res.transpose(1, 2).bmm(res)
    direction = res.clone()
    for _ in range(nb):
        rr = rr_new
        gd = gram.bmm(direction)
        step = rr / (direction.transpose(1, 2).bmm(gd) + 1e-6)
        x += step * direction
        res -= step * gd
        rr_new = res.transpose(1, 2).bmm(res)
        direction = res + (rr_new / (rr + 1e-6)) * direction
    return x.view(rows, nb)


def bcq_shift_quantize(w: torch.Tensor, nb: int, rounds: int = 5):
    """w [rows, gs] fp32 -> (B int8 [rows, gs, nb], alpha fp32 [rows, nb]) with
    alpha >= 0, sorted descending, each a power of two after refinement.

    The reference's quantize_shift(use_bst=True, apot_nums=1) with unit weighting
    (bcq_shift.py:82-192), float operation for float operation: on the committed
    fixture of the reference's own output it reproduces B and alpha exactly."""
    w = w.float()
    rows, gs = w.shape
    # greedy: peel off sign * mean|residual| (bcq_shift.py:131-161)
    B = torch.empty((rows, gs, nb), dtype=torch.float32, device=w.device)
    alpha = torch.empty((rows, nb), dtype=torch.float32, device=w.device)
    r = w.clone()
    for b in range(nb):
        # (the reference takes sign(r), which is 0 for an exact zero; +1 here, so
        # that every entry packs into one bit)
        s = torch.where(r >= 0, torch.ones_like(r), -torch.ones_like(r))
        a = r.abs().sum(dim=1) / float(gs)
        a[torch.isnan(a)] = 0.0
        B[:, :, b] = s
        alpha[:, b] = a
        r -= s * a.view(rows, 1)
    if rounds > 0 and nb > 1:
        for _ in range(rounds):
            # alpha given B: least squares by conjugate gradient from the current alpha,
            # magnitudes sorted, rounded to powers of two (bcq_shift.py:163-177)
            Bt = B.transpose(1, 2)
            sol = _least_squares_cg(Bt.bmm(B), Bt.bmm(w.unsqueeze(-1)).view(rows, nb), alpha)
            alpha = pow2_round(sol.abs().sort(dim=1, descending=True).values)
            # B given alpha (bcq_shift.py:187-189)
            B = assign_signs(w, alpha).float()
    return B.to(torch.int8), alpha


@dataclass
class RowwiseProblem:
    """One row-wise-alpha GEMV: kernel operands plus what made them."""
    N: int
    K: int
    nb: int
    group_size: int
    bW: torch.Tensor        # int32 [K/32, nb, N]
    alpha: torch.Tensor     # fp16  [K/group_size, nb, N]
    x: torch.Tensor         # fp16  [M, K]
    B: torch.Tensor | None = None      # int8 [N, K/gs, gs, nb]
    W: torch.Tensor | None = None      # fp32 [N, K] before quantisation

    @property
    def num_groups(self):
        return self.K // self.group_size


@dataclass
class BlockProblem:
    N: int
    K: int
    nb: int
    R: int
    bW: torch.Tensor        # int32 [K/32, nb, N]
    alpha: torch.Tensor     # fp16 [K/8, nb, R]
    x: torch.Tensor         # fp16 [M, K]
    disk_bWeight: torch.Tensor | None = None   # int32 [K, N/32, nb]
    disk_alpha: torch.Tensor | None = None     # fp32 [K/8, R, nb]


def _gen(seed: int) -> torch.Generator:
    return torch.Generator(device="cpu").manual_seed(seed)


def make_rowwise_problem(N, K, nb=3, group_size=128, M=1, seed=0, sigma=0.02, device="cpu",
                         rounds=5, quantize=True) -> RowwiseProblem:
    """Weights ~ N(0, sigma), x ~ N(0, 1) fp16, both drawn on the CPU generator
    so every machine sees the same bits.  quantize=False skips BCQ and draws
    random signs and power-of-two scales of the same distribution shape (for
    sizes where only throughput or size-independent properties are wanted)."""
    g = _gen(seed)
    x = torch.randn((M, K), generator=g).half().to(device)
    G = K // group_size
    if quantize:
        W = (torch.randn((N, K), generator=g) * sigma).to(device)
        Bq, a = bcq_shift_quantize(W.reshape(N * G, group_size), nb, rounds)
        B = Bq.reshape(N, G, group_size, nb)
        alpha = a.reshape(N, G, nb)
    else:
        W = None
        B = (torch.randint(0, 2, (N, G, group_size, nb), generator=g, dtype=torch.int8) * 2 - 1).to(device)
        e = torch.randint(-9, -5, (N, G, 1), generator=g).float() - torch.arange(nb).float()
        alpha = torch.exp2(e).to(device)
    bW = pack_binaryWeight(B).permute(1, 2, 0).contiguous()
    a16 = alpha.permute(1, 2, 0).contiguous().to(torch.float16)
    return RowwiseProblem(N, K, nb, group_size, bW, a16, x, B, W)


def make_block_problem(N, K, nb=2, R=8, M=1, seed=0, sigma=0.02, device="cpu", rounds=5,
                       quantize=True) -> BlockProblem:
    """ShiftAddLLM (Lat.) geometry: for every block of 8 adjacent input columns
    the N x 8 slab is cut into R row groups of N/R rows; each (block, row group)
    shares one power-of-two scale per bit plane."""
    g = _gen(seed)
    x = torch.randn((M, K), generator=g).half().to(device)
    rows = N // R
    C = K // 8
    if quantize:
        W = (torch.randn((N, K), generator=g) * sigma).to(device)
        # [N, K] -> [C, R, rows*8]: block c, row group r, the rows x 8 elements
        slabs = W.reshape(R, rows, C, 8).permute(2, 0, 1, 3).reshape(C * R, rows * 8)
        _, a = bcq_shift_quantize(slabs, nb, rounds)
        alpha = a.reshape(C, R, nb)                                   # on-disk order
        # signs per column with the block's scales (quantizer.py:9-37)
        a_col = alpha.repeat_interleave(8, dim=0).reshape(K * R, nb)  # [K*R, nb]
        cols = W.t().reshape(K * R, rows)                             # column k, row group r
        Bk = assign_signs(cols, a_col).reshape(K, R, rows, nb)        # [K, R, N/R, nb]
    else:
        Bk = (torch.randint(0, 2, (K, R, rows, nb), generator=g, dtype=torch.int8) * 2 - 1).to(device)
        e = torch.randint(-9, -5, (C, R, 1), generator=g).float() - torch.arange(nb).float()
        alpha = torch.exp2(e).to(device)
    disk_bW = pack_binaryWeight(Bk)                                   # [K, N/32, nb]
    by_row = Bk.reshape(K, N, nb).permute(1, 0, 2).reshape(N, 1, K, nb)
    bW = pack_binaryWeight(by_row).permute(1, 2, 0).contiguous()      # [K/32, nb, N]
    a16 = alpha.permute(0, 2, 1).contiguous().to(torch.float16)       # [K/8, nb, R]
    return BlockProblem(N, K, nb, R, bW, a16, x, disk_bW, alpha.float())


# ---- named configurations of the benchmark ---------------------------------

LLAMA2_7B_LINEARS = (
    ("q_proj", 4096, 4096), ("k_proj", 4096, 4096), ("v_proj", 4096, 4096), ("o_proj", 4096, 4096),
    ("gate_proj", 11008, 4096), ("up_proj", 11008, 4096), ("down_proj", 4096, 11008),
)
LLAMA2_13B_SHAPES = ((5120, 5120), (13824, 5120), (5120, 13824))
LLAMA2_70B_SHAPES = ((8192, 8192), (28672, 8192), (8192, 28672), (1024, 8192))
OPT125M_FC1 = (3072, 768)


def mixed_bit_config(n_layers=32, seed=0, prefix="model.layers"):
    """Per-linear bit widths drawn from {2,3,3,4} (ratio 1:2:1), in the
    `{"<module>": {"bits": b, "columnwise": bool}}` schema of the reference's
    --quant_config files (model/opt.py:83-88; sensitivity/mixbit/opt-125m.json)."""
    rng = random.Random(seed)
    names = ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
             "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj")
    return {f"{prefix}.{i}.{n}": {"bits": rng.choice((2, 3, 3, 4)), "columnwise": False}
            for i in range(n_layers) for n in names}
