"""Writes tests/golden/lutgemm_cases.npz: small seeded inputs and the oracle's
expected outputs for every operand format of the LUT-GEMM path.

The reference ships no golden vectors for this path (it has no tests at all), so
these are produced by this repo's CPU oracle (oracle/), whose functions are
pinned in tests/test_oracle_*.py by known answers, brute force and closed forms.
They freeze the oracle's answers: a later change of the oracle or of the workload
generator that alters any bit shows up as a fixture mismatch.

Run from the repo root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle as orc  # noqa: E402
from shiftaddllm_amd import workload  # noqa: E402
from shiftaddllm_amd.lut_gemm.quant import encode_apot_int8  # noqa: E402

out = {}

# row-wise alpha, real BCQ quantisation (3-bit, group 128), bias pre-filled
p = workload.make_rowwise_problem(96, 512, nb=3, group_size=128, M=2, seed=11)
bias = (torch.randn((2, 96), generator=torch.Generator().manual_seed(1)) * 0.1).half()
y16, y32 = orc.gemv_rowwise_c(p.bW.numpy(), p.alpha.numpy(), p.x.numpy(), p.num_groups, out=bias.numpy())
out.update(row_bW=p.bW.numpy(), row_alpha=p.alpha.numpy(), row_x=p.x.numpy(), row_bias=bias.numpy(),
           row_out=y16, row_y32=y32, row_B=p.B.numpy(), row_packed=orc.pack_binary_weight_np(p.B.numpy()))

# block alpha (Lat. geometry), real quantisation, 2-bit, R = 8; plus the on-disk tensors
b = workload.make_block_problem(64, 288, nb=2, R=8, M=1, seed=12)
y16, y32 = orc.gemv_block_c(b.bW.numpy(), b.alpha.numpy(), b.x.numpy(), 8, kind=orc.ALPHA_F16)
code = encode_apot_int8(b.alpha.float())
y16i, _ = orc.gemv_block_c(b.bW.numpy(), code.numpy(), b.x.numpy(), 8, kind=orc.ALPHA_APOT_I8)
out.update(blk_bW=b.bW.numpy(), blk_alpha=b.alpha.numpy(), blk_x=b.x.numpy(), blk_out=y16, blk_y32=y32,
           blk_disk_bW=b.disk_bWeight.numpy(), blk_disk_alpha=b.disk_alpha.numpy(),
           blk_apot=code.numpy(), blk_apot_out=y16i)

# uint16 shift fields and uniform mode on random operands
g = torch.Generator().manual_seed(13)
r = workload.make_rowwise_problem(64, 256, nb=3, group_size=64, M=1, seed=13, quantize=False)
u16 = torch.randint(0, 512, (256 // 8, 3, 4), generator=g).to(torch.int16)
xs = (r.x.float() * 0.01).half()
y16u, _ = orc.gemv_block_c(r.bW.numpy(), u16.numpy(), xs.numpy(), 4, kind=orc.ALPHA_SHIFT_U16)
ua = (torch.rand((4, 64), generator=g) * 0.05).half()
uq = (torch.randn((4, 64), generator=g) * 0.01).half()
y16q, _ = orc.gemv_uniform_c(r.bW.numpy(), ua.numpy(), uq.numpy(), r.x.numpy(), 4)
out.update(misc_bW=r.bW.numpy(), misc_x=r.x.numpy(), misc_xs=xs.numpy(), u16_alpha=u16.numpy(), u16_out=y16u,
           uni_alpha=ua.numpy(), uni_qbias=uq.numpy(), uni_out=y16q)

path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lutgemm_cases.npz")
np.savez_compressed(path, **out)
print("wrote", path, os.path.getsize(path), "bytes")
