"""The C ABI boundary without a GPU: the library loads, exports every symbol the
header declares, rejects malformed calls before touching the device, and quotes
the algorithmic byte counts the throughput figures are computed from."""
import ctypes
import os
import re

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(REPO, "include", "lutgemm_gfx950.h")


@pytest.fixture(scope="module")
def lib():
    from shiftaddllm_amd import native
    if not os.path.exists(native.KERNEL_LIB):
        from shiftaddllm_amd import build
        build.build_kernel_library()
    return native.cabi()


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lutgemm_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared_functions()
    for want in ("lutgemm_gemv_rowwise_f16", "lutgemm_gemv_rowwise_f16_grouped", "lutgemm_gemv_uniform_f16", "lutgemm_gemv_block_f16",
                 "lutgemm_gemv_block_shift_u16", "lutgemm_gemv_block_apot_i8"):
        assert want in names


def test_library_exports_every_declared_symbol(lib):
    from shiftaddllm_amd import native
    declared = _declared_functions()
    assert sorted(native.C_ABI_SYMBOLS) == declared
    for name in declared:
        assert getattr(lib, name) is not None, name


def test_strerror(lib):
    assert lib.lutgemm_strerror(0) == b"ok"
    for code in (-1, -2, -3, -4, -5):
        assert len(lib.lutgemm_strerror(code)) > 3
    assert b"unknown" in lib.lutgemm_strerror(-99)


def test_algorithmic_bytes_worked_examples(lib):
    f = lib.lutgemm_algorithmic_bytes
    # signs K*N*nb/8 + alphas + x (2MK) + out read and write (2 * 2MN)
    assert f(3072, 768, 3, 1, 6 * 3 * 3072, 2) == 1_009_152          # OPT-125m fc1
    assert f(4096, 4096, 3, 1, 32 * 3 * 4096, 2) == 7_102_464        # Llama-2-7B q/k/v/o
    assert f(11008, 4096, 3, 1, 32 * 3 * 11008, 2) == 19_074_048     # gate/up
    assert f(4096, 11008, 3, 1, 86 * 3 * 4096, 2) == 19_060_224      # down
    assert f(5120, 5120, 2, 1, 640 * 2 * 8, 2) == 6_604_800          # 13B block alpha
    assert f(13824, 5120, 2, 1, 640 * 2 * 8, 2) == 17_780_736
    assert f(5120, 13824, 2, 1, 1728 * 2 * 8, 2) == 17_798_144


def test_malformed_calls_are_rejected_on_the_host(lib):
    # Validation happens before any HIP call, so this needs no GPU.  Aligned dummy
    # addresses are never dereferenced because every call below must fail first.
    p = ctypes.c_void_p(0x1000)
    E_INVAL, E_ALIGN, E_UNSUP = -1, -2, -3
    row = lib.lutgemm_gemv_rowwise_f16
    assert row(None, p, p, p, 64, 64, 3, 2, 1, None) == E_INVAL          # null bW
    assert row(p, p, p, None, 64, 64, 3, 2, 1, None) == E_INVAL          # null out
    assert row(p, p, p, p, 64, 48, 3, 1, 1, None) == E_INVAL             # K % 32
    assert row(p, p, p, p, 66, 64, 3, 2, 1, None) == E_INVAL             # N % 4
    assert row(p, p, p, p, 64, 64, 0, 2, 1, None) == E_INVAL             # nb < 1
    assert row(p, p, p, p, 64, 64, 5, 2, 1, None) == E_INVAL             # nb > 4
    assert row(p, p, p, p, 64, 64, 3, 4, 1, None) == E_INVAL             # group of 16 inputs
    assert row(p, p, p, p, 64, 64, 3, 3, 1, None) == E_INVAL             # groups do not divide K
    assert row(p, p, p, p, 64, 64, 3, 2, 0, None) == E_INVAL             # M = 0
    assert row(p, p, p, p, -4, 64, 3, 2, 1, None) == E_INVAL
    assert row(ctypes.c_void_p(0x1004), p, p, p, 64, 64, 3, 2, 1, None) == E_ALIGN
    assert row(p, ctypes.c_void_p(0x1002), p, p, 64, 64, 3, 2, 1, None) == E_ALIGN
    blk = lib.lutgemm_gemv_block_f16
    assert blk(p, p, p, p, 64, 64, 2, 3, 1, None) == E_INVAL             # R does not divide N
    assert blk(p, p, p, p, 64, 64, 2, 32, 1, None) == E_INVAL            # 2 rows per group
    assert lib.lutgemm_gemv_block_shift_u16(p, p, p, p, 64, 64, 2, 8, 2, 1, None) == E_UNSUP
    assert lib.lutgemm_gemv_block_apot_i8(p, p, p, p, 64, 64, 2, 8, 1, 1, None) == E_UNSUP
    assert lib.lutgemm_gemv_uniform_f16(p, p, None, p, p, 64, 64, 3, 2, 1, None) == E_INVAL
    assert lib.lutgemm_copy_bytes(p, p, 24, None) == E_INVAL
    assert lib.lutgemm_copy_bytes(p, p, 0, None) == 0


def test_fused_call_rejects_bad_split_norm_slots_and_overlapping_operands(lib):
    # Host-side validation only: every call below must fail before anything is launched.
    from shiftaddllm_amd import native
    E_INVAL = -1
    base = 0x100000

    def problem(M=8, K=256, N=256, **kw):
        f = dict(bW=base, alpha_f16=base + 0x10000, x_f16=base + 0x20000, out_f16=base + 0x30000, N=N, K=K, nb=2,
                 num_groups=K // 128, M=M, overwrite=0, norm_weight_f16=None, gate_f16=None, norm_eps=1e-5,
                 next_norm_weight_f16=None, next_input_f16=None, sumsq_out_f32=None, sumsq_in_f32=None,
                 sumsq_in_slots=0)
        f.update(kw)
        return native.FusedProblem(**f)

    def call(*problems):
        arr = (native.FusedProblem * len(problems))(*problems)
        return lib.lutgemm_gemv_rowwise_f16_fused(len(problems), arr, None)

    sums = base + 0x40000
    # the slots of the consuming side are K / 32, whatever kernel the row count selects
    for M in (1, 8):
        assert call(problem(M=M, sumsq_in_f32=sums, sumsq_in_slots=1)) == E_INVAL
        assert call(problem(M=M, sumsq_in_f32=sums, sumsq_in_slots=6)) == E_INVAL
        assert call(problem(M=M, sumsq_in_f32=sums, sumsq_in_slots=9)) == E_INVAL
    assert call(problem(sumsq_in_f32=None, sumsq_in_slots=8)) == E_INVAL
    # outputs of two problems overlap
    assert call(problem(), problem(bW=base + 0x50000)) == E_INVAL
    # next_input of one problem is the input of another problem of the same call
    nw = base + 0x60000
    assert call(problem(next_norm_weight_f16=nw, next_input_f16=base + 0x70000),
                problem(x_f16=base + 0x70000, out_f16=base + 0x80000)) == E_INVAL
    # two problems share a row of sums of squares
    assert call(problem(sumsq_out_f32=sums), problem(out_f16=base + 0x80000, sumsq_out_f32=sums)) == E_INVAL
    # an output is another problem's gate row
    assert call(problem(gate_f16=base + 0x90000), problem(out_f16=base + 0x80000, gate_f16=base + 0x30000)) == E_INVAL


def test_python_module_exposes_reference_signatures():
    from shiftaddllm_amd import native
    if not os.path.exists(native.TORCH_EXT):
        pytest.skip("torch extension not built (python -m shiftaddllm_amd.build)")
    mod = native.lutgemm
    for fn in ("lutgemm_compute", "lutgemm_compute_shift_scale", "lutgemm_compute_block",
               "lutgemm_compute_block_shift", "lutgemm_compute_block_shiftInt8"):
        assert callable(getattr(mod, fn))
    import sys
    assert sys.modules["lutgemm"] is mod      # `import lutgemm` resolves to it

    import torch
    out = torch.zeros(1, 64, dtype=torch.float16)
    with pytest.raises(RuntimeError):         # CPU tensors are refused, not read
        mod.lutgemm_compute_shift_scale(out, torch.zeros(2, 3, 64, dtype=torch.int32),
                                        torch.zeros(2, 3, 64, dtype=torch.float16),
                                        torch.zeros(1, 64, dtype=torch.float16), 64, 64, 3, 2)
