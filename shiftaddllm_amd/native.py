"""Loader for the compiled pieces.  Fails loudly: no fallback path exists.

`lutgemm`  -- the CPython module with the reference's call signatures
              (lut_gemm/lutgemm_cuda.cpp:225-230 in the ShiftAddLLM checkout).
`cabi()`   -- ctypes handle on liblutgemm_gfx950.so with argtypes set from
              include/lutgemm_gfx950.h, for callers that bind the C ABI directly.
"""
from __future__ import annotations

import ctypes
import importlib.util
import os
import sys
import sysconfig

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
KERNEL_LIB = os.path.join(_PKG_DIR, "liblutgemm_gfx950.so")
KERNEL_LIB_TS = os.path.join(_PKG_DIR, "liblutgemm_gfx950_ts.so")
TORCH_EXT = os.path.join(_PKG_DIR, "lutgemm" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))

C_ABI_SYMBOLS = (
    "lutgemm_strerror",
    "lutgemm_last_hip_error",
    "lutgemm_gemv_rowwise_f16",
    "lutgemm_gemv_rowwise_pow2_f16",
    "lutgemm_gemv_rowwise_f16_noalloc",
    "lutgemm_gemv_rowwise_f16_grouped",
    "lutgemm_gemv_rowwise_f16_fused",
    "lutgemm_gemv_rowwise_f16_chain",
    "lutgemm_describe_chain_plan",
    "lutgemm_chain_tag_rows",
    "lutgemm_chain_untag_rows",
    "lutgemm_chain_advance_epoch",
    "lutgemm_chain_status",
    "lutgemm_gemv_uniform_f16",
    "lutgemm_gemv_block_f16",
    "lutgemm_gemv_block_shift_u16",
    "lutgemm_gemv_block_apot_i8",
    "lutgemm_algorithmic_bytes",
    "lutgemm_copy_bytes",
    "lutgemm_workspace_words",
    "lutgemm_reserve_workspace",
    "lutgemm_describe_plan",
    "lutgemm_describe_pow2_plan",
    "lutgemm_set_option",
    "lutgemm_set_timestamp_buffer",
    "lutgemm_get_option",
    "lutgemm_measure_stream_read",
    "lutgemm_measure_empty_launch",
    "lutgemm_release_workspaces",
    "lutgemm_decode_rmsnorm_f16",
    "lutgemm_decode_attention_f16",
    "lutgemm_decode_silu_mul_f16",
)


MAX_GROUP = 8
OPTIONS = {"TARGET_BLOCKS": 0, "FIRST_SHARE": 1, "MFMA_MIN_M": 2, "MFMA_BLOCKS": 3, "PAIR_TABLES": 4, "SINGLE_ITEM": 5,
           "CHAIN_BLOCKS": 6, "CHAIN_GRID": 7, "TWIN_ITEMS": 8, "BLOCK_SCALED": 9, "POW2_CONVERT": 10}
CHAIN_MAX_ROWS = 4
CHAIN_MAX_TAG = 65534
NOALLOC_MAX_WORDS = 1 << 18


class RowwiseProblem(ctypes.Structure):
    """struct lutgemm_rowwise_problem of include/lutgemm_gfx950.h."""
    _fields_ = [("bW", ctypes.c_void_p), ("alpha_f16", ctypes.c_void_p), ("x_f16", ctypes.c_void_p),
                ("out_f16", ctypes.c_void_p), ("N", ctypes.c_int), ("K", ctypes.c_int),
                ("nb", ctypes.c_int), ("num_groups", ctypes.c_int), ("M", ctypes.c_int)]


class Plan(ctypes.Structure):
    """struct lutgemm_plan of include/lutgemm_gfx950.h."""
    _fields_ = [(n, ctypes.c_int) for n in (
        "kernel", "workgroups", "rows_per_pass", "row_chunks", "tiles", "k_units", "ranges", "long_ranges",
        "items_per_long_range", "items_per_short_range", "k_slices", "units_per_slice", "needs_workspace", "tile_columns")]


class FusedProblem(ctypes.Structure):
    """struct lutgemm_fused_problem of include/lutgemm_gfx950.h."""
    _fields_ = [("bW", ctypes.c_void_p), ("alpha_f16", ctypes.c_void_p), ("x_f16", ctypes.c_void_p),
                ("out_f16", ctypes.c_void_p), ("N", ctypes.c_int), ("K", ctypes.c_int),
                ("nb", ctypes.c_int), ("num_groups", ctypes.c_int), ("M", ctypes.c_int),
                ("overwrite", ctypes.c_int), ("norm_weight_f16", ctypes.c_void_p),
                ("gate_f16", ctypes.c_void_p), ("norm_eps", ctypes.c_float),
                ("next_norm_weight_f16", ctypes.c_void_p), ("next_input_f16", ctypes.c_void_p),
                ("sumsq_out_f32", ctypes.c_void_p), ("sumsq_in_f32", ctypes.c_void_p),
                ("sumsq_in_slots", ctypes.c_int)]


class ChainProblem(ctypes.Structure):
    """struct lutgemm_chain_problem of include/lutgemm_gfx950.h."""
    _fields_ = [("p", FusedProblem), ("x_tag", ctypes.c_int), ("gate_tag", ctypes.c_int), ("out_tag", ctypes.c_int)]


class ChainControl(ctypes.Structure):
    """struct lutgemm_chain_control of include/lutgemm_gfx950.h."""
    _fields_ = [("epoch", ctypes.c_void_p), ("status", ctypes.c_void_p), ("spin_limit_us", ctypes.c_uint)]


class ChainPlan(ctypes.Structure):
    """struct lutgemm_chain_plan of include/lutgemm_gfx950.h."""
    _fields_ = [("workgroups", ctypes.c_int), ("units", ctypes.c_int), ("needs_workspace", ctypes.c_int),
                ("stage", ctypes.c_int * MAX_GROUP), ("first_unit", ctypes.c_int * MAX_GROUP),
                ("unit_count", ctypes.c_int * MAX_GROUP), ("items_per_unit", ctypes.c_int * MAX_GROUP)]


class NativeLibraryMissing(ImportError):
    pass


def _missing(path: str) -> NativeLibraryMissing:
    return NativeLibraryMissing(
        f"{path} has not been built. Run `python -m shiftaddllm_amd.build` "
        "(hipcc --offload-arch=gfx950). There is no fallback compute path.")


def _load_extension():
    if not os.path.exists(KERNEL_LIB):
        raise _missing(KERNEL_LIB)
    if not os.path.exists(TORCH_EXT):
        raise _missing(TORCH_EXT)
    import torch  # noqa: F401  (its HIP runtime must be the one already loaded)
    spec = importlib.util.spec_from_file_location("lutgemm", TORCH_EXT)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    # `import lutgemm` elsewhere in the process (the reference's quant.py does
    # exactly that) now resolves to this module.
    sys.modules.setdefault("lutgemm", module)
    return module


def _bind(lib: ctypes.CDLL) -> ctypes.CDLL:
    """Set argument and result types of every entry point of include/lutgemm_gfx950.h."""
    vp, ci, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    lib.lutgemm_strerror.argtypes = [ci]
    lib.lutgemm_strerror.restype = ctypes.c_char_p
    lib.lutgemm_last_hip_error.argtypes = []
    lib.lutgemm_last_hip_error.restype = ci
    lib.lutgemm_gemv_rowwise_f16.argtypes = [vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
    lib.lutgemm_gemv_rowwise_pow2_f16.argtypes = [vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
    lib.lutgemm_gemv_rowwise_pow2_f16.restype = ci
    lib.lutgemm_gemv_rowwise_f16_noalloc.argtypes = [vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
    lib.lutgemm_gemv_rowwise_f16_noalloc.restype = ci
    lib.lutgemm_gemv_rowwise_f16_grouped.argtypes = [ci, ctypes.POINTER(RowwiseProblem), vp]
    lib.lutgemm_gemv_rowwise_f16_grouped.restype = ci
    lib.lutgemm_gemv_rowwise_f16_fused.argtypes = [ci, ctypes.POINTER(FusedProblem), vp]
    lib.lutgemm_gemv_rowwise_f16_fused.restype = ci
    lib.lutgemm_gemv_rowwise_f16_chain.argtypes = [ci, ctypes.POINTER(ChainProblem), ctypes.POINTER(ChainControl), vp]
    lib.lutgemm_gemv_rowwise_f16_chain.restype = ci
    lib.lutgemm_describe_chain_plan.argtypes = [ci, ctypes.POINTER(ChainProblem), ci, ctypes.POINTER(ChainPlan)]
    lib.lutgemm_describe_chain_plan.restype = ci
    lib.lutgemm_chain_tag_rows.argtypes = [vp, vp, sz, ci, vp, vp]
    lib.lutgemm_chain_tag_rows.restype = ci
    lib.lutgemm_chain_untag_rows.argtypes = [vp, vp, sz, vp]
    lib.lutgemm_chain_untag_rows.restype = ci
    lib.lutgemm_chain_advance_epoch.argtypes = [vp, ctypes.c_uint, vp]
    lib.lutgemm_chain_advance_epoch.restype = ci
    lib.lutgemm_chain_status.argtypes = [vp, vp]
    lib.lutgemm_chain_status.restype = ci
    lib.lutgemm_gemv_uniform_f16.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
    lib.lutgemm_gemv_block_f16.argtypes = [vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
    lib.lutgemm_gemv_block_shift_u16.argtypes = [vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, vp]
    lib.lutgemm_gemv_block_apot_i8.argtypes = [vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, vp]
    for name in ("lutgemm_gemv_rowwise_f16", "lutgemm_gemv_uniform_f16", "lutgemm_gemv_block_f16",
                 "lutgemm_gemv_block_shift_u16", "lutgemm_gemv_block_apot_i8"):
        getattr(lib, name).restype = ci
    lib.lutgemm_algorithmic_bytes.argtypes = [ci, ci, ci, ci, sz, ci]
    lib.lutgemm_algorithmic_bytes.restype = sz
    lib.lutgemm_copy_bytes.argtypes = [vp, vp, sz, vp]
    lib.lutgemm_copy_bytes.restype = ci
    lib.lutgemm_describe_plan.argtypes = [ci, ci, ci, ci, ci, ci, ctypes.POINTER(Plan)]
    lib.lutgemm_describe_plan.restype = ci
    lib.lutgemm_describe_pow2_plan.argtypes = [ci, ci, ci, ci, ci, ctypes.POINTER(Plan)]
    lib.lutgemm_describe_pow2_plan.restype = ci
    lib.lutgemm_set_option.argtypes = [ci, ci]
    lib.lutgemm_set_option.restype = ci
    lib.lutgemm_get_option.argtypes = [ci]
    lib.lutgemm_get_option.restype = ci
    lib.lutgemm_workspace_words.argtypes = [ci, ci]
    lib.lutgemm_workspace_words.restype = sz
    lib.lutgemm_reserve_workspace.argtypes = [vp, sz]
    lib.lutgemm_reserve_workspace.restype = ci
    lib.lutgemm_measure_stream_read.argtypes = [vp, sz, vp, vp]
    lib.lutgemm_measure_stream_read.restype = ci
    lib.lutgemm_measure_empty_launch.argtypes = [ci, vp]
    lib.lutgemm_measure_empty_launch.restype = ci
    lib.lutgemm_release_workspaces.argtypes = []
    lib.lutgemm_release_workspaces.restype = ci
    lib.lutgemm_decode_rmsnorm_f16.argtypes = [vp, vp, vp, ci, ci, ctypes.c_float, vp, sz, vp]
    lib.lutgemm_decode_rmsnorm_f16.restype = ci
    lib.lutgemm_decode_attention_f16.argtypes = [vp] * 9 + [ci] * 5 + [vp]
    lib.lutgemm_decode_attention_f16.restype = ci
    lib.lutgemm_decode_silu_mul_f16.argtypes = [vp, vp, vp, sz, vp]
    lib.lutgemm_decode_silu_mul_f16.restype = ci
    lib.lutgemm_set_timestamp_buffer.argtypes = [vp, sz]
    lib.lutgemm_set_timestamp_buffer.restype = ci
    return lib


_cabi = None
_cabi_ts = None


def cabi() -> ctypes.CDLL:
    global _cabi
    if _cabi is None:
        if not os.path.exists(KERNEL_LIB):
            raise _missing(KERNEL_LIB)
        import torch  # noqa: F401
        _cabi = _bind(ctypes.CDLL(KERNEL_LIB))
    return _cabi


def cabi_timestamps() -> ctypes.CDLL:
    """The time-stamped build of the library (measurements only: its look-up kernels read the clock
    at fixed points, see lutgemm_set_timestamp_buffer)."""
    global _cabi_ts
    if _cabi_ts is None:
        if not os.path.exists(KERNEL_LIB_TS):
            raise _missing(KERNEL_LIB_TS)
        import torch  # noqa: F401
        _cabi_ts = _bind(ctypes.CDLL(KERNEL_LIB_TS))
    return _cabi_ts


def __getattr__(name):
    if name == "lutgemm":
        module = _load_extension()
        globals()["lutgemm"] = module
        return module
    raise AttributeError(name)
