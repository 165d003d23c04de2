"""numpy + C restatement of ShiftAddLLM's LUT-GEMM path (the checker).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
benchmark's CPU-baseline leg, never by the shipped package.

Two independent restatements live here on purpose:
  * numpy closed forms (vectorised, this file), and
  * scalar C loops that emulate the kernels' table look-ups
    (lutgemm_oracle.c, reached through ctypes),
so that each can be checked against the other as well as against
known-answer vectors.  Paths in the citations are relative to the ShiftAddLLM
checkout.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_lutgemm.so")
_lib = None

ALPHA_F16, ALPHA_SHIFT_U16, ALPHA_APOT_I8 = 0, 1, 2
APOT_ABSENT = -128  # int8 exponent meaning "this additive term is not present"


def build(force: bool = False) -> str:
    """Compile lutgemm_oracle.c with gcc (seconds).  Returns the library path."""
    src = os.path.join(_HERE, "lutgemm_oracle.c")
    stale = (not os.path.exists(_LIB_PATH)
             or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src))
    if force or stale:
        subprocess.check_call(
            ["gcc", "-O2", "-Wall", "-Wextra", "-fPIC", "-shared", "-o", _LIB_PATH, src, "-lm"])
    return _LIB_PATH


def _c():
    global _lib
    if _lib is None:
        build()
        lib = ctypes.CDLL(_LIB_PATH)
        vp, ci = ctypes.c_void_p, ctypes.c_int
        lib.orc_pack_binary_weight.argtypes = [vp, ci, ci, ci, vp]
        lib.orc_unpack_weight.argtypes = [vp, vp, ci, ci, ci, ci, vp]
        lib.orc_table_indices.argtypes = [vp, ci, ci, ci, vp]
        lib.orc_table_indices.restype = None
        lib.orc_build_lut.argtypes = [vp, vp]
        lib.orc_build_lut.restype = None
        lib.orc_gemv_rowwise.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci]
        lib.orc_gemv_uniform.argtypes = [vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci]
        lib.orc_gemv_block.argtypes = [vp, vp, ci, vp, vp, vp, ci, ci, ci, ci, ci]
        lib.orc_dense_gemv.argtypes = [vp, vp, vp, ci, ci, ci]
        lib.orc_dense_gemv.restype = None
        lib.orc_half_to_float.argtypes = [ctypes.c_uint16]
        lib.orc_half_to_float.restype = ctypes.c_float
        lib.orc_float_to_half.argtypes = [ctypes.c_float]
        lib.orc_float_to_half.restype = ctypes.c_uint16
        _lib = lib
    return _lib


def _ptr(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.c_void_p)


def _as(a, dtype):
    return np.ascontiguousarray(np.asarray(a), dtype=dtype)


def _half_bits(a) -> np.ndarray:
    """fp16 array -> uint16 bit patterns (C side has no _Float16)."""
    a = np.asarray(a)
    if a.dtype != np.float16:
        raise TypeError(f"expected float16, got {a.dtype}")
    return np.ascontiguousarray(a).view(np.uint16)


# --------------------------------------------------------------------------
# numpy closed forms
# --------------------------------------------------------------------------

def pack_binary_weight_np(B: np.ndarray) -> np.ndarray:
    """lut_gemm/kernel.py:9-23.  B [A, G, S, nb] of +-1 -> int32 [A, G*S/32, nb].

    Closed form: word[a, j, b] = sum_t [B[a, 32j+t, b] == +1] << t over the
    flattened (G, S) axis, as a two's-complement int32.
    """
    B = np.asarray(B)
    if B.ndim != 4:
        raise ValueError("expected [A, n_groups, group_size, wbit]")
    if not np.all((B == 1) | (B == -1)):
        raise ValueError("entries must be +1 or -1")
    A, G, S, nb = B.shape
    L = G * S
    if L % 32:
        raise ValueError("n_groups*group_size must be a multiple of 32")
    bits = (B.reshape(A, L // 32, 32, nb) == 1).astype(np.uint64)
    weights = (np.uint64(1) << np.arange(32, dtype=np.uint64))[None, None, :, None]
    words = (bits * weights).sum(axis=2).astype(np.uint32)
    return words.view(np.int32)


def unpack_bits_np(bW: np.ndarray) -> np.ndarray:
    """int32 [A, L/32, nb] -> +-1 int8 [A, L, nb] (inverse of the packing)."""
    bW = np.ascontiguousarray(bW, dtype=np.int32).view(np.uint32)
    A, J, nb = bW.shape
    t = np.arange(32, dtype=np.uint32)[None, None, :, None]
    bits = (bW[:, :, None, :] >> t) & np.uint32(1)
    return (bits.astype(np.int8) * 2 - 1).reshape(A, J * 32, nb)


def unpack_weight_np(bW: np.ndarray, alpha: np.ndarray) -> np.ndarray:
    """lut_gemm/kernel.py:26-56.  bW int32 [A, L/32, nb], alpha [A, G, nb]
    -> fp32 [A, L] with W[a, l] = sum_b alpha[a, l // (L/G), b] * (2*bit - 1),
    accumulated in fp32 in bit-plane order like the reference loop."""
    signs = unpack_bits_np(bW).astype(np.float32)              # [A, L, nb]
    alpha = np.asarray(alpha, dtype=np.float32)
    A, L, nb = signs.shape
    G = alpha.shape[1]
    if alpha.shape != (A, G, nb) or L % G:
        raise ValueError("alpha must be [A, G, nb] with G dividing L")
    a_full = np.repeat(alpha, L // G, axis=1)                   # [A, L, nb]
    W = np.zeros((A, L), dtype=np.float32)
    for b in range(nb):
        W += a_full[:, :, b] * signs[:, :, b]
    return W


def rowwise_to_kernel_layout(B: np.ndarray, alpha: np.ndarray):
    """BCQ output B [N, K/gs, gs, nb], alpha [N, K/gs, nb] -> kernel operands
    Wp int32 [K/32, nb, N], a fp16 [K/gs, nb, N]
    (lut_gemm/quant.py:25; mv_fp16_bias.hpp:52,86,543,551)."""
    Wp = np.ascontiguousarray(pack_binary_weight_np(B).transpose(1, 2, 0))
    a = np.ascontiguousarray(np.asarray(alpha, dtype=np.float32).transpose(1, 2, 0)).astype(np.float16)
    return Wp, a


def dequant_rowwise_kernel_layout(Wp: np.ndarray, a: np.ndarray) -> np.ndarray:
    """Kernel operands (Wp [K/32, nb, N], a [K/gs, nb, N]) -> W_q fp32 [N, K]."""
    bW = np.ascontiguousarray(np.asarray(Wp).transpose(2, 0, 1))
    al = np.ascontiguousarray(np.asarray(a, dtype=np.float32).transpose(2, 0, 1))
    return unpack_weight_np(bW, al)


def dequant_block_kernel_layout(Wp: np.ndarray, a_eff: np.ndarray) -> np.ndarray:
    """Block operands Wp [K/32, nb, N], effective alpha a_eff [K/8, nb, R]
    -> W_q fp32 [N, K]:  W[n, k] = sum_b a_eff[k//8, b, n//(N/R)] * sign."""
    Wp = np.asarray(Wp)
    a_eff = np.asarray(a_eff, dtype=np.float32)
    J, nb, N = Wp.shape
    K = 32 * J
    C, nb2, R = a_eff.shape
    if C != K // 8 or nb2 != nb or N % R:
        raise ValueError("alpha must be [K/8, nb, R] with R dividing N")
    signs = unpack_bits_np(np.ascontiguousarray(Wp.transpose(2, 0, 1))).astype(np.float32)  # [N,K,nb]
    a_full = np.repeat(np.repeat(a_eff, 8, axis=0), N // R, axis=2)     # [K, nb, N]
    W = np.zeros((N, K), dtype=np.float32)
    for b in range(nb):
        W += a_full[:, b, :].T * signs[:, :, b]
    return W


def lat_disk_to_kernel_layout(bWeight: np.ndarray, alpha: np.ndarray):
    """What lut_gemm/kernel.py:112-133 (convert_weight) is meant to do.

    On disk (quant_methods/shiftaddllm.py:193-211): bWeight int32
    [K, N/32, nb] packed along the OUTPUT axis (bit t <-> out row 32j+t) and
    alpha fp32 [K/8, R, nb].  Kernel: Wp int32 [K/32, nb, N] packed along the
    INPUT axis and alpha [K/8, nb, R]."""
    signs = unpack_bits_np(bWeight)                    # [K, N, nb]
    K, N, nb = signs.shape
    B = signs.transpose(1, 0, 2).reshape(N, 1, K, nb)  # [N, 1, K, nb]
    Wp = np.ascontiguousarray(pack_binary_weight_np(B).transpose(1, 2, 0))
    a = np.ascontiguousarray(np.asarray(alpha, dtype=np.float32).transpose(0, 2, 1))
    return Wp, a


def dequant_lat_disk(bWeight: np.ndarray, alpha: np.ndarray) -> np.ndarray:
    """lut_gemm/kernel.py:101-107: on-disk Lat. tensors -> dense W_q [N, K]
    (alpha repeated over the 8 columns of a block, unpack, transpose)."""
    a_rep = np.repeat(np.asarray(alpha, dtype=np.float32), 8, axis=0)
    return np.ascontiguousarray(unpack_weight_np(bWeight, a_rep).T)


def shift_u16_to_alpha(u: np.ndarray) -> np.ndarray:
    """mv_fp16_bias.hpp:286-297: three 3-bit shift fields -> 2^f0+2^f1+2^f2."""
    u = np.asarray(u).astype(np.int64) & 0xFFFF
    return (2.0 ** (u & 7) + 2.0 ** ((u >> 3) & 7) + 2.0 ** ((u >> 6) & 7)).astype(np.float32)


def apot_i8_to_alpha(s: np.ndarray) -> np.ndarray:
    """mv_fp16_bias.hpp:335-340,473-482: int8 [..., 3] exponents -> sum 2^s.
    Exponent -128 marks an absent term (contributes 0)."""
    s = np.asarray(s).astype(np.int64)
    terms = np.where(s == APOT_ABSENT, 0.0, np.ldexp(1.0, np.where(s == APOT_ABSENT, 0, s)))
    return terms.sum(axis=-1).astype(np.float32)


def pow2_round_np(a: np.ndarray) -> np.ndarray:
    """quantizers/bcq_quant/bcq_shift.py:15-39: sign(a) * 2^round(log2|a|),
    round half to even on the exponent (torch.round semantics)."""
    a = np.asarray(a, dtype=np.float32)
    with np.errstate(divide="ignore"):
        e = np.rint(np.log(np.abs(a)) / np.float32(np.log(2)))
    return (np.sign(a) * np.exp2(e)).astype(np.float32)


def dense_gemv_np(W: np.ndarray, x: np.ndarray) -> np.ndarray:
    """y = x.float() @ W^T with double accumulation.  W [N, K], x fp16 [M, K]."""
    return (np.asarray(x, dtype=np.float64) @ np.asarray(W, dtype=np.float64).T).astype(np.float32)


def accumulate_into_fp16(out: np.ndarray, y: np.ndarray) -> np.ndarray:
    """fp16(out.float() + y): the kernels accumulate into a caller-filled
    output (mv_fp16_bias.hpp:101,216,324,491,577)."""
    return (np.asarray(out, dtype=np.float32) + np.asarray(y, dtype=np.float32)).astype(np.float16)


# --------------------------------------------------------------------------
# C restatement (table-lookup emulation)
# --------------------------------------------------------------------------

def pack_binary_weight_c(B: np.ndarray) -> np.ndarray:
    B = np.asarray(B)
    A, G, S, nb = B.shape
    Bi = _as(B.reshape(A, G * S, nb), np.int8)
    if not np.array_equal(Bi, np.asarray(B).reshape(A, G * S, nb)):
        raise ValueError("entries must be +1 or -1")
    out = np.empty((A, G * S // 32, nb), dtype=np.int32)
    rc = _c().orc_pack_binary_weight(_ptr(Bi), A, G * S, nb, _ptr(out))
    if rc:
        raise ValueError(f"orc_pack_binary_weight failed ({rc})")
    return out


def unpack_weight_c(bW: np.ndarray, alpha: np.ndarray) -> np.ndarray:
    bW = _as(bW, np.int32)
    alpha = _as(alpha, np.float32)
    A, J, nb = bW.shape
    G = alpha.shape[1]
    W = np.empty((A, J * 32), dtype=np.float32)
    rc = _c().orc_unpack_weight(_ptr(bW), _ptr(alpha), A, J * 32, G, nb, _ptr(W))
    if rc:
        raise ValueError(f"orc_unpack_weight failed ({rc})")
    return W


def table_indices_c(Wp: np.ndarray) -> np.ndarray:
    """uint8 [K/8, nb, N]: the byte each look-up uses (mv_fp16_bias.hpp:86-90)."""
    Wp = _as(Wp, np.int32)
    J, nb, N = Wp.shape
    idx = np.empty((J * 4, nb, N), dtype=np.uint8)
    _c().orc_table_indices(_ptr(Wp), J * 32, nb, N, _ptr(idx))
    return idx


def build_lut_c(x8: np.ndarray) -> np.ndarray:
    x8 = _half_bits(np.asarray(x8, dtype=np.float16).reshape(8))
    lut = np.empty(256, dtype=np.float64)
    _c().orc_build_lut(_ptr(x8), _ptr(lut))
    return lut


def _prep_io(x, out, N, K):
    x = np.asarray(x)
    if x.dtype != np.float16:
        raise TypeError("x must be float16")
    x2 = np.ascontiguousarray(x.reshape(-1, K))
    M = x2.shape[0]
    if out is None:
        out = np.zeros((M, N), dtype=np.float16)
    out2 = np.ascontiguousarray(np.asarray(out, dtype=np.float16).reshape(M, N)).copy()
    y32 = np.empty((M, N), dtype=np.float32)
    return x2, out2, y32, M


def gemv_rowwise_c(Wp, alpha, x, num_groups, out=None):
    """lutgemm_compute_shift_scale semantics.  Returns (out_fp16, y_fp32)."""
    Wp = _as(Wp, np.int32)
    J, nb, N = Wp.shape
    K = 32 * J
    a = _half_bits(alpha)
    if a.shape != (num_groups, nb, N):
        raise ValueError("alpha must be [num_groups, nb, N]")
    x2, out2, y32, M = _prep_io(x, out, N, K)
    rc = _c().orc_gemv_rowwise(_ptr(Wp), _ptr(a), _ptr(_half_bits(x2)), _ptr(out2.view(np.uint16)),
                               _ptr(y32), N, K, nb, num_groups, M)
    if rc:
        raise ValueError(f"orc_gemv_rowwise failed ({rc})")
    return out2, y32


def gemv_uniform_c(Wp, alpha, q_bias, x, num_groups, out=None):
    """lutgemm_compute semantics.  Returns (out_fp16, y_fp32)."""
    Wp = _as(Wp, np.int32)
    J, nb, N = Wp.shape
    K = 32 * J
    a, q = _half_bits(alpha), _half_bits(q_bias)
    if a.shape != (num_groups, N) or q.shape != (num_groups, N):
        raise ValueError("alpha and q_bias must be [num_groups, N]")
    x2, out2, y32, M = _prep_io(x, out, N, K)
    rc = _c().orc_gemv_uniform(_ptr(Wp), _ptr(a), _ptr(q), _ptr(_half_bits(x2)),
                               _ptr(out2.view(np.uint16)), _ptr(y32), N, K, nb, num_groups, M)
    if rc:
        raise ValueError(f"orc_gemv_uniform failed ({rc})")
    return out2, y32


def gemv_block_c(Wp, alpha, x, num_groups, kind=ALPHA_F16, out=None):
    """lutgemm_compute_block / _block_shift / _block_shiftInt8 semantics.
    alpha: fp16 [K/8, nb, R] | int16/uint16 [K/8, nb, R] | int8 [K/8, nb, R, 3]."""
    Wp = _as(Wp, np.int32)
    J, nb, N = Wp.shape
    K = 32 * J
    R = num_groups
    if kind == ALPHA_F16:
        a = _half_bits(alpha)
        want = (K // 8, nb, R)
    elif kind == ALPHA_SHIFT_U16:
        a = np.ascontiguousarray(np.asarray(alpha)).view(np.uint16)
        want = (K // 8, nb, R)
    elif kind == ALPHA_APOT_I8:
        a = _as(alpha, np.int8)
        want = (K // 8, nb, R, 3)
    else:
        raise ValueError("unknown alpha kind")
    if a.shape != want:
        raise ValueError(f"alpha must be {want}, got {a.shape}")
    x2, out2, y32, M = _prep_io(x, out, N, K)
    rc = _c().orc_gemv_block(_ptr(Wp), _ptr(a), kind, _ptr(_half_bits(x2)),
                             _ptr(out2.view(np.uint16)), _ptr(y32), N, K, nb, R, M)
    if rc:
        raise ValueError(f"orc_gemv_block failed ({rc})")
    return out2, y32


def dense_gemv_c(W, x):
    W = _as(W, np.float32)
    N, K = W.shape
    x2 = np.ascontiguousarray(np.asarray(x, dtype=np.float16).reshape(-1, K))
    y = np.empty((x2.shape[0], N), dtype=np.float32)
    _c().orc_dense_gemv(_ptr(W), _ptr(_half_bits(x2)), _ptr(y), N, K, x2.shape[0])
    return y


def half_to_float_c(bits: int) -> float:
    return float(_c().orc_half_to_float(int(bits) & 0xFFFF))


def float_to_half_c(f: float) -> int:
    return int(_c().orc_float_to_half(float(f)))


# --------------------------------------------------------------------------
# CPU baseline: the reference's CPU-executable inference path
# --------------------------------------------------------------------------

def cpu_dense_path(Wp, alpha, num_threads=None):
    """Dequantise once (unpack_weight semantics, kernel.py:87-109) and return a
    callable running the ordinary fp32 linear on host cores with torch, which
    is what the reference's non-kernel path executes.  Used only to time a
    baseline."""
    import torch
    if num_threads:
        torch.set_num_threads(int(num_threads))
    W = torch.from_numpy(dequant_rowwise_kernel_layout(np.asarray(Wp), np.asarray(alpha)))

    def run(x):
        return torch.nn.functional.linear(x.float(), W)

    return run, W


def error_metrics(y, y_ref):
    """(relative L2 error, max abs diff / max |y_ref|) in double."""
    y = np.asarray(y, dtype=np.float64)
    r = np.asarray(y_ref, dtype=np.float64)
    den = np.linalg.norm(r)
    rel = float(np.linalg.norm(y - r) / den) if den > 0 else float(np.linalg.norm(y - r))
    mx = float(np.abs(r).max()) if r.size else 0.0
    mad = float(np.abs(y - r).max() / mx) if mx > 0 else float(np.abs(y - r).max() if r.size else 0.0)
    return rel, mad
