"""In-tree build of the two native pieces (no JIT cache, no install step).

  liblutgemm_gfx950.so          hipcc --offload-arch=gfx950, kernels + C ABI
  liblutgemm_gfx950_ts.so       the same sources with -DLUTGEMM_TIMESTAMPS: the look-up
                                kernels read the clock at fixed points (measurements only)
  lutgemm.cpython-*.so          g++, the `lutgemm` Python module (torch shim),
                                linked against the library above via $ORIGIN

Run `python -m shiftaddllm_amd.build` (add --force to rebuild everything).
hipcc cross-compiles for gfx950 without a GPU present.
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(REPO_DIR, "include")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

KERNEL_LIB = os.path.join(PKG_DIR, "liblutgemm_gfx950.so")
KERNEL_LIB_TS = os.path.join(PKG_DIR, "liblutgemm_gfx950_ts.so")
EXT_SUFFIX = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
TORCH_EXT = os.path.join(PKG_DIR, "lutgemm" + EXT_SUFFIX)

# -packed-fp32-ops is switched off for all device code: hipcc would otherwise
# form v_pk_*_f32 from ordinary float arithmetic.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _newer(target: str, *sources: str) -> bool:
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(s) <= t for s in sources)


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


KERNEL_SOURCES = ("lutgemm_host.hip", "lut_gemv_rowwise.hip", "lut_gemv_block.hip", "lut_gemv_block_staged.hip",
                  "lut_gemv_group.hip", "lut_gemv_fused.hip", "lut_gemv_chain.hip", "lut_gemm_mfma.hip", "lut_gemm_mx.hip", "decode_kernels.hip")
KERNEL_HEADERS = ("lutgemm_internal.h", "lutgemm_common.h", "lutgemm_launch.h", "lut_gemv_device.h",
                  "lut_gemm_mfma_device.h", "lut_gemm_mx_device.h")


def build_kernel_library(force: bool = False, timestamps: bool = False) -> str:
    """One object per source (only stale ones are recompiled, several at a time), linked into the library.
    `timestamps`: the variant whose look-up kernels read the clock (-DLUTGEMM_TIMESTAMPS)."""
    from concurrent.futures import ThreadPoolExecutor

    hdrs = [os.path.join(INCLUDE, "lutgemm_gfx950.h")] + [os.path.join(CSRC, h) for h in KERNEL_HEADERS]
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    obj_dir = os.path.join(CSRC, "build_ts" if timestamps else "build")
    target = KERNEL_LIB_TS if timestamps else KERNEL_LIB
    os.makedirs(obj_dir, exist_ok=True)
    flags = [f for f in HIPCC_FLAGS if f != "-shared"] + (["-DLUTGEMM_TIMESTAMPS"] if timestamps else [])
    objs, stale = [], []
    for name in KERNEL_SOURCES:
        src = os.path.join(CSRC, name)
        obj = os.path.join(obj_dir, os.path.splitext(name)[0] + ".o")
        if force or not _newer(obj, src, *hdrs):
            stale.append([hipcc, *flags, "-I", INCLUDE, "-I", CSRC, "-c", "-o", obj, src])
        objs.append(obj)
    jobs = max(1, min(len(stale), int(os.environ.get("MAX_JOBS", "0")) or (os.cpu_count() or 4), 8))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(_run, stale))
    if stale or force or not _newer(target, *objs):
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", target, *objs])
    return target


def build_torch_extension(force: bool = False) -> str:
    src = os.path.join(CSRC, "lutgemm_torch.cpp")
    hdr = os.path.join(INCLUDE, "lutgemm_gfx950.h")
    if not force and _newer(TORCH_EXT, src, hdr, KERNEL_LIB):
        return TORCH_EXT
    import torch
    from torch.utils import cpp_extension

    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = []
    for d in cpp_extension.include_paths():
        inc += ["-isystem", d]
    inc += ["-isystem", os.path.join(ROCM, "include"), "-isystem", sysconfig.get_paths()["include"]]
    abi = int(torch.compiled_with_cxx11_abi())
    cmd = [
        os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared",
        "-DTORCH_EXTENSION_NAME=lutgemm", "-DTORCH_API_INCLUDE_EXTENSION_H",
        "-DUSE_ROCM=1", "-D__HIP_PLATFORM_AMD__=1", f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
        "-I", INCLUDE, *inc, src, "-o", TORCH_EXT,
        "-L", PKG_DIR, "-llutgemm_gfx950",
        "-L", torch_lib, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
        "-Wl,-rpath,$ORIGIN", "-Wl,--no-as-needed",
    ]
    _run(cmd)
    return TORCH_EXT


def build_all(force: bool = False):
    return build_kernel_library(force), build_kernel_library(force, timestamps=True), build_torch_extension(force)


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
