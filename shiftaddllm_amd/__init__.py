"""MI355X-native LUT-GEMM engine behind ShiftAddLLM's quantised-linear API.

Layout of the package:
  csrc/lutgemm_kernels.hip   gfx950 kernels + the C ABI (include/lutgemm_gfx950.h)
  csrc/lutgemm_torch.cpp     Python module `lutgemm` with the reference signatures
  lut_gemm/quant.py          LutLinear, make_lut, load_lut
  lut_gemm/kernel.py         pack / unpack / convert / checkpoint loaders
  workload.py                seeded synthetic BCQ problems for tests and benchmarks
  build.py                   in-tree build of the two shared objects

`import shiftaddllm_amd.native as native; native.lutgemm` is the compiled
module; importing it raises if the shared objects have not been built -- there
is no Python or CPU fallback for the compute path.
"""

__all__ = ["native", "lut_gemm", "workload", "build"]
