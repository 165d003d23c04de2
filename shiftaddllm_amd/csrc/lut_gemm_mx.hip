// Block-scaled matrix-core kernel instances (row-wise alphas that are powers of two, several
// activation rows) and the kernel that splits the activations for them.
#include "lut_gemm_mx_device.h"
#include "lutgemm_launch.h"

namespace lutgemm {
namespace {

template <int NB, int MP>
hipError_t launch_one(const Problem &p, const MxActivations &act, hipStream_t stream)
{
    const dim3 grid((unsigned)p.n_blocks), block(kMfmaThreads);
    hipLaunchKernelGGL((lut_gemm_mx_kernel<NB, MP>), grid, block, 0, stream, p, act);
    return hipGetLastError();
}

template <int NB>
hipError_t launch_nb(const Problem &p, const MxActivations &act, hipStream_t stream)
{
    switch (mx_chunk_rows(p.M)) {
    case 5: return launch_one<NB, 5>(p, act, stream);
    case 8: return launch_one<NB, 8>(p, act, stream);
    default: return launch_one<NB, 16>(p, act, stream);
    }
}

}  // namespace

hipError_t launch_mx(const Problem &p, void *split, hipStream_t stream)
{
    // the activations first: three 8-bit floats per value, a row of zeros, a scale word per block of 32
    const long threads = (long)p.M * (p.K / 32) * 8;   // eight threads per block of 32
    unsigned char *pieces = (unsigned char *)split;
    uint32_t *scales = (uint32_t *)(pieces + (size_t)p.M * p.K * kMxPieces + p.K);
    hipLaunchKernelGGL(mx_split_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, p.x, pieces, scales, p.M,
                       p.K);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    MxActivations act;
    act.pieces = pieces;
    act.scales = scales;
    switch (p.nb) {
    case 1: return launch_nb<1>(p, act, stream);
    case 2: return launch_nb<2>(p, act, stream);
    case 3: return launch_nb<3>(p, act, stream);
    default: return launch_nb<4>(p, act, stream);
    }
}

}  // namespace lutgemm
