// Matrix-core kernel instances (row-wise alpha, several activation rows).
#include "lut_gemm_mfma_device.h"
#include "lutgemm_launch.h"

namespace lutgemm {
namespace {

template <int NB>
hipError_t launch_nb(const Problem &p, int mt, bool pow2, hipStream_t stream)
{
    const dim3 grid((unsigned)p.n_blocks), block(kMfmaThreads);
    const bool one = mt == 1 && p.sets_per_split == kMfmaWaves;  // one round per K-slice
    if (pow2 && one)
        hipLaunchKernelGGL((lut_gemm_mfma_kernel<NB, 1, true, true>), grid, block, 0, stream, p);
    else if (pow2 && mt == 2)
        hipLaunchKernelGGL((lut_gemm_mfma_kernel<NB, 2, false, true>), grid, block, 0, stream, p);
    else if (pow2)
        hipLaunchKernelGGL((lut_gemm_mfma_kernel<NB, 1, false, true>), grid, block, 0, stream, p);
    else if (one)
        hipLaunchKernelGGL((lut_gemm_mfma_kernel<NB, 1, true>), grid, block, 0, stream, p);
    else if (mt == 2)
        hipLaunchKernelGGL((lut_gemm_mfma_kernel<NB, 2>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((lut_gemm_mfma_kernel<NB, 1>), grid, block, 0, stream, p);
    return hipGetLastError();
}

template <int NB>
hipError_t launch_fused_nb(const Problem &p, int mt, hipStream_t stream)
{
    const dim3 grid((unsigned)p.n_blocks), block(kMfmaThreads);
    if (mt == 1 && p.sets_per_split == kMfmaWaves)  // one round per K-slice
        hipLaunchKernelGGL((lut_gemm_mfma_fused_kernel<NB, 1, true>), grid, block, 0, stream, p);
    else if (mt == 2)
        hipLaunchKernelGGL((lut_gemm_mfma_fused_kernel<NB, 2>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((lut_gemm_mfma_fused_kernel<NB, 1>), grid, block, 0, stream, p);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_mfma_fused(const Problem &p, int mt, hipStream_t stream)
{
    switch (p.nb) {
    case 1: return launch_fused_nb<1>(p, mt, stream);
    case 2: return launch_fused_nb<2>(p, mt, stream);
    case 3: return launch_fused_nb<3>(p, mt, stream);
    default: return launch_fused_nb<4>(p, mt, stream);
    }
}

hipError_t launch_mfma(const Problem &p, int mt, bool pow2, hipStream_t stream)
{
    switch (p.nb) {
    case 1: return launch_nb<1>(p, mt, pow2, stream);
    case 2: return launch_nb<2>(p, mt, pow2, stream);
    case 3: return launch_nb<3>(p, mt, pow2, stream);
    default: return launch_nb<4>(p, mt, pow2, stream);
    }
}

hipError_t launch_mfma_group(const Group &g, int mt, int blocks, hipStream_t stream)
{
    const dim3 grid((unsigned)blocks, (unsigned)g.count), block(kMfmaThreads);
    if (mt == 2)
        hipLaunchKernelGGL((lut_gemm_mfma_group_kernel<2>), grid, block, 0, stream, g);
    else
        hipLaunchKernelGGL((lut_gemm_mfma_group_kernel<1>), grid, block, 0, stream, g);
    return hipGetLastError();
}

}  // namespace lutgemm
