// Look-up kernel instances for ONE row-wise problem with the fused extras of a decoder
// block: an input transform (none, RMSNorm, SiLU(gate) * x) and the split-RMSNorm fields.
// The problem is the kernel argument itself and the bit width a template parameter, so
// that the start of the kernel is the plain kernel's: one round of scalar loads, no
// dispatch on the problem's fields.
#include <stdlib.h>

#include "lut_gemv_device.h"
#include "lutgemm_launch.h"

namespace lutgemm {
namespace {

// SINGLE: every range of the launch holds exactly one item.
template <int NB, int XF, bool SINGLE = false>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
lut_gemv_fused_kernel(const Problem p)
{
    __shared__ __attribute__((aligned(16))) float lut[kLutDwords + kStageDwords + kWindowDwords];
    gemv_range<NB, kRowF16, 1, XF, true, SINGLE ? 2 : 1>(p, (int)blockIdx.x, (int)blockIdx.y, lut);  // grid = (ranges, rows)
}

template <int NB>
hipError_t launch_nb(const Problem &p, int xform, hipStream_t stream)
{
    const dim3 grid((unsigned)p.wgs_per_chunk, (unsigned)p.mchunks), block(kThreads);
    const bool single_item = option(LUTGEMM_OPTION_SINGLE_ITEM) != 0;
    if (p.items_per_wg == 1 && p.short_items == 1 && single_item) {
        if (xform == kXNorm)
            hipLaunchKernelGGL((lut_gemv_fused_kernel<NB, kXNorm, true>), grid, block, 0, stream, p);
        else if (xform == kXGate)
            hipLaunchKernelGGL((lut_gemv_fused_kernel<NB, kXGate, true>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((lut_gemv_fused_kernel<NB, kXNone, true>), grid, block, 0, stream, p);
        return hipGetLastError();
    }
    if (xform == kXNorm)
        hipLaunchKernelGGL((lut_gemv_fused_kernel<NB, kXNorm>), grid, block, 0, stream, p);
    else if (xform == kXGate)
        hipLaunchKernelGGL((lut_gemv_fused_kernel<NB, kXGate>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((lut_gemv_fused_kernel<NB, kXNone>), grid, block, 0, stream, p);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_gemv_fused(const Problem &p, int xform, hipStream_t stream)
{
    switch (p.nb) {
    case 1: return launch_nb<1>(p, xform, stream);
    case 2: return launch_nb<2>(p, xform, stream);
    case 3: return launch_nb<3>(p, xform, stream);
    default: return launch_nb<4>(p, xform, stream);
    }
}

}  // namespace lutgemm
