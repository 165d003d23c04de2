// Look-up kernel instances: several row-wise problems per launch, with the fused input
// transforms (none, RMSNorm, SiLU(gate) * x).
#include "lut_gemv_device.h"
#include "lutgemm_launch.h"

namespace lutgemm {

hipError_t launch_gemv_group(const Group &g, int xform, int blocks, hipStream_t stream)
{
    const dim3 grid((unsigned)blocks, (unsigned)g.count), block(kThreads);
    if (xform == kXNorm)
        hipLaunchKernelGGL((lut_gemv_group_kernel<kXNorm>), grid, block, 0, stream, g);
    else if (xform == kXGate)
        hipLaunchKernelGGL((lut_gemv_group_kernel<kXGate>), grid, block, 0, stream, g);
    else
        hipLaunchKernelGGL((lut_gemv_group_kernel<kXNone>), grid, block, 0, stream, g);
    return hipGetLastError();
}

}  // namespace lutgemm
