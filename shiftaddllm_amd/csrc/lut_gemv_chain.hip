// Look-up kernel instance for chained launches: several row-wise problems per launch, some of
// which read the tagged rows that others of the same launch write.
#include "lut_gemv_device.h"
#include "lutgemm_launch.h"

namespace lutgemm {

// Several row-wise problems in one launch, some of which read what others of the same launch
// write (tagged rows).  grid = (workgroups of the largest problem, problems): workgroups are
// dispatched in that order, so every workgroup of a producer is resident or finished before a
// workgroup of one of its consumers takes a slot, and a consumer's wait cannot keep its producer
// from running.  Each problem has its own input transform (chosen at run time) and bit width.
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
lut_gemv_chain_kernel(const Chain c)
{
    __shared__ __attribute__((aligned(16))) float lut[kLutDwords + kStageDwords + kWindowDwords];
    const Problem &p = *(const Problem *)((const __attribute__((address_space(4))) Problem *)&c.g.p[0] + blockIdx.y);
    if ((int)blockIdx.x >= p.n_blocks) return;
    int range, m;
    decode_block(p, (int)blockIdx.x, range, m);
    ChainWait cw;
    cw.epoch = c.ctl.epoch ? *c.ctl.epoch : 0u;
    cw.status = c.ctl.status;
    cw.spin_ticks = c.ctl.spin_ticks;
    switch (p.nb) {
    case 1: gemv_range<1, kRowF16, 1, kXDynamic, false, 1, false, true>(p, range, m, lut, &cw); break;
    case 2: gemv_range<2, kRowF16, 1, kXDynamic, false, 1, false, true>(p, range, m, lut, &cw); break;
    case 3: gemv_range<3, kRowF16, 1, kXDynamic, false, 1, false, true>(p, range, m, lut, &cw); break;
    default: gemv_range<4, kRowF16, 1, kXDynamic, false, 1, false, true>(p, range, m, lut, &cw); break;
    }
}

hipError_t launch_gemv_chain(const Chain &c, int blocks, hipStream_t stream)
{
    const dim3 grid((unsigned)blocks, (unsigned)c.g.count), block(kThreads);
    hipLaunchKernelGGL(lut_gemv_chain_kernel, grid, block, 0, stream, c);
    return hipGetLastError();
}

}  // namespace lutgemm
