// Look-up kernel instance for chained launches: several row-wise problems per launch, some of
// which read the tagged rows that others of the same launch write.
#include <atomic>

#include "lut_gemv_device.h"
#include "lutgemm_launch.h"

namespace lutgemm {

// Several row-wise problems in one launch, some of which read what others of the same launch
// write (tagged rows).  The launch is persistent: its workgroups, all resident at once, take the
// launch's units (one workgroup's range of one problem; numbered problem by problem, producers
// before consumers) in steps of the grid size.  A unit waits only for units with smaller numbers,
// and every workgroup takes its units in increasing order, so the unfinished unit with the
// smallest number can always run: no wait can starve what it waits for.  Each problem has its
// own input transform (chosen at run time) and bit width.
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
lut_gemv_chain_kernel(const Chain c)
{
    __shared__ __attribute__((aligned(16))) float lut[kLutDwords + kStageDwords + kWindowDwords];
    ChainWait cw;
    cw.epoch = c.ctl.epoch ? *c.ctl.epoch : 0u;
    cw.status = c.ctl.status;
    cw.spin_ticks = c.ctl.spin_ticks;
    const int total = c.unit_start[c.g.count];
    int y = 0;
    for (int unit = (int)blockIdx.x; unit < total; unit += (int)gridDim.x) {
        while (unit >= c.unit_start[y + 1]) ++y;   // (units only grow: the search goes on where it stopped)
        const Problem &p = *(const Problem *)((const __attribute__((address_space(4))) Problem *)&c.g.p[0] + y);
        int range, m;
        decode_block(p, unit - c.unit_start[y], range, m);
        cw.unit = unit;
        cw.problem = y;
        bool ok;
        switch (p.nb) {
        case 1: ok = gemv_range<1, kRowF16, 1, kXDynamic, false, 1, false, true>(p, range, m, lut, &cw); break;
        case 2: ok = gemv_range<2, kRowF16, 1, kXDynamic, false, 1, false, true>(p, range, m, lut, &cw); break;
        case 3: ok = gemv_range<3, kRowF16, 1, kXDynamic, false, 1, false, true>(p, range, m, lut, &cw); break;
        default: ok = gemv_range<4, kRowF16, 1, kXDynamic, false, 1, false, true>(p, range, m, lut, &cw); break;
        }
        if (!ok) return;    // a wait gave up: the later units of this workgroup would wait in vain
        __syncthreads();    // the next unit's tables and window overwrite this one's
    }
}

hipError_t launch_gemv_chain(const Chain &c, int blocks, hipStream_t stream)
{
    const dim3 grid((unsigned)blocks), block(kThreads);
    hipLaunchKernelGGL(lut_gemv_chain_kernel, grid, block, 0, stream, c);
    return hipGetLastError();
}

hipError_t chain_resident_workgroups(int *count)
{
    constexpr int kMaxDevices = 64;
    static std::atomic<int> cached[kMaxDevices];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < kMaxDevices && cached[dev].load() > 0) {
        *count = cached[dev].load();
        return hipSuccess;
    }
    int per_cu = 0, cus = 0;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lut_gemv_chain_kernel, kThreads, 0);
    if (e != hipSuccess) return e;
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    *count = per_cu * cus;
    if (dev >= 0 && dev < kMaxDevices) cached[dev].store(*count);
    return hipSuccess;
}

}  // namespace lutgemm
