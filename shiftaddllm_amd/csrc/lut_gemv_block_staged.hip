// Look-up kernel instances: block alpha of ShiftAddLLM (Lat.), one multiplier per 8-input
// chunk, bit plane and row group, as fp16, uint16 shift fields or int8 exponents
// (lut_gemm/mv_fp16_bias.hpp:105-220,223-328,342-495 of the ShiftAddLLM checkout), for
// N-tiles that span at most two row groups: the workgroup stages an item's multipliers
// in LDS.
#include "lut_gemv_device.h"
#include "lutgemm_launch.h"

namespace lutgemm {
namespace {

template <int NB, int MODE>
hipError_t launch_nb(const Problem &p, int mrows, hipStream_t stream)
{
    const dim3 grid((unsigned)p.wgs_per_chunk, (unsigned)p.mchunks), block(kThreads);
    if (mrows == 4)
        hipLaunchKernelGGL((lut_gemv_kernel<NB, MODE, 4>), grid, block, 0, stream, p);
    else if (mrows == 2)
        hipLaunchKernelGGL((lut_gemv_kernel<NB, MODE, 2>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((lut_gemv_kernel<NB, MODE, 1>), grid, block, 0, stream, p);
    return hipGetLastError();
}

template <int MODE>
hipError_t launch_mode(const Problem &p, int mrows, hipStream_t stream)
{
    switch (p.nb) {
    case 1: return launch_nb<1, MODE>(p, mrows, stream);
    case 2: return launch_nb<2, MODE>(p, mrows, stream);
    case 3: return launch_nb<3, MODE>(p, mrows, stream);
    default: return launch_nb<4, MODE>(p, mrows, stream);
    }
}

}  // namespace

hipError_t launch_gemv_block_staged(const Problem &p, int mode, int mrows, hipStream_t stream)
{
    switch (mode) {
    case kBlockF16Staged: return launch_mode<kBlockF16Staged>(p, mrows, stream);
    case kBlockShiftU16Staged: return launch_mode<kBlockShiftU16Staged>(p, mrows, stream);
    default: return launch_mode<kBlockApotI8Staged>(p, mrows, stream);
    }
}

}  // namespace lutgemm
