// Look-up kernel instances: row-wise alpha (lut_gemm/mv_fp16_bias.hpp:498-579 of the
// ShiftAddLLM checkout) and uniform mode with q_bias (mv_fp16_bias.hpp:8-103).
#include <stdlib.h>

#include "lut_gemv_device.h"
#include "lutgemm_launch.h"

namespace lutgemm {
namespace {

template <int NB, int MODE>
hipError_t launch_nb(const Problem &p, int mrows, hipStream_t stream)
{
    // Rows are taken two at a time through tables whose entries hold both rows as fp16 halves
    // unless LUTGEMM_OPTION_PAIR_TABLES is 0 (one fp32 table set per row then); launches whose
    // ranges all hold one item take the instance that requests nothing for a second item unless
    // LUTGEMM_OPTION_SINGLE_ITEM is 0.
    const bool pair_tables = option(LUTGEMM_OPTION_PAIR_TABLES) != 0;
    const bool single_item = option(LUTGEMM_OPTION_SINGLE_ITEM) != 0;
    const dim3 grid((unsigned)p.wgs_per_chunk, (unsigned)p.mchunks), block(kThreads);
    if (mrows == 4 && pair_tables)
        hipLaunchKernelGGL((lut_gemv_kernel<NB, MODE, 4, true>), grid, block, 0, stream, p);
    else if (mrows == 2 && pair_tables)
        hipLaunchKernelGGL((lut_gemv_kernel<NB, MODE, 2, true>), grid, block, 0, stream, p);
    else if (mrows == 4)
        hipLaunchKernelGGL((lut_gemv_kernel<NB, MODE, 4>), grid, block, 0, stream, p);
    else if (mrows == 2)
        hipLaunchKernelGGL((lut_gemv_kernel<NB, MODE, 2>), grid, block, 0, stream, p);
    else if (p.twin)
        hipLaunchKernelGGL((lut_gemv_kernel<NB, MODE, 1, false, false, true>), grid, block, 0, stream, p);
    else if (p.items_per_wg == 1 && p.short_items == 1 && single_item)
        hipLaunchKernelGGL((lut_gemv_kernel<NB, MODE, 1, false, true>), grid, block, 0, stream, p);
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

hipError_t launch_gemv_rowwise(const Problem &p, int mode, int mrows, hipStream_t stream)
{
    return mode == kUniformF16 ? launch_mode<kUniformF16>(p, mrows, stream) : launch_mode<kRowF16>(p, mrows, stream);
}

}  // namespace lutgemm
