// Launchers of the kernel templates, one translation unit per family so that the
// library builds in parallel.  Each returns hipGetLastError() after the launch.
#ifndef LUTGEMM_LAUNCH_H
#define LUTGEMM_LAUNCH_H

#include "lutgemm_common.h"

namespace lutgemm {

// current value of a tuning option (LUTGEMM_OPTION_* of the public header)
int option(int which);

// look-up kernel, one problem; grid = (p.wgs_per_chunk, p.mchunks); mrows in {1, 2, 4}
hipError_t launch_gemv_rowwise(const Problem &p, int mode, int mrows, hipStream_t stream);       // kRowF16, kUniformF16
hipError_t launch_gemv_block(const Problem &p, int mode, int mrows, hipStream_t stream);         // kBlock*
hipError_t launch_gemv_block_staged(const Problem &p, int mode, int mrows, hipStream_t stream);  // kBlock*Staged
// look-up kernel, one row-wise problem with fused extras, one row per workgroup;
// grid = (p.wgs_per_chunk, p.mchunks)
hipError_t launch_gemv_fused(const Problem &p, int xform, hipStream_t stream);
// look-up kernel, several row-wise problems; grid = (blocks of the largest problem, problems)
hipError_t launch_gemv_group(const Group &g, int xform, int blocks, hipStream_t stream);
// look-up kernel, chained row-wise problems; persistent grid of `blocks` workgroups
hipError_t launch_gemv_chain(const Chain &c, int blocks, hipStream_t stream);
// workgroups of that kernel the current device holds at once (looked up once per device)
hipError_t chain_resident_workgroups(int *count);
// matrix-core kernel; mt = 1 (16-row tiles) or 2 (32-row tiles)
// pow2: the caller promises power-of-two alphas (signs through the LDS table and the fp4 conversion)
hipError_t launch_mfma(const Problem &p, int mt, bool pow2, hipStream_t stream);
hipError_t launch_mfma_fused(const Problem &p, int mt, hipStream_t stream);  // one problem with fused extras
hipError_t launch_mfma_group(const Group &g, int mt, int blocks, hipStream_t stream);
// block-scaled matrix-core kernel (alphas are powers of two): splits p.x into `split` (mx_split_bytes:
// three pieces per value, a row of zeros, a scale word per block of 32), then runs the problem; grid =
// p.n_blocks, row chunks of mx_chunk_rows(p.M) rows
hipError_t launch_mx(const Problem &p, void *split, hipStream_t stream);
inline int mx_chunk_rows(int M) { return M <= 5 ? 5 : M <= 8 ? 8 : 16; }
inline size_t mx_split_bytes(int M, int K) { return (size_t)M * K * 3 + (size_t)K + (size_t)M * (K / 32) * 4; }

}  // namespace lutgemm

#endif
