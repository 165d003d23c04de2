// LUT-GEMV kernels for BCQ linear layers on MI355X (gfx950, wave64) and the
// C ABI that launches them.  Written for this target only.
//
// One kernel template covers the five operand formats of the reference
// extension (lut_gemm/mv_fp16_bias.hpp:8-103,105-220,223-328,342-495,498-579
// in the ShiftAddLLM checkout); the operand layouts are the reference's, the
// execution scheme is not:
//
//  * A workgroup (256 threads = 4 waves) owns an N-tile of 128*NSTEPS outputs
//    and a contiguous K-slice, processed in "sets" of 256 inputs = 8 sign
//    words = 32 eight-input chunks.
//  * Per set it builds 32 partial-sum tables of 256 fp32 entries in LDS
//    (32 KiB).  Table t lives entirely in LDS bank t: entry i of table t is
//    dword i*32 + t.  A half-wave is arranged so that its 32 lanes always
//    look up 32 different tables, hence 32 different banks: no bank conflicts
//    by construction, whatever the data-dependent indices are.
//  * Lane l of a wave: q = l&3, kw = (l>>2)&7, h = l>>5.  The lane streams
//    128-bit loads of sign word (set*8 + kw) for the 4 outputs of quad
//    (h*4+q); rows of the sign matrix are read in 512-byte contiguous runs
//    per workgroup.  At look-up step j the lane uses byte (j+q)&3 of its
//    word, i.e. table kw*4 + ((j+q)&3) -- distinct over (kw, q).
//  * Accumulation is fp32; alphas are applied with one fma per look-up
//    (a power-of-two alpha is then an exact exponent shift).  The 8 kw-lanes
//    of an output are reduced with cross-lane shuffles.
//  * K is split over workgroups (grid.y).  Partial sums go to an fp32
//    workspace; the last workgroup to finish an N-tile (ticket counter) sums
//    them in slice order, adds the caller's fp16 output and rounds once.
//    Deterministic, no floating-point atomics.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <map>
#include <mutex>
#include <utility>

#include "lutgemm_gfx950.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kSetWords = 8;               // sign words (of 32 inputs) per table set
constexpr int kTables = 4 * kSetWords;     // 32 tables, one per LDS bank
constexpr int kWaveCols = 32;              // outputs a wave covers per step
constexpr int kStepCols = 4 * kWaveCols;   // outputs a workgroup covers per step

enum AlphaMode : int {
    kRowF16 = 0,      // fp16 [G][nb][N]
    kBlockF16 = 1,    // fp16 [K/8][nb][R]
    kBlockShiftU16 = 2,
    kBlockApotI8 = 3,
    kUniformF16 = 4,  // alpha, q_bias fp16 [G][N]
};

struct Problem {
    const uint32_t *W;
    const void *alpha;
    const __half *qbias;
    const __half *x;
    __half *out;
    float *partial;      // [ksplit][M][N] fp32, used when ksplit > 1
    unsigned *tickets;   // [M][n_tiles], zero between launches
    int N, K, M;
    int kwords;          // K / 32
    int nsets;           // ceil(kwords / 8)
    int sets_per_split;
    int ksplit;
    int group_words;     // row-wise / uniform: words per alpha group
    int R;               // block modes: row groups
    int rows_per_group;  // block modes: N / R
};

__device__ __forceinline__ float half_bits_to_float(uint32_t bits16)
{
    return __half2float(__ushort_as_half((unsigned short)bits16));
}

// Decode one block-alpha multiplier.
template <int MODE>
__device__ __forceinline__ float load_block_alpha(const void *alpha, size_t i)
{
    if constexpr (MODE == kBlockF16) {
        return __half2float(((const __half *)alpha)[i]);
    } else if constexpr (MODE == kBlockShiftU16) {
        const uint32_t u = ((const uint16_t *)alpha)[i];
        return (float)((1u << (u & 7u)) + (1u << ((u >> 3) & 7u)) + (1u << ((u >> 6) & 7u)));
    } else {
        const int8_t *s = (const int8_t *)alpha + 3 * i;
        float a = 0.0f;
#pragma unroll
        for (int t = 0; t < 3; ++t) {
            const int e = s[t];
            a += (e == -128) ? 0.0f : ldexpf(1.0f, e);  // exponent shift, no multiplier
        }
        return a;
    }
}

template <int NB, int NSTEPS, int MODE>
__global__ void __launch_bounds__(kThreads) lut_gemv_kernel(const Problem p)
{
    __shared__ __attribute__((aligned(16))) float lut[256 * kTables];
    __shared__ unsigned s_is_last;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int q = lane & 3;
    const int kw = (lane >> 2) & 7;
    const int h = lane >> 5;
    const int m = blockIdx.z;
    const int tile0 = blockIdx.x * (kStepCols * NSTEPS);
    const int n_lane = tile0 + wave * kWaveCols + (h * 4 + q) * 4;  // + s*kStepCols

    const __half *x = p.x + (size_t)m * p.K;

    // dword offset of "my" table inside an entry row, per look-up step
    int bank[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) bank[j] = kw * 4 + ((j + q) & 3);

    float acc[NSTEPS][4];
#pragma unroll
    for (int s = 0; s < NSTEPS; ++s)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[s][i] = 0.0f;

    // table-build role of this thread
    const int tb = tid & 31;  // table (bank)
    const int eb = tid >> 5;  // entries eb*32 .. eb*32+31

    const int set_begin = blockIdx.y * p.sets_per_split;
    const int set_end = min(set_begin + p.sets_per_split, p.nsets);

    for (int set = set_begin; set < set_end; ++set) {
        // ---- 1. issue the streaming loads for this set -------------------------
        const int row = set * kSetWords + kw;
        const bool row_ok = row < p.kwords;
        u32x4 wreg[NSTEPS][NB];
#pragma unroll
        for (int s = 0; s < NSTEPS; ++s) {
            const int n = n_lane + s * kStepCols;
            const bool ok = row_ok && n < p.N;
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                if (ok) {
                    const u32x4 *src = (const u32x4 *)(p.W + ((size_t)row * NB + b) * p.N + n);
                    wreg[s][b] = __builtin_nontemporal_load(src);
                } else {
                    wreg[s][b] = (u32x4){0u, 0u, 0u, 0u};
                }
            }
        }

        // alpha operands
        [[maybe_unused]] float a_row[NSTEPS][NB][4];    // row-wise: per (bit, output)
        [[maybe_unused]] float a_blk[NSTEPS][NB][4];    // block: per (bit, look-up step)
        [[maybe_unused]] float a_uni[NSTEPS][4];        // uniform: alpha per output
        [[maybe_unused]] float q_uni[NSTEPS][4];        // uniform: q_bias per output
        if constexpr (MODE == kRowF16) {
            const int g = row / p.group_words;
#pragma unroll
            for (int s = 0; s < NSTEPS; ++s) {
                const int n = n_lane + s * kStepCols;
                const bool ok = row_ok && n < p.N;
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    u32x2 raw = (u32x2){0u, 0u};
                    if (ok)
                        raw = *(const u32x2 *)((const __half *)p.alpha + ((size_t)g * NB + b) * p.N + n);
                    a_row[s][b][0] = half_bits_to_float(raw.x & 0xffffu);
                    a_row[s][b][1] = half_bits_to_float(raw.x >> 16);
                    a_row[s][b][2] = half_bits_to_float(raw.y & 0xffffu);
                    a_row[s][b][3] = half_bits_to_float(raw.y >> 16);
                }
            }
        } else if constexpr (MODE == kUniformF16) {
            const int g = row / p.group_words;
#pragma unroll
            for (int s = 0; s < NSTEPS; ++s) {
                const int n = n_lane + s * kStepCols;
                const bool ok = row_ok && n < p.N;
                u32x2 ra = (u32x2){0u, 0u}, rq = (u32x2){0u, 0u};
                if (ok) {
                    ra = *(const u32x2 *)((const __half *)p.alpha + (size_t)g * p.N + n);
                    rq = *(const u32x2 *)(p.qbias + (size_t)g * p.N + n);
                }
                a_uni[s][0] = half_bits_to_float(ra.x & 0xffffu);
                a_uni[s][1] = half_bits_to_float(ra.x >> 16);
                a_uni[s][2] = half_bits_to_float(ra.y & 0xffffu);
                a_uni[s][3] = half_bits_to_float(ra.y >> 16);
                q_uni[s][0] = half_bits_to_float(rq.x & 0xffffu);
                q_uni[s][1] = half_bits_to_float(rq.x >> 16);
                q_uni[s][2] = half_bits_to_float(rq.y & 0xffffu);
                q_uni[s][3] = half_bits_to_float(rq.y >> 16);
            }
        } else {
#pragma unroll
            for (int s = 0; s < NSTEPS; ++s) {
                const int n = n_lane + s * kStepCols;
                const bool ok = row_ok && n < p.N;
                const int r = ok ? n / p.rows_per_group : 0;
#pragma unroll
                for (int b = 0; b < NB; ++b)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int chunk = row * 4 + ((j + q) & 3);
                        a_blk[s][b][j] =
                            ok ? load_block_alpha<MODE>(p.alpha, ((size_t)chunk * NB + b) * p.R + r)
                               : 0.0f;
                    }
            }
        }

        // activations of the chunk whose table this thread helps to build
        float x2[8];  // 2 * x
        float base = 0.0f;
        {
            const int k0 = (set * kTables + tb) * 8;
            u32x4 raw = (u32x4){0u, 0u, 0u, 0u};
            if (k0 < p.K) raw = *(const u32x4 *)(x + k0);
            const uint32_t r4[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float lo = half_bits_to_float(r4[j] & 0xffffu);
                const float hi = half_bits_to_float(r4[j] >> 16);
                x2[2 * j] = lo + lo;
                x2[2 * j + 1] = hi + hi;
                base -= lo + hi;  // entry 0 = -sum x
            }
        }

        __syncthreads();  // look-ups of the previous set are done with the tables

        // ---- 2. build: this thread writes entries eb*32 .. +31 of table tb ----
        {
            // bits 5..7 of the entry index come from eb
            float top = base;
#pragma unroll
            for (int j = 5; j < 8; ++j)
                if ((eb >> (j - 5)) & 1) top += x2[j];
            float *col = lut + (eb * 32) * kTables + tb;
#pragma unroll
            for (int sb = 0; sb < 4; ++sb) {  // bits 3,4 fixed per sub-block: 4 short chains
                float v = top;
                if (sb & 1) v += x2[3];
                if (sb & 2) v += x2[4];
                unsigned gray = 0;
                col[(sb * 8) * kTables] = v;
#pragma unroll
                for (int i = 1; i < 8; ++i) {
                    const int bit = __builtin_ctz(i);
                    gray ^= 1u << bit;
                    v += ((gray >> bit) & 1u) ? x2[bit] : -x2[bit];
                    col[(sb * 8 + gray) * kTables] = v;
                }
            }
        }
        __syncthreads();

        // ---- 3. look-ups ---------------------------------------------------
        [[maybe_unused]] float sum_x = 0.0f;
        if constexpr (MODE == kUniformF16) {
#pragma unroll
            for (int j = 0; j < 4; ++j) sum_x += lut[255 * kTables + bank[j]];
        }
#pragma unroll
        for (int s = 0; s < NSTEPS; ++s) {
            if constexpr (MODE == kUniformF16) {
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[s][i] = fmaf(q_uni[s][i], sum_x, acc[s][i]);
            }
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const uint32_t w4[4] = {wreg[s][b].x, wreg[s][b].y, wreg[s][b].z, wreg[s][b].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t w = __builtin_rotateright32(w4[i], 8 * q);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t idx = (w >> (8 * j)) & 255u;
                        const float v = lut[idx * kTables + bank[j]];
                        float a;
                        if constexpr (MODE == kRowF16)
                            a = a_row[s][b][i];
                        else if constexpr (MODE == kUniformF16)
                            a = a_uni[s][i] * (1.0f / (float)(2 << b));
                        else
                            a = a_blk[s][b][j];
                        acc[s][i] = fmaf(v, a, acc[s][i]);
                    }
                }
            }
        }
    }

    // ---- 4. reduce the 8 kw-lanes of each output, write ---------------------
#pragma unroll
    for (int s = 0; s < NSTEPS; ++s)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float v = acc[s][i];
            v += __shfl_xor(v, 4);
            v += __shfl_xor(v, 8);
            v += __shfl_xor(v, 16);
            acc[s][i] = v;
        }

    __half *out = p.out + (size_t)m * p.N;
    if (p.ksplit == 1) {
        if (kw == 0) {
#pragma unroll
            for (int s = 0; s < NSTEPS; ++s) {
                const int n = n_lane + s * kStepCols;
                if (n < p.N) {
                    u32x2 raw = *(const u32x2 *)(out + n);
                    const float o0 = half_bits_to_float(raw.x & 0xffffu) + acc[s][0];
                    const float o1 = half_bits_to_float(raw.x >> 16) + acc[s][1];
                    const float o2 = half_bits_to_float(raw.y & 0xffffu) + acc[s][2];
                    const float o3 = half_bits_to_float(raw.y >> 16) + acc[s][3];
                    raw.x = (uint32_t)__half_as_ushort(__float2half_rn(o0)) |
                            ((uint32_t)__half_as_ushort(__float2half_rn(o1)) << 16);
                    raw.y = (uint32_t)__half_as_ushort(__float2half_rn(o2)) |
                            ((uint32_t)__half_as_ushort(__float2half_rn(o3)) << 16);
                    *(u32x2 *)(out + n) = raw;
                }
            }
        }
        return;
    }

    float *partial = p.partial + ((size_t)blockIdx.y * p.M + m) * p.N;
    if (kw == 0) {
#pragma unroll
        for (int s = 0; s < NSTEPS; ++s) {
            const int n = n_lane + s * kStepCols;
            if (n < p.N)
                *(f32x4 *)(partial + n) = (f32x4){acc[s][0], acc[s][1], acc[s][2], acc[s][3]};
        }
    }
    __threadfence();  // release: partials visible device-wide before the ticket
    __syncthreads();
    unsigned *ticket = p.tickets + (size_t)m * gridDim.x + blockIdx.x;
    if (tid == 0) {
        const unsigned t = atomicAdd(ticket, 1u);
        s_is_last = (t == (unsigned)(p.ksplit - 1)) ? 1u : 0u;
    }
    __syncthreads();
    if (!s_is_last) return;
    __threadfence();  // acquire: see every other workgroup's partials

    for (int quad = tid; quad < (kStepCols * NSTEPS) / 4; quad += kThreads) {
        const int n = tile0 + quad * 4;
        if (n >= p.N) continue;
        f32x4 sum = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
        const float *src = p.partial + (size_t)m * p.N + n;
        for (int ks = 0; ks < p.ksplit; ++ks)
            sum += *(const f32x4 *)(src + (size_t)ks * p.M * p.N);
        u32x2 raw = *(const u32x2 *)(out + n);
        const float o0 = half_bits_to_float(raw.x & 0xffffu) + sum.x;
        const float o1 = half_bits_to_float(raw.x >> 16) + sum.y;
        const float o2 = half_bits_to_float(raw.y & 0xffffu) + sum.z;
        const float o3 = half_bits_to_float(raw.y >> 16) + sum.w;
        raw.x = (uint32_t)__half_as_ushort(__float2half_rn(o0)) |
                ((uint32_t)__half_as_ushort(__float2half_rn(o1)) << 16);
        raw.y = (uint32_t)__half_as_ushort(__float2half_rn(o2)) |
                ((uint32_t)__half_as_ushort(__float2half_rn(o3)) << 16);
        *(u32x2 *)(out + n) = raw;
    }
    if (tid == 0) *ticket = 0u;  // ready for the next launch
}

__global__ void __launch_bounds__(256) copy_kernel(u32x4 *dst, const u32x4 *src, size_t n16)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n16; i += stride) dst[i] = src[i];
}

// ------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------

thread_local int g_last_hip_error = 0;

struct Workspace {
    float *partial = nullptr;
    size_t partial_floats = 0;
    unsigned *tickets = nullptr;
    size_t n_tickets = 0;
};

std::mutex g_ws_mutex;
std::map<std::pair<int, hipStream_t>, Workspace> g_workspaces;

int hip_fail(hipError_t e)
{
    g_last_hip_error = (int)e;
    return LUTGEMM_EHIP;
}

// Grow-only workspace per (device, stream).  Launches on one stream are
// ordered, so a stream can share one workspace across calls.
int get_workspace(hipStream_t stream, size_t partial_floats, size_t n_tickets, Workspace *out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e);
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Workspace &ws = g_workspaces[std::make_pair(dev, stream)];
    if (ws.partial_floats < partial_floats || ws.n_tickets < n_tickets) {
        // work queued on the stream may still use the old buffers
        e = hipStreamSynchronize(stream);
        if (e != hipSuccess) return hip_fail(e);
        if (ws.partial_floats < partial_floats) {
            if (ws.partial) (void)hipFree(ws.partial);
            ws.partial = nullptr;
            ws.partial_floats = 0;
            size_t want = partial_floats < (1u << 20) ? (1u << 20) : partial_floats;
            e = hipMalloc((void **)&ws.partial, want * sizeof(float));
            if (e != hipSuccess) { g_last_hip_error = (int)e; return LUTGEMM_ENOMEM; }
            ws.partial_floats = want;
        }
        if (ws.n_tickets < n_tickets) {
            if (ws.tickets) (void)hipFree(ws.tickets);
            ws.tickets = nullptr;
            ws.n_tickets = 0;
            size_t want = n_tickets < 4096 ? 4096 : n_tickets;
            e = hipMalloc((void **)&ws.tickets, want * sizeof(unsigned));
            if (e != hipSuccess) { g_last_hip_error = (int)e; return LUTGEMM_ENOMEM; }
            e = hipMemsetAsync(ws.tickets, 0, want * sizeof(unsigned), stream);
            if (e != hipSuccess) return hip_fail(e);
            e = hipStreamSynchronize(stream);
            if (e != hipSuccess) return hip_fail(e);
            ws.n_tickets = want;
        }
    }
    *out = ws;
    return LUTGEMM_OK;
}

struct Plan {
    int nsteps;   // 1, 2 or 4
    int ksplit;
    int sets_per_split;
    int n_tiles;
};

// Pick the N-tile and the K-split so that the launch has a few workgroups per
// CU (256 CUs) while each workgroup still does enough look-ups per table built.
Plan make_plan(int N, int K, int M)
{
    const int nsets = (K / 32 + kSetWords - 1) / kSetWords;
    const long target_blocks = 1024;
    Plan best{};
    int nsteps = 2;
    if (N <= 128) nsteps = 1;
    const int n_tiles = (N + kStepCols * nsteps - 1) / (kStepCols * nsteps);
    long want = target_blocks / ((long)n_tiles * M);
    if (want < 1) want = 1;
    if (want > nsets) want = nsets;
    int sets_per_split = (nsets + (int)want - 1) / (int)want;
    int ksplit = (nsets + sets_per_split - 1) / sets_per_split;
    best.nsteps = nsteps;
    best.ksplit = ksplit;
    best.sets_per_split = sets_per_split;
    best.n_tiles = n_tiles;
    return best;
}

template <int NB, int MODE>
int launch_nb(const Problem &p, const Plan &plan, hipStream_t stream)
{
    dim3 grid((unsigned)plan.n_tiles, (unsigned)plan.ksplit, (unsigned)p.M);
    dim3 block(kThreads);
    if (plan.nsteps == 1)
        hipLaunchKernelGGL((lut_gemv_kernel<NB, 1, MODE>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((lut_gemv_kernel<NB, 2, MODE>), grid, block, 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e);
    return LUTGEMM_OK;
}

template <int MODE>
int launch_mode(const Problem &p, int nb, const Plan &plan, hipStream_t stream)
{
    switch (nb) {
    case 1: return launch_nb<1, MODE>(p, plan, stream);
    case 2: return launch_nb<2, MODE>(p, plan, stream);
    case 3: return launch_nb<3, MODE>(p, plan, stream);
    case 4: return launch_nb<4, MODE>(p, plan, stream);
    default: return LUTGEMM_EINVAL;
    }
}

bool aligned(const void *ptr, size_t a) { return ((uintptr_t)ptr & (a - 1)) == 0; }

int run(int mode, const uint32_t *bW, const void *alpha, const void *qbias, const void *x,
        void *out, int N, int K, int nb, int num_groups, int M, void *stream_v)
{
    if (!bW || !alpha || !x || !out) return LUTGEMM_EINVAL;
    if (mode == kUniformF16 && !qbias) return LUTGEMM_EINVAL;
    if (N <= 0 || K <= 0 || M <= 0 || num_groups <= 0) return LUTGEMM_EINVAL;
    if (K % 32 != 0 || N % 4 != 0) return LUTGEMM_EINVAL;
    if (nb < 1 || nb > 4) return LUTGEMM_EINVAL;
    if (M > 65535) return LUTGEMM_EINVAL;
    if (!aligned(bW, 16) || !aligned(x, 16) || !aligned(out, 8)) return LUTGEMM_EALIGN;

    Problem p{};
    p.W = bW;
    p.alpha = alpha;
    p.qbias = (const __half *)qbias;
    p.x = (const __half *)x;
    p.out = (__half *)out;
    p.N = N;
    p.K = K;
    p.M = M;
    p.kwords = K / 32;
    p.nsets = (p.kwords + kSetWords - 1) / kSetWords;
    if (mode == kRowF16 || mode == kUniformF16) {
        if (K % num_groups != 0) return LUTGEMM_EINVAL;
        const int gs = K / num_groups;
        if (gs % 32 != 0) return LUTGEMM_EINVAL;  // a sign word may not straddle two groups
        p.group_words = gs / 32;
        if (!aligned(alpha, 8)) return LUTGEMM_EALIGN;
        if (mode == kUniformF16 && !aligned(qbias, 8)) return LUTGEMM_EALIGN;
    } else {
        if (N % num_groups != 0) return LUTGEMM_EINVAL;
        p.R = num_groups;
        p.rows_per_group = N / num_groups;
        if (p.rows_per_group % 4 != 0) return LUTGEMM_EINVAL;
    }
    // x rows must stay 16-byte aligned for the table build
    if (M > 1 && (K % 8) != 0) return LUTGEMM_EINVAL;

    hipStream_t stream = (hipStream_t)stream_v;
    Plan plan = make_plan(N, K, M);
    p.ksplit = plan.ksplit;
    p.sets_per_split = plan.sets_per_split;
    if (plan.ksplit > 1) {
        Workspace ws;
        int rc = get_workspace(stream, (size_t)plan.ksplit * M * N, (size_t)plan.n_tiles * M, &ws);
        if (rc != LUTGEMM_OK) return rc;
        p.partial = ws.partial;
        p.tickets = ws.tickets;
    }
    switch (mode) {
    case kRowF16: return launch_mode<kRowF16>(p, nb, plan, stream);
    case kBlockF16: return launch_mode<kBlockF16>(p, nb, plan, stream);
    case kBlockShiftU16: return launch_mode<kBlockShiftU16>(p, nb, plan, stream);
    case kBlockApotI8: return launch_mode<kBlockApotI8>(p, nb, plan, stream);
    case kUniformF16: return launch_mode<kUniformF16>(p, nb, plan, stream);
    default: return LUTGEMM_EINVAL;
    }
}

}  // namespace

extern "C" {

const char *lutgemm_strerror(int code)
{
    switch (code) {
    case LUTGEMM_OK: return "ok";
    case LUTGEMM_EINVAL:
        return "invalid argument (null pointer, K % 32 != 0, N % 4 != 0, nb outside 1..4, "
               "group size not a multiple of 32, or rows per group not a multiple of 4)";
    case LUTGEMM_EALIGN: return "operand pointer is not aligned (bW, x: 16 bytes; alpha, out: 8 bytes)";
    case LUTGEMM_EUNSUP: return "unsupported configuration";
    case LUTGEMM_EHIP: return "HIP runtime error (see lutgemm_last_hip_error)";
    case LUTGEMM_ENOMEM: return "workspace allocation failed";
    default: return "unknown lutgemm error";
    }
}

int lutgemm_last_hip_error(void) { return g_last_hip_error; }

int lutgemm_gemv_rowwise_f16(const uint32_t *bW, const void *alpha_f16, const void *x_f16,
                             void *out_f16, int N, int K, int nb, int num_groups, int M,
                             void *stream)
{
    return run(kRowF16, bW, alpha_f16, nullptr, x_f16, out_f16, N, K, nb, num_groups, M, stream);
}

int lutgemm_gemv_uniform_f16(const uint32_t *bW, const void *alpha_f16, const void *qbias_f16,
                             const void *x_f16, void *out_f16, int N, int K, int nb,
                             int num_groups, int M, void *stream)
{
    return run(kUniformF16, bW, alpha_f16, qbias_f16, x_f16, out_f16, N, K, nb, num_groups, M,
               stream);
}

int lutgemm_gemv_block_f16(const uint32_t *bW, const void *alpha_f16, const void *x_f16,
                           void *out_f16, int N, int K, int nb, int num_groups, int M,
                           void *stream)
{
    return run(kBlockF16, bW, alpha_f16, nullptr, x_f16, out_f16, N, K, nb, num_groups, M, stream);
}

int lutgemm_gemv_block_shift_u16(const uint32_t *bW, const uint16_t *alpha_u16, const void *x_f16,
                                 void *out_f16, int N, int K, int nb, int num_groups,
                                 int num_apot, int M, void *stream)
{
    if (num_apot != 3) return LUTGEMM_EUNSUP;
    return run(kBlockShiftU16, bW, alpha_u16, nullptr, x_f16, out_f16, N, K, nb, num_groups, M,
               stream);
}

int lutgemm_gemv_block_apot_i8(const uint32_t *bW, const int8_t *alpha_i8, const void *x_f16,
                               void *out_f16, int N, int K, int nb, int num_groups, int num_apot,
                               int M, void *stream)
{
    if (num_apot != 3) return LUTGEMM_EUNSUP;
    return run(kBlockApotI8, bW, alpha_i8, nullptr, x_f16, out_f16, N, K, nb, num_groups, M,
               stream);
}

size_t lutgemm_algorithmic_bytes(int N, int K, int nb, int M, size_t alpha_entries,
                                 int alpha_bytes_per_entry)
{
    const size_t signs = (size_t)K / 8 * (size_t)N * (size_t)nb;
    const size_t alphas = alpha_entries * (size_t)alpha_bytes_per_entry;
    const size_t xin = 2u * (size_t)M * (size_t)K;
    const size_t yio = 2u * 2u * (size_t)M * (size_t)N;  // read (accumulate) + write
    return signs + alphas + xin + yio;
}

int lutgemm_copy_bytes(void *dst, const void *src, size_t bytes, void *stream)
{
    if (!dst || !src || bytes % 16 != 0) return LUTGEMM_EINVAL;
    if (!aligned(dst, 16) || !aligned(src, 16)) return LUTGEMM_EALIGN;
    if (bytes == 0) return LUTGEMM_OK;
    const size_t n16 = bytes / 16;
    size_t blocks = (n16 + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (u32x4 *)dst, (const u32x4 *)src, n16);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e);
    return LUTGEMM_OK;
}

int lutgemm_release_workspaces(void)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e);
    e = hipDeviceSynchronize();
    if (e != hipSuccess) return hip_fail(e);
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    for (auto it = g_workspaces.begin(); it != g_workspaces.end();) {
        if (it->first.first == dev) {
            if (it->second.partial) (void)hipFree(it->second.partial);
            if (it->second.tickets) (void)hipFree(it->second.tickets);
            it = g_workspaces.erase(it);
        } else {
            ++it;
        }
    }
    return LUTGEMM_OK;
}

}  // extern "C"
