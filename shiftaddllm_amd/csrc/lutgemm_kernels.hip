// LUT-GEMV kernels for BCQ linear layers on MI355X (gfx950, wave64) and the
// C ABI that launches them.  Written for this target only.
//
// One kernel template covers the five operand formats of the reference
// extension (lut_gemm/mv_fp16_bias.hpp:8-103,105-220,223-328,342-495,498-579
// in the ShiftAddLLM checkout); the operand layouts are the reference's, the
// execution scheme is not:
//
//  * A workgroup (512 threads = 8 waves) owns an N-tile of 256*NSTEPS outputs
//    and a contiguous K-slice, processed in "sets" of 256 inputs = 8 sign
//    words = 32 eight-input chunks.
//  * Per set it builds 32 partial-sum tables of 256 fp32 entries in LDS.
//    Entry i of table t of buffer f sits at byte i*256 + 4*(t + 32*f): every
//    table lives entirely in LDS bank t, and two buffers interleave in the same
//    64 KiB so that the tables of set i+1 are built while set i is looked up
//    (one barrier per set).  A half-wave is arranged so that its 32 lanes always
//    look up 32 different tables, hence 32 different banks: no bank conflicts by
//    construction, whatever the data-dependent indices are.
//  * The 256-byte entry stride makes a look-up address "index byte in bits
//    8..15, per-lane bank offset in bits 0..7", which ONE v_perm_b32 assembles
//    from the sign word and a per-lane constant; a look-up costs that, the
//    ds_read_b32 and one fma.
//  * Lane l of a wave: q = l&3, kw = (l>>2)&7, h = l>>5.  The lane streams
//    128-bit loads of sign word (set*8 + kw) for the 4 outputs of quad
//    (h*4+q); rows of the sign matrix are read in 1 KiB contiguous runs per
//    workgroup.  At look-up step j the lane uses byte (j+q)&3 of its word,
//    i.e. table kw*4 + ((j+q)&3) -- distinct over (kw, q).
//  * The loads of set i+1 are issued before the look-ups of set i, so the
//    HBM latency of a workgroup's own stream hides behind its LDS work.
//  * Accumulation is fp32; alphas are applied with one fma per look-up
//    (a power-of-two alpha is then an exact exponent shift).  The 8 kw-lanes
//    of an output are reduced with cross-lane shuffles.
//  * K is split over workgroups.  Each workgroup adds its partial sums, as
//    64-bit fixed point (2^-32 units), into a per-output accumulator word with
//    ONE returning atomic; the top byte of the word counts contributions, so
//    the contributor that sees count == ksplit-1 owns the complete sum, adds
//    the caller's fp16 output, rounds once and clears the word.  Integer
//    addition is associative: the result does not depend on arrival order.
//    No fences (a device-scope release costs tens of microseconds here) and
//    no second pass.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdlib.h>

#include <map>
#include <mutex>
#include <type_traits>
#include <utility>
#include <vector>

#include "lutgemm_gfx950.h"
#include "lutgemm_internal.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / 64;
constexpr int kSetWords = 8;               // sign words (of 32 inputs) per table set
constexpr int kTables = 4 * kSetWords;     // 32 tables, one per LDS bank
constexpr int kWaveCols = 32;              // outputs a wave covers per step
constexpr int kStepCols = kWaves * kWaveCols;  // outputs a workgroup covers per step
constexpr int kEntryStride = 64;           // dwords between consecutive entries of a table
constexpr int kLutDwords = 256 * kEntryStride;  // 64 KiB: two interleaved table buffers
constexpr int kStageDwords = 2 * 2 * 4 * kTables;  // staged block alphas: [buffer][row group][bit][chunk]
constexpr int kMaxKSplit = 32;             // bounded by the fixed-point accumulator layout
constexpr int kMaxGroup = LUTGEMM_MAX_GROUP;  // problems per grouped launch

// fixed-point accumulator word: [63:56] contributions, [55:0] sum of (v + kBias),
// v = partial * 2^32 with |partial| <= 2^16
constexpr unsigned long long kCountOne = 1ull << 56;
constexpr unsigned long long kSumMask = kCountOne - 1;
constexpr long long kBias = 1ll << 49;

enum AlphaMode : int {
    kRowF16 = 0,      // fp16 [G][nb][N]
    kBlockF16 = 1,    // fp16 [K/8][nb][R]
    kBlockShiftU16 = 2,
    kBlockApotI8 = 3,
    kUniformF16 = 4,  // alpha, q_bias fp16 [G][N]
    // block formats when an N-tile spans at most two alpha row groups: the set's
    // alphas are staged in LDS by the workgroup instead of loaded lane by lane
    kBlockF16Staged = 5,
    kBlockShiftU16Staged = 6,
    kBlockApotI8Staged = 7,
};

constexpr bool is_block(int mode) { return mode == kBlockF16 || mode == kBlockShiftU16 || mode == kBlockApotI8; }
constexpr bool is_staged(int mode) { return mode >= kBlockF16Staged; }
constexpr int base_mode(int mode) { return is_staged(mode) ? mode - 4 : mode; }

struct Problem {
    const uint32_t *W;
    const void *alpha;
    const __half *qbias;
    const __half *x;
    __half *out;
    unsigned long long *accum;  // [M][N] fixed-point words, zero between launches (ksplit > 1)
    int N, K, M;
    int kwords;          // K / 32
    int nsets;           // ceil(kwords / 8)
    int sets_per_split;
    int ksplit;
    int n_tiles;
    int group_words;     // row-wise / uniform: words per alpha group
    int group_shift;     // log2(group_words) when it is a power of two, else -1
    int R;               // block modes: row groups
    int rows_per_group;  // block modes: N / R
    int nb;
    int block_begin;     // grouped launches: first flat workgroup index of this problem
    int mchunks;         // activation rows are handled in chunks of MROWS
    int n_blocks;        // workgroups of this problem in the flat grid
    // fused input transforms and output mode (row-wise look-up path only)
    const __half *norm_w;  // non-null: the input is fp16(fp16(x * rsqrt(mean(x^2) + norm_eps)) * norm_w)
    const __half *gate;    // non-null [M][K]: the input is fp16(fp16(silu(gate)) * x)
    float norm_eps;
    int overwrite;         // 1: out = y instead of out += y
};

// Flat workgroup index (relative to the problem) -> (tile, kslice, m).
__device__ __forceinline__ void decode_block(const Problem &p, int local, int &tile, int &kslice, int &m)
{
    tile = local % p.n_tiles;
    local /= p.n_tiles;
    kslice = local % p.ksplit;
    m = local / p.ksplit;  // row chunk
}

struct Group {
    int count;
    Problem p[kMaxGroup];
};

__device__ __forceinline__ float half_bits_to_float(uint32_t bits16)
{
    return __half2float(__ushort_as_half((unsigned short)bits16));
}

__device__ __forceinline__ uint32_t float_to_half_bits(float f)
{
    return (uint32_t)__half_as_ushort(__float2half_rn(f));
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

// Everything one lane needs from global memory for one table set.
template <int NB, int NSTEPS, int MODE>
struct SetOperands {
    u32x4 w[NSTEPS][NB];        // sign words: 4 outputs x 32 inputs per register quad
    u32x2 a_row[NSTEPS][NB];    // row-wise: 4 fp16 alphas (one per output)
    float a_blk[NSTEPS][NB][4]; // block: one multiplier per look-up step
    u32x2 a_uni[NSTEPS];        // uniform: alpha per output
    u32x2 q_uni[NSTEPS];        // uniform: q_bias per output
    float a_stage;              // staged block modes: the one alpha this thread stages
};

// Per-lane address parts that do not change from set to set.
template <int NSTEPS>
struct LaneCols {
    uint32_t col4[NSTEPS];  // byte offset of the lane's output quad inside a row of sign words
    uint32_t col2[NSTEPS];  // same, inside a row of fp16 alphas
    int rgroup[NSTEPS];     // block modes: alpha row group of the quad (staged: relative to the tile's first)
    int rg0;                // staged block modes: first row group of the tile
    int tid;
};

// Issue every global load of one table set for this lane.  Branch-free on
// purpose: out-of-range rows and columns are clamped to valid addresses instead
// of predicated, so the loads sit in straight-line code and the compiler can
// keep later sets' loads in flight (s_waitcnt vmcnt(n), n > 0) while the
// current set is consumed.  Clamped data is harmless: tables of inputs beyond K
// are all zero, and outputs beyond N are never written.  Addresses are a
// uniform 64-bit base plus a 32-bit per-lane offset.
template <int NB, int NSTEPS, int MODE>
__device__ __forceinline__ void load_set(SetOperands<NB, NSTEPS, MODE> &r, const Problem &p, int set,
                                         int kw, int q, const LaneCols<NSTEPS> &lc)
{
    const int kwc = min(kw, p.kwords - 1 - set * kSetWords);  // only the last set of K can clamp
    const uint32_t row_bytes = (uint32_t)p.N * 4u;            // one bit plane of one sign word row
    const char *wbase = (const char *)p.W + (size_t)set * kSetWords * NB * row_bytes;
    const uint32_t wrow = (uint32_t)kwc * (NB * row_bytes);
    [[maybe_unused]] const int row = set * kSetWords + kwc;
    [[maybe_unused]] const int g = p.group_shift >= 0 ? (row >> p.group_shift) : (row / p.group_words);
#pragma unroll
    for (int s = 0; s < NSTEPS; ++s) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const char *src = wbase + (size_t)b * row_bytes;
            r.w[s][b] = __builtin_nontemporal_load((const u32x4 *)(src + (wrow + lc.col4[s])));
        }
        if constexpr (MODE == kRowF16) {
            const uint32_t arow = (uint32_t)g * (NB * (uint32_t)p.N * 2u);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const char *src = (const char *)p.alpha + (size_t)b * p.N * 2u;
                r.a_row[s][b] = *(const u32x2 *)(src + (arow + lc.col2[s]));
            }
        } else if constexpr (MODE == kUniformF16) {
            const uint32_t arow = (uint32_t)g * ((uint32_t)p.N * 2u);
            r.a_uni[s] = *(const u32x2 *)((const char *)p.alpha + (arow + lc.col2[s]));
            r.q_uni[s] = *(const u32x2 *)((const char *)p.qbias + (arow + lc.col2[s]));
        } else if constexpr (is_block(MODE)) {
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int chunk = row * 4 + ((j + q) & 3);
                    r.a_blk[s][b][j] =
                        load_block_alpha<MODE>(p.alpha, ((size_t)chunk * NB + b) * p.R + lc.rgroup[s]);
                }
        }
    }
    if constexpr (is_staged(MODE)) {
        // thread t stages alpha(chunk c of the set, bit b, row group rg0 + g2)
        const int t = lc.tid % (2 * NB * kTables);
        const int c = t % kTables, b = (t / kTables) % NB, g2 = t / (NB * kTables);
        const int chunk = min(set * kTables + c, p.K / 8 - 1);
        const int rg = min(lc.rg0 + g2, p.R - 1);
        r.a_stage = load_block_alpha<base_mode(MODE)>(p.alpha, ((size_t)chunk * NB + b) * p.R + rg);
    }
}

// Staged block modes: publish this thread's alpha of a set into stage buffer `abuf`.
template <int NB, int NSTEPS, int MODE>
__device__ __forceinline__ void stage_alpha(const SetOperands<NB, NSTEPS, MODE> &ops, float *stage, int abuf,
                                            int tid)
{
    if constexpr (is_staged(MODE)) {
        if (tid < 2 * NB * kTables) {
            const int c = tid % kTables, b = (tid / kTables) % NB, g2 = tid / (NB * kTables);
            stage[((abuf * 2 + g2) * 4 + b) * kTables + c] = ops.a_stage;
        }
    }
}

// The 8 activations (fp16) of the chunk whose table this thread helps to build:
// chunk tb of set `set` of activation row x.  Fetching and finishing are separate
// so that the loads stay in flight across the look-ups of the current item.
// FUSED kernels also fetch the matching chunk of the norm weight or of the gate row.
// compile-time input transform of a kernel instance
constexpr int kXNone = 0, kXNorm = 1, kXGate = 2;

struct XChunk {
    u32x4 x, other;
    int kc;     // first input of the chunk (clamped into the row)
    bool live;  // chunks beyond K read as zero
};

template <int XF>
__device__ __forceinline__ XChunk fetch_x_chunk(const Problem &p, const __half *x, const __half *gate, int set,
                                                int tb)
{
    const int k0 = (set * kTables + tb) * 8;
    const int kc = min(k0, p.K - 8);
    XChunk c;
    c.x = *(const u32x4 *)(x + kc);
    c.other = (u32x4){0u, 0u, 0u, 0u};
    // (the norm weight is read when the chunk is finished: every workgroup reads the
    // same few KB, an L1/L2 hit, and four registers less are held across the look-ups)
    if constexpr (XF == kXGate) c.other = *(const u32x4 *)(gate + kc);
    c.kc = kc;
    c.live = k0 < p.K;
    return c;
}

// With a norm weight the chunk is scaled by `rscale` (the row's reciprocal RMS) and
// the weight; with a gate row it is multiplied by silu(gate); both with the
// roundings of the separate fp16 operations they replace.
template <int XF>
__device__ __forceinline__ u32x4 finish_x_chunk(const Problem &p, const XChunk &c, float rscale)
{
    u32x4 xr = c.x;
    if constexpr (XF != kXNone) {
        {
            u32x4 other = c.other;
            if constexpr (XF == kXNorm) other = *(const u32x4 *)(p.norm_w + c.kc);
            const uint32_t a[4] = {c.x.x, c.x.y, c.x.z, c.x.w};
            const uint32_t b[4] = {other.x, other.y, other.z, other.w};
            uint32_t o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float v[2];
#pragma unroll
                for (int hh = 0; hh < 2; ++hh) {
                    const float xv = half_bits_to_float((a[j] >> (16 * hh)) & 0xffffu);
                    const float bv = half_bits_to_float((b[j] >> (16 * hh)) & 0xffffu);
                    if constexpr (XF == kXGate)
                        v[hh] = half_bits_to_float(float_to_half_bits(__fdividef(bv, 1.0f + __expf(-bv)))) * xv;
                    else
                        v[hh] = half_bits_to_float(float_to_half_bits(xv * rscale)) * bv;
                }
                o[j] = float_to_half_bits(v[0]) | (float_to_half_bits(v[1]) << 16);
            }
            xr = (u32x4){o[0], o[1], o[2], o[3]};
        }
    }
    u32x4 r;
    r.x = c.live ? xr.x : 0u;
    r.y = c.live ? xr.y : 0u;
    r.z = c.live ? xr.z : 0u;
    r.w = c.live ? xr.w : 0u;
    return r;
}

// Build the 32 tables of one set into buffer `buf` (0/1).  Thread (tb, eb)
// writes entries eb*16 .. eb*16+15 of table tb: bits 4..7 of the entry index
// come from eb, bits 0..3 are walked in Gray-code order, one add per entry.
__device__ __forceinline__ void build_tables(const u32x4 &xraw, float *lut, int buf, int tb, int eb)
{
    float x2[8];  // 2 * x
    float base = 0.0f;
    const uint32_t r4[4] = {xraw.x, xraw.y, xraw.z, xraw.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float lo = half_bits_to_float(r4[j] & 0xffffu);
        const float hi = half_bits_to_float(r4[j] >> 16);
        x2[2 * j] = lo + lo;
        x2[2 * j + 1] = hi + hi;
        base -= lo + hi;  // entry 0 = -sum x
    }
    float top = base;
#pragma unroll
    for (int j = 4; j < 8; ++j)
        if ((eb >> (j - 4)) & 1) top += x2[j];
    float *col = lut + (eb * 16) * kEntryStride + buf * kTables + tb;
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {  // bit 3 fixed per sub-block: two short chains
        float v = top;
        if (sb & 1) v += x2[3];
        unsigned gray = 0;
        col[(sb * 8) * kEntryStride] = v;
#pragma unroll
        for (int i = 1; i < 8; ++i) {
            const int bit = __builtin_ctz(i);
            gray ^= 1u << bit;
            v += ((gray >> bit) & 1u) ? x2[bit] : -x2[bit];
            col[(sb * 8 + gray) * kEntryStride] = v;
        }
    }
}

// This lane's look-ups of one set against table buffer `lane_off` selects.
// lane_off: byte j = 4*(bank of the table used at step j + 32*buffer).
// sel[j]  : v_perm_b32 selector putting byte (j+q)&3 of the sign word into
//           bits 8..15 and byte j of lane_off into bits 0..7.
// Software pipelined in units of 16 look-ups (one bit plane of one step): the
// LDS reads of unit u+1 are issued before the fmas of unit u.
template <int NB, int NSTEPS, int MODE>
__device__ __forceinline__ void lookup_set(const SetOperands<NB, NSTEPS, MODE> &cur, const float *lut,
                                           float (&acc)[NSTEPS][4], uint32_t lane_off,
                                           const uint32_t (&sel)[4], const float *stage_lane,
                                           const LaneCols<NSTEPS> &lc)
{
    const char *lut_bytes = (const char *)lut;
    constexpr int kUnits = NSTEPS * NB;
    float val[2][16];
    [[maybe_unused]] float aval[2][4];
    auto issue = [&](int u, float (&v)[16], float (&av)[4]) {
        const int s = u / NB, b = u % NB;
        const uint32_t w4[4] = {cur.w[s][b].x, cur.w[s][b].y, cur.w[s][b].z, cur.w[s][b].w};
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                v[4 * i + j] = *(const float *)(lut_bytes + __builtin_amdgcn_perm(w4[i], lane_off, sel[j]));
        if constexpr (is_staged(MODE)) {
            // stage_lane points at [this set's buffer][group 0][bit 0][kw*4]; the four
            // alphas of the lane's sign word, in look-up step order
            const float *a4 = stage_lane + (lc.rgroup[s] * 4 + b) * kTables;
#pragma unroll
            for (int j = 0; j < 4; ++j) av[j] = a4[(j + (lc.tid & 3)) & 3];
        }
    };
    auto retire = [&](int u, const float (&v)[16], const float (&av)[4]) {
        const int s = u / NB, b = u % NB;
        [[maybe_unused]] const uint32_t ar[2] = {cur.a_row[s][b].x, cur.a_row[s][b].y};
        [[maybe_unused]] const uint32_t au[2] = {cur.a_uni[s].x, cur.a_uni[s].y};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float a = 0.0f;
            if constexpr (MODE == kRowF16)
                a = half_bits_to_float((ar[i >> 1] >> (16 * (i & 1))) & 0xffffu);
            else if constexpr (MODE == kUniformF16)
                a = half_bits_to_float((au[i >> 1] >> (16 * (i & 1))) & 0xffffu) * (1.0f / (float)(2 << b));
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if constexpr (is_block(MODE))
                    a = cur.a_blk[s][b][j];
                else if constexpr (is_staged(MODE))
                    a = av[j];
                acc[s][i] = fmaf(v[4 * i + j], a, acc[s][i]);
            }
        }
    };
    issue(0, val[0], aval[0]);
    if constexpr (MODE == kUniformF16) {
        // sum of the lane's 32 inputs = entry 255 of its four tables
        float sum_x = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            sum_x += *(const float *)(lut_bytes + 255 * 4 * kEntryStride + ((lane_off >> (8 * j)) & 255u));
#pragma unroll
        for (int s = 0; s < NSTEPS; ++s) {
            const uint32_t rq[2] = {cur.q_uni[s].x, cur.q_uni[s].y};
#pragma unroll
            for (int i = 0; i < 4; ++i)
                acc[s][i] = fmaf(half_bits_to_float((rq[i >> 1] >> (16 * (i & 1))) & 0xffffu), sum_x, acc[s][i]);
        }
    }
#pragma unroll
    for (int u = 0; u < kUnits; ++u) {
        if (u + 1 < kUnits) issue(u + 1, val[(u + 1) & 1], aval[(u + 1) & 1]);
        retire(u, val[u & 1], aval[u & 1]);
    }
}

// One workgroup's share: N-tile `tile`, K-slice `kslice`, activation rows
// mchunk*MROWS .. +MROWS-1.  The sign words of a set are loaded once and used
// for all MROWS rows; tables are built per (set, row) and double buffered, so the
// work items of the pipeline are the (set, row) pairs in order.
template <int NB, int NSTEPS, int MODE, int MROWS, int XF = kXNone>
__device__ __forceinline__ void gemv_tile(const Problem &p, int tile, int kslice, int mchunk, float *lut)
{
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int q = lane & 3;
    const int kw = (lane >> 2) & 7;
    const int h = lane >> 5;
    const int tile0 = tile * (kStepCols * NSTEPS);
    const int n_lane = tile0 + wave * kWaveCols + (h * 4 + q) * 4;  // + s*kStepCols
    const int m0 = mchunk * MROWS;

    // rows beyond M are clamped to the last row (computed twice, written once)
    const __half *xrow[MROWS];
#pragma unroll
    for (int r = 0; r < MROWS; ++r) xrow[r] = p.x + (size_t)min(m0 + r, p.M - 1) * p.K;
    const __half *grow[MROWS];
#pragma unroll
    for (int r = 0; r < MROWS; ++r)
        grow[r] = (XF == kXGate) ? p.gate + (size_t)min(m0 + r, p.M - 1) * p.K : nullptr;

    // per-lane look-up constants (see lookup_set)
    uint32_t lane_off = 0;
    uint32_t sel[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int jj = (j + q) & 3;
        lane_off |= (uint32_t)(4 * (kw * 4 + jj)) << (8 * j);
        sel[j] = 0x0c0c0000u | ((uint32_t)(4 + jj) << 8) | (uint32_t)j;
    }

    float acc[MROWS][NSTEPS][4];
#pragma unroll
    for (int r = 0; r < MROWS; ++r)
#pragma unroll
        for (int s = 0; s < NSTEPS; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[r][s][i] = 0.0f;

    // table-build role of this thread
    const int tb = tid & 31;  // table (bank)
    const int eb = tid >> 5;  // entries eb*16 .. eb*16+15

    const int set_begin = kslice * p.sets_per_split;
    const int set_end = min(set_begin + p.sets_per_split, p.nsets);

    LaneCols<NSTEPS> lc;
#pragma unroll
    for (int s = 0; s < NSTEPS; ++s) {
        const int n = min(n_lane + s * kStepCols, p.N - 4);
        lc.col4[s] = (uint32_t)n * 4u;
        lc.col2[s] = (uint32_t)n * 2u;
        lc.rgroup[s] = 0;
        if constexpr (is_block(MODE)) lc.rgroup[s] = n / p.rows_per_group;
        if constexpr (is_staged(MODE)) lc.rgroup[s] = n / p.rows_per_group - tile0 / p.rows_per_group;
    }
    lc.rg0 = is_staged(MODE) ? tile0 / p.rows_per_group : 0;
    lc.tid = tid;
    float *stage = lut + kLutDwords;
    int abuf = 0;

    // Two operand buffers used alternately: while set i is looked up, the loads of
    // set i+1 are in flight.  No register copies between them (a copy would have
    // to wait for the loads), and the has-next test is peeled out of the load
    // path so that the compiler can count the loads in flight exactly.
    // fused RMSNorm: every workgroup forms the reciprocal RMS of its rows itself (K
    // fp16 values per row, from L2).  The row is requested BEFORE the first sign
    // words so that, loads returning in order, it can be waited for alone.
    constexpr int kNormChunks = 2;  // 16-byte chunks per thread held in registers: K <= 8192
    u32x4 nx[XF == kXNorm ? MROWS : 1][kNormChunks];
    if constexpr (XF == kXNorm) {
        {
#pragma unroll
            for (int r = 0; r < MROWS; ++r)
#pragma unroll
                for (int u = 0; u < kNormChunks; ++u)
                    nx[r][u] = *(const u32x4 *)(xrow[r] + 8 * min(tid + kThreads * u, p.K / 8 - 1));
        }
    }
    XChunk xc0 = fetch_x_chunk<XF>(p, xrow[0], grow[0], set_begin, tb);

    SetOperands<NB, NSTEPS, MODE> opA, opB;
    load_set<NB, NSTEPS, MODE>(opA, p, set_begin, kw, q, lc);

    // the caller's output, needed only by whoever completes a sum: fetched now,
    // off the critical path
    u32x2 out_raw[MROWS][NSTEPS];
#pragma unroll
    for (int r = 0; r < MROWS; ++r)
#pragma unroll
        for (int s = 0; s < NSTEPS; ++s)
            out_raw[r][s] = *(const u32x2 *)((const char *)(p.out + (size_t)min(m0 + r, p.M - 1) * p.N) + lc.col2[s]);

    float rscale[MROWS];
#pragma unroll
    for (int r = 0; r < MROWS; ++r) rscale[r] = 1.0f;
    if constexpr (XF == kXNorm) {
        {
            float ss[MROWS];
#pragma unroll
            for (int r = 0; r < MROWS; ++r) {
                ss[r] = 0.0f;
                auto add_chunk = [&](const u32x4 &v) {
                    const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float lo = half_bits_to_float(w4[j] & 0xffffu), hi = half_bits_to_float(w4[j] >> 16);
                        ss[r] = fmaf(lo, lo, fmaf(hi, hi, ss[r]));
                    }
                };
#pragma unroll
                for (int u = 0; u < kNormChunks; ++u)
                    if (tid + kThreads * u < p.K / 8) add_chunk(nx[r][u]);
                for (int c = tid + kThreads * kNormChunks; c < p.K / 8; c += kThreads)  // K > 16384
                    add_chunk(*(const u32x4 *)(xrow[r] + 8 * c));
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) ss[r] += __shfl_xor(ss[r], off);
                if (lane == 0) lut[wave * MROWS + r] = ss[r];
            }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < MROWS; ++r) {
                float t = 0.0f;
#pragma unroll
                for (int w = 0; w < kWaves; ++w) t += lut[w * MROWS + r];
                rscale[r] = rsqrtf(t / (float)p.K + p.norm_eps);
            }
            __syncthreads();  // the tables are built over the same LDS words
        }
    }

    int buf = 0;
    build_tables(finish_x_chunk<XF>(p, xc0, rscale[0]), lut, 0, tb, eb);
    stage_alpha<NB, NSTEPS, MODE>(opA, stage, 0, tid);
    __syncthreads();
    // Steady state, per (set, row) item: fetch the activations of the next item,
    // look the current item up in table buffer f, build the next item's tables into
    // buffer f^1, one barrier.  The barrier both publishes buffer f^1 and retires
    // the readers of buffer f, which the item after next overwrites.
    constexpr uint32_t kFlip = 0x80808080u;  // +128 bytes = the other table buffer
    auto rows_of_set = [&](const SetOperands<NB, NSTEPS, MODE> &ops, const SetOperands<NB, NSTEPS, MODE> &nxt,
                           int set, auto has_next_set) {
#pragma unroll
        for (int r = 0; r < MROWS; ++r) {
            const bool more = (r + 1 < MROWS) || decltype(has_next_set)::value;
            XChunk xn{};
            if (more)
                xn = (r + 1 < MROWS) ? fetch_x_chunk<XF>(p, xrow[(r + 1) % MROWS], grow[(r + 1) % MROWS], set, tb)
                                     : fetch_x_chunk<XF>(p, xrow[0], grow[0], set + 1, tb);
            // opaque to the optimiser: otherwise the 48 look-up addresses of a set are
            // kept in registers across all rows instead of being recomputed (1 op each)
            asm volatile("" : "+v"(lane_off));
            lookup_set<NB, NSTEPS, MODE>(ops, lut, acc[r], lane_off, sel,
                                         stage + abuf * (2 * 4 * kTables) + kw * 4, lc);
            if (more) {
                buf ^= 1;
                lane_off ^= kFlip;
                build_tables(finish_x_chunk<XF>(p, xn, rscale[(r + 1) % MROWS]), lut, buf, tb, eb);
                if (r + 1 == MROWS) {  // moving on to the next set: its alphas go to the other stage buffer
                    abuf ^= 1;
                    stage_alpha<NB, NSTEPS, MODE>(nxt, stage, abuf, tid);
                }
                __syncthreads();
            }
        }
    };
    for (int set = set_begin;;) {
        if (set + 1 >= set_end) {
            rows_of_set(opA, opA, set, std::false_type{});
            break;
        }
        load_set<NB, NSTEPS, MODE>(opB, p, set + 1, kw, q, lc);
        rows_of_set(opA, opB, set, std::true_type{});
        ++set;
        if (set + 1 >= set_end) {
            rows_of_set(opB, opB, set, std::false_type{});
            break;
        }
        load_set<NB, NSTEPS, MODE>(opA, p, set + 1, kw, q, lc);
        rows_of_set(opB, opA, set, std::true_type{});
        ++set;
    }

    // ---- reduce the 8 kw-lanes of each output --------------------------------
#pragma unroll
    for (int r = 0; r < MROWS; ++r)
#pragma unroll
        for (int s = 0; s < NSTEPS; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float v = acc[r][s][i];
                v += __shfl_xor(v, 4);
                v += __shfl_xor(v, 8);
                v += __shfl_xor(v, 16);
                acc[r][s][i] = v;
            }
    if (kw != 0) return;

#pragma unroll
    for (int r = 0; r < MROWS; ++r) {
        const int m = m0 + r;
        if (m >= p.M) break;
        __half *out = p.out + (size_t)m * p.N;
        if (p.ksplit == 1) {
#pragma unroll
            for (int s = 0; s < NSTEPS; ++s) {
                const int n = n_lane + s * kStepCols;
                if (n < p.N) {
                    u32x2 raw = out_raw[r][s];
                    if (p.overwrite) raw = (u32x2){0u, 0u};
                    const float o0 = half_bits_to_float(raw.x & 0xffffu) + acc[r][s][0];
                    const float o1 = half_bits_to_float(raw.x >> 16) + acc[r][s][1];
                    const float o2 = half_bits_to_float(raw.y & 0xffffu) + acc[r][s][2];
                    const float o3 = half_bits_to_float(raw.y >> 16) + acc[r][s][3];
                    raw.x = float_to_half_bits(o0) | (float_to_half_bits(o1) << 16);
                    raw.y = float_to_half_bits(o2) | (float_to_half_bits(o3) << 16);
                    *(u32x2 *)(out + n) = raw;
                }
            }
            continue;
        }

        // ---- K-split: one returning fixed-point atomic per output ---------------
        unsigned long long *accum = p.accum + (size_t)m * p.N;
        unsigned long long contrib[NSTEPS][4], old[NSTEPS][4];
#pragma unroll
        for (int s = 0; s < NSTEPS; ++s) {
            const int n = n_lane + s * kStepCols;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // non-finite or out-of-range partial sums saturate (fp16 rounds them to inf)
                float v = acc[r][s][i];
                v = (v == v) ? v : 65536.0f;
                v = fminf(fmaxf(v, -65536.0f), 65536.0f);
                const long long fx = __double2ll_rn((double)v * 4294967296.0);
                contrib[s][i] = (unsigned long long)(fx + kBias) + kCountOne;
                old[s][i] = 0;
                if (n < p.N)
                    old[s][i] = __hip_atomic_fetch_add(accum + n + i, contrib[s][i], __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
            }
        }
#pragma unroll
        for (int s = 0; s < NSTEPS; ++s) {
            const int n = n_lane + s * kStepCols;
            if (n >= p.N) continue;
            const uint32_t raw2[2] = {out_raw[r][s].x, out_raw[r][s].y};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if ((int)(old[s][i] >> 56) != p.ksplit - 1) continue;
                // this contribution completed the sum
                const long long total =
                    (long long)((old[s][i] + contrib[s][i]) & kSumMask) - (long long)p.ksplit * kBias;
                const float y = (float)((double)total * (1.0 / 4294967296.0));
                const float prev = p.overwrite ? 0.0f : half_bits_to_float((raw2[i >> 1] >> (16 * (i & 1))) & 0xffffu);
                out[n + i] = __float2half_rn(prev + y);
                __hip_atomic_store(accum + n + i, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
}

template <int NB, int NSTEPS, int MODE, int MROWS>
__global__ void __launch_bounds__(kThreads) lut_gemv_kernel(const Problem p)
{
    __shared__ __attribute__((aligned(16))) float lut[kLutDwords + kStageDwords];
    int tile, kslice, mchunk;
    decode_block(p, (int)blockIdx.x, tile, kslice, mchunk);
    gemv_tile<NB, NSTEPS, MODE, MROWS>(p, tile, kslice, mchunk, lut);
}

// Several row-wise problems in one launch (flat 1-D grid).  Bit widths may
// differ between the problems of a group.
// XF: the input transform shared by all problems of the launch.
template <int NSTEPS, int XF>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
lut_gemv_group_kernel(const Group g)
{
    __shared__ __attribute__((aligned(16))) float lut[kLutDwords + kStageDwords];
    const int b = blockIdx.x;
    int pi = 0;
#pragma unroll
    for (int i = 1; i < kMaxGroup; ++i)
        if (i < g.count && b >= g.p[i].block_begin) pi = i;
    const Problem &p = g.p[pi];
    int tile, kslice, m;
    decode_block(p, b - p.block_begin, tile, kslice, m);
    switch (p.nb) {
    case 1: gemv_tile<1, NSTEPS, kRowF16, 1, XF>(p, tile, kslice, m, lut); break;
    case 2: gemv_tile<2, NSTEPS, kRowF16, 1, XF>(p, tile, kslice, m, lut); break;
    case 3: gemv_tile<3, NSTEPS, kRowF16, 1, XF>(p, tile, kslice, m, lut); break;
    default: gemv_tile<4, NSTEPS, kRowF16, 1, XF>(p, tile, kslice, m, lut); break;
    }
}

// ---------------------------------------------------------------------------
// Small-batch path (row-wise alpha, several activation rows): matrix cores.
//
// Table look-ups cost one LDS read and two VALU operations per sign byte PER
// ROW, so beyond a couple of rows the look-up kernel is VALU/LDS bound
// (measured: ~21 us per extra row on a 132 MB matrix whose stream takes 18 us).
// Here the sign bits are expanded to +-1.0 fp16 in registers (one VALU
// operation per two signs) and multiplied with 16 activation rows at a time by
// v_mfma_f32_16x16x32_f16, fp32 accumulation; alpha scales each (group, bit
// plane) partial product with one fma per output.
//
// Work split: a workgroup of 8 waves owns 64 outputs; its waves take different
// K-steps (128 inputs = 4 sign words = one alpha group of 128) and their
// accumulators meet in LDS at the end, so that the number of cross-workgroup
// atomics does not grow with the K parallelism.  Lane l (li = l&15, kb = l>>4)
// loads the four sign words of outputs n = base + 4*li .. +3 for word kb of its
// step (256-byte runs per row).  MFMA instance (e, beta) takes from every lane 8
// signs of its word e: bits 4*beta+i and 16+4*beta+i, i < 4 -- two bits 16 apart
// land in the sign positions of a packed fp16 pair with ONE shift and ONE
// and-or.  So the instance's A rows are outputs base + 4*i + e and its K block
// kb is word kb; the activations of a round (8 steps) are staged in LDS in
// exactly that K order.
// ---------------------------------------------------------------------------
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kMfmaThreads = 512;
constexpr int kMfmaWaves = kMfmaThreads / 64;
constexpr int kMfmaTileCols = 64;     // outputs per workgroup
constexpr int kMfmaStepK = 128;
constexpr int kXRowBytes = 256 + 16;  // one activation row of a K-step, padded against bank conflicts

constexpr int kAlphaStepHalves = 64;  // alphas of one (K-step, bit plane): the workgroup's 64 outputs

// Sign words of one K-step of a wave: word kb of 4 outputs per bit plane.
template <int NB>
struct MfmaSigns {
    u32x4 w[NB];
};

template <int NB>
__device__ __forceinline__ void mfma_load_signs(MfmaSigns<NB> &r, const Problem &p, int step, int kb, uint32_t wcol4)
{
    const uint32_t row_bytes = (uint32_t)p.N * 4u;
    const char *wbase = (const char *)p.W + (size_t)step * 4 * NB * row_bytes;
    const uint32_t wrow = (uint32_t)kb * (NB * row_bytes);
#pragma unroll
    for (int b = 0; b < NB; ++b)
        r.w[b] = __builtin_nontemporal_load((const u32x4 *)(wbase + (size_t)b * row_bytes + (wrow + wcol4)));
}

// What a thread fetches for the staging of one round (8 K-steps): 4*MT activation
// targets (16 bytes each after the shuffle into MFMA K order) and one 8-byte run of
// alphas.
template <int MT>
struct MfmaStage {
    u32x2 lo[4 * MT], hi[4 * MT];
    u32x2 alpha;
};

// 8 signs of sign word `w` -> 8 fp16 +-1.0 (bit set = +1.0): pair i holds
// bit 4*beta+i (low half) and bit 16+4*beta+i (high half).
__device__ __forceinline__ f16x8 expand_signs(uint32_t w, int beta)
{
    // (~shifted & 0x80008000) | 0x3c003c00 as ONE three-input bit operation
    // (truth table 0xae = (~a & b) | c); the compiler otherwise emits not + and + or.
    const uint32_t sign = 0x80008000u, one = 0x3c003c00u;
    u32x4 r;
    r.x = __builtin_amdgcn_bitop3_b32(w << (15 - (4 * beta + 0)), sign, one, 0xae);
    r.y = __builtin_amdgcn_bitop3_b32(w << (15 - (4 * beta + 1)), sign, one, 0xae);
    r.z = __builtin_amdgcn_bitop3_b32(w << (15 - (4 * beta + 2)), sign, one, 0xae);
    r.w = __builtin_amdgcn_bitop3_b32(w << (15 - (4 * beta + 3)), sign, one, 0xae);
    return __builtin_bit_cast(f16x8, r);
}

// xs: activations of one round, [wave's step][row][word][instance][8 halves],
// kMfmaWaves * 16 * MT * kXRowBytes bytes (reused for the final reduction), followed
// by the alphas of the round, kMfmaWaves * NB * 64 halves.
template <int NB, int MT>
__device__ __forceinline__ void mfma_tile(const Problem &p, int local_block, char *xs)
{
    constexpr int kWaveXBytes = 16 * MT * kXRowBytes;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int li = lane & 15;
    const int kb = lane >> 4;
    int tile, kslice, mchunk;
    decode_block(p, local_block, tile, kslice, mchunk);
    const int m0 = mchunk * 16 * MT;
    const int n_base = tile * kMfmaTileCols;

    const uint32_t wcol4 = (uint32_t)min(n_base + 4 * li, p.N - 4) * 4u;

    const int step_begin = kslice * p.sets_per_split;
    const int step_end = min(step_begin + p.sets_per_split, p.nsets);

    // Staging of a round (8 K-steps, one per wave), fetched one round ahead into
    // registers and written to LDS between two barriers:
    //  * activations: target t = (step s of the round, row rr, word w, instance beta)
    //    gets 8 halves in MFMA K order;
    //  * alphas: thread t < 128*NB fetches alpha[group of step s][plane b][base + 4q .. +3]
    //    (s, b, q from t) and scatters it to as[s][b][kb][e][r], so that a lane reads
    //    the four alphas of its D rows (one e, r = 0..3) as one 8-byte word.
    char *as = xs + kMfmaWaves * kWaveXBytes;
    const int a_q = tid & 15, a_sb = tid >> 4;          // alpha role: 4 outputs 4q.., (step, plane)
    const int a_s = a_sb / NB, a_b = a_sb % NB;
    const bool a_role = tid < 16 * kMfmaWaves * NB;
    const uint32_t acol2 = (uint32_t)min(n_base + 4 * a_q, p.N - 4) * 2u;

    auto fetch_stage = [&](MfmaStage<MT> &st, int r0) {
#pragma unroll
        for (int u = 0; u < 4 * MT; ++u) {
            const int t = tid + kMfmaThreads * u;
            const int beta = t & 3, w = (t >> 2) & 3, rr = (t >> 4) % (16 * MT), sidx = t / (256 * MT);
            const int step = min(r0 + sidx, p.nsets - 1);
            const __half *src = p.x + (size_t)min(m0 + rr, p.M - 1) * p.K + step * kMfmaStepK + 32 * w + 4 * beta;
            st.lo[u] = *(const u32x2 *)src;
            st.hi[u] = *(const u32x2 *)(src + 16);
        }
        const int g = (min(r0 + (a_role ? a_s : 0), p.nsets - 1) * 4) / p.group_words;
        st.alpha = *(const u32x2 *)((const char *)p.alpha + ((size_t)g * NB + (a_role ? a_b : 0)) * p.N * 2u + acol2);
    };
    auto store_stage = [&](const MfmaStage<MT> &st) {
#pragma unroll
        for (int u = 0; u < 4 * MT; ++u) {
            const int t = tid + kMfmaThreads * u;
            const int beta = t & 3, w = (t >> 2) & 3, rr = (t >> 4) % (16 * MT), sidx = t / (256 * MT);
            u32x4 v;
            v.x = __builtin_amdgcn_perm(st.hi[u].x, st.lo[u].x, 0x05040100u);
            v.y = __builtin_amdgcn_perm(st.hi[u].x, st.lo[u].x, 0x07060302u);
            v.z = __builtin_amdgcn_perm(st.hi[u].y, st.lo[u].y, 0x05040100u);
            v.w = __builtin_amdgcn_perm(st.hi[u].y, st.lo[u].y, 0x07060302u);
            *(u32x4 *)(xs + sidx * kWaveXBytes + rr * kXRowBytes + w * 64 + beta * 16) = v;
        }
        if (a_role) {
            // outputs 4q + e, e = 0..3: kb = q >> 2, r = q & 3
            unsigned short *dst = (unsigned short *)as + ((a_s * NB + a_b) * 4 + (a_q >> 2)) * 16 + (a_q & 3);
            dst[0] = (unsigned short)(st.alpha.x & 0xffffu);
            dst[4] = (unsigned short)(st.alpha.x >> 16);
            dst[8] = (unsigned short)(st.alpha.y & 0xffffu);
            dst[12] = (unsigned short)(st.alpha.y >> 16);
        }
    };

    f32x4 acc[4][MT];
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[e][mt] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};

    auto compute = [&](const MfmaSigns<NB> &ops) {
        const char *xw = xs + wave * kWaveXBytes;
        const u32x2 *aw = (const u32x2 *)as + (wave * NB * 4 + kb) * 4;   // + b*16 + e
        f16x8 bx[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int beta = 0; beta < 4; ++beta)
                bx[mt][beta] = *(const f16x8 *)(xw + (16 * mt + li) * kXRowBytes + kb * 64 + beta * 16);
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const uint32_t w4[4] = {ops.w[b].x, ops.w[b].y, ops.w[b].z, ops.w[b].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const u32x2 al = aw[b * 16 + e];  // alphas of D rows r = 0..3 (outputs base + 16*kb + 4*r + e)
                f32x4 d[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) d[mt] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int beta = 0; beta < 4; ++beta) {
                    const f16x8 a = expand_signs(w4[e], beta);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        d[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bx[mt][beta], d[mt], 0, 0, 0);
                }
                const uint32_t araw[4] = {al.x & 0xffffu, al.x >> 16, al.y & 0xffffu, al.y >> 16};
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float alr = half_bits_to_float(araw[r]);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) acc[e][mt][r] = fmaf(d[mt][r], alr, acc[e][mt][r]);
                }
            }
        }
    };

    // Rounds of 8 steps, one per wave, software pipelined: while round i is
    // multiplied, the sign words of round i+1 (the HBM stream) are in flight; two sign
    // buffers alternate (no register copies) and loads are clamped, not predicated, so
    // that the waits can count them.  The staging data (activations and alphas, L2
    // hits) is fetched a round ahead too where registers allow: in the 32-row tile,
    // which has one workgroup per CU anyway.  The 16-row tile keeps to 128 registers
    // so that two workgroups share a CU (measured, 28672x8192x4: 62 us with two
    // resident workgroups and no look-ahead, 70-74 us with one and full look-ahead).
    constexpr bool kStageAhead = MT == 2 && NB >= 3;
    MfmaSigns<NB> sgA, sgB;
    MfmaStage<MT> st;
    mfma_load_signs<NB>(sgA, p, min(step_begin + wave, p.nsets - 1), kb, wcol4);
    if constexpr (kStageAhead) fetch_stage(st, step_begin);
    // (the look-ahead of the last round re-reads clamped addresses and is discarded)
    auto round = [&](const MfmaSigns<NB> &cur, MfmaSigns<NB> &nxt, int r0) {
        __syncthreads();  // the previous round's readers are done with the staged data
        if constexpr (!kStageAhead) fetch_stage(st, r0);
        store_stage(st);
        mfma_load_signs<NB>(nxt, p, min(r0 + kMfmaWaves + wave, p.nsets - 1), kb, wcol4);
        if constexpr (kStageAhead) fetch_stage(st, r0 + kMfmaWaves);
        __syncthreads();
        if (r0 + wave < step_end) compute(cur);
    };
    for (int r0 = step_begin; r0 < step_end; r0 += 2 * kMfmaWaves) {
        round(sgA, sgB, r0);
        if (r0 + kMfmaWaves < step_end) round(sgB, sgA, r0 + kMfmaWaves);
    }

    // ---- the 8 waves' accumulators meet in LDS -----------------------------------
    // red[wave][j = (e*MT + mt)*4 + r][lane], rows padded to 65 words so that the
    // read-out below (consecutive threads = consecutive outputs) spreads over the banks
    constexpr int kRedRow = 65;
    __syncthreads();
    float *red = (float *)xs;
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                red[(wave * (16 * MT) + (e * MT + mt) * 4 + r) * kRedRow + lane] = acc[e][mt][r];
    __syncthreads();
    // Thread t finishes output column t & 63 of rows (t >> 6) + 8*i: a wave covers 64
    // consecutive outputs of one row, so its atomics and its fp16 read-modify-write
    // fall into whole cache lines.
    const int nl = tid & 63;
    const int n = n_base + nl;
    const int src_lane = (nl >> 4) * 16;            // kb of the column; + li of the row below
    const int src_j = (nl & 3) * MT * 4 + ((nl >> 2) & 3);  // e and r of the column; + mt*4 of the row
    float val[2 * MT];
    unsigned long long contrib[2 * MT], old[2 * MT];
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i) {
        const int ml = (tid >> 6) + 8 * i;          // row within the chunk
        const int j = src_j + (ml >> 4) * 4, sl = src_lane + (ml & 15);
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < kMfmaWaves; ++w) v += red[(w * (16 * MT) + j) * kRedRow + sl];
        val[i] = v;
        old[i] = 0;
        contrib[i] = 0;
        const int m = m0 + ml;
        if (p.ksplit > 1 && m < p.M && n < p.N) {
            v = (v == v) ? v : 65536.0f;
            v = fminf(fmaxf(v, -65536.0f), 65536.0f);
            const long long fx = __double2ll_rn((double)v * 4294967296.0);
            contrib[i] = (unsigned long long)(fx + kBias) + kCountOne;
            old[i] = __hip_atomic_fetch_add(p.accum + (size_t)m * p.N + n, contrib[i], __ATOMIC_RELAXED,
                                            __HIP_MEMORY_SCOPE_AGENT);
        }
    }
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i) {
        const int m = m0 + (tid >> 6) + 8 * i;
        if (m >= p.M || n >= p.N) continue;
        __half *dst = p.out + (size_t)m * p.N + n;
        if (p.ksplit == 1) {
            *dst = __float2half_rn((p.overwrite ? 0.0f : __half2float(*dst)) + val[i]);
            continue;
        }
        if ((int)(old[i] >> 56) != p.ksplit - 1) continue;
        const long long total = (long long)((old[i] + contrib[i]) & kSumMask) - (long long)p.ksplit * kBias;
        const float y = (float)((double)total * (1.0 / 4294967296.0));
        *dst = __float2half_rn((p.overwrite ? 0.0f : __half2float(*dst)) + y);
        __hip_atomic_store(p.accum + (size_t)m * p.N + n, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <int NB, int MT>
__global__ void __launch_bounds__(kMfmaThreads) lut_gemm_mfma_kernel(const Problem p)
{
    __shared__ __attribute__((aligned(16))) char xs[kMfmaWaves * 16 * MT * kXRowBytes + kMfmaWaves * NB * kAlphaStepHalves * 2];
    mfma_tile<NB, MT>(p, (int)blockIdx.x, xs);
}

// Several problems in one launch (flat 1-D grid); bit widths may differ.
template <int MT>
__global__ void __launch_bounds__(kMfmaThreads) lut_gemm_mfma_group_kernel(const Group g)
{
    __shared__ __attribute__((aligned(16))) char xs[kMfmaWaves * 16 * MT * kXRowBytes + kMfmaWaves * 4 * kAlphaStepHalves * 2];
    const int b = blockIdx.x;
    int pi = 0;
#pragma unroll
    for (int i = 1; i < kMaxGroup; ++i)
        if (i < g.count && b >= g.p[i].block_begin) pi = i;
    const Problem &p = g.p[pi];
    switch (p.nb) {
    case 1: mfma_tile<1, MT>(p, b - p.block_begin, xs); break;
    case 2: mfma_tile<2, MT>(p, b - p.block_begin, xs); break;
    case 3: mfma_tile<3, MT>(p, b - p.block_begin, xs); break;
    default: mfma_tile<4, MT>(p, b - p.block_begin, xs); break;
    }
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
    unsigned long long *accum = nullptr;
    size_t words = 0;
    std::vector<unsigned long long *> retired;  // outgrown buffers: captured graphs may still name them
};

std::mutex g_ws_mutex;
std::map<std::pair<int, hipStream_t>, Workspace> g_workspaces;

int hip_fail(hipError_t e)
{
    g_last_hip_error = (int)e;
    return LUTGEMM_EHIP;
}

// Grow-only, zero-initialised accumulator words per (device, stream).  Launches
// on one stream are ordered and every launch leaves its words at zero again, so
// a stream shares one workspace across calls.  Growing synchronises the stream
// and allocates: do a first call of each shape before capturing a graph.  An
// outgrown buffer is kept (zero, unused by new launches) until
// lutgemm_release_workspaces(): a graph captured earlier still points at it.
int get_workspace(hipStream_t stream, size_t words, unsigned long long **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e);
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Workspace &ws = g_workspaces[std::make_pair(dev, stream)];
    if (ws.words < words) {
        e = hipStreamSynchronize(stream);  // queued work may still use the old buffer
        if (e != hipSuccess) return hip_fail(e);
        if (ws.accum) ws.retired.push_back(ws.accum);
        ws.accum = nullptr;
        ws.words = 0;
        size_t want = words < (1u << 18) ? (1u << 18) : words;
        e = hipMalloc((void **)&ws.accum, want * sizeof(unsigned long long));
        if (e != hipSuccess) {
            g_last_hip_error = (int)e;
            return LUTGEMM_ENOMEM;
        }
        e = hipMemsetAsync(ws.accum, 0, want * sizeof(unsigned long long), stream);
        if (e != hipSuccess) return hip_fail(e);
        e = hipStreamSynchronize(stream);
        if (e != hipSuccess) return hip_fail(e);
        ws.words = want;
    }
    *out = ws.accum;
    return LUTGEMM_OK;
}

int env_int(const char *name, int fallback)
{
    const char *v = getenv(name);
    return (v && *v) ? atoi(v) : fallback;
}

// Tuning knobs (read once): LUTGEMM_TARGET_BLOCKS = workgroups a launch aims
// for (64 KiB of tables per workgroup lets two be resident per CU),
// LUTGEMM_NSTEPS = 1 or 2 output steps per workgroup.
int target_blocks()
{
    static const int v = env_int("LUTGEMM_TARGET_BLOCKS", 512);  // 2 workgroups x 256 CUs
    return v;
}
int forced_nsteps()
{
    static const int v = env_int("LUTGEMM_NSTEPS", 0);
    return v;
}

// Pick the N-tile and the K-split so that `want_blocks` workgroups exist while
// each still does enough look-ups per table built.
void plan_problem(Problem &p, int nsteps, int mrows, long want_blocks)
{
    p.n_tiles = (p.N + kStepCols * nsteps - 1) / (kStepCols * nsteps);
    p.mchunks = (p.M + mrows - 1) / mrows;
    long want = want_blocks / ((long)p.n_tiles * p.mchunks);
    if (want < 1) want = 1;
    if (want > p.nsets) want = p.nsets;
    if (want > kMaxKSplit) want = kMaxKSplit;
    p.sets_per_split = (p.nsets + (int)want - 1) / (int)want;
    // One set per workgroup leaves nothing to overlap inside it and doubles the
    // accumulator atomics; two sets cost the same time as long as one workgroup per
    // two CUs remains (4096x4096: 256 x 1 set 7.1 us, 128 x 2 sets 6.9 us).
    if (p.sets_per_split == 1 && p.nsets >= 2 && (long)p.n_tiles * ((p.nsets + 1) / 2) * p.mchunks >= 128)
        p.sets_per_split = 2;
    p.ksplit = (p.nsets + p.sets_per_split - 1) / p.sets_per_split;
    p.n_blocks = p.n_tiles * p.ksplit * p.mchunks;
}

int pick_nsteps(int N)
{
    // One step (128 outputs per workgroup) measured faster than two on every
    // shape tried: twice the workgroups to spread the stream over, and a shorter
    // tail, outweigh building each table for half as many look-ups.
    const int f = forced_nsteps();
    if (f == 1 || f == 2) return f;
    (void)N;
    return 1;
}

int pick_mrows(int M) { return M >= 3 ? 4 : M; }

template <int NB, int MODE>
int launch_nb(const Problem &p, int nsteps, int mrows, hipStream_t stream)
{
    dim3 grid((unsigned)p.n_blocks);
    dim3 block(kThreads);
    if (mrows == 4)
        hipLaunchKernelGGL((lut_gemv_kernel<NB, 1, MODE, 4>), grid, block, 0, stream, p);
    else if (mrows == 2)
        hipLaunchKernelGGL((lut_gemv_kernel<NB, 1, MODE, 2>), grid, block, 0, stream, p);
    else if (nsteps == 1)
        hipLaunchKernelGGL((lut_gemv_kernel<NB, 1, MODE, 1>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((lut_gemv_kernel<NB, 2, MODE, 1>), grid, block, 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e);
    return LUTGEMM_OK;
}

template <int MODE>
int launch_mode(const Problem &p, int nsteps, int mrows, hipStream_t stream)
{
    switch (p.nb) {
    case 1: return launch_nb<1, MODE>(p, nsteps, mrows, stream);
    case 2: return launch_nb<2, MODE>(p, nsteps, mrows, stream);
    case 3: return launch_nb<3, MODE>(p, nsteps, mrows, stream);
    case 4: return launch_nb<4, MODE>(p, nsteps, mrows, stream);
    default: return LUTGEMM_EINVAL;
    }
}

bool aligned(const void *ptr, size_t a) { return ((uintptr_t)ptr & (a - 1)) == 0; }

// Validate one problem and fill everything but the launch plan.
int fill_problem(Problem &p, int mode, const uint32_t *bW, const void *alpha, const void *qbias,
                 const void *x, void *out, int N, int K, int nb, int num_groups, int M)
{
    if (!bW || !alpha || !x || !out) return LUTGEMM_EINVAL;
    if (mode == kUniformF16 && !qbias) return LUTGEMM_EINVAL;
    if (N <= 0 || K <= 0 || M <= 0 || num_groups <= 0) return LUTGEMM_EINVAL;
    if (K % 32 != 0 || N % 4 != 0) return LUTGEMM_EINVAL;
    if (nb < 1 || nb > 4) return LUTGEMM_EINVAL;
    if (M > 65535) return LUTGEMM_EINVAL;
    if (!aligned(bW, 16) || !aligned(x, 16) || !aligned(out, 8)) return LUTGEMM_EALIGN;

    p = Problem{};
    p.W = bW;
    p.alpha = alpha;
    p.qbias = (const __half *)qbias;
    p.x = (const __half *)x;
    p.out = (__half *)out;
    p.N = N;
    p.K = K;
    p.M = M;
    p.nb = nb;
    p.kwords = K / 32;
    p.nsets = (p.kwords + kSetWords - 1) / kSetWords;
    if (mode == kRowF16 || mode == kUniformF16) {
        if (K % num_groups != 0) return LUTGEMM_EINVAL;
        const int gs = K / num_groups;
        if (gs % 32 != 0) return LUTGEMM_EINVAL;  // a sign word may not straddle two groups
        p.group_words = gs / 32;
        p.group_shift = -1;
        for (int sh = 0; sh < 20; ++sh)
            if ((1 << sh) == p.group_words) p.group_shift = sh;
        if (!aligned(alpha, 8)) return LUTGEMM_EALIGN;
        if (mode == kUniformF16 && !aligned(qbias, 8)) return LUTGEMM_EALIGN;
    } else {
        if (N % num_groups != 0) return LUTGEMM_EINVAL;
        p.R = num_groups;
        p.rows_per_group = N / num_groups;
        if (p.rows_per_group % 4 != 0) return LUTGEMM_EINVAL;
    }
    return LUTGEMM_OK;
}

int mfma_min_rows()
{
    static const int v = env_int("LUTGEMM_MFMA_MIN_M", 3);
    return v;
}

// The matrix-core path needs whole 128-input steps inside one alpha group and
// 16-output alpha runs.
bool mfma_eligible(const Problem &p, int mode)
{
    if (!(mode == kRowF16 && p.K % kMfmaStepK == 0 && p.group_words % 4 == 0 && p.N % 16 == 0 && p.N >= 16))
        return false;
    if (p.M >= mfma_min_rows()) return true;
    // two rows: the look-up kernel wins only where the sign stream is long enough to
    // hide its per-row work (measured, look-up vs matrix core: 4096x4096x3 13.4 us vs
    // 7.4; 8192x8192x4 21.8 vs 19.9; 28672x8192x2 about 30 vs 38.9; 28672x8192x4 46 vs 62)
    return p.M == 2 && mfma_min_rows() == 3 && (long)p.N * (p.K / 8) * p.nb <= (32l << 20);
}

template <int NB>
int launch_mfma_nb(const Problem &p, int mt, hipStream_t stream)
{
    dim3 grid((unsigned)p.n_blocks), block(kMfmaThreads);
    if (mt == 2)
        hipLaunchKernelGGL((lut_gemm_mfma_kernel<NB, 2>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((lut_gemm_mfma_kernel<NB, 1>), grid, block, 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e);
    return LUTGEMM_OK;
}

// K-steps are split 8 ways inside a workgroup already; across workgroups only as
// far as needed to reach `want_blocks`.
void plan_mfma(Problem &p, int mt, long want_blocks)
{
    p.n_tiles = (p.N + kMfmaTileCols - 1) / kMfmaTileCols;
    p.mchunks = (p.M + 16 * mt - 1) / (16 * mt);
    p.nsets = p.K / kMfmaStepK;  // K-steps
    long want = want_blocks / ((long)p.n_tiles * p.mchunks);
    if (want < 1) want = 1;
    if (want > p.nsets / kMfmaWaves) want = p.nsets / kMfmaWaves;
    if (want < 1) want = 1;
    if (want > kMaxKSplit) want = kMaxKSplit;
    p.sets_per_split = (p.nsets + (int)want - 1) / (int)want;
    p.sets_per_split = (p.sets_per_split + kMfmaWaves - 1) / kMfmaWaves * kMfmaWaves;  // whole rounds
    p.ksplit = (p.nsets + p.sets_per_split - 1) / p.sets_per_split;
    p.n_blocks = p.n_tiles * p.ksplit * p.mchunks;
}

// Workgroups wanted per launch: two per CU for the 16-row tile (its register count
// lets two be resident), one per CU for the 32-row tile.  Measured, 8192x8192x2:
// 16 rows 16.9 us at 256 and 15.1 at 512; 32 rows 36.4 at 256 and 40.0 at 512 (4 bits).
int mfma_blocks(int mt)
{
    static const int v = env_int("LUTGEMM_MFMA_BLOCKS", 0);
    if (v > 0) return v;
    return mt == 1 ? 512 : 256;
}

int run_mfma(Problem &p, hipStream_t stream)
{
    const int mt = p.M > 16 ? 2 : 1;
    plan_mfma(p, mt, mfma_blocks(mt));
    if (p.ksplit > 1) {
        int rc = get_workspace(stream, (size_t)p.M * p.N, &p.accum);
        if (rc != LUTGEMM_OK) return rc;
    }
    switch (p.nb) {
    case 1: return launch_mfma_nb<1>(p, mt, stream);
    case 2: return launch_mfma_nb<2>(p, mt, stream);
    case 3: return launch_mfma_nb<3>(p, mt, stream);
    case 4: return launch_mfma_nb<4>(p, mt, stream);
    default: return LUTGEMM_EINVAL;
    }
}

// All problems of a group on the matrix-core kernel in one launch (they share the
// row-tile height: all M <= 16 or all M > 16).
int run_mfma_group(Group &g, hipStream_t stream)
{
    const int mt = g.p[0].M > 16 ? 2 : 1;
    long total_bytes = 0;
    size_t words = 0;
    for (int i = 0; i < g.count; ++i) {
        total_bytes += (long)g.p[i].N * (g.p[i].K / 8) * g.p[i].nb;
        words += (size_t)g.p[i].M * g.p[i].N;
    }
    int begin = 0;
    bool any_split = false;
    for (int i = 0; i < g.count; ++i) {
        Problem &p = g.p[i];
        const long mine = (long)p.N * (p.K / 8) * p.nb;
        plan_mfma(p, mt, (long)mfma_blocks(mt) * mine / (total_bytes > 0 ? total_bytes : 1));
        p.block_begin = begin;
        begin += p.n_blocks;
        any_split = any_split || p.ksplit > 1;
    }
    if (any_split) {
        unsigned long long *base = nullptr;
        int rc = get_workspace(stream, words, &base);
        if (rc != LUTGEMM_OK) return rc;
        size_t off = 0;
        for (int i = 0; i < g.count; ++i) {
            g.p[i].accum = base + off;
            off += (size_t)g.p[i].M * g.p[i].N;
        }
    }
    const dim3 grid((unsigned)begin), block(kMfmaThreads);
    if (mt == 2)
        hipLaunchKernelGGL((lut_gemm_mfma_group_kernel<2>), grid, block, 0, stream, g);
    else
        hipLaunchKernelGGL((lut_gemm_mfma_group_kernel<1>), grid, block, 0, stream, g);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e);
    return LUTGEMM_OK;
}

int run(int mode, const uint32_t *bW, const void *alpha, const void *qbias, const void *x,
        void *out, int N, int K, int nb, int num_groups, int M, void *stream_v)
{
    Problem p;
    int rc = fill_problem(p, mode, bW, alpha, qbias, x, out, N, K, nb, num_groups, M);
    if (rc != LUTGEMM_OK) return rc;
    hipStream_t stream = (hipStream_t)stream_v;
    if (mfma_eligible(p, mode)) return run_mfma(p, stream);
    const int mrows = pick_mrows(M);
    const int nsteps = mrows > 1 ? 1 : pick_nsteps(N);
    plan_problem(p, nsteps, mrows, target_blocks());
    if (p.ksplit > 1) {
        rc = get_workspace(stream, (size_t)M * N, &p.accum);
        if (rc != LUTGEMM_OK) return rc;
    }
    if (is_block(mode) && p.rows_per_group >= kStepCols * nsteps) mode += 4;  // tile spans <= 2 row groups
    switch (mode) {
    case kBlockF16Staged: return launch_mode<kBlockF16Staged>(p, nsteps, mrows, stream);
    case kBlockShiftU16Staged: return launch_mode<kBlockShiftU16Staged>(p, nsteps, mrows, stream);
    case kBlockApotI8Staged: return launch_mode<kBlockApotI8Staged>(p, nsteps, mrows, stream);
    case kRowF16: return launch_mode<kRowF16>(p, nsteps, mrows, stream);
    case kBlockF16: return launch_mode<kBlockF16>(p, nsteps, mrows, stream);
    case kBlockShiftU16: return launch_mode<kBlockShiftU16>(p, nsteps, mrows, stream);
    case kBlockApotI8: return launch_mode<kBlockApotI8>(p, nsteps, mrows, stream);
    case kUniformF16: return launch_mode<kUniformF16>(p, nsteps, mrows, stream);
    default: return LUTGEMM_EINVAL;
    }
}

// Up to kMaxGroup row-wise problems in one launch of the look-up kernel.  Problems
// with enough rows for the matrix-core kernel (and no fused transform) are launched
// one by one on that path instead.
int run_group(int count, const lutgemm_fused_problem *problems, hipStream_t stream)
{
    Group g{};
    g.count = count;
    size_t words = 0;
    long total_bytes = 0;
    bool plain = true, all_mfma = true;
    int xform = kXNone;
    for (int i = 0; i < count; ++i) {
        const lutgemm_fused_problem &q = problems[i];
        Problem &p = g.p[i];
        int rc = fill_problem(p, kRowF16, q.bW, q.alpha_f16, nullptr, q.x_f16, q.out_f16, q.N, q.K, q.nb,
                              q.num_groups, q.M);
        if (rc != LUTGEMM_OK) return rc;
        if (q.norm_weight_f16 && q.gate_f16) return LUTGEMM_EINVAL;
        if (q.overwrite != 0 && q.overwrite != 1) return LUTGEMM_EINVAL;
        if (q.norm_weight_f16 && !(q.norm_eps >= 0.0f)) return LUTGEMM_EINVAL;
        if (!aligned(q.norm_weight_f16, 16) || !aligned(q.gate_f16, 16)) return LUTGEMM_EALIGN;
        p.norm_w = (const __half *)q.norm_weight_f16;
        p.gate = (const __half *)q.gate_f16;
        p.norm_eps = q.norm_eps;
        p.overwrite = q.overwrite;
        // one kernel instance per transform: the problems of a launch share theirs
        const int mine = p.norm_w ? kXNorm : p.gate ? kXGate : kXNone;
        if (i > 0 && mine != xform) return LUTGEMM_EUNSUP;
        xform = mine;
        plain = plain && !p.norm_w && !p.gate && !p.overwrite;
        all_mfma = all_mfma && mfma_eligible(p, kRowF16);
        words += (size_t)q.M * q.N;
        total_bytes += (long)q.N * (q.K / 8) * q.nb * q.M;
    }
    // every problem finishes its outputs with a plain read-modify-write: two problems
    // of one launch may not write the same memory
    for (int i = 0; i < count; ++i)
        for (int j = i + 1; j < count; ++j) {
            const char *a0 = (const char *)g.p[i].out, *a1 = a0 + (size_t)g.p[i].M * g.p[i].N * 2;
            const char *b0 = (const char *)g.p[j].out, *b1 = b0 + (size_t)g.p[j].M * g.p[j].N * 2;
            if (a0 < b1 && b0 < a1) return LUTGEMM_EINVAL;
        }
    // The matrix-core kernel takes plain and (as a group launch) overwriting problems.
    // Input transforms stay with the look-up kernel: there a workgroup transforms only
    // its K-slice of one row, while every 64-output workgroup of the matrix-core kernel
    // would redo the transform of all rows (measured slower than a separate kernel).
    bool same_height = true;
    for (int i = 1; i < count; ++i) same_height = same_height && ((g.p[i].M > 16) == (g.p[0].M > 16));
    if (all_mfma && xform == kXNone && same_height && (count > 1 || !plain)) return run_mfma_group(g, stream);
    if (plain && all_mfma) {
        for (int i = 0; i < count; ++i) {
            int rc = run_mfma(g.p[i], stream);
            if (rc != LUTGEMM_OK) return rc;
        }
        return LUTGEMM_OK;
    }
    // Share the launch's workgroup budget in proportion to each problem's sign
    // bytes.  The budget is what is resident at once (two workgroups on each of 256
    // CUs): a launch a little above it runs a second, mostly empty round that costs
    // as much as the first (3 x 4096x4096: 15.6 us with 768 workgroups, 10.8 with 384).
    const long budget = (long)target_blocks();
    int begin = 0;
    bool any_split = false;
    for (int i = 0; i < count; ++i) {
        Problem &p = g.p[i];
        const long mine = (long)p.N * (p.K / 8) * p.nb * p.M;
        long want = budget * mine / (total_bytes > 0 ? total_bytes : 1);
        if (want < 1) want = 1;
        plan_problem(p, 1, 1, want);
        p.block_begin = begin;
        begin += p.n_blocks;
        any_split = any_split || p.ksplit > 1;
    }
    if (any_split) {
        unsigned long long *base = nullptr;
        int rc = get_workspace(stream, words, &base);
        if (rc != LUTGEMM_OK) return rc;
        size_t off = 0;
        for (int i = 0; i < count; ++i) {
            g.p[i].accum = base + off;
            off += (size_t)g.p[i].M * g.p[i].N;
        }
    }
    const dim3 grid((unsigned)begin), block(kThreads);
    if (xform == kXNorm)
        hipLaunchKernelGGL((lut_gemv_group_kernel<1, kXNorm>), grid, block, 0, stream, g);
    else if (xform == kXGate)
        hipLaunchKernelGGL((lut_gemv_group_kernel<1, kXGate>), grid, block, 0, stream, g);
    else
        hipLaunchKernelGGL((lut_gemv_group_kernel<1, kXNone>), grid, block, 0, stream, g);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e);
    return LUTGEMM_OK;
}

}  // namespace

int lutgemm_internal_hip_fail(int hip_error) { return hip_fail((hipError_t)hip_error); }

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

int lutgemm_gemv_rowwise_f16_grouped(int count, const lutgemm_rowwise_problem *problems,
                                     void *stream_v)
{
    if (!problems || count < 1 || count > kMaxGroup) return LUTGEMM_EINVAL;
    lutgemm_fused_problem f[kMaxGroup] = {};
    for (int i = 0; i < count; ++i) {
        const lutgemm_rowwise_problem &q = problems[i];
        f[i].bW = q.bW;
        f[i].alpha_f16 = q.alpha_f16;
        f[i].x_f16 = q.x_f16;
        f[i].out_f16 = q.out_f16;
        f[i].N = q.N;
        f[i].K = q.K;
        f[i].nb = q.nb;
        f[i].num_groups = q.num_groups;
        f[i].M = q.M;
    }
    return run_group(count, f, (hipStream_t)stream_v);
}

int lutgemm_gemv_rowwise_f16_fused(int count, const lutgemm_fused_problem *problems, void *stream_v)
{
    if (!problems || count < 1 || count > kMaxGroup) return LUTGEMM_EINVAL;
    return run_group(count, problems, (hipStream_t)stream_v);
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
            if (it->second.accum) (void)hipFree(it->second.accum);
            for (unsigned long long *old : it->second.retired) (void)hipFree(old);
            it = g_workspaces.erase(it);
        } else {
            ++it;
        }
    }
    return LUTGEMM_OK;
}

}  // extern "C"
