// Matrix-core kernel templates for BCQ linear layers with several activation rows on
// MI355X (gfx950, wave64): row-wise alpha, the semantics of lut_gemm/mv_fp16_bias.hpp:
// 498-579 in the ShiftAddLLM checkout extended to M rows.
#ifndef LUT_GEMM_MFMA_DEVICE_H
#define LUT_GEMM_MFMA_DEVICE_H

#include "lutgemm_common.h"

namespace lutgemm {

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
    // flat workgroup index (relative to the problem) -> (tile, K-slice, row chunk)
    const int tile = local_block % p.n_tiles;
    const int kslice = (local_block / p.n_tiles) % p.ksplit;
    const int mchunk = local_block / (p.n_tiles * p.ksplit);
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
        const int g = fast_div(min(r0 + (a_role ? a_s : 0), p.nsets - 1) * 4, p.by_group_words);
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
    Contribution contrib[2 * MT];
    unsigned long long old[2 * MT];
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i) {
        const int ml = (tid >> 6) + 8 * i;          // row within the chunk
        const int j = src_j + (ml >> 4) * 4, sl = src_lane + (ml & 15);
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < kMfmaWaves; ++w) v += red[(w * (16 * MT) + j) * kRedRow + sl];
        val[i] = v;
        old[i] = 0;
        contrib[i] = Contribution{0ull, 0ull};
        const int m = m0 + ml;
        if (p.ksplit > 1 && m < p.M && n < p.N) {
            unsigned long long *word = p.accum + (size_t)m * p.N + n;
            contrib[i] = fixed_contribution(v);
            if (contrib[i].flags)
                __hip_atomic_fetch_or(word, contrib[i].flags, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            old[i] = __hip_atomic_fetch_add(word, contrib[i].add, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
        const float y = fixed_total((old[i] | contrib[i].flags) + contrib[i].add, p.ksplit);
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

}  // namespace lutgemm

#endif
