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
// Here the sign bits are expanded to +-alpha fp16 in registers (one VALU
// operation per two signs plus the shift that brings them into place) and
// multiplied with 16 activation rows at a time by v_mfma_f32_16x16x32_f16, fp32
// accumulation over all bit planes and groups: alpha is an fp16 number, so
// +-alpha is exact and the products are the reference's alpha * (+-x).
//
// Work split: a workgroup of 8 waves owns 64 outputs; its waves take different
// K-steps (128 inputs = 4 sign words, inside one alpha group) and their
// accumulators meet in LDS at the end, so that the number of cross-workgroup
// atomics does not grow with the K parallelism.  Lane l (li = l&15, kb = l>>4)
// loads the four sign words of outputs n = base + 4*li .. +3 for word kb of its
// step (256-byte runs per row).  MFMA instance (e, beta) takes from every lane 8
// signs of its word e: bits 4*beta+i and 16+4*beta+i, i < 4 -- two bits 16 apart
// land in the sign positions of a packed fp16 pair with ONE shift and ONE
// three-input bit operation.  So the instance's A rows are outputs base + 4*i + e
// and its K block kb is word kb.
//
// Nothing is staged through LDS in the main loop and there is no barrier in it: a
// lane's B operands of a step are the 32 activations of row li under its word kb,
// 64 contiguous bytes that it loads itself (L2 hits: the activations are M*K*2
// bytes in all), and instance beta's operand is halves 4*beta+i and 16+4*beta+i of
// them, paired like the signs by four byte permutes.  Each wave runs its own
// two-deep pipeline of (signs, alphas, activations) and the waves of a workgroup
// drift freely until the final reduction.
// ---------------------------------------------------------------------------
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kMfmaThreads = 512;
constexpr int kMfmaWaves = kMfmaThreads / 64;
constexpr int kMfmaTileCols = 64;     // outputs per workgroup
constexpr int kMfmaStepK = 128;
constexpr int kRedRow = 65;           // the final reduction's LDS rows, padded against bank conflicts
template <int MT>
constexpr int kMfmaRedBytes = kMfmaWaves * 16 * MT * kRedRow * 4;
// POW2 instances keep a 64 KiB table in front (sign byte -> eight 4-bit floats, see mfma_tile); the
// final reduction takes its place afterwards, the rows' reciprocal RMS sit behind both.
constexpr int kSignLutBytes = 256 * 64 * 4;   // 256 entries x 64 copies: copy l for lane l, one bank per lane of a half-wave
template <int MT, bool POW2 = false>
constexpr int kMfmaScaleOffset = (POW2 && kSignLutBytes > kMfmaRedBytes<MT>) ? kSignLutBytes : kMfmaRedBytes<MT>;
template <int MT, bool POW2 = false>
constexpr int kMfmaLdsBytes = kMfmaScaleOffset<MT, POW2> + 16 * MT * 4;

// Operands of one K-step of a wave: per bit plane word kb of 4 outputs; the alphas of
// those 4 outputs for bit plane kb (one load covers all planes: lane group kb of the wave
// takes plane kb, and hands them to the other groups by lane permutes when the plane's
// turn comes); per 16-row tile the lane's 32 activations.
template <int NB, int MT>
struct MfmaOperands {
    u32x4 w[NB];
    u32x2 alpha;
    u32x4 x[MT][4];
};

template <int NB, int MT>
__device__ __forceinline__ void mfma_load(MfmaOperands<NB, MT> &r, const Problem &p, int step, int kb, uint32_t wcol4,
                                          const __half *const (&xlane)[MT])
{
    const uint32_t row_bytes = (uint32_t)p.N * 4u;
    const char *wbase = (const char *)p.W + (size_t)step * 4 * NB * row_bytes;
    const uint32_t wrow = (uint32_t)kb * (NB * row_bytes);
#pragma unroll
    for (int b = 0; b < NB; ++b)
        r.w[b] = __builtin_nontemporal_load((const u32x4 *)(wbase + (size_t)b * row_bytes + (wrow + wcol4)));
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int c = 0; c < 4; ++c) r.x[mt][c] = *(const u32x4 *)(xlane[mt] + step * kMfmaStepK + 8 * c);
    const int g = fast_div(step * 4, p.by_group_words);
    const char *abase = (const char *)p.alpha + (size_t)g * NB * (p.N * 2u) + (wcol4 >> 1);
    r.alpha = *(const u32x2 *)(abase + (size_t)min(kb, NB - 1) * (p.N * 2u));
}

// 8 signs of sign word `w` -> 8 fp16 values +-alpha (bit set = +alpha): pair i holds
// bit 4*beta+i (low half) and bit 16+4*beta+i (high half).  `alpha2` is the output's
// alpha in both halves; the sign rides on it, so the matrix cores multiply and add
// alpha * sign * x directly and no per-plane scaling of partial sums is left over.
__device__ __forceinline__ f16x8 expand_signs(uint32_t w, int beta, uint32_t alpha2)
{
    // (~shifted & 0x80008000) ^ alpha2 as ONE three-input bit operation (truth table
    // 0xa6 = (~a & b) ^ c); the compiler otherwise emits not + and + xor.
    const uint32_t sign = 0x80008000u;
    u32x4 r;
    r.x = __builtin_amdgcn_bitop3_b32(w << (15 - (4 * beta + 0)), sign, alpha2, 0xa6);
    r.y = __builtin_amdgcn_bitop3_b32(w << (15 - (4 * beta + 1)), sign, alpha2, 0xa6);
    r.z = __builtin_amdgcn_bitop3_b32(w << (15 - (4 * beta + 2)), sign, alpha2, 0xa6);
    r.w = __builtin_amdgcn_bitop3_b32(w << (15 - (4 * beta + 3)), sign, alpha2, 0xa6);
    return __builtin_bit_cast(f16x8, r);
}

// xs: kMfmaLdsBytes<MT, POW2> bytes of LDS for the final reduction (and, behind them, the
// reciprocal RMS of the tile's rows).
// EXTRA: the launch honours the split-RMSNorm fields of the problem (next_in, sumsq_*).
// ONE: every K-slice of the launch is a single round, i.e. a wave takes at most one step (the
//      host's choice): nothing is requested beyond that step.
// POW2: the caller promises that every alpha is a positive normal fp16 power of two.  Sign bits then
//      become fp16 +-alpha without the per-pair shift and bit operation: a byte of the sign word
//      (eight signs) indexes a table in LDS whose entries hold eight 4-bit floats +-1 (e2m1 codes
//      0x2 / 0xA), and v_cvt_scalef32_pk_f16_fp4 turns two of them into a packed fp16 pair times a
//      scale of which the hardware uses the exponent only (measured: scale 3.0 gives +-2), which for
//      a power of two is the alpha itself.  One table read and four conversions per matrix
//      instruction instead of eight vector operations, the eight signs come out in input order, so
//      the activations need no permutes either.
template <int NB, int MT, bool EXTRA = false, bool ONE = false, bool POW2 = false>
__device__ __forceinline__ void mfma_tile(const Problem &p, int local_block, char *xs)
{
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

    // the lane's activations: row li of each 16-row tile (rows beyond M are clamped to
    // the last one: computed twice, written once), the 32 inputs under word kb
    const __half *xlane[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xlane[mt] = p.x + (size_t)min(m0 + 16 * mt + li, p.M - 1) * p.K + 32 * kb;

    // split RMSNorm, consuming side: wave w sums the slots of rows w, w + 8, ... and leaves
    // their reciprocal RMS in LDS for the hand-over
    // The slots are requested here, ahead of everything else, and summed once the first
    // step's operands have been requested behind them (see the main loop): loads return in
    // order, so that wait is for the slots alone.
    float *row_scale = (float *)(xs + kMfmaScaleOffset<MT, POW2>);
    typedef float f32x4v __attribute__((ext_vector_type(4)));
    constexpr int kScaleRows = 2 * MT;  // rows per wave
    bool scaled = false;
    [[maybe_unused]] f32x4v slot4[kScaleRows];
    // (the wave index as a scalar, so that the rows' addresses are a scalar base plus one lane offset)
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    if constexpr (EXTRA) {
        scaled = p.sumsq_in != nullptr;
        if (scaled) {
            // one 16-byte request per row and lane: 256 slots, inputs up to 8192 (slots = K / 32
            // and K % 128 == 0 on this path)
            const int quads = p.sumsq_slots >> 2;
#pragma unroll
            for (int i = 0; i < kScaleRows; ++i) {
                const float *slots = p.sumsq_in + (size_t)min(m0 + wave_s + kMfmaWaves * i, p.M - 1) * p.sumsq_slots;
                slot4[i] = *((const f32x4v *)slots + min(lane, quads - 1));
            }
        }
    }
    auto row_scales = [&]() {
        const int quads = p.sumsq_slots >> 2;
#pragma unroll
        for (int i = 0; i < kScaleRows; ++i) {
            const int row = wave_s + kMfmaWaves * i;
            const float *slots = p.sumsq_in + (size_t)min(m0 + row, p.M - 1) * p.sumsq_slots;
            float t = lane < quads ? (slot4[i].x + slot4[i].y) + (slot4[i].z + slot4[i].w) : 0.0f;
            for (int c = 4 * 64 + lane; c < p.sumsq_slots; c += 64) t += slots[c];  // inputs beyond 8192
            t = wave_sum(t);
            if (lane == 0) row_scale[row] = rsqrtf(t / (float)p.K + p.norm_eps);
        }
    };

    f32x4 acc[4][MT];
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[e][mt] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};

    // POW2: the sign table.  Entry i, copy c at byte i * 256 + 4 * c; lane l reads copy l, so one
    // v_perm_b32 of (sign word, per-lane constant) is the address: index byte in bits 8..15, the
    // lane's copy offset in bits 0..7.
    [[maybe_unused]] const uint32_t lane_off = (uint32_t)(4 * lane) * 0x01010101u;
    if constexpr (POW2) {
        uint32_t *lut = (uint32_t *)xs;
#pragma unroll 4
        for (int idx = tid; idx < kSignLutBytes / 4; idx += kMfmaThreads) {   // a wave writes one entry's 64 copies
            // (the entry index is the same for the whole wave: scalar arithmetic)
            uint32_t v = (uint32_t)__builtin_amdgcn_readfirstlane(idx >> 6);   // bit j of it -> bit 4 * j + 3
            v = (v | (v << 12)) & 0x000f000fu;
            v = (v | (v << 6)) & 0x03030303u;
            v = (v | (v << 3)) & 0x11111111u;
            lut[idx] = 0xaaaaaaaau ^ (v << 3);
        }
        __syncthreads();
    }

    auto compute = [&](const MfmaOperands<NB, MT> &ops) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const uint32_t w4[4] = {ops.w[b].x, ops.w[b].y, ops.w[b].z, ops.w[b].w};
            const int from = 4 * (16 * b + li);   // the lane of group b that holds this lane's outputs
            const u32x2 al = {(uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)ops.alpha.x),
                              (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)ops.alpha.y)};
            if constexpr (POW2) {
                // the alpha of output e as the conversion's fp32 scale
                const float scale[4] = {half_bits_to_float(al.x & 0xffffu), half_bits_to_float(al.x >> 16),
                                        half_bits_to_float(al.y & 0xffffu), half_bits_to_float(al.y >> 16)};
                constexpr uint32_t sel[4] = {0x0c0c0400u, 0x0c0c0501u, 0x0c0c0602u, 0x0c0c0703u};
#pragma unroll
                for (int beta = 0; beta < 4; ++beta) {
                    // byte beta of the sign word = inputs 8 * beta .. + 7 of the lane's 32, in order
                    f16x8 bx[MT];
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) bx[mt] = __builtin_bit_cast(f16x8, ops.x[mt][beta]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t nib = *(const uint32_t *)(xs + __builtin_amdgcn_perm(w4[e], lane_off, sel[beta]));
                        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
                        const f16x2 p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(nib, scale[e], 0);
                        const f16x2 p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(nib, scale[e], 1);
                        const f16x2 p2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(nib, scale[e], 2);
                        const f16x2 p3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(nib, scale[e], 3);
                        const f16x8 a = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt)
                            acc[e][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bx[mt], acc[e][mt], 0, 0, 0);
                    }
                }
                continue;
            }
            // the alpha of output e in both halves of a register
            const uint32_t a2[4] = {__builtin_amdgcn_perm(al.x, al.x, 0x01000100u), __builtin_amdgcn_perm(al.x, al.x, 0x03020302u),
                                    __builtin_amdgcn_perm(al.y, al.y, 0x01000100u), __builtin_amdgcn_perm(al.y, al.y, 0x03020302u)};
#pragma unroll
            for (int beta = 0; beta < 4; ++beta) {
                f16x8 bx[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    // halves 4*beta+i and 16+4*beta+i of the lane's 32 activations, interleaved
                    // like the sign pairs
                    const u32x4 lo4 = ops.x[mt][beta >> 1], hi4 = ops.x[mt][2 + (beta >> 1)];
                    const uint32_t lo0 = (beta & 1) ? lo4.z : lo4.x, lo1 = (beta & 1) ? lo4.w : lo4.y;
                    const uint32_t hi0 = (beta & 1) ? hi4.z : hi4.x, hi1 = (beta & 1) ? hi4.w : hi4.y;
                    u32x4 v;
                    v.x = __builtin_amdgcn_perm(hi0, lo0, 0x05040100u);
                    v.y = __builtin_amdgcn_perm(hi0, lo0, 0x07060302u);
                    v.z = __builtin_amdgcn_perm(hi1, lo1, 0x05040100u);
                    v.w = __builtin_amdgcn_perm(hi1, lo1, 0x07060302u);
                    bx[mt] = __builtin_bit_cast(f16x8, v);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const f16x8 a = expand_signs(w4[e], beta, a2[e]);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc[e][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bx[mt], acc[e][mt], 0, 0, 0);
                }
            }
        }
    };

    // This wave's steps: step_begin + wave, + 8, ...  Two operand buffers alternate and
    // each step's loads are issued one compute phase ahead.  Steps are taken in pairs by
    // a counted loop with one load site per buffer (a second site makes the register
    // allocator reconcile the two with copies that wait for the loads): the first
    // iteration skips its first compute at run time, and a load beyond the wave's last
    // step re-reads that last step (the lines the wave has just asked for) and is
    // discarded, so that the waits can count it.
    MfmaOperands<NB, MT> opA, opB;
    const int last_step = p.nsets - 1;
    const int first_step = step_begin + wave;
    const int n_steps = first_step < step_end ? (step_end - first_step + kMfmaWaves - 1) / kMfmaWaves : 0;
    const int own_last = n_steps > 0 ? first_step + kMfmaWaves * (n_steps - 1) : last_step;
    const int pairs = ONE ? 0 : (n_steps + 1) / 2;
    if constexpr (ONE) {
        // One round per slice: the general loop would request a second, discarded step behind
        // the first one, and a wave cannot end before those loads have come back.
        mfma_load<NB, MT>(opA, p, min(first_step, last_step), kb, wcol4, xlane);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (EXTRA)
            if (scaled) row_scales();
        __builtin_amdgcn_sched_barrier(0);
        if (n_steps > 0) compute(opA);
    }
#pragma clang loop unroll(disable)
    for (int j = 0; j < pairs; ++j) {
        // (opaque, which keeps the compiler from peeling the first iteration)
        int first = __builtin_amdgcn_readfirstlane(j == 0);
        asm volatile("" : "+s"(first));
        const int s = first_step + 2 * kMfmaWaves * j;
        mfma_load<NB, MT>(opA, p, min(s, own_last), kb, wcol4, xlane);
        __builtin_amdgcn_sched_barrier(0);
        if (!first) compute(opB);
        if constexpr (EXTRA)
            if (first && scaled) row_scales();
        __builtin_amdgcn_sched_barrier(0);
        mfma_load<NB, MT>(opB, p, min(s + kMfmaWaves, own_last), kb, wcol4, xlane);
        __builtin_amdgcn_sched_barrier(0);
        compute(opA);
    }
    if (!ONE && n_steps > 0 && (n_steps & 1) == 0) compute(opB);
    if constexpr (EXTRA && !ONE)
        if (n_steps == 0 && scaled) row_scales();  // (a wave without steps still owes its rows)

    // ---- the 8 waves' accumulators meet in LDS -----------------------------------
    // red[wave][j = (e*MT + mt)*4 + r][lane], rows padded to 65 words so that the
    // read-out below (consecutive threads = consecutive outputs) spreads over the banks
    if constexpr (POW2) __syncthreads();   // (the table's memory: every wave is done with it)
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
    [[maybe_unused]] float next_w = 0.0f;
    if constexpr (EXTRA)
        if (p.next_w) next_w = __half2float(p.next_w[min(n, p.N - 1)]);
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
        if (scaled) v *= row_scale[ml];
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
        [[maybe_unused]] float sq = 0.0f;  // square of the output this thread completed
        if (m < p.M && n < p.N && (p.ksplit == 1 || (int)(old[i] >> 56) == p.ksplit - 1)) {
            __half *dst = p.out + (size_t)m * p.N + n;
            const float y = p.ksplit == 1 ? val[i] : fixed_total((old[i] | contrib[i].flags) + contrib[i].add, p.ksplit);
            const __half y16 = __float2half_rn((p.overwrite ? 0.0f : __half2float(*dst)) + y);
            *dst = y16;
            if (p.ksplit > 1)
                __hip_atomic_store(p.accum + (size_t)m * p.N + n, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if constexpr (EXTRA) {
                const float yf = __half2float(y16);
                sq = yf * yf;
                if (p.next_in) p.next_in[(size_t)m * p.N + n] = __float2half_rn(yf * next_w);
            }
        }
        if constexpr (EXTRA) {
            // the wave's 64 columns of row m: one add into the first of their two slots
            if (p.sumsq_out) {
                const float s = wave_sum(sq);
                if (lane == 0 && m < p.M && s != 0.0f)
                    unsafeAtomicAdd(p.sumsq_out + (size_t)m * (p.N / 32) + n_base / 32, s);
            }
        }
    }
}

template <int NB, int MT, bool ONE = false, bool POW2 = false>
__global__ void __launch_bounds__(kMfmaThreads) lut_gemm_mfma_kernel(const Problem p)
{
    __shared__ __attribute__((aligned(16))) char xs[kMfmaLdsBytes<MT, POW2>];
    mfma_tile<NB, MT, false, ONE, POW2>(p, (int)blockIdx.x, xs);
}

// One problem with the split-RMSNorm fields honoured.
template <int NB, int MT, bool ONE = false>
__global__ void __launch_bounds__(kMfmaThreads) lut_gemm_mfma_fused_kernel(const Problem p)
{
    __shared__ __attribute__((aligned(16))) char xs[kMfmaLdsBytes<MT>];
    mfma_tile<NB, MT, true, ONE>(p, (int)blockIdx.x, xs);
}

// Several problems in one launch; bit widths may differ.
template <int MT>
__global__ void __launch_bounds__(kMfmaThreads) lut_gemm_mfma_group_kernel(const Group g)
{
    __shared__ __attribute__((aligned(16))) char xs[kMfmaLdsBytes<MT>];
    // grid = (workgroups of the largest problem, problems)
    // (through the constant address space, which the kernel arguments live in: the fields are
    // then scalar loads that may be repeated at will instead of values to keep in registers)
    const Problem &p = *(const Problem *)((const __attribute__((address_space(4))) Problem *)&g.p[0] + blockIdx.y);
    const int b = blockIdx.x;
    if (b >= p.n_blocks) return;
    switch (p.nb) {
    case 1: mfma_tile<1, MT, true>(p, b, xs); break;
    case 2: mfma_tile<2, MT, true>(p, b, xs); break;
    case 3: mfma_tile<3, MT, true>(p, b, xs); break;
    default: mfma_tile<4, MT, true>(p, b, xs); break;
    }
}

}  // namespace lutgemm

#endif
