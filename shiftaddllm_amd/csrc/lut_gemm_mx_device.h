// Block-scaled matrix-core kernel templates for BCQ linear layers whose alphas are powers of two,
// with several activation rows, on MI355X (gfx950, wave64): the semantics of
// lut_gemm/mv_fp16_bias.hpp:498-579 in the ShiftAddLLM checkout extended to M rows.
//
// ShiftAddLLM's alphas are powers of two: multiplying by one is a shift.  gfx950's block-scaled
// matrix instruction (v_mfma_scale_f32_16x16x128_f8f6f4) takes exactly that as an operand: one
// power-of-two scale (an exponent byte) per row and per block of 32 inputs, applied inside the
// matrix core.  So here
//   * a sign bit becomes a 4-bit float +-1 (e2m1 codes 0x2 / 0xA): eight signs = one byte of the
//     sign word = one 32-bit table entry, one LDS read per eight signs instead of a vector
//     instruction per sign (which is what bounds the fp16 matrix-core kernel);
//   * the alpha of (output, bit plane, group) rides as the A-side block scale: its fp16 exponent
//     field plus 112 is the exponent byte, no multiplication anywhere;
//   * the activations are split ahead of the launch into three 8-bit floats (e4m3) per value with
//     a power-of-two scale per block of 32: x = s * (p1 + p2 / 16 + p3 / 256) holds exactly for
//     every fp16 value within 2^14 of its block's largest one (three times four significant bits
//     cover fp16's eleven), so the products are the reference's alpha * (+-x) as before and the
//     fp32 accumulation is the matrix core's.
// The instruction has 16 columns for the activations.  With up to 5 rows the three pieces of all rows
// sit side by side in ONE instruction's columns (piece q of row m in column 5 * q + m, each column
// with its own scale) and the pieces' partial sums are added at the end; with up to 8 rows two
// instructions hold them (pieces 0 and 1, then piece 2 beside eight columns of zeros), with up to 16
// rows three.  Matrix instructions take about the same time whatever their format and depth when
// every CU issues them (measured: 16 ns for v_mfma_f32_16x16x32_f16, 17 to 20 ns for this one), so
// what counts is their number: per (bit plane, 16 outputs, 128 inputs) one, two or three here
// against four of the fp16 instruction, which also needs 128 vector instructions of sign expansion.
//
// Operand layout of the instruction (measured on the device, not documented here elsewhere):
//   A (4-bit): lane l holds row l % 16, inputs 32 * (l / 16) .. + 31, eight per register, low
//              nibble first;
//   B (8-bit): lane l holds column l % 16; bytes 0..15 are inputs 16 * (l / 16) .. + 15, bytes
//              16..31 inputs 64 + 16 * (l / 16) .. + 15;
//   scales:    byte `opsel` of the scale register of lane l applies to row (column) l % 16 and to
//              inputs 32 * (l / 16) .. + 31, wherever the operand layout keeps them;
//   D:         lane l holds column l % 16, rows 4 * (l / 16) + r in register r.
#ifndef LUT_GEMM_MX_DEVICE_H
#define LUT_GEMM_MX_DEVICE_H

#include <type_traits>
#include <utility>

#include "lut_gemm_mfma_device.h"

namespace lutgemm {

typedef int i32x8 __attribute__((ext_vector_type(8)));

constexpr int kMxPieces = 3;
constexpr int kMxLutBytes = 256 * 256;   // 256 entries x 64 copies x 4 bytes: copy l % 64 for lane l, one bank each

// ---- activations: fp16 -> three e4m3 pieces and a scale word per block of 32 ---------------------
// Eight threads per (row, block of 32 consecutive inputs).  The pieces of a 128-input step are stored
// in the order the B operand wants them (see above): the bytes a lane loads are contiguous.
//   pieces: [3][M][K] bytes; within each 128-input step, block q's inputs 0..15 go to byte
//           32 * (2 * (q & 1)) + 16 * (q >> 1), its inputs 16..31 to byte 32 * (2 * (q & 1) + 1) + 16 * (q >> 1);
//           behind them one row of K zero bytes;
//   scales: [M][K / 32] words: byte j = exponent byte of piece j (s, s - 4, s - 8), byte 3 = 0.
__device__ __forceinline__ uint32_t e4m3_encode(float v, float *decoded)
{
    // round to nearest even onto the e4m3 grid (|v| <= 256 here); returns the code, leaves the value
    const uint32_t bits = __builtin_bit_cast(uint32_t, v);
    const uint32_t sign = (bits >> 24) & 0x80u;
    const uint32_t mag = bits & 0x7fffffffu;
    if (mag < 0x3c800000u) {  // below 2^-6: multiples of 2^-9
        const float q = rintf(__builtin_bit_cast(float, mag) * 512.0f);
        *decoded = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, q * (1.0f / 512.0f)) | (bits & 0x80000000u));
        return sign | (uint32_t)q;          // (q == 8 is the smallest normal: the same code)
    }
    // keep three mantissa bits: add half of the last kept place (less one, plus the kept place's own
    // bit: ties to even), cut the rest; a carry runs into the exponent as it should
    const uint32_t rounded = (mag + 0x7ffffu + ((mag >> 20) & 1u)) & 0xfff00000u;
    *decoded = __builtin_bit_cast(float, rounded | (bits & 0x80000000u));
    return sign | ((rounded >> 20) - (120u << 3));   // exponent field: fp32's less 127 plus 7
}

// Eight threads per block of 32 (four values each); the block's largest magnitude is found across
// the eight by lane exchanges.
__global__ void __launch_bounds__(256) mx_split_kernel(const __half *__restrict__ x, unsigned char *__restrict__ pieces,
                                                       uint32_t *__restrict__ scales, int M, int K)
{
    const uint32_t blocks_per_row = (uint32_t)K / 32u;
    const uint32_t id = blockIdx.x * 256u + threadIdx.x;
    const uint32_t total = (uint32_t)M * blocks_per_row * 8u;   // (the host keeps M * K below 2^31)
    const uint32_t cid = id < total ? id : total - 1u;   // (clamped: the lane exchanges below need every lane)
    const int part = (int)(cid & 7u);
    const uint32_t bid = cid >> 3;
    const int m = (int)(bid / blocks_per_row), blk = (int)(bid % blocks_per_row);
    const int step = blk >> 2, q = blk & 3;
    const u32x2 w = *(const u32x2 *)(x + (size_t)m * K + 32 * blk + 4 * part);
    const uint32_t h[4] = {w.x & 0xffffu, w.x >> 16, w.y & 0xffffu, w.y >> 16};
    // largest magnitude as fp16 bits (they order like the values; NaN and inf on top)
    uint32_t mxbits = max(max(h[0] & 0x7fffu, h[1] & 0x7fffu), max(h[2] & 0x7fffu, h[3] & 0x7fffu));
    mxbits = max(mxbits, (uint32_t)__shfl_xor((int)mxbits, 1));
    mxbits = max(mxbits, (uint32_t)__shfl_xor((int)mxbits, 2));
    mxbits = max(mxbits, (uint32_t)__shfl_xor((int)mxbits, 4));
    // Scale 2^(e - 7) for a largest value in [2^e, 2^(e+1)): scaled values stay below 256.  A block of
    // zeros takes the smallest scale; an infinity or NaN in the block poisons its scale word (exponent
    // byte 255 = NaN), so every output the block's row reaches comes out NaN.
    const bool finite = mxbits < 0x7c00u;
    int e = -24;
    if (finite && mxbits != 0u) e = (int)((__builtin_bit_cast(uint32_t, half_bits_to_float(mxbits)) >> 23) & 0xffu) - 127;
    int sb = e - 7 + 127;           // exponent byte of piece 0
    if (sb < 9) sb = 9;             // (keeps the bytes of pieces 1 and 2 at 1 or more)
    const float inv = __builtin_bit_cast(float, (uint32_t)(254 - sb) << 23);   // 2^(127 - sb)
    uint32_t code[kMxPieces] = {0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float r = finite ? half_bits_to_float(h[i]) * inv : 0.0f;   // exact: a power of two
#pragma unroll
        for (int pc = 0; pc < kMxPieces; ++pc) {
            float dec;
            code[pc] |= e4m3_encode(r, &dec) << (8 * i);
            r = (r - dec) * 16.0f;              // the next piece's scale is 2^-4 of this one's
        }
    }
    // (a row of zeros behind the pieces: the source of matrix-instruction columns that hold nothing)
    if (id < (uint32_t)K / 16u) *(u32x4 *)(pieces + (size_t)kMxPieces * M * K + 16u * id) = (u32x4){0u, 0u, 0u, 0u};
    if (id >= total) return;
    const size_t row = (size_t)m * K + (size_t)step * 128;
    // block q's values 0..15 go to byte 32 * (2 * (q & 1)) + 16 * (q >> 1), its values 16..31 32 bytes on
    const int at = 32 * (2 * (q & 1) + (part >> 2)) + 16 * (q >> 1) + 4 * (part & 3);
#pragma unroll
    for (int pc = 0; pc < kMxPieces; ++pc) *(uint32_t *)(pieces + (size_t)pc * M * K + row + at) = code[pc];
    if (part == 0)
        scales[(size_t)m * blocks_per_row + blk] =
            finite ? ((uint32_t)sb | ((uint32_t)(sb - 4) << 8) | ((uint32_t)(sb - 8) << 16)) : 0x00ffffffu;
}

// ---- the kernel ---------------------------------------------------------------------------------
static_assert(kMxLutBytes >= kMfmaRedBytes<1> + 16 * 4, "the final reduction reuses the table's memory");

// Operands that come from HBM, for U K-steps (128 inputs each) of a wave: per bit plane word kb of 4
// outputs, and the alphas of those 4 outputs for bit plane kb (one load covers all planes: lane group
// kb of the wave takes plane kb).
template <int NB, int U>
struct MxOperands {
    u32x4 w[U][NB];
    u32x2 alpha[U];
};

// The lane's share of the activations of one K-step: per matrix instruction J of a (bit plane, 16
// outputs) the 32 values of the lane's column (a piece of a row, or zeros) and their exponent byte
// (L2 hits).
template <int NMF>
struct MxX {
    u32x4 x[NMF][2];
    uint32_t xs[NMF];
};

struct MxActivations {
    const unsigned char *pieces;   // [3][M][K], then K zero bytes
    const uint32_t *scales;        // [M][K / 32]
};

template <int NB>
__device__ __forceinline__ void mx_load_step(u32x4 (&w)[NB], u32x2 &alpha, const Problem &p, int step, int kb, uint32_t wcol4)
{
    const uint32_t row_bytes = (uint32_t)p.N * 4u;
    const char *wbase = (const char *)p.W + (size_t)step * 4 * NB * row_bytes;
    const uint32_t wrow = (uint32_t)kb * (NB * row_bytes);
#pragma unroll
    for (int b = 0; b < NB; ++b)
        w[b] = __builtin_nontemporal_load((const u32x4 *)(wbase + (size_t)b * row_bytes + (wrow + wcol4)));
    const int g = fast_div(step * 4, p.by_group_words);
    const char *abase = (const char *)p.alpha + (size_t)g * NB * (p.N * 2u) + (wcol4 >> 1);
    alpha = *(const u32x2 *)(abase + (size_t)min(kb, NB - 1) * (p.N * 2u));
}

template <int OA, int OB>
__device__ __forceinline__ f32x4 mx_mfma(const i32x8 &a, const i32x8 &b, const f32x4 &c, int scale_a, int scale_b)
{
    // A: 4-bit floats (cbsz 4), B: 8-bit floats e4m3 (blgp 0); byte OA of scale_a, byte OB of scale_b
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 4, 0, OA, scale_a, OB, scale_b);
}

template <int... Is, class F>
__device__ __forceinline__ void mx_static_for(std::integer_sequence<int, Is...>, F &&f)
{
    (f(std::integral_constant<int, Is>{}), ...);
}

// Flat workgroup index (relative to the problem) -> (row chunk, unit = tile and K-slice).  The row
// chunks of a unit stream the same sign words: they sit 8 workgroups apart, which puts them on the
// same XCD (workgroups go to the 8 XCDs in turn) and so behind the same L2.
__device__ __forceinline__ void mx_decode_block(const Problem &p, int local_block, int &mchunk, int &unit)
{
    const int units = p.n_tiles * p.ksplit;
    const int span = 8 * p.mchunks;
    const int g = local_block / span, r = local_block - g * span;
    const int width = min(8, units - 8 * g);   // (the last group may hold fewer than 8 units)
    mchunk = r / width;
    unit = 8 * g + (r - mchunk * width);
}

// xs: kMxLutBytes of LDS: the sign table during the main loop, the final reduction afterwards.
// A workgroup of 8 waves owns 64 outputs, up to MP activation rows (5, 8 or 16) and a K-slice; its
// waves take different K-steps of the slice.
template <int NB, int MP>
__device__ __forceinline__ void mx_tile(const Problem &p, const MxActivations &act, int local_block, char *xs)
{
    constexpr int NMF = MP <= 5 ? 1 : MP == 8 ? 2 : 3;   // matrix instructions per (bit plane, 16 outputs, K-step)
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int li = lane & 15;
    const int kb = lane >> 4;
    int mchunk, unit;
    mx_decode_block(p, local_block, mchunk, unit);
    const int tile = unit % p.n_tiles;
    const int kslice = unit / p.n_tiles;
    const int m0 = mchunk * MP;
    const int n_base = tile * kMfmaTileCols;
    const uint32_t wcol4 = (uint32_t)min(n_base + 4 * li, p.N - 4) * 4u;
    const int step_begin = kslice * p.sets_per_split;
    const int step_end = min(step_begin + p.sets_per_split, p.nsets);

    // ---- the sign table: byte -> eight 4-bit floats, +1 (0x2) where the bit is set, -1 (0xA) where not;
    // entry i, copy c at byte i * 256 + 4 * c; lane l reads copy l (one bank per lane of a half-wave)
    {
        uint32_t *lut = (uint32_t *)xs;
#pragma unroll 4
        for (int idx = tid; idx < kMxLutBytes / 4; idx += kMfmaThreads) {   // a wave writes one entry's 64 copies
            // (the entry index is the same for the whole wave: scalar arithmetic)
            uint32_t v = (uint32_t)__builtin_amdgcn_readfirstlane(idx >> 6);   // bit j of it -> bit 4 * j + 3
            v = (v | (v << 12)) & 0x000f000fu;
            v = (v | (v << 6)) & 0x03030303u;
            v = (v | (v << 3)) & 0x11111111u;
            lut[idx] = 0xaaaaaaaau ^ (v << 3);
        }
    }

    // The lane's column li of matrix instruction J holds piece (16 * J + li) / MP of row
    // (16 * J + li) % MP of the chunk (rows beyond M are clamped: computed twice, never read), or zeros
    // where that piece number is 3 or more.
    const unsigned char *xcol[NMF];
    const unsigned char *scol[NMF];
#pragma unroll
    for (int J = 0; J < NMF; ++J) {
        const int v = 16 * J + li;
        const int piece = v / MP, mrow = min(m0 + v % MP, p.M - 1);
        const size_t piece_stride = (size_t)p.M * p.K;
        xcol[J] = act.pieces + (piece < kMxPieces ? (size_t)piece * piece_stride + (size_t)mrow * p.K : (size_t)kMxPieces * piece_stride) +
                  32 * kb;
        scol[J] = (const unsigned char *)(act.scales + (size_t)mrow * (p.K / 32) + kb) + min(piece, kMxPieces - 1);
    }
    auto load_x = [&](MxX<NMF> &r, int J, int step) {
        const u32x4 *src = (const u32x4 *)(xcol[J] + (size_t)step * kMfmaStepK);
        r.x[J][0] = src[0];
        r.x[J][1] = src[1];
        r.xs[J] = scol[J][(size_t)step * 16];
    };

    f32x4 acc[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};

    // per-lane look-up constants: v_perm_b32 puts byte j of the sign word into bits 8..15 and the lane's
    // copy offset into bits 0..7
    const uint32_t lane_off = (uint32_t)(4 * lane) * 0x01010101u;
    const uint32_t sel[4] = {0x0c0c0400u, 0x0c0c0501u, 0x0c0c0602u, 0x0c0c0703u};
    const char *lut_bytes = xs;
    __syncthreads();

    // This wave's steps: step_begin + wave, + 8, ...: own step t is K-step first_step + 8 * t.
    const int first_step = step_begin + wave;
    const int n_steps = first_step < step_end ? (step_end - first_step + kMfmaWaves - 1) / kMfmaWaves : 0;
    auto step_of = [&](int t) { return min(first_step + kMfmaWaves * min(t, n_steps - 1), p.nsets - 1); };

    // One K-step: per bit plane the four sign words become four A operands (sixteen table reads), then
    // each of them meets the NMF operands of activations: 4 * NMF matrix instructions on four
    // independent accumulators.  The alphas' exponent bytes (fp16 exponent field + 112: 2^(field - 15) =
    // 2^(byte - 127)) of the lane's four outputs are packed into one register by the lane group that
    // loaded the plane's alphas and handed to the other groups by a lane permute; the instruction
    // picks its output's byte.  The activations live in one register set: in the last bit plane each
    // operand is re-loaded for the wave's next step as soon as its last instruction has been issued.
    constexpr int U = 1;   // steps per operand set
    auto compute = [&](const MxOperands<NB, U> &ops, MxX<NMF> &xq, int t_base) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int t = t_base + u;
            if (U > 1 && t >= n_steps) break;   // (the wave's last set may be half empty)
            const uint32_t lo = ops.alpha[u].x, hi = ops.alpha[u].y;
            const int packed = (int)((__builtin_amdgcn_ubfe(lo, 10, 5) | (__builtin_amdgcn_ubfe(lo, 26, 5) << 8) |
                                      (__builtin_amdgcn_ubfe(hi, 10, 5) << 16) | (__builtin_amdgcn_ubfe(hi, 26, 5) << 24)) +
                                     0x70707070u);
            const int next = step_of(t + 1);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const uint32_t w4[4] = {ops.w[u][b].x, ops.w[u][b].y, ops.w[u][b].z, ops.w[u][b].w};
                const int scale_a = __builtin_amdgcn_ds_bpermute(4 * (16 * b + li), packed);
                i32x8 a[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        a[e][j] = *(const int *)(lut_bytes + __builtin_amdgcn_perm(w4[e], lane_off, sel[j]));
                    a[e][4] = a[e][5] = a[e][6] = a[e][7] = 0;
                }
#pragma unroll
                for (int J = 0; J < NMF; ++J) {
                    i32x8 bv;
                    bv[0] = (int)xq.x[J][0].x;
                    bv[1] = (int)xq.x[J][0].y;
                    bv[2] = (int)xq.x[J][0].z;
                    bv[3] = (int)xq.x[J][0].w;
                    bv[4] = (int)xq.x[J][1].x;
                    bv[5] = (int)xq.x[J][1].y;
                    bv[6] = (int)xq.x[J][1].z;
                    bv[7] = (int)xq.x[J][1].w;
                    const int scale_b = (int)xq.xs[J];
                    mx_static_for(std::make_integer_sequence<int, 4>{}, [&](auto e_c) {
                        constexpr int e = decltype(e_c)::value;
                        acc[e] = mx_mfma<e, 0>(a[e], bv, acc[e], scale_a, scale_b);
                    });
                    // the next plane's table reads may move up to here, not further: only two planes'
                    // operands are live at a time
                    if (J == (NMF > 1 ? NMF - 2 : 0)) __builtin_amdgcn_sched_barrier(0);
                    if (b == NB - 1) {
                        __builtin_amdgcn_sched_barrier(0);
                        load_x(xq, J, next);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        }
    };
    auto load = [&](MxOperands<NB, U> &r, int t_base) {
#pragma unroll
        for (int u = 0; u < U; ++u) mx_load_step<NB>(r.w[u], r.alpha[u], p, step_of(t_base + u), kb, wcol4);
    };

    // Two operand sets alternate and each set's loads are issued one compute phase ahead.  Sets are
    // taken in pairs by a counted loop with one load site per set; the first iteration loads the
    // activations instead of its first compute, and a load beyond the wave's last step re-reads that
    // step and is discarded, so that the waits can count it.
    MxOperands<NB, U> opA, opB;
    MxX<NMF> xq;
    const int n_sets = (n_steps + U - 1) / U;
    const int pairs = (n_sets + 1) / 2;
#pragma clang loop unroll(disable)
    for (int j = 0; j < pairs; ++j) {
        int first = __builtin_amdgcn_readfirstlane(j == 0);
        asm volatile("" : "+s"(first));   // (opaque, which keeps the compiler from peeling the first iteration)
        load(opA, U * 2 * j);
        __builtin_amdgcn_sched_barrier(0);
        if (!first) {
            compute(opB, xq, U * (2 * j - 1));
        } else {
#pragma unroll
            for (int J = 0; J < NMF; ++J) load_x(xq, J, step_of(0));
        }
        __builtin_amdgcn_sched_barrier(0);
        load(opB, U * (2 * j + 1));
        __builtin_amdgcn_sched_barrier(0);
        compute(opA, xq, U * 2 * j);
    }
    if (n_sets > 0 && (n_sets & 1) == 0) compute(opB, xq, U * (n_sets - 1));

    // ---- the 8 waves' accumulators meet in LDS (the table's memory: every wave is done with it) -----
    __syncthreads();
    float *red = (float *)xs;
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[(wave * 16 + e * 4 + r) * kRedRow + lane] = acc[e][r];
    __syncthreads();
    // Thread t finishes output column t & 63 of rows (t >> 6) and (t >> 6) + 8 (where MP has them): a
    // wave covers 64 consecutive outputs of one row.  Row m's pieces sit in columns m, MP + m, ...
    const int nl = tid & 63;
    const int n = n_base + nl;
    const int src_lane = (nl >> 4) * 16;
    const int src_j = (nl & 3) * 4 + ((nl >> 2) & 3);
    constexpr int kRowsPerThread = MP == 16 ? 2 : 1;
    float val[kRowsPerThread];
    Contribution contrib[kRowsPerThread];
    unsigned long long old[kRowsPerThread];
    bool mine[kRowsPerThread];
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        const int ml = (tid >> 6) + 8 * i;
        const int m = m0 + ml;
        mine[i] = ml < MP && m < p.M && n < p.N;
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < kMfmaWaves; ++w)
#pragma unroll
            for (int q = 0; q < 16 / MP; ++q) v += red[(w * 16 + src_j) * kRedRow + src_lane + q * MP + min(ml, MP - 1)];
        val[i] = v;
        old[i] = 0;
        contrib[i] = Contribution{0ull, 0ull};
        if (p.ksplit > 1 && mine[i]) {
            unsigned long long *word = p.accum + (size_t)m * p.N + n;
            contrib[i] = fixed_contribution(v);
            if (contrib[i].flags) __hip_atomic_fetch_or(word, contrib[i].flags, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            old[i] = __hip_atomic_fetch_add(word, contrib[i].add, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        const int m = m0 + (tid >> 6) + 8 * i;
        if (mine[i] && (p.ksplit == 1 || (int)(old[i] >> 56) == p.ksplit - 1)) {
            __half *dst = p.out + (size_t)m * p.N + n;
            const float y = p.ksplit == 1 ? val[i] : fixed_total((old[i] | contrib[i].flags) + contrib[i].add, p.ksplit);
            *dst = __float2half_rn((p.overwrite ? 0.0f : __half2float(*dst)) + y);
            if (p.ksplit > 1)
                __hip_atomic_store(p.accum + (size_t)m * p.N + n, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

template <int NB, int MP>
__global__ void __launch_bounds__(kMfmaThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
lut_gemm_mx_kernel(const Problem p, const MxActivations act)
{
    __shared__ __attribute__((aligned(16))) char xs[kMxLutBytes];
    mx_tile<NB, MP>(p, act, (int)blockIdx.x, xs);
}

}  // namespace lutgemm

#endif
