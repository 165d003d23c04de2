/*
 * lutgemm_oracle.c -- CPU restatement of the ShiftAddLLM LUT-GEMM hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against.  Nothing in the shipped package may link, import or call
 * it; only the test-suite, the smoke check and the CPU-baseline leg of the
 * benchmark do.  It is written for clarity, not speed: scalar loops, double
 * accumulation, one thread.
 *
 * Every function names the reference lines it restates (paths relative to the
 * ShiftAddLLM checkout).  What pins each function (known-answer vectors,
 * brute force, closed forms) lives in tests/test_oracle_*.py.
 *
 * Conventions:  y[N] = W[N,K] x[K];  N = out features ("mSize"),
 * K = in features ("kSize"), nb = bit planes, B in {-1,+1}.
 * Kernel sign tensor  Wp[K/32][nb][N] (uint32), bit t of Wp[w][b][n] set
 * <=> B[n][32w+t][b] = +1  (lut_gemm/mv_fp16_bias.hpp:19-26,52,86-90).
 */
#include <stdint.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

/* ---------- IEEE binary16 <-> binary32 (no _Float16 in this gcc) ---------- */

static float half_bits_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: renormalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* round-to-nearest-even, like v_cvt_f16_f32 and torch's .half() */
static uint16_t float_to_half_bits(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u : 0));
    if (ax >= 0x477ff000u) /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    if (ax < 0x33000001u) /* < 2^-25 (or == 2^-25: ties to even -> 0) */
        return (uint16_t)sign;
    int e = (int)(ax >> 23) - 127;
    uint32_t man = (ax & 0x7fffffu) | 0x800000u;
    int shift;
    uint32_t base;
    if (e < -14) { /* subnormal half */
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x7fffffu;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u)))
        q++;
    return (uint16_t)(sign | (base + q)); /* carry into exponent is correct */
}

float orc_half_to_float(uint16_t h) { return half_bits_to_float(h); }
uint16_t orc_float_to_half(float f) { return float_to_half_bits(f); }

/* ---------- A8: pack_binaryWeight (lut_gemm/kernel.py:9-23) ----------
 * B    : int8 [A][L][nb], entries must be +1 or -1 (kernel.py:18 asserts it).
 *        The reference's 4-D input [A, n_groups, group_size, nb] is this with
 *        L = n_groups*group_size flattened (kernel.py:16).
 * out  : int32 [A][L/32][nb]; bit t of out[a][j][b] = (B[a][32j+t][b] == +1),
 *        LSB first (mask 2**arange(32), kernel.py:20); the int64 sum is cast
 *        to int32, so bit 31 lands in the sign (kernel.py:21).
 * returns 0, or -1 if L%32 != 0, -2 if an entry is not +-1.
 */
int orc_pack_binary_weight(const int8_t *B, int A, int L, int nb, int32_t *out)
{
    if (L % 32) return -1;
    for (int a = 0; a < A; a++)
        for (int j = 0; j < L / 32; j++)
            for (int b = 0; b < nb; b++) {
                uint32_t word = 0;
                for (int t = 0; t < 32; t++) {
                    int8_t v = B[((size_t)a * L + 32 * j + t) * nb + b];
                    if (v != 1 && v != -1) return -2;
                    if (v == 1) word |= (1u << t);
                }
                out[((size_t)a * (L / 32) + j) * nb + b] = (int32_t)word;
            }
    return 0;
}

/* ---------- A9: unpack_weight, the dequantisation oracle (kernel.py:26-56) --
 * bW    : int32 [A][L/32][nb]
 * alpha : float [A][G][nb]   (G groups along L, group = L/G entries)
 * W     : float [A][L],  W[a][l] = sum_b alpha[a][l/(L/G)][b] * (2*bit - 1)
 * fp32 accumulation in bit-plane order b = 0,1,.. starting from 0, which is
 * the order of the `ret_weight += alpha * (2*bin-1)` loop (kernel.py:48-53).
 */
int orc_unpack_weight(const int32_t *bW, const float *alpha, int A, int L, int G,
                      int nb, float *W)
{
    if (L % 32 || G <= 0 || L % G) return -1;
    int gs = L / G;
    for (int a = 0; a < A; a++)
        for (int l = 0; l < L; l++) {
            float acc = 0.0f;
            for (int b = 0; b < nb; b++) {
                uint32_t word = (uint32_t)bW[((size_t)a * (L / 32) + l / 32) * nb + b];
                float s = ((word >> (l % 32)) & 1u) ? 1.0f : -1.0f;
                acc += alpha[((size_t)a * G + l / gs) * nb + b] * s;
            }
            W[(size_t)a * L + l] = acc;
        }
    return 0;
}

/* ---------- table indices of the kernel layout (mv_fp16_bias.hpp:86-90) -----
 * Wp  : uint32 [K/32][nb][N]
 * idx : uint8  [K/8][nb][N]; idx[c][b][n] = byte (c%4) of Wp[c/4][b][n].
 */
void orc_table_indices(const uint32_t *Wp, int K, int nb, int N, uint8_t *idx)
{
    for (int c = 0; c < K / 8; c++)
        for (int b = 0; b < nb; b++)
            for (int n = 0; n < N; n++) {
                uint32_t w = Wp[((size_t)(c / 4) * nb + b) * N + n];
                idx[((size_t)c * nb + b) * N + n] = (uint8_t)((w >> (8 * (c % 4))) & 255u);
            }
}

/* ---------- the 256-entry partial-sum table (mv_fp16_bias.hpp:19-45) --------
 * lut[i] = sum_{j<8} (2*bit_j(i) - 1) * x[j]; bit j set means +x[j].
 * The reference builds it in fp16 with a doubling recurrence; the oracle
 * evaluates the defining sum exactly in double.
 */
void orc_build_lut(const uint16_t *x8, double *lut)
{
    double xv[8];
    for (int j = 0; j < 8; j++) xv[j] = (double)half_bits_to_float(x8[j]);
    for (int i = 0; i < 256; i++) {
        double s = 0.0;
        for (int j = 0; j < 8; j++) s += ((i >> j) & 1) ? xv[j] : -xv[j];
        lut[i] = s;
    }
}

/* finish: out (fp16, pre-filled by the caller with bias or zeros) += y.
 * All five reference kernels accumulate into `output` (mv_fp16_bias.hpp:101,
 * 216,324,491,577).  y32 (optional) receives the un-rounded GEMV result. */
static void accumulate_out(uint16_t *out, float *y32, size_t i, double y)
{
    if (y32) y32[i] = (float)y;
    out[i] = float_to_half_bits((float)((double)half_bits_to_float(out[i]) + y));
}

/* ---------- A3: row-wise alpha GEMV (mv_fp16_bias.hpp:498-579) --------------
 * lutgemm_compute_shift_scale.  alpha fp16 [K/gs][nb][N], gs = K/num_groups.
 * out[m][n] += sum_g sum_b alpha[g][b][n] * sum_{k in g} B[n][k][b] x[m][k]
 * evaluated the way the kernel does: per 8-input chunk c a 256-entry table,
 * indexed by byte (c%4) of word c/4.   x fp16 [M][K], out fp16 [M][N].
 * returns 0 or <0 on a shape the layout cannot express.
 */
int orc_gemv_rowwise(const uint32_t *Wp, const uint16_t *alpha, const uint16_t *x,
                     uint16_t *out, float *y32, int N, int K, int nb, int num_groups,
                     int M)
{
    if (K % 32 || num_groups <= 0 || K % num_groups) return -1;
    int gs = K / num_groups;
    if (gs % 8) return -2;
    double lut[256];
    size_t total = (size_t)M * N;
    double *acc = (double *)malloc(total * sizeof(double));
    if (!acc) return -3;
    memset(acc, 0, total * sizeof(double));
    for (int m = 0; m < M; m++)
        for (int c = 0; c < K / 8; c++) {
            orc_build_lut(x + (size_t)m * K + 8 * c, lut);
            int g = (8 * c) / gs;
            for (int b = 0; b < nb; b++)
                for (int n = 0; n < N; n++) {
                    uint32_t w = Wp[((size_t)(c / 4) * nb + b) * N + n];
                    int idx = (w >> (8 * (c % 4))) & 255;
                    double a = (double)half_bits_to_float(alpha[((size_t)g * nb + b) * N + n]);
                    acc[(size_t)m * N + n] += a * lut[idx];
                }
        }
    for (size_t i = 0; i < total; i++) accumulate_out(out, y32, i, acc[i]);
    free(acc);
    return 0;
}

/* ---------- A7: uniform-quant mode (mv_fp16_bias.hpp:8-103) -----------------
 * lutgemm_compute.  alpha, q_bias fp16 [K/gs][N].
 * out[n] += sum_g ( q_bias[g][n] * sum_{k in g} x[k]
 *                   + sum_b alpha[g][n] / 2^(b+1) * sum_{k in g} B x )
 * (the kernel halves alpha before each bit-plane, l.77-84, and takes sum x
 *  from table entry 255, l.59-76).  The reference is batch-1; M>1 applies the
 * same formula per row.
 */
int orc_gemv_uniform(const uint32_t *Wp, const uint16_t *alpha, const uint16_t *q_bias,
                     const uint16_t *x, uint16_t *out, float *y32, int N, int K, int nb,
                     int num_groups, int M)
{
    if (K % 32 || num_groups <= 0 || K % num_groups) return -1;
    int gs = K / num_groups;
    if (gs % 8) return -2;
    double lut[256];
    size_t total = (size_t)M * N;
    double *acc = (double *)malloc(total * sizeof(double));
    if (!acc) return -3;
    memset(acc, 0, total * sizeof(double));
    for (int m = 0; m < M; m++)
        for (int c = 0; c < K / 8; c++) {
            orc_build_lut(x + (size_t)m * K + 8 * c, lut);
            int g = (8 * c) / gs;
            for (int n = 0; n < N; n++) {
                double a = (double)half_bits_to_float(alpha[(size_t)g * N + n]);
                double q = (double)half_bits_to_float(q_bias[(size_t)g * N + n]);
                double s = q * lut[255];
                for (int b = 0; b < nb; b++) {
                    uint32_t w = Wp[((size_t)(c / 4) * nb + b) * N + n];
                    int idx = (w >> (8 * (c % 4))) & 255;
                    a *= 0.5;
                    s += a * lut[idx];
                }
                acc[(size_t)m * N + n] += s;
            }
        }
    for (size_t i = 0; i < total; i++) accumulate_out(out, y32, i, acc[i]);
    free(acc);
    return 0;
}

/* decode one block-alpha multiplier; kind selects the storage format */
enum { ORC_ALPHA_F16 = 0, ORC_ALPHA_SHIFT_U16 = 1, ORC_ALPHA_APOT_I8 = 2 };

static double block_alpha(const void *alpha, int kind, size_t i)
{
    if (kind == ORC_ALPHA_F16)
        return (double)half_bits_to_float(((const uint16_t *)alpha)[i]);
    if (kind == ORC_ALPHA_SHIFT_U16) {
        /* three 3-bit left-shift fields, multiplier 2^f0 + 2^f1 + 2^f2
         * (mv_fp16_bias.hpp:286-297) */
        uint16_t u = ((const uint16_t *)alpha)[i];
        return (double)(1 << (u & 7)) + (double)(1 << ((u >> 3) & 7)) +
               (double)(1 << ((u >> 6) & 7));
    }
    /* int8 [..][3] signed exponents; each table value is "shifted" by the three
     * and the results summed = multiply by 2^s0 + 2^s1 + 2^s2
     * (mv_fp16_bias.hpp:335-340,406-420,473-482).  Exponent -128 is this
     * project's "term absent" marker (the reference has no way to write a
     * one- or two-term alpha; it is documented as an extension). */
    const int8_t *s = (const int8_t *)alpha + 3 * i;
    double a = 0.0;
    for (int t = 0; t < 3; t++)
        if (s[t] != -128) a += ldexp(1.0, (int)s[t]);
    return a;
}

/* ---------- A4/A5/A6: block-alpha GEMV (mv_fp16_bias.hpp:105-220,223-328,
 * 342-495).  alpha [K/8][nb][R] (+[3] for int8), R = num_groups row-groups of
 * N/R consecutive outputs (l.110,160-175):
 * out[m][n] += sum_c sum_b alpha[c][b][n/(N/R)] * LUT_c[idx(c,b,n)]
 * x fp16 [M][K] (row m at x + m*K), out fp16 [M][N].
 */
int orc_gemv_block(const uint32_t *Wp, const void *alpha, int alpha_kind,
                   const uint16_t *x, uint16_t *out, float *y32, int N, int K, int nb,
                   int num_groups, int M)
{
    if (K % 32 || num_groups <= 0 || N % num_groups) return -1;
    int R = num_groups, rows = N / R;
    double lut[256];
    size_t total = (size_t)M * N;
    double *acc = (double *)malloc(total * sizeof(double));
    if (!acc) return -3;
    memset(acc, 0, total * sizeof(double));
    for (int m = 0; m < M; m++)
        for (int c = 0; c < K / 8; c++) {
            orc_build_lut(x + (size_t)m * K + 8 * c, lut);
            for (int b = 0; b < nb; b++)
                for (int n = 0; n < N; n++) {
                    uint32_t w = Wp[((size_t)(c / 4) * nb + b) * N + n];
                    int idx = (w >> (8 * (c % 4))) & 255;
                    double a = block_alpha(alpha, alpha_kind, ((size_t)c * nb + b) * R + n / rows);
                    acc[(size_t)m * N + n] += a * lut[idx];
                }
        }
    for (size_t i = 0; i < total; i++) accumulate_out(out, y32, i, acc[i]);
    free(acc);
    return 0;
}

/* ---------- dense path: y = x @ W^T in fp32-in / double-accumulate ----------
 * The reference's CPU-executable inference path is "dequantise once, then an
 * ordinary Linear" (kernel.py:87-109).  W float [N][K], x fp16 [M][K].
 */
void orc_dense_gemv(const float *W, const uint16_t *x, float *y, int N, int K, int M)
{
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            double s = 0.0;
            for (int k = 0; k < K; k++)
                s += (double)W[(size_t)n * K + k] *
                     (double)half_bits_to_float(x[(size_t)m * K + k]);
            y[(size_t)m * N + n] = (float)s;
        }
}
