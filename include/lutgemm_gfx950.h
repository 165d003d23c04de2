/*
 * lutgemm_gfx950.h -- C ABI of the MI355X (gfx950) LUT-GEMM engine for
 * binary-coding-quantised (BCQ) linear layers.
 *
 * This is the boundary a host binding sits on: plain pointers and sizes, no
 * torch types.  All pointers are DEVICE pointers on the current HIP device;
 * `stream` is a hipStream_t passed as void* (NULL = the null stream).  Every
 * call is asynchronous with respect to the host and returns 0 on success or a
 * negative LUTGEMM_E* code; nothing throws and nothing is printed.
 *
 * Shared operand conventions (paths are relative to the ShiftAddLLM
 * reference checkout):
 *   N = out features ("mSize"), K = in features ("kSize"), nb = bit planes.
 *   bW    : uint32 [K/32][nb][N]; bit t of bW[w][b][n] set <=> sign
 *           B[n][32w+t][b] = +1; byte j of the word indexes the 256-entry
 *           table of inputs 32w+8j .. 32w+8j+7
 *           (lut_gemm/mv_fp16_bias.hpp:19-26,52,86-90; lut_gemm/quant.py:25).
 *   x     : fp16 [M][K] row-major (row m at x + m*K).
 *   out   : fp16 [M][N] row-major.  The engine ACCUMULATES: out += W_q x,
 *           the caller pre-fills out with the bias or zeros
 *           (mv_fp16_bias.hpp:101,216,324,491,577; lut_gemm/quant.py:46).
 *           Unlike the reference's fp16 atomics the sum is formed in fp32 and
 *           rounded to fp16 once, and it is deterministic.  (Two to four rows
 *           of a per-column-alpha problem on the table look-up kernel share
 *           tables whose entries are fp16, like the reference's
 *           (mv_fp16_bias.hpp:342-380): one more fp16 rounding per eight
 *           inputs, output error about 3e-4 relative instead of 2e-4.)
 *           A NaN input gives NaN and an infinite input gives an infinity
 *           or NaN in every output it reaches, whatever the launch plan.
 *           Finite inputs have a guaranteed range: while every partial sum
 *           over a run of K stays within +-65536, and (calls with two or
 *           more rows on the look-up kernel, whose tables are fp16) every
 *           sum of eight |x| stays below 65504, the result is the rounded
 *           exact sum under every launch plan.  Beyond that range the
 *           result depends on the plan: a partial sum beyond +-65536 counts
 *           as infinite where K is split over workgroups and is carried as
 *           fp32 where it is not, so the same finite problem may give an
 *           infinity for one M or grouping and a finite value for another.
 * Shape rules enforced here (the reference checks nothing and reads or writes
 * out of bounds instead): K % 32 == 0, N % 4 == 0, 1 <= nb <= 4,
 * 1 <= M <= 65535, 16-byte aligned bW and x, 8-byte aligned row-wise alpha and out.
 *
 * Workspace.  K is split over workgroups whose partial sums meet in one 64-bit
 * word per output, M * N words per call, which the library keeps per (device,
 * stream): grow-only, zero between launches.  The first call that needs more
 * words than the stream has synchronises the stream and allocates; that cannot
 * happen while the stream is being captured (LUTGEMM_ECAPTURE), so either make
 * one call of each shape before capturing or reserve the words up front with
 * lutgemm_reserve_workspace().  A captured graph names the workspace of the
 * stream it was captured on: replay graphs captured on ONE stream one at a
 * time (whatever stream they are replayed on), and do not run eager calls on
 * that stream while one of its graphs is replaying -- both would share
 * accumulator words.  Graphs captured on different streams are independent.
 */
#ifndef LUTGEMM_GFX950_H
#define LUTGEMM_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LUTGEMM_OK 0
#define LUTGEMM_EINVAL (-1)   /* bad shape / size / null pointer            */
#define LUTGEMM_EALIGN (-2)   /* pointer not aligned as required            */
#define LUTGEMM_EUNSUP (-3)   /* legal in the reference API, not built here */
#define LUTGEMM_EHIP (-4)     /* a HIP runtime call failed                  */
#define LUTGEMM_ENOMEM (-5)   /* workspace allocation failed                */
#define LUTGEMM_ECAPTURE (-6) /* the stream is being captured and its workspace
                                 would have to grow: reserve it beforehand   */
#define LUTGEMM_ETOOBIG (-7)  /* beyond the fixed buffer of the entry point
                                 that does not allocate                      */
#define LUTGEMM_ETIMEDOUT (-8) /* lutgemm_chain_status: a wait of a chained
                                  launch gave up                             */

/* Human-readable text for a return code (static storage). */
const char *lutgemm_strerror(int code);

/* HIP error of the last LUTGEMM_EHIP on this thread (hipError_t as int). */
int lutgemm_last_hip_error(void);

/*
 * Row-wise alpha, groups along K.
 * Replaces lutgemm_compute_shift_scale -> nqmv_bias_shift_mulq ->
 * _nqmv_bias_shift_mulq<32>  (lut_gemm/lutgemm_cuda.cpp:43-52;
 * lutgemm_cuda_kernel.cu:268-285; mv_fp16_bias.hpp:498-579,766-774).
 *   alpha : fp16 [num_groups][nb][N], group g covers inputs
 *           g*(K/num_groups) .. ; K/num_groups must be a multiple of 32.
 *   out[m][n] += sum_g sum_b alpha[g][b][n] * sum_{k in g} B[n][k][b] x[m][k]
 * The reference entry point is batch-1; M > 1 rows are a superset.
 */
int lutgemm_gemv_rowwise_f16(const uint32_t *bW, const void *alpha_f16, const void *x_f16,
                             void *out_f16, int N, int K, int nb, int num_groups, int M,
                             void *stream);

/*
 * lutgemm_gemv_rowwise_f16 for alphas that are POWERS OF TWO, which is what ShiftAddLLM's
 * quantiser produces (quantizers/bcq_quant/bcq_shift.py:15-24,34: every alpha is rounded
 * to 2^round(log2 |alpha|)) and what gives the method its name: multiplying by such an
 * alpha is a shift.  Same arguments and semantics; the caller PROMISES that every alpha
 * is a positive normal fp16 power of two (mantissa bits zero, exponent field 1..30).
 * With that promise a call of 3 to 8 rows on a large matrix (K a multiple of 128, groups of a
 * multiple of 128 inputs, N a multiple of 16; up to 5 rows from 48 MB of sign words on, up
 * to 8 rows from 96 MB on; option LUTGEMM_OPTION_BLOCK_SCALED widens or switches off the
 * rule, lutgemm_describe_pow2_plan tells what a call takes) runs on gfx950's block-scaled
 * matrix instruction: sign bits become 4-bit floats +-1 through a table (one LDS read per
 * eight signs), the alpha's exponent rides as the instruction's per-block power-of-two
 * scale, and the activations are split, by a small kernel in front, into three 8-bit floats
 * per value with a power-of-two scale per 32 (exact for every fp16 value within 2^14 of the
 * largest of its 32; smaller ones are cut off at 2^-25 of it); the three pieces of up to
 * 5 rows share the 16 columns of one instruction.  Accumulation is fp32, one rounding to
 * fp16 at the end, as in every other entry point.  An infinity or NaN among the activations
 * gives NaN in every output of its row.  Calls of up to 16 rows that take the fp16
 * matrix-core kernel with long K extents per workgroup form their sign operands through
 * the same kind of table and gfx950's scaled fp4 -> fp16 conversion (option
 * LUTGEMM_OPTION_POW2_CONVERT): the same exact products as lutgemm_gemv_rowwise_f16,
 * summed in another order.  Other calls run exactly as lutgemm_gemv_rowwise_f16 does.  With an alpha that breaks the promise the result is that
 * of the alpha with its mantissa bits cleared (zero counts as 2^-15).
 * The split activations (3 * M * K + K + M * K / 8 bytes) live in a second per-stream
 * buffer that grows like the accumulator workspace: make one call of each size before
 * capturing a graph.  No counterpart in the reference.
 */
int lutgemm_gemv_rowwise_pow2_f16(const uint32_t *bW, const void *alpha_f16, const void *x_f16,
                                  void *out_f16, int N, int K, int nb, int num_groups, int M,
                                  void *stream);

/*
 * lutgemm_gemv_rowwise_f16 for callers that cannot allocate device memory: code
 * under HIP graph capture, tight serving loops, harnesses that forbid it.  It
 * has no counterpart in the reference.  Same arguments, semantics and results,
 * but the accumulator words come from a fixed array inside the library
 * (LUTGEMM_NOALLOC_MAX_WORDS words of 8 bytes = 2 MiB, which every GPU the
 * library runs on holds until the process ends) instead of a per-stream
 * workspace: the call never calls hipMalloc or hipFree and never synchronises.
 * M * N may be at most LUTGEMM_NOALLOC_MAX_WORDS (LUTGEMM_ETOOBIG otherwise).
 * All calls on one GPU share the array, whatever their stream, and each leaves
 * the words it used at zero again: calls that overlap in time on one GPU race
 * (order them, e.g. on one stream).  The first call on a device looks the
 * array's address up, which may load the code object: make that call outside
 * graph capture.
 */
#define LUTGEMM_NOALLOC_MAX_WORDS (1 << 18)
int lutgemm_gemv_rowwise_f16_noalloc(const uint32_t *bW, const void *alpha_f16, const void *x_f16,
                                     void *out_f16, int N, int K, int nb, int num_groups, int M,
                                     void *stream);

/*
 * Several row-wise-alpha GEMVs in ONE kernel launch.  No counterpart in the
 * reference, which launches every linear layer separately; it exists because a
 * launch on this hardware has a fixed cost of about 2 microseconds, more than
 * a 7B-sized GEMV needs at HBM speed, so projections that do not depend on each
 * other (q/k/v, gate/up) are best issued together.  Each entry has the
 * arguments and the semantics of lutgemm_gemv_rowwise_f16; bit widths and
 * shapes may differ between entries; outputs must not overlap (LUTGEMM_EINVAL).
 * 1 <= count <= LUTGEMM_MAX_GROUP.
 */
#define LUTGEMM_MAX_GROUP 8
typedef struct lutgemm_rowwise_problem {
    const uint32_t *bW;
    const void *alpha_f16;
    const void *x_f16;
    void *out_f16;
    int N, K, nb, num_groups, M;
} lutgemm_rowwise_problem;

int lutgemm_gemv_rowwise_f16_grouped(int count, const lutgemm_rowwise_problem *problems,
                                     void *stream);

/*
 * Uniform-quantisation mode of the original LUT-GEMM.
 * Replaces lutgemm_compute -> nqmv_bias -> _nqmv_bias<32>
 * (lutgemm_cuda.cpp:88-98; lutgemm_cuda_kernel.cu:287-315;
 *  mv_fp16_bias.hpp:8-103,726-734).
 *   alpha, q_bias : fp16 [num_groups][N]
 *   out[m][n] += sum_g ( q_bias[g][n] * sum_{k in g} x[m][k]
 *                + sum_b alpha[g][n] / 2^(b+1) * sum_{k in g} B[n][k][b] x[m][k] )
 */
int lutgemm_gemv_uniform_f16(const uint32_t *bW, const void *alpha_f16, const void *qbias_f16,
                             const void *x_f16, void *out_f16, int N, int K, int nb,
                             int num_groups, int M, void *stream);

/*
 * Block alpha (ShiftAddLLM "Lat."): one alpha per 8-input chunk, bit plane and
 * row group.  R = num_groups row groups of N/R consecutive outputs.
 *   out[m][n] += sum_c sum_b A(c, b, n / (N/R)) * LUT_c[byte(c,b,n)]
 * (N/R) % 4 == 0 is required.
 *
 * _f16      : A = alpha fp16 [K/8][nb][R].  Replaces lutgemm_compute_block ->
 *             _nqmv_bias_block<32> (lutgemm_cuda.cpp:54-63;
 *             lutgemm_cuda_kernel.cu:318-346; mv_fp16_bias.hpp:105-220,736-744).
 * _shift_u16: alpha uint16 [K/8][nb][R] of three 3-bit shift fields,
 *             A = 2^(u&7) + 2^((u>>3)&7) + 2^((u>>6)&7).  Replaces
 *             lutgemm_compute_block_shift -> _nqmv_bias_block_shift<32>
 *             (lutgemm_cuda.cpp:65-74; lutgemm_cuda_kernel.cu:349-377;
 *             mv_fp16_bias.hpp:223-328,746-754).
 * _apot_i8  : alpha int8 [K/8][nb][R][3] signed exponents,
 *             A = 2^s0 + 2^s1 + 2^s2, a term with s = -128 is absent.
 *             Replaces lutgemm_compute_block_shiftInt8 ->
 *             _nqmv_bias_block_shiftInt8<32> (lutgemm_cuda.cpp:76-85;
 *             lutgemm_cuda_kernel.cu:380-408; mv_fp16_bias.hpp:335-340,
 *             342-495,756-764) -- the call LutLinear.forward makes
 *             (lut_gemm/quant.py:50-51).
 * num_apot must be 3: the reference ignores the argument and hard-codes three
 * terms (mv_fp16_bias.hpp:294,473-482).
 */
int lutgemm_gemv_block_f16(const uint32_t *bW, const void *alpha_f16, const void *x_f16,
                           void *out_f16, int N, int K, int nb, int num_groups, int M,
                           void *stream);
int lutgemm_gemv_block_shift_u16(const uint32_t *bW, const uint16_t *alpha_u16, const void *x_f16,
                                 void *out_f16, int N, int K, int nb, int num_groups,
                                 int num_apot, int M, void *stream);
int lutgemm_gemv_block_apot_i8(const uint32_t *bW, const int8_t *alpha_i8, const void *x_f16,
                               void *out_f16, int N, int K, int nb, int num_groups, int num_apot,
                               int M, void *stream);

/*
 * Algorithmic HBM bytes of one call (signs + alphas + x + out read + out
 * write), the figure throughput is quoted against.  alpha_bytes_per_entry is
 * 2 (fp16, uint16) or 3 (int8 x 3); alpha_entries is the alpha element count.
 */
size_t lutgemm_algorithmic_bytes(int N, int K, int nb, int M, size_t alpha_entries,
                                 int alpha_bytes_per_entry);

/*
 * Measurement helper: a plain device-to-device copy of `bytes` (multiple of
 * 16) done by a kernel of this library, used to calibrate profiler byte
 * counters against a known traffic.  No counterpart in the reference.
 */
int lutgemm_copy_bytes(void *dst, const void *src, size_t bytes, void *stream);

/*
 * Words (8 bytes each) of accumulator workspace a call with these sizes needs at
 * most, and a way to provide them ahead of time: after
 * lutgemm_reserve_workspace(stream, w) no call on `stream` whose sizes need at
 * most w words synchronises or allocates, so such calls can be captured into a
 * HIP graph without a warm-up call.  For a grouped or fused call add up the
 * words of its problems.  Reserving synchronises `stream` and may not be done
 * while it is being captured (LUTGEMM_ECAPTURE).  No counterpart in the
 * reference, whose kernels accumulate with fp16 atomics straight into `out`.
 */
size_t lutgemm_workspace_words(int N, int M);
int lutgemm_reserve_workspace(void *stream, size_t words);

/*
 * How a lone call with these sizes would be launched: which kernel, how many
 * workgroups, how the work is cut.  Pure host arithmetic: no device is touched,
 * so launch plans can be inspected (and tested) on a machine without a GPU.
 * `format` is one of LUTGEMM_FORMAT_*; `groups` is num_groups for the row-wise
 * and uniform formats and the number of row groups R for the block formats.
 * Returns what the compute entry point would return for the same sizes
 * (LUTGEMM_EINVAL, LUTGEMM_EUNSUP) without launching anything.  The tuning knobs
 * of the environment apply as they do to the compute calls.  No counterpart in
 * the reference, whose launch geometry is fixed at compile time
 * (mv_fp16_bias.hpp:726-774).
 */
#define LUTGEMM_FORMAT_ROWWISE_F16 0
#define LUTGEMM_FORMAT_BLOCK_F16 1
#define LUTGEMM_FORMAT_BLOCK_SHIFT_U16 2
#define LUTGEMM_FORMAT_BLOCK_APOT_I8 3
#define LUTGEMM_FORMAT_UNIFORM_F16 4

typedef struct lutgemm_plan {
    int kernel;          /* 0: table look-up kernel, 1: matrix-core kernel, 2: block-scaled matrix-core kernel */
    int workgroups;      /* of the launch */
    int rows_per_pass;   /* activation rows a workgroup handles together */
    int row_chunks;      /* ceil(M / rows_per_pass) */
    int tiles;           /* output tiles of tile_columns columns */
    int k_units;         /* sets of 256 inputs (look-up), steps of 128 (matrix cores) */
    /* look-up kernel: the tiles x k_units items of a row chunk, tile-major, are cut into
     * `ranges` contiguous ranges: the first `long_ranges` of `items_per_long_range`
     * items, the others of `items_per_short_range` (the last one may be shorter) */
    int ranges, long_ranges, items_per_long_range, items_per_short_range;
    /* matrix-core kernel: every tile is cut into `k_slices` slices of
     * `units_per_slice` steps (the last one may be shorter) */
    int k_slices, units_per_slice;
    int needs_workspace; /* 1: the launch uses lutgemm_workspace_words(N, M) accumulator words */
    int tile_columns;    /* output columns per tile: 256 (look-up), 512 (look-up, twin items), 64 (matrix cores) */
} lutgemm_plan;

int lutgemm_describe_plan(int format, int N, int K, int nb, int groups, int M, lutgemm_plan *plan);
/* The same for lutgemm_gemv_rowwise_pow2_f16: kernel 2 is the block-scaled matrix-core kernel
 * (rows_per_pass 5, 8 or 16; tiles of 64 columns, steps of 128 inputs); a call that takes one
 * of the other kernels is described as lutgemm_describe_plan describes it. */
int lutgemm_describe_pow2_plan(int N, int K, int nb, int groups, int M, lutgemm_plan *plan);

/*
 * Tuning options (no counterpart in the reference, whose launch geometry is fixed at
 * compile time).  Each starts from the environment variable of the same name
 * (LUTGEMM_TARGET_BLOCKS ...), read once per process; lutgemm_set_option changes it
 * for every later call of the process (a negative value restores the start value),
 * lutgemm_get_option reads it.  Results stay within the documented tolerances under
 * every setting; the options exist for measurements and tests.
 *   TARGET_BLOCKS : workgroups a look-up launch aims for (0 = 256 up to 24 MB of
 *                   sign words, 512 beyond: one or two resident workgroups per CU)
 *   FIRST_SHARE   : per cent of a CU's items its first-dispatched workgroup takes in
 *                   a 512-workgroup look-up launch (default 60; 50 = equal ranges)
 *   MFMA_MIN_M    : rows from which a row-wise problem takes the matrix-core kernel
 *                   (default 3; a large value switches that kernel off)
 *   MFMA_BLOCKS   : workgroups aimed at per matrix-core launch (0 = the cost model)
 *   PAIR_TABLES   : 1 = two rows share one table set of fp16 pairs on the look-up
 *                   kernel, 0 = one fp32 table set per row
 *   SINGLE_ITEM   : 1 = launches whose ranges all hold one item take the kernel
 *                   instance that requests nothing beyond it, 0 = the general one
 *   TWIN_ITEMS    : one-row look-up launches whose workgroups would all hold at least this
 *                   many items take twin items instead (one table build per 512 outputs
 *                   instead of per 256; default 4, 0 = never)
 *   BLOCK_SCALED  : lutgemm_gemv_rowwise_pow2_f16 takes the block-scaled matrix-core
 *                   kernel 1 = where it is the faster one (few rows, large matrices),
 *                   2 = wherever it applies, 0 = never (the call then behaves like
 *                   lutgemm_gemv_rowwise_f16); default 1
 *   POW2_CONVERT  : calls of lutgemm_gemv_rowwise_pow2_f16 that take the fp16 matrix-core
 *                   kernel form its sign operands through an LDS table and the scaled
 *                   fp4 -> fp16 conversion instruction (which applies a power-of-two alpha
 *                   as its scale) instead of a shift and a bit operation per fp16 pair
 *                   1 = where that is faster (up to 16 rows, six or more rounds of K-steps
 *                   per workgroup), 2 = always, 0 = never; default 1
 *   CHAIN_GRID    : workgroups of a chained launch (0 = as many as the device holds
 *                   at once, which is also the upper limit)
 *   CHAIN_BLOCKS  : ranges the problems of one stage of a chained launch are cut into
 *                   (0 = one per workgroup of the launch)
 */
#define LUTGEMM_OPTION_TARGET_BLOCKS 0
#define LUTGEMM_OPTION_FIRST_SHARE 1
#define LUTGEMM_OPTION_MFMA_MIN_M 2
#define LUTGEMM_OPTION_MFMA_BLOCKS 3
#define LUTGEMM_OPTION_PAIR_TABLES 4
#define LUTGEMM_OPTION_SINGLE_ITEM 5
#define LUTGEMM_OPTION_CHAIN_BLOCKS 6
#define LUTGEMM_OPTION_CHAIN_GRID 7
#define LUTGEMM_OPTION_TWIN_ITEMS 8
#define LUTGEMM_OPTION_BLOCK_SCALED 9
#define LUTGEMM_OPTION_POW2_CONVERT 10
#define LUTGEMM_OPTION_COUNT 11
int lutgemm_set_option(int which, int value);
int lutgemm_get_option(int which);

/*
 * Measurement helpers for the floors any kernel of this library sits on (no
 * counterpart in the reference): a kernel that streams `bytes` (multiple of 16)
 * from `src` with the same 128-bit non-temporal loads as the look-up kernel and
 * does nothing with them (`sink`: 4 writable bytes, or NULL), and an empty
 * kernel with the look-up kernel's workgroup size and LDS footprint.
 */
int lutgemm_measure_stream_read(const void *src, size_t bytes, void *sink, void *stream);
int lutgemm_measure_empty_launch(int workgroups, void *stream);

/*
 * Measurement helper of the time-stamped build of the library
 * (liblutgemm_gfx950_ts.so, same sources compiled with -DLUTGEMM_TIMESTAMPS;
 * the ordinary build returns LUTGEMM_EUNSUP).  After this call every wave of every
 * look-up kernel launch writes LUTGEMM_STAMPS_PER_WAVE readings of the 100 MHz
 * wall clock, taken at fixed points of the kernel (entry, first operands
 * requested, activations arrived, first tables built, first item looked up, all
 * items looked up, sums handed over, exit), into
 *   readings[((workgroup of the grid) * 8 + wave) * LUTGEMM_STAMPS_PER_WAVE + point]
 * (uint64, device memory, `count` readings of capacity; what does not fit is
 * dropped; NULL switches the readings off).  The low 56 bits of a reading are the
 * clock, the top byte is the workgroup's row of the grid: the problem of a grouped
 * or chained launch, the row chunk of a lone one.  No counterpart in the reference.
 */
#define LUTGEMM_STAMPS_PER_WAVE 8
int lutgemm_set_timestamp_buffer(void *readings, size_t count);

/* Release the per-stream workspaces this library allocated on the current
 * device (optional; they otherwise live until the process ends).  HIP graphs
 * captured from calls of this library name those workspaces: destroy such
 * graphs first.  A workspace that a later, larger call outgrew is kept until
 * this call for the same reason. */
int lutgemm_release_workspaces(void);

/*
 * Row-wise GEMVs with the neighbouring element-wise work of a decoder block
 * folded in (no counterpart in the reference, whose modules run them as
 * separate framework kernels).  Up to LUTGEMM_MAX_GROUP problems per launch.
 *   norm_weight_f16 : NULL, or fp16 [K]: the GEMV input is
 *                     x * rsqrt(mean(x^2) + norm_eps) * norm_weight
 *                     per row of x (RMSNorm), formed inside the kernel;
 *   gate_f16        : NULL, or fp16 [M][K]: the GEMV input is
 *                     fp16(fp16(silu(gate)) * x)  (SwiGLU);
 *                     at most one of the two per problem; both 16-byte aligned;
 *   overwrite       : 0 = out += y like every other entry point, 1 = out = y
 *                     (out need not be initialised).
 * A problem with none of the three is the plain row-wise GEMV.  The problems of
 * one call must share their transform (all norm, all gate or all none;
 * LUTGEMM_EUNSUP otherwise).  Problems with a transform always run on the
 * look-up kernel, whatever M (with several rows a separate transform kernel in
 * front of a plain call is faster); overwriting problems with several rows take
 * the matrix-core kernel like plain ones.
 *
 * With norm_weight_f16 the kernel multiplies x by the weight first (x * weight is
 * held as fp16 and must stay below 65504) and applies rsqrt(mean(x^2) + norm_eps)
 * to the finished sums, which is the same product.
 *
 * RMSNorm split over two launches, for a residual stream that one GEMV completes
 * and the next reads normalised (either look-up or matrix-core kernel, any M):
 *   the completing problem (out = residual, accumulated into) names
 *     next_norm_weight_f16 : fp16 [N], the weight of the norm that follows,
 *     next_input_f16       : fp16 [M][N], receives fp16(out * next_norm_weight),
 *     sumsq_out_f32        : float [M][N/32], ZERO before the call (N % 32 == 0):
 *                            receives, spread over a row's slots, the sum of the
 *                            squares of the row's final outputs;
 *   the consuming problem takes x_f16 = that next_input, K = that N, and
 *     sumsq_in_f32 / sumsq_in_slots : that array (16-byte aligned) and its slots per row,
 *                            which must be K / 32 (LUTGEMM_EINVAL otherwise):
 *                            y = rsqrt(sum(slots) / K + norm_eps) * W x.
 *   All five may be NULL / 0; next_norm_weight and next_input come together;
 *   sumsq_in excludes norm_weight_f16.  Which slot receives which columns is
 *   unspecified.  On the look-up kernel a slot normally receives one float add
 *   (two when outputs of a 32-column run were completed by different
 *   workgroups), and two adds commute, so the sums are reproducible from run to
 *   run; on the matrix-core kernel with K cut into three or more slices a slot
 *   may receive that many adds in arrival order, and the sums (hence the
 *   consuming problem's outputs) may differ in the last bits between runs.
 *   Nothing a problem of the call writes (out, next_input, sumsq_out) may overlap
 *   what another write or a read (x, gate, sumsq_in) of the same call touches
 *   (LUTGEMM_EINVAL).
 */
typedef struct lutgemm_fused_problem {
    const uint32_t *bW;
    const void *alpha_f16;
    const void *x_f16;
    void *out_f16;
    int N, K, nb, num_groups, M;
    int overwrite;
    const void *norm_weight_f16;
    const void *gate_f16;
    float norm_eps;
    const void *next_norm_weight_f16;
    void *next_input_f16;
    float *sumsq_out_f32;
    const float *sumsq_in_f32;
    int sumsq_in_slots;
} lutgemm_fused_problem;

int lutgemm_gemv_rowwise_f16_fused(int count, const lutgemm_fused_problem *problems, void *stream);

/*
 * Row-wise GEMVs that DEPEND on each other in ONE launch (no counterpart in the
 * reference, which launches every linear layer separately and waits for each).
 * Of a GEMV's bytes all but the activation row are independent of the GEMV in
 * front of it, but a launch boundary makes all of them wait: about 2 us of launch
 * gap, the first memory round trip and the ramp of the stream, per dependent GEMV.
 * Here up to LUTGEMM_MAX_GROUP problems form one grid; a problem that consumes
 * another's output requests its sign words and alphas at once and then waits for
 * the activations only.
 *
 * The hand-over goes through TAGGED rows: uint32 [M][N], one word per value =
 * fp16 bits | tag << 16.  The producer writes every finished value with its tag
 * (one store past its L2); the consumer re-reads the words it needs until all
 * carry the tag it expects.  Per problem:
 *   x_tag    0: x_f16 is plain fp16 [M][K], written before the call;
 *            t >= 1: x_f16 points at a tagged row uint32 [M][K] and the problem
 *            waits until the words it needs carry tag t;
 *   gate_tag the same for gate_f16;
 *   out_tag  0: out_f16 is plain fp16 [M][N]; t >= 1: a tagged row uint32 [M][N],
 *            every output is written with tag t (accumulation reads the old
 *            values whatever their tags).
 * The other fields of `p` mean what they mean in the fused call (norm_weight:
 * RMSNorm formed from the row itself, K <= 8192 when it is tagged; gate:
 * SiLU(gate) * x; overwrite); the split-RMSNorm fields must be NULL / 0
 * (LUTGEMM_EUNSUP).  1 <= M <= LUTGEMM_CHAIN_MAX_ROWS (one row per workgroup,
 * look-up kernel).  Tags lie in 1..LUTGEMM_CHAIN_MAX_TAG.
 *
 * Order.  The launch is persistent: as many workgroups as the device holds of the
 * kernel at once walk the call's units (one workgroup's range of one problem,
 * numbered in the order the problems are given) in increasing order, which is
 * what keeps a wait from starving the problem it waits for (see
 * lutgemm_describe_chain_plan).  So a problem must come AFTER every problem of
 * the call whose tag it waits for (LUTGEMM_EINVAL), and problems must be listed
 * stage by stage (those that wait for nothing, then those that wait for them,
 * ...).  A tag that no problem of the call writes is waited for all the same:
 * the row may be written by other work of the process, but nothing guarantees
 * that such work runs while the call waits, and kernels of other streams that
 * run at the same time may keep part of the launch from being resident, so every
 * wait is bounded (control->spin_limit_us, 0 = 100000).  A wait that gives up
 * sets bit 0 of *control->status (device memory, zero before the call); the
 * waiting workgroups of the call then exit without writing, the kernel ends
 * normally, and lutgemm_chain_status() reports LUTGEMM_ETIMEDOUT.
 *
 * Epoch.  A captured launch is replayed with the same tags, and last replay's
 * rows would satisfy this replay's waits: the effective tag of base t is
 * 1 + (t + *control->epoch) % 65535 (epoch: device memory, may be NULL = 0).
 * Advance the epoch word between replays (lutgemm_chain_advance_epoch, by at
 * least the number of tag bases in use) so that no row still carries a tag that a
 * later call waits for before its producer has written it.
 *
 * Overlap.  The same tagged row may be written by several problems of a call with
 * different tags (a residual row that two GEMVs complete one after the other) and
 * read in between, if the waits order them: a later writer must wait, directly
 * or through other problems, for the earlier writer and for every reader of the
 * earlier contents (LUTGEMM_EINVAL otherwise).  Plain rows may not be shared
 * between a writer and any other problem of the call.
 * Workspace, capture and error conventions are those of the other entry points.
 */
#define LUTGEMM_CHAIN_MAX_ROWS 4
#define LUTGEMM_CHAIN_MAX_TAG 65534
typedef struct lutgemm_chain_problem {
    lutgemm_fused_problem p;
    int x_tag, gate_tag, out_tag;
} lutgemm_chain_problem;

typedef struct lutgemm_chain_control {
    const uint32_t *epoch;
    uint32_t *status;
    unsigned spin_limit_us;
} lutgemm_chain_control;

int lutgemm_gemv_rowwise_f16_chain(int count, const lutgemm_chain_problem *problems,
                                   const lutgemm_chain_control *control, void *stream);

/*
 * How a chained call would be launched (pure host arithmetic when `workgroups` > 0; with 0 the
 * device is asked how many workgroups of the kernel it holds at once, which is what the compute
 * call uses).  The launch is persistent: `workgroups` workgroups, all resident at the same time,
 * take the call's `units` (one workgroup's range of one problem, numbered problem by problem in
 * the order given) in steps of `workgroups`: workgroup w takes units w, w + workgroups, ...
 * A unit waits only for units with smaller numbers, and every workgroup takes its units in
 * increasing order, so the unfinished unit with the smallest number can always run: no wait can
 * starve the unit it waits for.  That argument needs every workgroup of the launch resident,
 * which other kernels running at the same time can prevent: hence the bounded waits.
 * Per problem: its stage (0 = waits for nothing in the call), its first unit, its units, and the
 * (tile, set) items of a unit (the last unit of a problem may hold fewer).  Returns what the
 * compute call would return for the same problems without launching anything.
 */
typedef struct lutgemm_chain_plan {
    int workgroups, units, needs_workspace;
    int stage[LUTGEMM_MAX_GROUP], first_unit[LUTGEMM_MAX_GROUP], unit_count[LUTGEMM_MAX_GROUP],
        items_per_unit[LUTGEMM_MAX_GROUP];
} lutgemm_chain_plan;
int lutgemm_describe_chain_plan(int count, const lutgemm_chain_problem *problems, int workgroups,
                                lutgemm_chain_plan *plan);

/* dst_tagged[i] = src_f16[i] | effective tag << 16 (count values), and back. */
int lutgemm_chain_tag_rows(void *dst_tagged, const void *src_f16, size_t count, int tag, const uint32_t *epoch,
                           void *stream);
int lutgemm_chain_untag_rows(void *dst_f16, const void *src_tagged, size_t count, void *stream);
/* *epoch += by, on the stream. */
int lutgemm_chain_advance_epoch(uint32_t *epoch, uint32_t by, void *stream);
/* Synchronises `stream`, reads *status: LUTGEMM_OK or LUTGEMM_ETIMEDOUT. */
int lutgemm_chain_status(const uint32_t *status, void *stream);

/*
 * ---- decode-step glue (no counterpart in the reference) ----------------------
 * The reference times token-by-token decoding through an eager framework model
 * (model/opt.py:367-423); around each LUT-GEMV that costs some forty small
 * framework kernels per decoder block.  These three entry points replace them,
 * so that a block is eight launches.  fp16 tensors, row-major, contiguous.
 */

/* y[r] = fp16(fp16(x[r] * rsqrt(mean(x[r]^2) + eps)) * weight), r < rows;
 * hidden % 8 == 0.  The same launch also zero-fills `clear_bytes` (multiple of
 * 16, may be 0) at `clear`: the accumulate-into outputs of the GEMVs that
 * consume y.  x, weight, y, clear 16-byte aligned. */
int lutgemm_decode_rmsnorm_f16(const void *x, const void *weight, void *y, int rows, int hidden, float eps,
                               void *clear, size_t clear_bytes, void *stream);

/* One new token per sequence: rotary embedding of q and k at position
 * *position (rotate-half convention: cos/sin tables [max_positions][head_dim],
 * the two halves of a row equal), append k and v to the caches
 * [batch][kv_heads][max_positions][head_dim], softmax(q k^T / sqrt(head_dim))
 * v over cache positions 0..*position.  q [batch][heads*head_dim], k and v
 * [batch][kv_heads*head_dim], out [batch][heads*head_dim]; heads a multiple of
 * kv_heads; head_dim a multiple of 8, at most 256; max_positions at most 8192.
 * `position` is a DEVICE pointer so that a captured graph can be replayed for
 * successive tokens; the kernel clamps *position into 0..max_positions-1 (it
 * cannot report an error), so the caller must keep it inside the cache. */
int lutgemm_decode_attention_f16(const void *q, const void *k, const void *v, const void *cos_table,
                                 const void *sin_table, void *k_cache, void *v_cache, const int64_t *position,
                                 void *out, int batch, int heads, int kv_heads, int head_dim, int max_positions,
                                 void *stream);

/* out = fp16(fp16(silu(gate)) * up) over `count` values (multiple of 8);
 * pointers 16-byte aligned. */
int lutgemm_decode_silu_mul_f16(const void *gate, const void *up, void *out, size_t count, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* LUTGEMM_GFX950_H */
