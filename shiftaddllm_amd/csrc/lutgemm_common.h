// Types and constants shared by the device templates and the host side of
// liblutgemm_gfx950.so.  Not installed; gfx950 (wave64) only.
#ifndef LUTGEMM_COMMON_H
#define LUTGEMM_COMMON_H

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stddef.h>
#include <stdint.h>

#include "lutgemm_gfx950.h"

namespace lutgemm {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / 64;
constexpr int kSetWords = 8;               // sign words (of 32 inputs) per table set
constexpr int kTables = 4 * kSetWords;     // 32 tables, one per LDS bank
constexpr int kWaveCols = 32;              // outputs a wave covers
constexpr int kTileCols = kWaves * kWaveCols;  // outputs a workgroup covers (256)
constexpr int kEntryStride = 64;           // dwords between consecutive entries of a table
constexpr int kLutDwords = 256 * kEntryStride;  // 64 KiB: two interleaved table buffers
constexpr int kStageDwords = 2 * 2 * 4 * kTables;  // staged block alphas: [buffer][row group][bit][chunk]
constexpr int kMaxContrib = 40;            // contributions per accumulator word (see below)
constexpr int kMaxSlices = 32;             // matrix-core kernel: K-slices per tile
constexpr int kMaxGroup = LUTGEMM_MAX_GROUP;  // problems per grouped launch

// Fixed-point accumulator word of one output (K split over workgroups):
//   [63:56] contributions so far
//   [55]    a contribution was -inf, below -2^16, or NaN
//   [54]    a contribution was +inf, above +2^16, or NaN
//   [53:0]  sum of (v + kBias), v = partial * 2^31 rounded, |partial| <= 2^16
// kMaxContrib contributions of at most 2^48 + 2^47 each stay below 2^54 (40 * 1.5 = 60 < 64).  Integer
// addition is associative, so the total does not depend on the arrival order.
// The two flags are set with an atomic OR that precedes the contributor's add
// (same lane, same address: performed in program order), so they are sticky and
// every later reader of the word sees them.
constexpr unsigned long long kCountOne = 1ull << 56;
constexpr unsigned long long kFlagNeg = 1ull << 55;
constexpr unsigned long long kFlagPos = 1ull << 54;
constexpr unsigned long long kSumMask = kFlagPos - 1;
constexpr long long kBias = 1ll << 48;
constexpr double kFixedScale = 2147483648.0;  // 2^31
constexpr float kFixedScaleF = 2147483648.0f;

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

// compile-time input transform of a kernel instance
constexpr int kXNone = 0, kXNorm = 1, kXGate = 2;
constexpr int kXDynamic = 3;  // chained problems: one of the three, chosen at run time

// Division by a run-time constant without a divide: n / d == umulhi((2 * n) >> shift,
// magic), with the pair prepared on the host (kernels here start and end within a
// few microseconds; a software division is some thirty instructions on that path).
// d = 2^t * o (o odd): for o == 1 the pair is (t, 2^31 + 1), i.e. (2n >> t) / 2;
// otherwise (t + 1, floor(2^32 / o) + 1), i.e. (n >> t) / o.  The multiply-high is
// exact while 2 * n * d < 2^32, which the host checks for every divisor it hands over.
struct Divisor {
    int shift;
    uint32_t magic;
};

inline Divisor make_divisor(int d_in)
{
    int t = 0;
    unsigned d = (unsigned)d_in;
    while ((d & 1u) == 0) {
        d >>= 1;
        ++t;
    }
    Divisor r;
    if (d == 1) {
        r.shift = t;
        r.magic = 0x80000001u;
    } else {
        r.shift = t + 1;
        r.magic = (uint32_t)((1ull << 32) / d) + 1u;
    }
    return r;
}

__device__ __forceinline__ int fast_div(int n, const Divisor &d)
{
    return (int)__umulhi((uint32_t)(2 * n) >> d.shift, d.magic);
}

// Field order: a kernel fetches its arguments a cache line at a time, on demand, and
// each line touched for the first time before the sign words are requested is a round
// trip on the start-up path.  What the kernels need to issue their first loads comes
// first (two 64-byte lines), what the hand-over of finished sums needs comes last.
struct Problem {
    // ---- cache line 0: every kernel's first requests ---------------------------------------
    const uint32_t *W;
    const void *alpha;
    const __half *x;
    const float *sumsq_in;  // split RMSNorm, consuming side: [M][sumsq_slots] (see below)
    int N, K, M;
    int kwords;          // K / 32
    int nsets;           // look-up kernel: ceil(kwords / 8); matrix-core kernel: K-steps
    int n_tiles;
    int group_words;     // row-wise / uniform: words per alpha group
    int nb;
    // ---- cache line 1: the rest of what is needed to request the first operands ------------
    Divisor by_group_words;  // row / group_words
    Divisor by_nsets;        // item / nsets
    // Look-up kernel: the (tile, set) items of one row chunk, tile-major, are cut
    // into `wgs_per_chunk` contiguous ranges: the first `long_ranges` of `items_per_wg`
    // items, the others, from item `split_item` on, of `short_items`.
    int items_per_wg;
    int long_ranges;
    int short_items;
    int split_item;      // long_ranges * items_per_wg
    int mchunks;         // activation rows are handled in chunks
    int n_blocks;        // workgroups of this problem
    int wgs_per_chunk;
    int sumsq_slots;
    int R;               // block modes: row groups
    int rows_per_group;  // block modes: N / R
    const __half *norm_w;  // non-null: y = rsqrt(mean(x^2) + norm_eps) * W(fp16(x * norm_w))
    // ---- cache line 2 ----------------------------------------------------------------------
    const __half *gate;    // non-null [M][K]: the input is fp16(fp16(silu(gate)) * x)
    const __half *qbias;
    __half *out;
    unsigned long long *accum;  // [M][N] fixed-point words, zero between launches
    Divisor by_items;        // item / items_per_wg
    Divisor by_short_items;  // item / short_items
    // Matrix-core kernel: K-steps per K-slice and slices per tile.
    int sets_per_split;
    int ksplit;
    float norm_eps;
    int twin;            // look-up kernel: 1 = the items are twin items (n_tiles counts tile pairs)
    // ---- cache line 3: needed when sums are handed over --------------------------------------
    int overwrite;       // 1: out = y instead of out += y
    // RMSNorm split over two launches (fused entry point only).  The launch that completes
    // a residual row also leaves next_in = fp16(out * next_w) and adds the squares of its
    // outputs, 32 columns at a time, into sumsq_out[m][n / 32]; the launch that consumes
    // next_in scales its sums by rsqrt(sum(sumsq_in[m][0 .. sumsq_slots)) / K + norm_eps).
    const __half *next_w;   // [N]
    __half *next_in;        // [M][N]
    float *sumsq_out;       // [M][N / 32], zero before the launch
    // Chained launches (lut_gemv_chain_kernel): a tag base of 0 means plain fp16 values; otherwise
    // x / gate / out point at TAGGED rows, one 32-bit word per value = fp16 bits | tag << 16
    // (see tagged_word below), x and gate are waited for, out is written with its tag.
    int x_tag, gate_tag, out_tag;
    int reserved2_;
#ifdef LUTGEMM_TIMESTAMPS
    // Build with per-wave time stamps (the library variant bench.py --profile-phases loads):
    // kStampsPerWave readings of the 100 MHz wall clock per wave, at fixed points of the
    // look-up kernel, into stamps[((workgroup of the grid) * kWaves + wave) * kStampsPerWave + point].
    unsigned long long *stamps;
    long long stamp_slots;   // capacity in readings
#endif
};
static_assert(offsetof(Problem, by_group_words) == 64 && offsetof(Problem, gate) == 128 && offsetof(Problem, overwrite) == 192,
              "Problem: fields are grouped by cache line");

struct Group {
    int count;
    Problem p[kMaxGroup];
};

// Tagged rows: how the problems of ONE launch hand activations to each other while all of them are
// in flight.  A producer writes every finished value as one 32-bit word, fp16 bits | tag << 16,
// with an agent-scope store (written through to memory, past the producer's L2); a consumer reads
// the words it needs with agent-scope loads until all of them carry the tag it expects.  Value and
// tag travel in one word, so no counter, no fence and no second round trip are needed: the
// hand-over costs one store and one load latency.  The effective tag of base b in a launch whose
// epoch word reads e is 1 + (b + e) % 65535: never 0, so zero-filled memory never matches, and
// advancing the epoch between replays of a captured launch makes last replay's words stale.
__host__ __device__ inline uint32_t effective_tag(int base, uint32_t epoch)
{
    return 1u + (uint32_t)(((unsigned long long)(uint32_t)base + epoch) % 65535ull);
}

struct ChainControl {
    const uint32_t *epoch;   // device word added to every tag base (may be null: 0)
    uint32_t *status;        // device word: bit 0 is set when a wait gave up
    long long spin_ticks;    // bound of every wait, in ticks of the 100 MHz wall clock
};

// A chained launch is persistent: `grid` workgroups, all resident at once, walk the launch's
// units (a unit = one workgroup's range of one problem, numbered problem by problem) in steps of
// `grid`.  unit_start[y] is the first unit of problem y, unit_start[count] the number of units.
struct Chain {
    Group g;
    ChainControl ctl;
    int unit_start[kMaxGroup + 1];
    int reserved_;
};

// Points of the look-up kernel at which the time-stamped build reads the clock.
constexpr int kStampsPerWave = 8;
enum StampPoint : int {
    kStampEntry = 0,       // first instruction of the workgroup
    kStampRequested = 1,   // the first operands (sign words, alphas) have been requested
    kStampInputs = 2,      // the activations have arrived (and, in a chained launch, carry their tags)
    kStampTables = 3,      // first tables built, first barrier passed
    kStampFirstItem = 4,   // first item looked up
    kStampItems = 5,       // all items looked up (the last hand-over is next)
    kStampHandedOver = 6,  // sums handed over: atomics returned, outputs written
    kStampExit = 7,
};

// `wg`: the workgroup's slot among the readings (its place in the grid, or the unit it works on in a
// persistent launch); `row`: its row of the grid or the problem it works on.
__device__ __forceinline__ void stamp(const Problem &p, int point, long long wg, int row)
{
#ifdef LUTGEMM_TIMESTAMPS
    if (p.stamps && (threadIdx.x & 63) == 0) {
        const long long at = (wg * kWaves + (threadIdx.x >> 6)) * kStampsPerWave + point;
        // (the clock needs 56 bits in 22 years: the top byte names the row)
        if (at < p.stamp_slots) p.stamps[at] = (wall_clock64() & ((1ull << 56) - 1)) | ((unsigned long long)row << 56);
    }
#else
    (void)p;
    (void)point;
    (void)wg;
    (void)row;
#endif
}

__device__ __forceinline__ float half_bits_to_float(uint32_t bits16)
{
    return __half2float(__ushort_as_half((unsigned short)bits16));
}

__device__ __forceinline__ uint32_t float_to_half_bits(float f)
{
    return (uint32_t)__half_as_ushort(__float2half_rn(f));
}

// The value of another lane of the same row of 16, by a data-parallel-primitive move.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v)
{
    const int vi = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(vi, vi, CTRL, 0xf, 0xf, false));
}

// Sum over the 64 lanes of a wave, on the vector ALU: xor 1 and 2 inside quads, then the
// mirrored quad and the mirrored half of each row of 16, then the four rows.
__device__ __forceinline__ float wave_sum(float v)
{
    v += dpp_move<0xb1>(v);   // quad_perm [1,0,3,2]
    v += dpp_move<0x4e>(v);   // quad_perm [2,3,0,1]
    v += dpp_move<0x141>(v);  // row_half_mirror
    v += dpp_move<0x140>(v);  // row_mirror
    const int vi = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 0)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 16)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 32)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 48));
}

// One partial sum as a contribution to an accumulator word: the addend, and the
// flags to OR in first (0 for every finite partial sum within range).
struct Contribution {
    unsigned long long add, flags;
};

__device__ __forceinline__ Contribution fixed_contribution(float v)
{
    Contribution c;
    c.flags = 0;
    if (!(v <= 65536.0f)) c.flags |= kFlagPos;   // +inf, too large, NaN
    if (!(v >= -65536.0f)) c.flags |= kFlagNeg;  // -inf, too small, NaN
    v = c.flags ? 0.0f : v;
    // rn(v * 2^31) without double arithmetic: v = hi + lo with hi = rn(v * 2^7) / 2^7 (an
    // integer of at most 24 bits times 2^-7) and lo = v - hi (exact, |lo| <= 2^-8), so
    // v * 2^31 = (hi * 2^7) * 2^24 + lo * 2^31, and only the second term needs rounding.
    const float hi7 = rintf(v * 128.0f);
    const float lo = fmaf(hi7, -1.0f / 128.0f, v);
    const long long fx = ((long long)(int)hi7 << 24) + (long long)(int)rintf(lo * kFixedScaleF);
    c.add = (unsigned long long)(fx + kBias) + kCountOne;
    return c;
}

// The value of a complete accumulator word (`count` contributions).
__device__ __forceinline__ float fixed_total(unsigned long long word, int count)
{
    const long long total = (long long)(word & kSumMask) - (long long)count * kBias;
    float y = (float)((double)total * (1.0 / kFixedScale));
    const bool pos = word & kFlagPos, neg = word & kFlagNeg;
    if (pos || neg) y = (pos && neg) ? __builtin_nanf("") : pos ? __builtin_inff() : -__builtin_inff();
    return y;
}

}  // namespace lutgemm

#endif
