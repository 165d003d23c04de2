// Table look-up GEMV kernel templates for BCQ linear layers on MI355X (gfx950,
// wave64).  One template covers the five operand formats of the reference
// extension (lut_gemm/mv_fp16_bias.hpp:8-103,105-220,223-328,342-495,498-579 in
// the ShiftAddLLM checkout); the operand layouts are the reference's, the
// execution scheme is not:
//
//  * Work items are (N-tile of 256 outputs, "set" of 256 inputs = 8 sign words =
//    32 eight-input chunks), numbered tile-major.  A workgroup (512 threads = 8
//    waves) takes a contiguous range of items, so every workgroup of a launch
//    has the same amount of work whatever the shape; a range may end one tile's
//    K-slice and begin the next tile's.
//  * Per item the workgroup builds 32 partial-sum tables of 256 fp32 entries in
//    LDS.  Entry i of table t of buffer f sits at byte i*256 + 4*(t + 32*f):
//    every table lives entirely in LDS bank t, and two buffers interleave in the
//    same 64 KiB so that the tables of item i+1 are built while item i is looked
//    up (one barrier per item).  A half-wave is arranged so that its 32 lanes
//    always look up 32 different tables, hence 32 different banks: no bank
//    conflicts by construction, whatever the data-dependent indices are.
//  * The 256-byte entry stride makes a look-up address "index byte in bits
//    8..15, per-lane bank offset in bits 0..7", which ONE v_perm_b32 assembles
//    from the sign word and a per-lane constant; a look-up costs that, the
//    ds_read_b32 and one fma.
//  * Lane l of a wave: q = l&3, kw = (l>>2)&7, h = l>>5.  The lane streams
//    128-bit loads of sign word (set*8 + kw) for the 4 outputs of quad
//    (h*4+q); rows of the sign matrix are read in 1 KiB contiguous runs per
//    workgroup.  At look-up step j the lane uses byte (j+q)&3 of its word,
//    i.e. table kw*4 + ((j+q)&3) -- distinct over (kw, q).
//  * Two register buffers hold the operands of items i and i+1: the loads of
//    item i+1 are issued before the tables of item i are built and looked up,
//    so a load has a whole item's time to arrive, and the first two items of a
//    range are requested before anything is waited for.
//  * Accumulation is fp32; alphas are applied with one fma per look-up (a
//    power-of-two alpha is then an exact exponent shift).  At the end of a
//    tile's K-slice the 8 kw-lanes of an output are combined by a reduce-scatter
//    over ds_swizzle (4 exchanges), which leaves ONE output per lane, 32
//    consecutive outputs per wave.
//  * K is split over workgroups.  Each adds its partial sums, as 64-bit fixed
//    point, into a per-output accumulator word with ONE returning atomic per
//    lane (a wave's 32 atomics fall into two cache lines); the top byte of the
//    word counts contributions, so the contributor that completes the count owns
//    the sum, adds the caller's fp16 output, rounds once and clears the word.
//    Integer addition is associative: the result does not depend on arrival
//    order.  No fences (a device-scope release costs tens of microseconds here)
//    and no second pass.
#ifndef LUT_GEMV_DEVICE_H
#define LUT_GEMV_DEVICE_H

#include <type_traits>

#include "lutgemm_common.h"

namespace lutgemm {

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

// Everything one lane needs from global memory for one item.
template <int NB, int MODE>
struct ItemOperands {
    u32x4 w[NB];        // sign words: 4 outputs x 32 inputs per register quad
    u32x2 a_row[NB];    // row-wise: 4 fp16 alphas (one per output)
    float a_blk[NB][4]; // block: one multiplier per look-up step
    u32x2 a_uni;        // uniform: alpha per output
    u32x2 q_uni;        // uniform: q_bias per output
    float a_stage;      // staged block modes: the one alpha this thread stages
    int rgroup;         // staged block modes: alpha row group of the lane's quad, relative to the tile's first
};

// Issue every global load of item (tile, set) for this lane.  Branch-free on
// purpose: out-of-range rows and columns are clamped to valid addresses instead
// of predicated, so the loads sit in straight-line code and the compiler can
// keep later items' loads in flight (s_waitcnt vmcnt(n), n > 0) while the
// current item is consumed.  Clamped data is harmless: tables of inputs beyond K
// are all zero, and outputs beyond N are never written.  An item that does not
// exist (`valid` false, the slot after the last item of a range) is "loaded" too,
// with every lane pointed at the first words of the operands: a handful of cache
// lines instead of a conditional load.  Addresses are a uniform 64-bit base plus a
// 32-bit per-lane offset.
// PARTS: 1 = the sign words only, 2 = everything else (alphas), 3 = both.
template <int NB, int MODE, int PARTS = 3>
__device__ __forceinline__ void load_item(ItemOperands<NB, MODE> &r, const Problem &p, int tile, int set, bool valid,
                                          int kw, int q, int lane_col, int tid)
{
    tile = valid ? tile : 0;
    set = valid ? set : 0;
    const uint32_t lane_mask = valid ? ~0u : 0u;
    const int tile0 = tile * kTileCols;
    const int n = min(tile0 + lane_col, p.N - 4);
    const uint32_t col4 = (uint32_t)n * 4u, col2 = (uint32_t)n * 2u;
    const int kwc = min(kw, p.kwords - 1 - set * kSetWords);  // only the last set of K can clamp
    const uint32_t row_bytes = (uint32_t)p.N * 4u;            // one bit plane of one sign word row
    const char *wbase = (const char *)p.W + (size_t)set * kSetWords * NB * row_bytes;
    const uint32_t wrow = (uint32_t)kwc * (NB * row_bytes);
    [[maybe_unused]] const int row = set * kSetWords + kwc;
    [[maybe_unused]] const int g = fast_div(row, p.by_group_words);  // alpha group of the row
    const uint32_t woff = (wrow + col4) & lane_mask;
    if constexpr (PARTS & 1) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const char *src = wbase + (size_t)b * row_bytes;
            r.w[b] = __builtin_nontemporal_load((const u32x4 *)(src + woff));
        }
    }
    if constexpr (!(PARTS & 2)) return;
    if constexpr (MODE == kRowF16) {
        const uint32_t aoff = ((uint32_t)g * (NB * (uint32_t)p.N * 2u) + col2) & lane_mask;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const char *src = (const char *)p.alpha + (size_t)b * p.N * 2u;
            r.a_row[b] = *(const u32x2 *)(src + aoff);
        }
    } else if constexpr (MODE == kUniformF16) {
        const uint32_t aoff = ((uint32_t)g * ((uint32_t)p.N * 2u) + col2) & lane_mask;
        r.a_uni = *(const u32x2 *)((const char *)p.alpha + aoff);
        r.q_uni = *(const u32x2 *)((const char *)p.qbias + aoff);
    } else if constexpr (is_block(MODE)) {
        const int rgroup = n / p.rows_per_group;
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int chunk = row * 4 + ((j + q) & 3);
                r.a_blk[b][j] = load_block_alpha<MODE>(p.alpha, ((size_t)chunk * NB + b) * p.R + rgroup);
            }
    }
    if constexpr (is_staged(MODE)) {
        // thread t stages alpha(chunk c of the set, bit b, row group rg0 + g2)
        const int rg0 = tile0 / p.rows_per_group;
        r.rgroup = n / p.rows_per_group - rg0;
        const int t = tid % (2 * NB * kTables);
        const int c = t % kTables, b = (t / kTables) % NB, g2 = t / (NB * kTables);
        const int chunk = min(set * kTables + c, p.K / 8 - 1);
        const int rg = min(rg0 + g2, p.R - 1);
        r.a_stage = load_block_alpha<base_mode(MODE)>(p.alpha, ((size_t)chunk * NB + b) * p.R + rg);
    }
}

// Staged block modes: publish this thread's alpha of an item into stage buffer `abuf`.
template <int NB, int MODE>
__device__ __forceinline__ void stage_alpha(const ItemOperands<NB, MODE> &ops, float *stage, int abuf, int tid)
{
    if constexpr (is_staged(MODE)) {
        if (tid < 2 * NB * kTables) {
            const int c = tid % kTables, b = (tid / kTables) % NB, g2 = tid / (NB * kTables);
            stage[((abuf * 2 + g2) * 4 + b) * kTables + c] = ops.a_stage;
        }
    }
}

// Activation window.  The activations a workgroup needs are few (512 bytes per item
// and row), so they are not fetched item by item: thread t of the workgroup loads ONE
// 16-byte chunk (8 inputs) of a window of kWindowSlots/MROWS consecutive items, applies
// the fused input transform to it once, and parks it in LDS, where the table builds
// read it.  The builds then wait for no global load at all, and the loads that stream
// sign words are the only ones in the (in-order) return queue of the steady state.
// Window layout: [row][slot = item index within the range, modulo slots per row][chunk].
constexpr int kWindowSlots = kThreads / kTables;       // 16 (item, row) slots of 32 chunks
constexpr int kWindowDwords = kWindowSlots * kTables * 4;  // 8 KiB

// What thread `tid` fetches for the window that starts `first_rel` items into the range.
struct WindowChunk {
    u32x4 x, other;
    int kc;     // first input of the chunk (clamped into the row)
    bool live;  // chunks beyond K, or of items beyond the range, read as zero
};

// Which chunk of the window that starts `first_rel` items into the range thread `tid` fetches:
// the element offset of its first input in x (and gate), the first input itself (clamped into the
// row) and whether the chunk is live.
struct WindowIndex {
    size_t base;
    int kc;
    bool live;
};

template <int MROWS>
__device__ __forceinline__ WindowIndex window_index(const Problem &p, int m0, int set0, int first_rel, int n_items, int tid)
{
    constexpr int kSlots = kWindowSlots / MROWS;  // items per window
    const int c = tid % kTables, slot = (tid / kTables) % kSlots, row = tid / (kTables * kSlots);
    const int rel = first_rel + slot;
    const int v = set0 + rel;
    const int set = v - fast_div(v, p.by_nsets) * p.nsets;
    const int k0 = (set * kTables + c) * 8;
    WindowIndex w;
    w.kc = min(k0, p.K - 8);
    w.base = (size_t)min(m0 + row, p.M - 1) * p.K + w.kc;
    w.live = k0 < p.K && rel < n_items;
    return w;
}

template <int MROWS, int XF>
__device__ __forceinline__ WindowChunk fetch_window(const Problem &p, int m0, int set0, int first_rel, int n_items,
                                                    int tid)
{
    const WindowIndex i = window_index<MROWS>(p, m0, set0, first_rel, n_items, tid);
    WindowChunk w;
    w.x = *(const u32x4 *)(p.x + i.base);
    w.other = (u32x4){0u, 0u, 0u, 0u};
    if constexpr (XF == kXGate) w.other = *(const u32x4 *)(p.gate + i.base);
    if constexpr (XF == kXNorm) w.other = *(const u32x4 *)(p.norm_w + i.kc);
    w.kc = i.kc;
    w.live = i.live;
    return w;
}

// ---- tagged rows (chained launches) ------------------------------------------------------------
// What a workgroup of a chained launch needs to wait: the launch's epoch, where to report a wait
// that gave up, and how long a wait may last.
struct ChainWait {
    uint32_t epoch;
    uint32_t *status;
    long long spin_ticks;
    int unit, problem;   // of the launch (for the time-stamped build)
};

// Read NCH chunks of eight tagged words each (32 bytes at src[c]) until every word of every lane
// of the wave carries its tag want[c] (already shifted into the upper half); returns the eight
// fp16 values of each chunk packed into 16 bytes.  Returns false when the wait gave up: the
// launch's status word is set (by this wave after spin_ticks, or by another wave earlier) and
// the values are meaningless.  The loads bypass the L2 (agent scope), which other workgroups'
// stores are written through.  One asm statement holds the requests and their wait: the
// compiler may place nothing that reads the destination registers in between.
// A wave that finds a word without its tag does not read everything again at once (two thousand
// waves re-reading kilobytes each microsecond would take a good part of the memory system from
// the producers they wait for): it watches that one word, one four-byte request per round trip,
// and reads everything again when the word has arrived.
template <int NCH>
__device__ __forceinline__ bool poll_tagged(const uint32_t *const (&src)[NCH], const uint32_t (&want)[NCH], u32x4 (&out)[NCH],
                                            const ChainWait &cw)
{
    static_assert(NCH >= 1 && NCH <= 3, "one to three chunks per thread");
    const long long t0 = wall_clock64();
    for (;;) {
        u32x4 lo[NCH], hi[NCH];
        if constexpr (NCH == 1)
            asm volatile("global_load_dwordx4 %0, %2, off sc1\n\t"
                         "global_load_dwordx4 %1, %2, off offset:16 sc1\n\t"
                         "s_waitcnt vmcnt(0)"
                         : "=&v"(lo[0]), "=&v"(hi[0]) : "v"(src[0]) : "memory");
        else if constexpr (NCH == 2)
            asm volatile("global_load_dwordx4 %0, %4, off sc1\n\t"
                         "global_load_dwordx4 %1, %4, off offset:16 sc1\n\t"
                         "global_load_dwordx4 %2, %5, off sc1\n\t"
                         "global_load_dwordx4 %3, %5, off offset:16 sc1\n\t"
                         "s_waitcnt vmcnt(0)"
                         : "=&v"(lo[0]), "=&v"(hi[0]), "=&v"(lo[1]), "=&v"(hi[1]) : "v"(src[0]), "v"(src[1]) : "memory");
        else
            asm volatile("global_load_dwordx4 %0, %6, off sc1\n\t"
                         "global_load_dwordx4 %1, %6, off offset:16 sc1\n\t"
                         "global_load_dwordx4 %2, %7, off sc1\n\t"
                         "global_load_dwordx4 %3, %7, off offset:16 sc1\n\t"
                         "global_load_dwordx4 %4, %8, off sc1\n\t"
                         "global_load_dwordx4 %5, %8, off offset:16 sc1\n\t"
                         "s_waitcnt vmcnt(0)"
                         : "=&v"(lo[0]), "=&v"(hi[0]), "=&v"(lo[1]), "=&v"(hi[1]), "=&v"(lo[2]), "=&v"(hi[2])
                         : "v"(src[0]), "v"(src[1]), "v"(src[2]) : "memory");
        // the first word that does not carry its tag yet (-1: all of this lane's words do)
        int missing = -1;
#pragma unroll
        for (int c = NCH - 1; c >= 0; --c) {
            const uint32_t w = want[c];
            const uint32_t got8[8] = {lo[c].x, lo[c].y, lo[c].z, lo[c].w, hi[c].x, hi[c].y, hi[c].z, hi[c].w};
#pragma unroll
            for (int i = 7; i >= 0; --i) missing = ((got8[i] ^ w) & 0xffff0000u) ? 8 * c + i : missing;
        }
        const unsigned long long late = __builtin_amdgcn_ballot_w64(missing >= 0);
        if (late == 0) {
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                out[c].x = __builtin_amdgcn_perm(lo[c].y, lo[c].x, 0x05040100u);
                out[c].y = __builtin_amdgcn_perm(lo[c].w, lo[c].z, 0x05040100u);
                out[c].z = __builtin_amdgcn_perm(hi[c].y, hi[c].x, 0x05040100u);
                out[c].w = __builtin_amdgcn_perm(hi[c].w, hi[c].z, 0x05040100u);
            }
            return true;
        }
        // watch the missing word of the first lane that has one (the same address in every lane:
        // one request)
        const int first = (int)__builtin_ctzll(late);
        const int which = __builtin_amdgcn_readlane(missing, first);
        const uint32_t *chunk = src[0];
        uint32_t watch_want = want[0];
#pragma unroll
        for (int c = 1; c < NCH; ++c)
            if ((which >> 3) == c) {
                chunk = src[c];
                watch_want = want[c];
            }
        const unsigned long long addr = (unsigned long long)(chunk + (which & 7));
        const uint32_t *watch = (const uint32_t *)(((unsigned long long)(uint32_t)__builtin_amdgcn_readlane((int)(addr >> 32), first) << 32) |
                                                   (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)addr, first));
        watch_want = (uint32_t)__builtin_amdgcn_readlane((int)watch_want, first);
        for (;;) {
            const uint32_t v = __hip_atomic_load(watch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (((v ^ watch_want) & 0xffff0000u) == 0) break;
            if (__hip_atomic_load(cw.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) return false;
            if (wall_clock64() - t0 > cw.spin_ticks) {
                if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_or(cw.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                return false;
            }
            __builtin_amdgcn_s_sleep(4);
        }
    }
}

// Transform the chunk and park it in the window.  With a gate row the chunk is
// multiplied by silu(gate), with the roundings of the separate fp16 operations this
// replaces.  With a norm weight it is multiplied by the weight only: the tables are
// linear in their inputs, so the row's reciprocal RMS is applied to the finished sums
// instead (flush_tile) and the reduction that yields it is not waited for here.
// (x * weight is held as fp16: it must stay below 65504.)
// XF == kXDynamic: the transform is `xf`, known at run time (uniform over the workgroup).
template <int MROWS, int XF>
__device__ __forceinline__ void store_window(const WindowChunk &w, float *window, int tid, int xf = XF)
{
    u32x4 xr = w.x;
    // (opaque: the work on the fetched chunk stays here, after the sign-word requests,
    // instead of being hoisted to where it would have to wait for the chunk first)
    asm volatile("" : "+v"(xr.x), "+v"(xr.y), "+v"(xr.z), "+v"(xr.w));
    if constexpr (XF == kXDynamic) {
        if (xf != kXNone) {
            const u32x4 other = w.other;
            const uint32_t a[4] = {xr.x, xr.y, xr.z, xr.w};
            const uint32_t b[4] = {other.x, other.y, other.z, other.w};
            uint32_t o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float v[2];
#pragma unroll
                for (int hh = 0; hh < 2; ++hh) {
                    const float xv = half_bits_to_float((a[j] >> (16 * hh)) & 0xffffu);
                    const float bv = half_bits_to_float((b[j] >> (16 * hh)) & 0xffffu);
                    const float silu = half_bits_to_float(float_to_half_bits(__fdividef(bv, 1.0f + __expf(-bv))));
                    v[hh] = xv * (xf == kXGate ? silu : bv);
                }
                o[j] = float_to_half_bits(v[0]) | (float_to_half_bits(v[1]) << 16);
            }
            xr = (u32x4){o[0], o[1], o[2], o[3]};
        }
    } else if constexpr (XF != kXNone) {
        const u32x4 other = w.other;
        const uint32_t a[4] = {xr.x, xr.y, xr.z, xr.w};
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
                    v[hh] = xv * bv;
            }
            o[j] = float_to_half_bits(v[0]) | (float_to_half_bits(v[1]) << 16);
        }
        xr = (u32x4){o[0], o[1], o[2], o[3]};
    }
    u32x4 r;
    r.x = w.live ? xr.x : 0u;
    r.y = w.live ? xr.y : 0u;
    r.z = w.live ? xr.z : 0u;
    r.w = w.live ? xr.w : 0u;
    *(u32x4 *)(window + 4 * tid) = r;
}

// Build the 32 tables of one item into buffer `buf` (0/1).  Thread (tb, eb)
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

// The same for two activation rows at once: an entry is the pair (row a, row b) as two
// fp16 halves of one word, so that one look-up serves both rows.  The sums are formed
// in fp32 like the single-row tables and rounded once when packed (the reference's own
// tables are fp16 sums of fp16 values, mv_fp16_bias.hpp:342-380).
__device__ __forceinline__ uint32_t pack_entry(float a, float b)
{
    const __half2 h = __floats2half2_rn(a, b);
    return __builtin_bit_cast(uint32_t, h);
}

__device__ __forceinline__ void build_tables_pair(const u32x4 &xa, const u32x4 &xb, float *lut, int buf, int tb, int eb)
{
    float a2[8], b2[8];  // 2 * x of either row
    float base_a = 0.0f, base_b = 0.0f;
    const uint32_t ra[4] = {xa.x, xa.y, xa.z, xa.w};
    const uint32_t rb[4] = {xb.x, xb.y, xb.z, xb.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float alo = half_bits_to_float(ra[j] & 0xffffu), ahi = half_bits_to_float(ra[j] >> 16);
        const float blo = half_bits_to_float(rb[j] & 0xffffu), bhi = half_bits_to_float(rb[j] >> 16);
        a2[2 * j] = alo + alo;
        a2[2 * j + 1] = ahi + ahi;
        b2[2 * j] = blo + blo;
        b2[2 * j + 1] = bhi + bhi;
        base_a -= alo + ahi;
        base_b -= blo + bhi;
    }
    float top_a = base_a, top_b = base_b;
#pragma unroll
    for (int j = 4; j < 8; ++j)
        if ((eb >> (j - 4)) & 1) {
            top_a += a2[j];
            top_b += b2[j];
        }
    uint32_t *col = (uint32_t *)lut + (eb * 16) * kEntryStride + buf * kTables + tb;
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
        float va = top_a, vb = top_b;
        if (sb & 1) {
            va += a2[3];
            vb += b2[3];
        }
        unsigned gray = 0;
        col[(sb * 8) * kEntryStride] = pack_entry(va, vb);
#pragma unroll
        for (int i = 1; i < 8; ++i) {
            const int bit = __builtin_ctz(i);
            gray ^= 1u << bit;
            const bool up = (gray >> bit) & 1u;
            va += up ? a2[bit] : -a2[bit];
            vb += up ? b2[bit] : -b2[bit];
            col[(sb * 8 + gray) * kEntryStride] = pack_entry(va, vb);
        }
    }
}

// This lane's look-ups of one item against the table buffer `lane_off` selects.
// lane_off: byte j = 4*(bank of the table used at step j + 32*buffer).
// sel[j]  : v_perm_b32 selector putting byte (j+q)&3 of the sign word into
//           bits 8..15 and byte j of lane_off into bits 0..7.
// Software pipelined in units of 8 look-ups (one bit plane of two outputs): the LDS
// reads of unit u+1 are issued before the fmas of unit u.  (Units of 16 cost 16 more
// registers, which four bit planes do not have to spare.)
template <int NB, int MODE>
__device__ __forceinline__ void lookup_item(const ItemOperands<NB, MODE> &cur, const float *lut, float (&acc)[4],
                                            uint32_t lane_off, const uint32_t (&sel)[4], const float *stage_lane,
                                            int q)
{
    const char *lut_bytes = (const char *)lut;
    constexpr int kUnits = 2 * NB;   // a unit = 8 look-ups: one bit plane of two outputs
    float val[2][8];
    [[maybe_unused]] float aval[2][4];
    auto issue = [&](int u, float (&v)[8], float (&av)[4]) {
        const int b = u >> 1, i0 = (u & 1) * 2;
        const uint32_t w4[4] = {cur.w[b].x, cur.w[b].y, cur.w[b].z, cur.w[b].w};
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                v[4 * i + j] = *(const float *)(lut_bytes + __builtin_amdgcn_perm(w4[i0 + i], lane_off, sel[j]));
        if constexpr (is_staged(MODE)) {
            // stage_lane points at [this item's buffer][group 0][bit 0][kw*4]; the four
            // alphas of the lane's sign word, in look-up step order
            const float *a4 = stage_lane + (cur.rgroup * 4 + b) * kTables;
#pragma unroll
            for (int j = 0; j < 4; ++j) av[j] = a4[(j + q) & 3];
        }
    };
    // Row-wise alphas: the entries of a bit plane are summed as they are and the plane's
    // alpha is applied once, after the item's last look-up, so the alphas (requested after
    // the sign words) are not waited for before that.
    [[maybe_unused]] float part[NB][4];
    if constexpr (MODE == kRowF16) {
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int i = 0; i < 4; ++i) part[b][i] = 0.0f;
    }
    auto retire = [&](int u, const float (&v)[8], const float (&av)[4]) {
        const int b = u >> 1, i0 = (u & 1) * 2;
        if constexpr (MODE == kRowF16) {
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) part[b][i0 + i] += v[4 * i + j];
            if (u == kUnits - 1) {
#pragma unroll
                for (int bb = 0; bb < NB; ++bb) {
                    const uint32_t a2[2] = {cur.a_row[bb].x, cur.a_row[bb].y};
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        acc[i] = fmaf(part[bb][i], half_bits_to_float((a2[i >> 1] >> (16 * (i & 1))) & 0xffffu), acc[i]);
                }
            }
            return;
        }
        [[maybe_unused]] const uint32_t au = (u & 1) ? cur.a_uni.y : cur.a_uni.x;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            float a = 0.0f;
            if constexpr (MODE == kUniformF16)
                a = half_bits_to_float((au >> (16 * i)) & 0xffffu) * (1.0f / (float)(2 << b));
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if constexpr (is_block(MODE))
                    a = cur.a_blk[b][j];
                else if constexpr (is_staged(MODE))
                    a = av[j];
                acc[i0 + i] = fmaf(v[4 * i + j], a, acc[i0 + i]);
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
        const uint32_t rq[2] = {cur.q_uni.x, cur.q_uni.y};
#pragma unroll
        for (int i = 0; i < 4; ++i)
            acc[i] = fmaf(half_bits_to_float((rq[i >> 1] >> (16 * (i & 1))) & 0xffffu), sum_x, acc[i]);
    }
#pragma unroll
    for (int u = 0; u < kUnits; ++u) {
        if (u + 1 < kUnits) issue(u + 1, val[(u + 1) & 1], aval[(u + 1) & 1]);
        retire(u, val[u & 1], aval[u & 1]);
    }
}

// The same against pair tables (build_tables_pair): one look-up, two rows.  Row-wise and
// uniform alphas only.
template <int NB, int MODE>
__device__ __forceinline__ void lookup_item_pair(const ItemOperands<NB, MODE> &cur, const float *lut, float (&acc_a)[4],
                                                 float (&acc_b)[4], uint32_t lane_off, const uint32_t (&sel)[4])
{
    static_assert(MODE == kRowF16 || MODE == kUniformF16, "pair tables: per-column alphas only");
    const char *lut_bytes = (const char *)lut;
    constexpr int kUnits = 2 * NB;
    uint32_t val[2][8];
    auto lo = [](uint32_t w) { return half_bits_to_float(w & 0xffffu); };
    auto hi = [](uint32_t w) { return half_bits_to_float(w >> 16); };
    auto issue = [&](int u, uint32_t (&v)[8]) {
        const int b = u >> 1, i0 = (u & 1) * 2;
        const uint32_t w4[4] = {cur.w[b].x, cur.w[b].y, cur.w[b].z, cur.w[b].w};
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                v[4 * i + j] = *(const uint32_t *)(lut_bytes + __builtin_amdgcn_perm(w4[i0 + i], lane_off, sel[j]));
    };
    auto retire = [&](int u, const uint32_t (&v)[8]) {
        const int b = u >> 1, i0 = (u & 1) * 2;
        [[maybe_unused]] const uint32_t ar = (u & 1) ? cur.a_row[b].y : cur.a_row[b].x;
        [[maybe_unused]] const uint32_t au = (u & 1) ? cur.a_uni.y : cur.a_uni.x;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            float a;
            if constexpr (MODE == kRowF16)
                a = half_bits_to_float((ar >> (16 * i)) & 0xffffu);
            else
                a = half_bits_to_float((au >> (16 * i)) & 0xffffu) * (1.0f / (float)(2 << b));
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc_a[i0 + i] = fmaf(lo(v[4 * i + j]), a, acc_a[i0 + i]);
                acc_b[i0 + i] = fmaf(hi(v[4 * i + j]), a, acc_b[i0 + i]);
            }
        }
    };
    issue(0, val[0]);
    if constexpr (MODE == kUniformF16) {
        // sums of the lane's 32 inputs = entry 255 of its four tables
        float sum_a = 0.0f, sum_b = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t e = *(const uint32_t *)(lut_bytes + 255 * 4 * kEntryStride + ((lane_off >> (8 * j)) & 255u));
            sum_a += lo(e);
            sum_b += hi(e);
        }
        const uint32_t rq[2] = {cur.q_uni.x, cur.q_uni.y};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float qb = half_bits_to_float((rq[i >> 1] >> (16 * (i & 1))) & 0xffffu);
            acc_a[i] = fmaf(qb, sum_a, acc_a[i]);
            acc_b[i] = fmaf(qb, sum_b, acc_b[i]);
        }
    }
#pragma unroll
    for (int u = 0; u < kUnits; ++u) {
        if (u + 1 < kUnits) issue(u + 1, val[(u + 1) & 1]);
        retire(u, val[u & 1]);
    }
}

// ds_swizzle in bit-mask mode: the value of lane (l ^ XOR) within each group of 32.
template <int XOR>
__device__ __forceinline__ float swizzle_xor(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), (XOR << 10) | 0x1f));
}

// Reduce-scatter of the 8 kw-lanes of a quad: each lane comes in with its partial
// sums of 4 outputs and leaves with the complete sum of output
// i = 2*(kw>>2 & 1) + (kw>>1 & 1); lanes kw and kw^1 hold the same value.
__device__ __forceinline__ float reduce_scatter_kw(const float (&acc)[4], int kw)
{
    const bool b2 = (kw >> 2) & 1, b1 = (kw >> 1) & 1;
    float k0 = b2 ? acc[2] : acc[0], k1 = b2 ? acc[3] : acc[1];   // kept
    const float s0 = b2 ? acc[0] : acc[2], s1 = b2 ? acc[1] : acc[3];  // sent to lane ^ 16
    k0 += swizzle_xor<16>(s0);
    k1 += swizzle_xor<16>(s1);
    float k = b1 ? k1 : k0;
    const float s = b1 ? k0 : k1;
    k += swizzle_xor<8>(s);
    k += swizzle_xor<4>(k);
    return k;
}

// One workgroup's share: items [range*items_per_wg, +items_per_wg) of row chunk
// `mchunk` (activation rows mchunk*MROWS .. +MROWS-1).  The sign words of an item
// are loaded once and used for all MROWS rows; tables are built per (item, row)
// and double buffered.
// EXTRA: the launch honours the split-RMSNorm fields of the problem (next_in, sumsq_*).
// ALONE: 1: the first item is requested on its own (see the main loop); 2: the same when no
//       range of the launch holds more than that one item (the host's choice).
// PAIR: rows are taken two at a time through pair tables (fp16 entries; MROWS even,
//       per-column alphas).
// DEP: a problem of a chained launch (`cw` non-null): x, gate and out may be tagged rows.  The
//      operands that depend on nothing (sign words and alphas of the first two items) are
//      requested at once; the activations are waited for, tag by tag, behind them.
// TWIN: the items are "twin" items: the same set of 256 inputs against TWO neighbouring output
//       tiles (512 outputs), so that one table build and one barrier serve two look-up passes.
//       The problem's n_tiles counts tile pairs then, and the planner's items are twin items.
template <int NB, int MODE, int MROWS, int XF = kXNone, bool EXTRA = false, int ALONE = MROWS == 1 && !is_block(MODE),
          bool PAIR = false, bool DEP = false, bool TWIN = false>
__device__ __forceinline__ bool gemv_range(const Problem &p, int range, int mchunk, float *lut, const ChainWait *cw = nullptr)
{
    // Returns false when a chained problem gave up waiting for its inputs (nothing was written).
    [[maybe_unused]] auto stamp = [&](const Problem &pp, int point) {
        if constexpr (DEP)
            lutgemm::stamp(pp, point, cw->unit, cw->problem);
        else
            lutgemm::stamp(pp, point, (long long)blockIdx.y * gridDim.x + blockIdx.x, (int)blockIdx.y);
    };
    static_assert(!PAIR || (MROWS % 2 == 0 && (MODE == kRowF16 || MODE == kUniformF16)), "pair tables: even row count, per-column alphas");
    static_assert(!(EXTRA || XF == kXNorm) || !is_staged(MODE), "the per-wave sums live in the alpha staging area");
    static_assert(!DEP || (MROWS == 1 && MODE == kRowF16 && !EXTRA && !PAIR), "chained launches: one row per workgroup, row-wise alphas");
    static_assert(DEP == (XF == kXDynamic), "chained problems choose their transform at run time, the others at compile time");
    static_assert(!TWIN || (MROWS == 1 && ALONE == 1 && !EXTRA && !PAIR && !DEP), "twin items: one row, first item alone, no extras");
    constexpr int kMembers = TWIN ? 2 : 1;   // output tiles per item
    // the transform: a compile-time constant except for chained problems (one kernel holds them
    // all, and an instance per bit width and transform is more than the compiler digests: from
    // eight instances of this function on, it emits an empty kernel)
    [[maybe_unused]] const int xf = XF != kXDynamic ? XF : p.norm_w ? kXNorm : p.gate ? kXGate : kXNone;
    constexpr bool kMayNorm = XF == kXNorm || XF == kXDynamic;
    stamp(p, kStampEntry);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int q = lane & 3;
    const int kw = (lane >> 2) & 7;
    const int h = lane >> 5;
    const int lane_col = wave * kWaveCols + (h * 4 + q) * 4;  // first of the lane's 4 outputs within a tile
    const int m0 = mchunk * MROWS;
    // The output this lane owns after the reduce-scatter: own_col(kw2) with kw2 = kw.  (A
    // function of the caller's copy of kw so that uses late in the kernel can pass an
    // opaque copy and keep their setup out of the start-up path.)
    auto own_col_of = [&](int kw2) { return lane_col + 2 * ((kw2 >> 2) & 1) + ((kw2 >> 1) & 1); };

    // rows beyond M are clamped to the last row (computed twice, written once)
    const __half *xrow[MROWS];
#pragma unroll
    for (int r = 0; r < MROWS; ++r) xrow[r] = p.x + (size_t)min(m0 + r, p.M - 1) * p.K;

    // Per-lane look-up constants (see lookup_item).  Like everything else that the first
    // requests do not depend on, they are formed after those requests have been issued
    // (late_setup below): a workgroup's waves share their SIMDs' issue slots, and each
    // hundred instructions ahead of the first load are a third of a microsecond.
    uint32_t lane_off = 0;
    uint32_t sel[4] = {0u, 0u, 0u, 0u};

    float acc[MROWS][4];
#pragma unroll
    for (int r = 0; r < MROWS; ++r)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[r][i] = 0.0f;
    [[maybe_unused]] float acc_twin[4] = {0.0f, 0.0f, 0.0f, 0.0f};   // the item's second tile

    // table-build role of this thread
    const int tb = tid & 31;  // table (bank)
    const int eb = tid >> 5;  // entries eb*16 .. eb*16+15

    // this workgroup's items; (tile, set) is the current one
    const int total = p.n_tiles * p.nsets;
    // (branch-free: a branch here becomes one more round of scalar loads ahead of the first requests)
    const int beyond = range - p.long_ranges;  // >= 0: a short range
    const int item0 = min(range, p.long_ranges) * p.items_per_wg + max(beyond, 0) * p.short_items;
    int rem = min(p.short_items + (beyond < 0 ? p.items_per_wg - p.short_items : 0), total - item0);
    int tile = fast_div(item0, p.by_nsets), set = item0 - tile * p.nsets;
    auto advance = [&](int &t, int &s) {
        if (++s == p.nsets) {
            s = 0;
            ++t;
        }
    };

    float *stage = lut + kLutDwords;
    int abuf = 0;

    // The first activation window is requested before anything else.
    constexpr int kSlots = kWindowSlots / MROWS;  // items per window
    const int set0 = set, n_items = rem;
    float *window = stage + kStageDwords;
    // (a chained problem that waits for a tag requests its activations later, behind the first
    // item's sign words)
    WindowChunk w0;
    if constexpr (!DEP) w0 = fetch_window<MROWS, XF>(p, m0, set0, 0, n_items, tid);
    [[maybe_unused]] const bool chain_waits = DEP && (p.x_tag != 0 || p.gate_tag != 0);
    constexpr bool kDirectFirst = XF == kXNone && !PAIR && !DEP;
    // Without an input transform the tables of the first item (row 0) are built straight
    // from a second request for this thread's own chunk, so that nothing but that chunk
    // stands between the start of the kernel and the first table.
    u32x4 x0 = (u32x4){0u, 0u, 0u, 0u};
    if constexpr (kDirectFirst) {
        const int k0 = (set0 * kTables + tb) * 8;
        x0 = *(const u32x4 *)(xrow[0] + min(k0, p.K - 8));
    }

    // fused RMSNorm: every workgroup forms the reciprocal RMS of its rows itself (K
    // fp16 values per row, from L2), requested right behind the window.
    constexpr int kNormChunks = 2;  // 16-byte chunks per thread held in registers: K <= 8192
    u32x4 nx[kMayNorm ? MROWS : 1][kNormChunks];
    if constexpr (XF == kXNorm && !DEP) {
#pragma unroll
        for (int r = 0; r < MROWS; ++r)
#pragma unroll
            for (int u = 0; u < kNormChunks; ++u)
                nx[r][u] = *(const u32x4 *)(xrow[r] + 8 * min(tid + kThreads * u, p.K / 8 - 1));
    }
    // Chained problem: the activations this thread needs (its chunk of the first window, with a
    // gate row the same chunk of that, with a norm its share of the whole row), each from a plain
    // fp16 row (written before the launch) or from a tagged row that an earlier problem of the
    // launch is still writing.  False when a wait gave up.
    [[maybe_unused]] uint32_t out_tagw = 0;
    auto chain_inputs = [&]() -> bool {
        if constexpr (!DEP) {
            return true;
        } else {
            const WindowIndex wi = window_index<MROWS>(p, m0, set0, 0, n_items, tid);
            w0.kc = wi.kc;
            w0.live = wi.live;
            w0.other = (u32x4){0u, 0u, 0u, 0u};
            const uint32_t xw = effective_tag(p.x_tag, cw->epoch) << 16;
            const uint32_t *xt = (const uint32_t *)p.x;  // tagged: one word per value
            bool ok = true;
            if (xf == kXNorm) {
                w0.other = *(const u32x4 *)(p.norm_w + wi.kc);
                const size_t row0 = (size_t)min(m0, p.M - 1) * p.K;
                const int c0 = 8 * min(tid, p.K / 8 - 1), c1 = 8 * min(tid + kThreads, p.K / 8 - 1);
                if (p.x_tag) {
                    const uint32_t *src[3] = {xt + wi.base, xt + row0 + c0, xt + row0 + c1};
                    const uint32_t want[3] = {xw, xw, xw};
                    u32x4 got[3];
                    ok = poll_tagged<3>(src, want, got, *cw);
                    w0.x = got[0];
                    nx[0][0] = got[1];
                    nx[0][1] = got[2];
                } else {
                    w0.x = *(const u32x4 *)(p.x + wi.base);
                    nx[0][0] = *(const u32x4 *)(p.x + row0 + c0);
                    nx[0][1] = *(const u32x4 *)(p.x + row0 + c1);
                }
            } else if (xf == kXGate) {
                const uint32_t gw = effective_tag(p.gate_tag, cw->epoch) << 16;
                const uint32_t *gt = (const uint32_t *)p.gate;
                if (!p.x_tag) w0.x = *(const u32x4 *)(p.x + wi.base);
                if (!p.gate_tag) w0.other = *(const u32x4 *)(p.gate + wi.base);
                if (p.x_tag && p.gate_tag) {
                    const uint32_t *src[2] = {xt + wi.base, gt + wi.base};
                    const uint32_t want[2] = {xw, gw};
                    u32x4 got[2];
                    ok = poll_tagged<2>(src, want, got, *cw);
                    w0.x = got[0];
                    w0.other = got[1];
                } else if (p.x_tag || p.gate_tag) {
                    const uint32_t *src[1] = {p.x_tag ? xt + wi.base : gt + wi.base};
                    const uint32_t want[1] = {p.x_tag ? xw : gw};
                    u32x4 got[1];
                    ok = poll_tagged<1>(src, want, got, *cw);
                    if (p.x_tag) w0.x = got[0]; else w0.other = got[0];
                }
            } else {
                if (p.x_tag) {
                    const uint32_t *src[1] = {xt + wi.base};
                    const uint32_t want[1] = {xw};
                    u32x4 got[1];
                    ok = poll_tagged<1>(src, want, got, *cw);
                    w0.x = got[0];
                } else {
                    w0.x = *(const u32x4 *)(p.x + wi.base);
                }
            }
            return ok;
        }
    };
    if constexpr (DEP)
        if (!chain_waits) (void)chain_inputs();   // plain rows: requested first, like a lone problem's
    // split RMSNorm, consuming side: this thread's share of the rows' sums of squares
    float slot_sum[MROWS];
#pragma unroll
    for (int r = 0; r < MROWS; ++r) slot_sum[r] = 0.0f;
    if constexpr (EXTRA) {
        // one clamped, unconditional request per row here (a loop would wait for each load,
        // and with it for everything requested above); more than kThreads slots are rare
        // and fetched in first_window
        if (p.sumsq_in) {
#pragma unroll
            for (int r = 0; r < MROWS; ++r)
                slot_sum[r] = p.sumsq_in[(size_t)min(m0 + r, p.M - 1) * p.sumsq_slots + min(tid, p.sumsq_slots - 1)];
        }
    }
    // the caller's output, needed only by whoever completes a sum: fetched early,
    // off the critical path (again whenever the range moves on to another tile)
    unsigned short out_prev[MROWS];
    [[maybe_unused]] unsigned short out_prev_twin = 0;
    auto fetch_out = [&](int t) {
        if constexpr (TWIN) {
            // t counts tile pairs
            const int na = min(2 * t * kTileCols + own_col_of(kw), p.N - 1);
            const int nb2 = min((2 * t + 1) * kTileCols + own_col_of(kw), p.N - 1);
            const unsigned short *row = (const unsigned short *)(p.out + (size_t)min(m0, p.M - 1) * p.N);
            out_prev[0] = row[na];
            out_prev_twin = row[nb2];
            return;
        }
        const int n = min(t * kTileCols + own_col_of(kw), p.N - 1);
        if constexpr (DEP) {
            // a tagged row that an earlier problem of the launch may have completed: its values
            // (whatever their tags) are read past the L2
            if (p.out_tag) {
                out_prev[0] = (unsigned short)__hip_atomic_load((const uint32_t *)p.out + (size_t)min(m0, p.M - 1) * p.N + n,
                                                                __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                return;
            }
        }
#pragma unroll
        for (int r = 0; r < MROWS; ++r)
            out_prev[r] = *((const unsigned short *)(p.out + (size_t)min(m0 + r, p.M - 1) * p.N) + n);
    };
    __builtin_amdgcn_sched_barrier(0);  // keep these requests ahead of the sign words

    // Runs once, after the first operand loads have been issued: everything the look-ups
    // and the hand-over need but the first requests did not.
    auto late_setup = [&]() {
        int t = tid;
        asm volatile("" : "+v"(t));  // (opaque, so that none of this is hoisted ahead of the requests)
        const int lq = t & 3, lkw = (t >> 2) & 7;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int jj = (j + lq) & 3;
            lane_off |= (uint32_t)(4 * (lkw * 4 + jj)) << (8 * j);
            sel[j] = 0x0c0c0000u | ((uint32_t)(4 + jj) << 8) | (uint32_t)j;
        }
    };
    // Also once, after that: park the first window and, with a fused RMSNorm, leave each
    // wave's share of the rows' sums of squares in LDS.  The reciprocal RMS is formed
    // from those behind the barrier and is first needed when sums are handed over.
    auto first_window = [&]() {
        if constexpr (kMayNorm) {
#pragma unroll
            for (int r = 0; r < MROWS; ++r) {
                if (xf != kXNorm) break;
                float ss = 0.0f;
                auto add_chunk = [&](const u32x4 &v) {
                    const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float lo = half_bits_to_float(w4[j] & 0xffffu), hi = half_bits_to_float(w4[j] >> 16);
                        ss = fmaf(lo, lo, fmaf(hi, hi, ss));
                    }
                };
#pragma unroll
                for (int u = 0; u < kNormChunks; ++u)
                    if (tid + kThreads * u < p.K / 8) add_chunk(nx[r][u]);
                if constexpr (!DEP)  // (the host keeps chained norm problems to K <= 8192)
                    for (int c = tid + kThreads * kNormChunks; c < p.K / 8; c += kThreads)  // K > 8192
                        add_chunk(*(const u32x4 *)(xrow[r] + 8 * c));
                ss = wave_sum(ss);
                if (lane == 0) stage[wave * MROWS + r] = ss;
            }
        }
        if constexpr (EXTRA) {
            if (p.sumsq_in) {
#pragma unroll
                for (int r = 0; r < MROWS; ++r) {
                    // (opaque: the work on the fetched value stays here, behind the sign-word
                    // requests, instead of being hoisted to where it would have to wait first)
                    asm volatile("" : "+v"(slot_sum[r]));
                    float v = tid < p.sumsq_slots ? slot_sum[r] : 0.0f;
                    for (int c = tid + kThreads; c < p.sumsq_slots; c += kThreads)
                        v += p.sumsq_in[(size_t)min(m0 + r, p.M - 1) * p.sumsq_slots + c];
                    const float s = wave_sum(v);
                    if (lane == 0) stage[wave * MROWS + r] = s;
                }
            }
        }
        store_window<MROWS, XF>(w0, window, tid, xf);
        stamp(p, kStampInputs);
        // (without a transform the first build does not read the window, and the barrier
        // that follows that build publishes the window as well)
        if constexpr (!kDirectFirst) __syncthreads();
    };
    // A row's reciprocal RMS from the per-wave sums (any time after the first barrier
    // that follows first_window; formed where it is used rather than kept in a register).
    auto row_scale = [&](int r) {
        float t = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) t += stage[w * MROWS + r];
        return rsqrtf(t / (float)p.K + p.norm_eps);
    };

    // ---- hand a tile's complete K-slice over ---------------------------------------
    auto flush_tile = [&](int t) {
        // contributions this tile receives: the ranges that overlap its items
        auto range_of = [&](int item) {
            const int in_long = fast_div(item, p.by_items);
            const int in_short = p.long_ranges + fast_div(max(item - p.split_item, 0), p.by_short_items);
            return item < p.split_item ? in_long : in_short;
        };
        const int count = range_of(t * p.nsets + p.nsets - 1) - range_of(t * p.nsets) + 1;
        int kw2 = kw;
        asm volatile("" : "+v"(kw2));  // (opaque: see own_col_of)
        const bool owner = (kw2 & 1) == 0;
        if constexpr (TWIN) {
            // both tiles of the pair (one row, no extras): both atomics are issued before either
            // result is looked at, so that their round trips overlap
            int n2[2];
            float v2[2];
            Contribution c2[2];
            unsigned long long old2[2] = {0ull, 0ull};
            bool mine[2];
#pragma unroll
            for (int member = 0; member < 2; ++member) {
                n2[member] = (2 * t + member) * kTileCols + own_col_of(kw2);
                v2[member] = reduce_scatter_kw(member ? acc_twin : acc[0], kw2);
#pragma unroll
                for (int i = 0; i < 4; ++i) (member ? acc_twin : acc[0])[i] = 0.0f;
                mine[member] = owner && n2[member] < p.N;
                c2[member] = fixed_contribution(v2[member]);
                if (mine[member] && count > 1) {
                    unsigned long long *word = p.accum + (size_t)m0 * p.N + n2[member];
                    if (c2[member].flags)
                        __hip_atomic_fetch_or(word, c2[member].flags, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    old2[member] = __hip_atomic_fetch_add(word, c2[member].add, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
#pragma unroll
            for (int member = 0; member < 2; ++member) {
                if (!mine[member]) continue;
                __half *dst = p.out + (size_t)m0 * p.N + n2[member];
                const float prev = p.overwrite ? 0.0f : half_bits_to_float(member ? out_prev_twin : out_prev[0]);
                if (count == 1) {
                    *dst = __float2half_rn(prev + v2[member]);
                    continue;
                }
                if ((int)(old2[member] >> 56) != count - 1) continue;
                *dst = __float2half_rn(prev + fixed_total((old2[member] | c2[member].flags) + c2[member].add, count));
                __hip_atomic_store(p.accum + (size_t)m0 * p.N + n2[member], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            return;
        }
        const int n = t * kTileCols + own_col_of(kw2);
        bool scaled = xf == kXNorm;
        if constexpr (EXTRA) scaled = scaled || p.sumsq_in != nullptr;
        // the next norm's weight for this lane's column: requested here, used once the
        // sums are complete
        [[maybe_unused]] unsigned short next_w_bits = 0;
        if constexpr (EXTRA)
            if (p.next_w) next_w_bits = *((const unsigned short *)p.next_w + min(n, p.N - 1));
        [[maybe_unused]] float sq[MROWS];  // squares of the outputs this lane completed
        // An output is complete: round it, write it and, with a split RMSNorm, its product
        // with the next norm's weight beside it.
        auto complete = [&](int r, __half *dst, float y) {
            const __half y16 = __float2half_rn(y);
            if constexpr (DEP) {
                if (p.out_tag) {
                    __hip_atomic_store((uint32_t *)p.out + (dst - p.out), out_tagw | (uint32_t)__half_as_ushort(y16),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    return;
                }
            }
            *dst = y16;
            if constexpr (EXTRA) {
                const float yf = __half2float(y16);
                sq[r] = yf * yf;
                if (p.next_in) p.next_in[dst - p.out] = __float2half_rn(yf * half_bits_to_float(next_w_bits));
            }
        };
#pragma unroll
        for (int r = 0; r < MROWS; ++r) {
            float v = reduce_scatter_kw(acc[r], kw2);
            if (scaled) v *= row_scale(r);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[r][i] = 0.0f;
            if constexpr (EXTRA) sq[r] = 0.0f;
            const int m = m0 + r;
            if (!owner || n >= p.N || m >= p.M) continue;
            __half *dst = p.out + (size_t)m * p.N + n;
            const float prev = p.overwrite ? 0.0f : half_bits_to_float(out_prev[r]);
            if (count == 1) {
                complete(r, dst, prev + v);
                continue;
            }
            unsigned long long *word = p.accum + (size_t)m * p.N + n;
            const Contribution c = fixed_contribution(v);
            if (c.flags) __hip_atomic_fetch_or(word, c.flags, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned long long old =
                __hip_atomic_fetch_add(word, c.add, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((int)(old >> 56) != count - 1) continue;
            // this contribution completed the sum
            complete(r, dst, prev + fixed_total((old | c.flags) + c.add, count));
            __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if constexpr (EXTRA) {
            // The wave's 32 columns are one slot of the row's sums of squares.  Normally one
            // wave completes all 32 and the slot receives a single add; when completions
            // are split between workgroups it receives one add from each.
            if (p.sumsq_out) {
#pragma unroll
                for (int r = 0; r < MROWS; ++r) {
                    const float s = wave_sum(sq[r]);
                    if (lane == 0 && s != 0.0f)
                        unsafeAtomicAdd(p.sumsq_out + (size_t)(m0 + r) * (p.N / kWaveCols) + t * kWaves + wave, s);
                }
            }
        }
    };

    // Pipeline step for one item whose operands `ops` were requested earlier: per row,
    // build the row's tables into buffer f, barrier, look them up.  The barrier both
    // publishes buffer f and retires the readers of buffer f^1, which the next build
    // overwrites.
    constexpr uint32_t kFlip = 0x80808080u;  // +128 bytes = the other table buffer
    int buf = 0;
    int rel = 0;  // items of the range done so far
    // `after_first_barrier` runs behind the barrier of the item's first row (see the first item below).
    // Twin items: the item's second tile is looked up against the tables that stand already.
    [[maybe_unused]] auto twin_second = [&](const ItemOperands<NB, MODE> &ops, bool last) {
        int nt = tile, ns = set;
        advance(nt, ns);
        asm volatile("" : "+v"(lane_off));
        lookup_item<NB, MODE>(ops, lut, acc_twin, lane_off, sel, stage + abuf * (2 * 4 * kTables) + kw * 4, q);
        buf ^= 1;
        lane_off ^= kFlip;
        if (rel == 0) stamp(p, kStampFirstItem);
        ++rel;
        if (last) stamp(p, kStampItems);
        if (last || nt != tile) {
            flush_tile(tile);
            if (!last) fetch_out(nt);
        }
        if (last) stamp(p, kStampHandedOver);
        tile = nt;
        set = ns;
    };
    auto item_step = [&](const ItemOperands<NB, MODE> &ops, bool last, auto &&after_first_barrier) {
        int nt = tile, ns = set;
        advance(nt, ns);
        const int slot = rel % kSlots;
        if (rel > 0 && slot == 0) {
            // The window is used up (every thread has passed the barrier that followed its
            // last read): fetch and park the next one.  Not prefetched: ranges of more than
            // a window's items only occur beyond half a billion weights per call, and a
            // conditional load in flight would make every later wait conservative.
            // (never reached by a chained problem: the host keeps its ranges within one window)
            const WindowChunk w = fetch_window<MROWS, XF>(p, m0, set0, rel, n_items, tid);
            store_window<MROWS, XF>(w, window, tid, xf);
            __syncthreads();
        }
        if constexpr (PAIR) {
#pragma unroll
            for (int rp = 0; rp < MROWS / 2; ++rp) {
                const u32x4 xa = *(const u32x4 *)(window + 4 * (((2 * rp) * kSlots + slot) * kTables + tb));
                const u32x4 xb = *(const u32x4 *)(window + 4 * (((2 * rp + 1) * kSlots + slot) * kTables + tb));
                build_tables_pair(xa, xb, lut, buf, tb, eb);
                __syncthreads();
                if (rp == 0) {
                    __builtin_amdgcn_sched_barrier(0);
                    after_first_barrier();
                    __builtin_amdgcn_sched_barrier(0);
                }
                asm volatile("" : "+v"(lane_off));
                lookup_item_pair<NB, MODE>(ops, lut, acc[2 * rp], acc[2 * rp + 1], lane_off, sel);
                buf ^= 1;
                lane_off ^= kFlip;
            }
        }
#pragma unroll
        for (int r = 0; r < (PAIR ? 0 : MROWS); ++r) {
            u32x4 xr = x0;
            if (!kDirectFirst || r > 0 || rel > 0) {
                xr = *(const u32x4 *)(window + 4 * ((r * kSlots + slot) * kTables + tb));
            } else {
                // (opaque, so that the chunk is not waited for before it is needed)
                asm volatile("" : "+v"(xr.x), "+v"(xr.y), "+v"(xr.z), "+v"(xr.w));
                if ((set0 * kTables + tb) * 8 >= p.K) xr = (u32x4){0u, 0u, 0u, 0u};  // inputs beyond K
            }
            build_tables(xr, lut, buf, tb, eb);
            if (r == 0) stage_alpha<NB, MODE>(ops, stage, abuf, tid);
            __syncthreads();
            if (r == 0) {
                if (rel == 0) stamp(p, kStampTables);
                __builtin_amdgcn_sched_barrier(0);
                after_first_barrier();
                __builtin_amdgcn_sched_barrier(0);
            }
            // opaque to the optimiser: otherwise the look-up addresses of an item are
            // kept in registers across all rows instead of being recomputed (1 op each)
            asm volatile("" : "+v"(lane_off));
            lookup_item<NB, MODE>(ops, lut, acc[r], lane_off, sel, stage + abuf * (2 * 4 * kTables) + kw * 4, q);
            if constexpr (TWIN) return;   // (the buffers turn, and the range moves on, behind the second tile)
            buf ^= 1;
            lane_off ^= kFlip;
        }
        abuf ^= 1;
        if (rel == 0) stamp(p, kStampFirstItem);
        ++rel;
        if (last) stamp(p, kStampItems);
        if (last || nt != tile) {
            flush_tile(tile);
            if (!last) fetch_out(nt);
        }
        if (last) stamp(p, kStampHandedOver);
        tile = nt;
        set = ns;
    };
    // Two operand buffers alternate: while one item is processed the next one's loads
    // are in flight.
    //
    // The FIRST item is taken outside the loop, and as little as possible is requested
    // before its tables stand.  A CU keeps only so many vector memory instructions in
    // flight (about 64, all waves together); a wave whose next load does not fit stalls at
    // that instruction, whatever else it could do.  With everything requested up front
    // (activations, two items, the caller's outputs: 15 loads per wave at three bit
    // planes) the second wave of every SIMD got stuck behind the first one's loads and
    // reached its table build a memory latency late (measured per wave: activations usable
    // at 1.3 us in waves 0-3, at 2.1 us in waves 4-7, and the workgroup's first barrier
    // waits for the last).  So: activations and the first item's sign words first; its
    // alphas once the activation window is parked; the second item and the caller's
    // outputs behind the first barrier.  4096x4096 3-bit: 5.98 -> 4.93 us per call.
    //
    // The other items are taken in pairs by a counted loop with ONE exit and one load site
    // per buffer inside it:
    //  * with a second load site in the loop the register allocator gives the two sites
    //    different registers and reconciles them with copies that wait for the loads;
    //  * with a second exit the loop is restructured with edges that are never taken but
    //    on which loads are still pending, and every iteration then starts by waiting
    //    for everything in flight.
    // An item that does not exist (the second of the last pair of an odd range) is requested
    // as a dummy (see load_item).
    ItemOperands<NB, MODE> opA, opB;
    int ld_tile = tile, ld_set = set;  // next item to request
    const int pairs = (n_items + 1) / 2;
    auto no_hook = []() {};
    if constexpr (ALONE == 2) {
        // One item per range, known at launch: nothing is requested for a second item.  In the
        // general form below a range that ends requests a dummy in place of the item that
        // does not exist (so that every wait can count its loads), and those six to eight
        // requests per wave sit in the CU's memory pipeline ahead of the hand-over atomics:
        // 4096x4096 3-bit 5.1 -> 4.8 us, 4-bit 6.1 -> 5.3, 3072x768 3-bit 4.4 -> 3.8.
        load_item<NB, MODE, 1>(opA, p, ld_tile, ld_set, true, kw, q, lane_col, tid);
        __builtin_amdgcn_sched_barrier(0);
        stamp(p, kStampRequested);
        late_setup();
        first_window();
        load_item<NB, MODE, 2>(opA, p, ld_tile, ld_set, true, kw, q, lane_col, tid);
        item_step(opA, true, [&]() { fetch_out(tile); });
    } else if constexpr (TWIN) {
        // Twin items: buffer A holds the item's first tile, buffer B its second.  The first tile's
        // step builds the tables (first item alone, as below), the second tile's step only looks up.
        load_item<NB, MODE, 1>(opA, p, 2 * ld_tile, ld_set, true, kw, q, lane_col, tid);
        __builtin_amdgcn_sched_barrier(0);
        stamp(p, kStampRequested);
        late_setup();
        first_window();
        load_item<NB, MODE, 2>(opA, p, 2 * ld_tile, ld_set, true, kw, q, lane_col, tid);
        item_step(opA, false, [&]() {
            fetch_out(tile);
            load_item<NB, MODE>(opB, p, 2 * ld_tile + 1, ld_set, true, kw, q, lane_col, tid);
            advance(ld_tile, ld_set);
        });
#pragma clang loop unroll(disable)
        for (int j = 1; j < n_items; ++j) {
            load_item<NB, MODE>(opA, p, 2 * ld_tile, ld_set, true, kw, q, lane_col, tid);
            twin_second(opB, false);
            load_item<NB, MODE>(opB, p, 2 * ld_tile + 1, ld_set, true, kw, q, lane_col, tid);
            advance(ld_tile, ld_set);
            item_step(opA, false, no_hook);
        }
        twin_second(opB, true);
    } else if constexpr (ALONE == 1) {
        load_item<NB, MODE, 1>(opA, p, ld_tile, ld_set, true, kw, q, lane_col, tid);
        __builtin_amdgcn_sched_barrier(0);
        stamp(p, kStampRequested);
        late_setup();
        if constexpr (DEP) {
            // Chained problem that waits: its activations are read, tag by tag, behind the first
            // item's sign words (which depend on nothing and stream meanwhile).  Every wave leaves
            // its verdict where the others read it behind first_window's barrier: a workgroup
            // goes on or gives up as a whole.
            out_tagw = effective_tag(p.out_tag, cw->epoch) << 16;
            bool ok = true;
            if (chain_waits) ok = chain_inputs();
            if (lane == 0) stage[64 + wave] = ok ? 0.0f : 1.0f;
        }
        first_window();
        if constexpr (DEP) {
            float gave_up = 0.0f;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) gave_up += stage[64 + w];
            if (gave_up != 0.0f) return false;
        }
        load_item<NB, MODE, 2>(opA, p, ld_tile, ld_set, true, kw, q, lane_col, tid);
        advance(ld_tile, ld_set);
        item_step(opA, n_items == 1, [&]() {
            fetch_out(tile);
            load_item<NB, MODE>(opB, p, ld_tile, ld_set, 1 < n_items, kw, q, lane_col, tid);
            advance(ld_tile, ld_set);
        });
#pragma clang loop unroll(disable)
        for (int j = 1; j < pairs; ++j) {
            load_item<NB, MODE>(opA, p, ld_tile, ld_set, true, kw, q, lane_col, tid);
            advance(ld_tile, ld_set);
            item_step(opB, false, no_hook);
            const bool has_b = 2 * j + 1 < n_items;
            load_item<NB, MODE>(opB, p, ld_tile, ld_set, has_b, kw, q, lane_col, tid);
            advance(ld_tile, ld_set);
            item_step(opA, !has_b, no_hook);
        }
        if ((n_items & 1) == 0) item_step(opB, true, no_hook);
    } else {
        // Several rows per pass, per-lane block alphas (the register budget does not allow the
        // first item a code path of its own: up to 300 bytes of spills per lane measured), and
        // four-plane problems of grouped launches.  Everything is requested up front and the
        // first iteration skips its first step at run time (opaque, which keeps the compiler
        // from peeling it).
#pragma clang loop unroll(disable)
        for (int j = 0; j < pairs; ++j) {
            int first = __builtin_amdgcn_readfirstlane(j == 0);
            asm volatile("" : "+s"(first));
            load_item<NB, MODE>(opA, p, ld_tile, ld_set, true, kw, q, lane_col, tid);
            advance(ld_tile, ld_set);
            if (!first) item_step(opB, false, no_hook);
            const bool has_b = 2 * j + 1 < n_items;
            load_item<NB, MODE>(opB, p, ld_tile, ld_set, has_b, kw, q, lane_col, tid);
            advance(ld_tile, ld_set);
            if (first) {
                stamp(p, kStampRequested);
                late_setup();
                fetch_out(tile);
                first_window();
            }
            item_step(opA, !has_b, no_hook);
        }
        if ((n_items & 1) == 0) item_step(opB, true, no_hook);
    }
    stamp(p, kStampExit);
    return true;
}

// Flat workgroup index (relative to the problem) -> (range, row chunk), for launches
// that hold several problems.
__device__ __forceinline__ void decode_block(const Problem &p, int local, int &range, int &mchunk)
{
    mchunk = p.mchunks == 1 ? 0 : local / p.wgs_per_chunk;
    range = local - mchunk * p.wgs_per_chunk;
}

// (at most 128 registers, so that two workgroups share a CU)
// SINGLE: every range of the launch holds exactly one item (see ALONE == 2 in gemv_range).
// TWIN: the launch's items are twin items (two output tiles per table build, see gemv_range).
template <int NB, int MODE, int MROWS, bool PAIR = false, bool SINGLE = false, bool TWIN = false>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
lut_gemv_kernel(const Problem p)
{
    __shared__ __attribute__((aligned(16))) float lut[kLutDwords + kStageDwords + kWindowDwords];
    // grid = (ranges, row chunks)
    gemv_range<NB, MODE, MROWS, kXNone, false, SINGLE ? 2 : (MROWS == 1 && !is_block(MODE)), PAIR, false, TWIN>(
        p, (int)blockIdx.x, (int)blockIdx.y, lut);
}

// Several row-wise problems in one launch.  Bit widths may differ between the
// problems of a group.
// XF: the input transform shared by all problems of the launch.
// (Up to three bit planes take the first item on its own, like a lone problem; four planes
// keep the loop that requests two items up front: with the peeled first item as well the
// kernel, whose register count is that of its largest bit width, spills 10-19 registers per
// lane, and everything slows down: q,k,v of a 7B block 10.3 us per launch with the spills,
// 9.6 with the old loop throughout, 9.1 this way; gate,up 14.4 / 13.4 / 12.8.)
template <int XF>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
lut_gemv_group_kernel(const Group g)
{
    __shared__ __attribute__((aligned(16))) float lut[kLutDwords + kStageDwords + kWindowDwords];
    // grid = (workgroups of the largest problem, problems): the problem is known from the
    // dispatch, so its fields are one scalar-load round trip away like a lone problem's
    // (through the constant address space, which the kernel arguments live in: the fields are
    // then scalar loads that may be repeated at will instead of values to keep in registers)
    const Problem &p = *(const Problem *)((const __attribute__((address_space(4))) Problem *)&g.p[0] + blockIdx.y);
    if ((int)blockIdx.x >= p.n_blocks) return;
    int range, m;
    decode_block(p, (int)blockIdx.x, range, m);
    switch (p.nb) {
    case 1: gemv_range<1, kRowF16, 1, XF, true, true>(p, range, m, lut); break;
    case 2: gemv_range<2, kRowF16, 1, XF, true, true>(p, range, m, lut); break;
    case 3: gemv_range<3, kRowF16, 1, XF, true, true>(p, range, m, lut); break;
    default: gemv_range<4, kRowF16, 1, XF, true, false>(p, range, m, lut); break;
    }
}

}  // namespace lutgemm

#endif
