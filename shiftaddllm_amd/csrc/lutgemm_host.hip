// Host side of liblutgemm_gfx950.so: operand validation, launch planning, the
// accumulator workspaces and the C ABI of include/lutgemm_gfx950.h.  The kernels live
// in lut_gemv_device.h (table look-ups) and lut_gemm_mfma_device.h (matrix cores).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <atomic>
#include <map>
#include <mutex>
#include <utility>
#include <vector>

#include "lutgemm_common.h"
#include "lutgemm_gfx950.h"
#include "lutgemm_internal.h"
#include "lutgemm_launch.h"

namespace lutgemm {
namespace {

constexpr int kMfmaWaves = 8;       // waves of a matrix-core workgroup: K-steps of a round
constexpr int kMfmaTileCols = 64;   // outputs per matrix-core workgroup
constexpr int kMfmaStepK = 128;
constexpr int kMaxDevices = 64;

thread_local int g_last_hip_error = 0;

// time-stamped build only: where the kernels leave their clock readings
std::atomic<unsigned long long *> g_stamps{nullptr};
std::atomic<long long> g_stamp_slots{0};

int hip_fail(hipError_t e)
{
    g_last_hip_error = (int)e;
    return LUTGEMM_EHIP;
}

// ---- accumulator words ------------------------------------------------------------
// K is split over workgroups; their partial sums meet in one 64-bit word per output
// (lutgemm_common.h).  Every launch leaves the words it used at zero, which is the
// state the next launch needs, so launches that are ordered on a stream can share
// one buffer.

// Fixed buffer of the entry point that may not allocate.  Zero when the code object is
// loaded; each GPU holds its own copy at its own address until the process ends.
static __device__ __align__(256) unsigned long long scratch[LUTGEMM_NOALLOC_MAX_WORDS];

std::mutex g_scratch_mutex;
unsigned long long *g_scratch_ptr[kMaxDevices] = {};

// Address of `scratch` on the current device, resolved once per device (in host code
// the array's name is a stand-in, not a device address).
int scratch_address(unsigned long long **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e);
    if (dev < 0 || dev >= kMaxDevices) return LUTGEMM_EUNSUP;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_fail(e);
        g_scratch_ptr[dev] = (unsigned long long *)ptr;
    }
    *out = g_scratch_ptr[dev];
    return LUTGEMM_OK;
}

struct Workspace {
    unsigned long long *accum = nullptr;
    size_t words = 0;
    std::vector<unsigned long long *> retired;  // outgrown buffers: captured graphs may still name them
    // second buffer of the block-scaled matrix-core path: the split activations of the call in flight
    void *split = nullptr;
    size_t split_bytes = 0;
    std::vector<void *> retired_split;
};

std::mutex g_ws_mutex;
std::map<std::pair<int, hipStream_t>, Workspace> g_workspaces;

// Grow-only, zero-initialised accumulator words per (device, stream).  Growing
// synchronises the stream and allocates, which a stream under capture cannot do: that
// case is refused before anything is touched (reserve the words beforehand).  An
// outgrown buffer is kept (zero, unused by new launches) until
// lutgemm_release_workspaces(): a graph captured earlier still points at it.
int stream_workspace(hipStream_t stream, size_t words, unsigned long long **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e);
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Workspace &ws = g_workspaces[std::make_pair(dev, stream)];
    if (ws.words < words) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        e = hipStreamIsCapturing(stream, &cap);
        if (e != hipSuccess) return hip_fail(e);
        if (cap != hipStreamCaptureStatusNone) return LUTGEMM_ECAPTURE;
        e = hipStreamSynchronize(stream);  // queued work may still use the old buffer
        if (e != hipSuccess) return hip_fail(e);
        if (ws.accum) ws.retired.push_back(ws.accum);
        ws.accum = nullptr;
        ws.words = 0;
        const size_t want = words < (1u << 18) ? (1u << 18) : words;
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

// The same for the split activations of the block-scaled path (not zeroed: every call writes what it
// reads).  Calls on one stream are ordered, so they can share the buffer.
int stream_split_buffer(hipStream_t stream, size_t bytes, void **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e);
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Workspace &ws = g_workspaces[std::make_pair(dev, stream)];
    if (ws.split_bytes < bytes) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        e = hipStreamIsCapturing(stream, &cap);
        if (e != hipSuccess) return hip_fail(e);
        if (cap != hipStreamCaptureStatusNone) return LUTGEMM_ECAPTURE;
        e = hipStreamSynchronize(stream);
        if (e != hipSuccess) return hip_fail(e);
        if (ws.split) ws.retired_split.push_back(ws.split);
        ws.split = nullptr;
        ws.split_bytes = 0;
        const size_t want = bytes < (1u << 20) ? (1u << 20) : bytes;
        e = hipMalloc(&ws.split, want);
        if (e != hipSuccess) {
            g_last_hip_error = (int)e;
            return LUTGEMM_ENOMEM;
        }
        ws.split_bytes = want;
    }
    *out = ws.split;
    return LUTGEMM_OK;
}

// Where a call takes its accumulator words from.
struct Accum {
    hipStream_t stream;
    bool fixed = false;  // the fixed device array instead of the stream's workspace
};

int accum_words(const Accum &a, size_t words, unsigned long long **out)
{
    if (!a.fixed) return stream_workspace(a.stream, words, out);
    if (words > (size_t)LUTGEMM_NOALLOC_MAX_WORDS) return LUTGEMM_ETOOBIG;
    return scratch_address(out);
}

int env_int(const char *name, int fallback)
{
    const char *v = getenv(name);
    return (v && *v) ? atoi(v) : fallback;
}

// Tuning options (lutgemm_set_option): each starts from its environment variable, read once.
struct Option {
    const char *env;
    int fallback;
};
constexpr Option kOptions[LUTGEMM_OPTION_COUNT] = {
    {"LUTGEMM_TARGET_BLOCKS", 0}, {"LUTGEMM_FIRST_SHARE", 60}, {"LUTGEMM_MFMA_MIN_M", 3},
    {"LUTGEMM_MFMA_BLOCKS", 0},   {"LUTGEMM_PAIR_TABLES", 1},  {"LUTGEMM_SINGLE_ITEM", 1},
    {"LUTGEMM_CHAIN_BLOCKS", 0}, {"LUTGEMM_CHAIN_GRID", 0},  {"LUTGEMM_TWIN_ITEMS", 4},
    {"LUTGEMM_BLOCK_SCALED", 1}, {"LUTGEMM_POW2_CONVERT", 1},
};
std::atomic<int> g_option[LUTGEMM_OPTION_COUNT];
std::once_flag g_option_once;

void load_options()
{
    std::call_once(g_option_once, [] {
        for (int i = 0; i < LUTGEMM_OPTION_COUNT; ++i) g_option[i].store(env_int(kOptions[i].env, kOptions[i].fallback));
    });
}

// LUTGEMM_OPTION_TARGET_BLOCKS = workgroups a look-up launch aims
// for.  74 KiB of LDS per workgroup lets two be resident per CU, and a launch above
// what is resident at once runs a second, mostly empty round that costs as much as
// the first.
// Short streams do better with ONE workgroup per CU and more items each: a workgroup's
// second and third item cost less than the start and the hand-over of another workgroup.
// Measured, one row, 256 vs 512 workgroups: 11008x4096x3 8.78 vs 9.04 us, 4096x11008x3 8.59
// vs 9.12, 13824x5120x2 8.92 vs 9.64, 8192x8192x2 8.27 vs 8.49; 8192x8192x4 11.74 vs 11.06,
// 28672x8192x2 18.75 vs 16.62.
// The block-alpha formats pay more per item (their alphas are staged per item), so a long
// range hurts them sooner: beyond four items per workgroup they take two workgroups per CU
// (13824x5120x2 in eight row groups 9.16 vs 8.58 us, 5120x13824x2 10.0 vs 8.54; 5120x5120x2,
// 1.6 items per workgroup, 5.91 vs 6.37).
int target_blocks(long sign_bytes, long items = 0, bool block_alpha = false)
{
    const int v = option(LUTGEMM_OPTION_TARGET_BLOCKS);
    if (v > 0) return v;
    if (block_alpha && items > 4 * 256) return 512;
    return sign_bytes <= (24l << 20) ? 256 : 512;  // 1 or 2 workgroups x 256 CUs
}

// Of the two workgroups that share a CU the one dispatched first runs faster (the older
// waves win the arbitration for issue slots and memory requests): with equal ranges the
// first half of a 512-workgroup grid ends 6-7 us before the second on the 132 MB shapes.
// So the first 256 workgroups get this share (per cent) of each pair's items.  Measured,
// equal ranges vs 60 %: 28672x8192x2 17.3 vs 16.3 us, 8192x28672x2 17.1 vs 15.8, 8192x28672x4
// 27.7 vs 27.0, 13824x5120x4 14.8 vs 13.1 (there mostly because 412 workgroups of 3 and 2
// items fill the CUs better than 360 of 3), 8192x8192x4 unchanged.
int first_share()
{
    return option(LUTGEMM_OPTION_FIRST_SHARE);
}

// Cut the (tile, set) items of a problem into contiguous ranges, one per workgroup,
// aiming at `want_blocks` workgroups.
// `twin`: the items are twin items, one set of inputs against a PAIR of output tiles (one table
// build for 512 outputs); n_tiles counts pairs then.
int plan_lookup(Problem &p, int mrows, long want_blocks, bool twin = false)
{
    p.n_tiles = (p.N + kTileCols - 1) / kTileCols;
    if (twin) p.n_tiles = (p.n_tiles + 1) / 2;
    p.twin = twin ? 1 : 0;
    p.mchunks = (p.M + mrows - 1) / mrows;
    const long total = (long)p.n_tiles * p.nsets;
    long wgs = want_blocks / p.mchunks;
    if (wgs < 1) wgs = 1;
    long ipw = (total + wgs - 1) / wgs;
    // an accumulator word takes at most kMaxContrib contributions: a tile of nsets items
    // overlaps at most ceil(nsets / ipw) + 1 ranges
    const long cap = (p.nsets + kMaxContrib - 2) / (kMaxContrib - 1);
    if (ipw < cap) ipw = cap;
    if (ipw > total) ipw = total;
    long n_long = (total + ipw - 1) / ipw, short_items = ipw, n_short = 0;
    // two resident workgroups per CU, one row chunk: unequal shares within each pair
    const int share = first_share();
    if (p.mchunks == 1 && want_blocks == 512 && total >= 2 * 256 * 2 && share > 50 && share < 100) {
        const long pair = (total + 255) / 256;
        long a = (pair * share + 99) / 100, b = pair - a;
        // (the smaller range may not fall below what the contribution count allows: give it
        // items of the larger one while the larger one stays the larger)
        while (b < cap && a - 1 > b + 1) {
            --a;
            ++b;
        }
        // (a split far beyond the share, 3 and 1 of 4, is worse than none: 8192x8192x4 11.4 us against 10.5)
        if (b >= 1 && b >= cap && a > b && 100 * a <= (share + 12) * pair) {
            ipw = a;
            n_long = 256;
            short_items = b;
            const long rest = total - n_long * a;
            n_short = rest > 0 ? (rest + b - 1) / b : 0;
            if (rest <= 0) n_long = (total + a - 1) / a;
        }
    }
    p.items_per_wg = (int)ipw;
    p.long_ranges = (int)n_long;
    p.short_items = (int)short_items;
    p.split_item = (int)(n_long * ipw);
    p.wgs_per_chunk = (int)(n_long + n_short);
    p.n_blocks = p.wgs_per_chunk * p.mchunks;
    p.by_items = make_divisor(p.items_per_wg);
    p.by_short_items = make_divisor(p.short_items);
    p.by_nsets = make_divisor(p.nsets);
    // the multiply-high divisions of the kernel are exact within this bound
    if (2ull * (unsigned long long)(total + p.nsets) * (unsigned long long)ipw >= (1ull << 32)) return LUTGEMM_EUNSUP;
    return LUTGEMM_OK;
}

// true when some tile is shared between ranges, i.e. accumulator words are needed
bool lookup_splits_k(const Problem &p)
{
    if (p.items_per_wg % p.nsets != 0) return true;
    return p.wgs_per_chunk > p.long_ranges && (p.short_items % p.nsets != 0 || p.split_item % p.nsets != 0);
}

int pick_mrows(int M) { return M >= 3 ? 4 : M; }

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
    p.group_words = 1;
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
    p.by_group_words = make_divisor(p.group_words);
#ifdef LUTGEMM_TIMESTAMPS
    p.stamps = g_stamps.load();
    p.stamp_slots = g_stamp_slots.load();
#endif
    // the multiply-high divisions of the kernels are exact within these bounds
    const unsigned long long tiles = (unsigned long long)(N + kTileCols - 1) / kTileCols;
    if (2ull * p.kwords * p.group_words >= (1ull << 32)) return LUTGEMM_EUNSUP;
    if (2ull * (tiles + 1) * p.nsets * p.nsets >= (1ull << 32)) return LUTGEMM_EUNSUP;
    return LUTGEMM_OK;
}

int mfma_min_rows()
{
    return option(LUTGEMM_OPTION_MFMA_MIN_M);
}

// The matrix-core path needs whole 128-input steps inside one alpha group and
// 16-output alpha runs.
bool mfma_eligible(const Problem &p, int mode)
{
    if (!(mode == kRowF16 && p.K % kMfmaStepK == 0 && p.group_words % 4 == 0 && p.N % 16 == 0 && p.N >= 16))
        return false;
    if (p.M >= mfma_min_rows()) return true;
    // two rows: the look-up kernel (one table set for both rows, fp16 entry pairs) wins from
    // about 12 MB of sign words on (measured, look-up vs matrix core: 4096x4096x3 7.3 us vs 6.4;
    // 11008x4096x2 10.5 vs 9.6; 5120x5120x4 9.8 vs 10.5; 11008x4096x3 11.9 vs 12.8; 8192x8192x4
    // 14.2 vs 16.6; 28672x8192x4 34.7 vs 52)
    return p.M == 2 && mfma_min_rows() == 3 && (long)p.N * (p.K / 8) * p.nb <= (12l << 20);
}

// K-steps are split 8 ways inside a workgroup already; across workgroups `want` ways
// at most (whole rounds of eight steps per slice).
void plan_mfma(Problem &p, int mt, long want)
{
    p.n_tiles = (p.N + kMfmaTileCols - 1) / kMfmaTileCols;
    p.mchunks = (p.M + 16 * mt - 1) / (16 * mt);
    p.nsets = p.K / kMfmaStepK;  // K-steps
    if (want > p.nsets / kMfmaWaves) want = p.nsets / kMfmaWaves;
    if (want < 1) want = 1;
    if (want > kMaxSlices) want = kMaxSlices;
    p.sets_per_split = (p.nsets + (int)want - 1) / (int)want;
    p.sets_per_split = (p.sets_per_split + kMfmaWaves - 1) / kMfmaWaves * kMfmaWaves;  // whole rounds
    p.ksplit = (p.nsets + p.sets_per_split - 1) / p.sets_per_split;
    p.n_blocks = p.n_tiles * p.ksplit * p.mchunks;
}

// Workgroups wanted per launch of the 32-row tile: one per CU (its register count allows
// no second one).  Measured, 8192x8192x4: 36.4 us at 256 and 40.0 at 512.
int mfma_blocks_override()
{
    return option(LUTGEMM_OPTION_MFMA_BLOCKS);
}

// K-slices per tile for the problems of one launch (all get the same number, each up to
// its own limit).
//   32-row tile: as many as reach one workgroup per CU.
//   16-row tile: the kernel is bound by the vector ALU work of expanding sign bits, two
//   workgroups share a CU, and the launch ends when the busiest CU does.  With w =
//   ceil(workgroups / 256) workgroups on that CU and R rounds (one K-step per wave, about
//   2.2 us at three bit planes) per workgroup, the slice count that minimises
//       w * R  +  0.18 * w  +  0.9 * max(0, w - 2)
//   is taken, the smaller one on ties: a workgroup's start and hand-over cost a fifth of a
//   round, and one that has to wait for a slot on its CU most of a round.  A lone workgroup
//   of four or more rounds hides its loads badly when there are many of them (more than
//   eight activation rows, or nine CUs in ten busy) and is charged 12 % more.  Fitted to
//   launches at 4 and 16 rows (us, slices -> time): 8192x8192x4: 2 -> 17.9, 4 -> 16.7;
//   11008x4096x3: 1 -> 13.0, 2 -> 13.4 (16 rows: 16.7, 14.9); 22016x4096x3: 1 -> 21.4, 2 -> 18.3;
//   28672x8192x2: 1 -> 28.1, 4 -> 32.5; 5120x13824x3: 3 -> 16.2, 5 -> 18.4.
int mfma_slices(const Group &g, int mt)
{
    constexpr long kCUs = 256;
    long tiles = 0;
    int max_rounds = 1, rows = 0;
    for (int i = 0; i < g.count; ++i) {
        const Problem &p = g.p[i];
        tiles += (long)((p.N + kMfmaTileCols - 1) / kMfmaTileCols) * ((p.M + 16 * mt - 1) / (16 * mt));
        const int rounds = p.K / kMfmaStepK / kMfmaWaves;
        if (rounds > max_rounds) max_rounds = rounds;
        if (p.M > rows) rows = p.M;
    }
    if (max_rounds > kMaxSlices) max_rounds = kMaxSlices;
    if (const int blocks = mfma_blocks_override()) return (int)(blocks / tiles > 1 ? blocks / tiles : 1);
    if (mt != 1) return (int)(kCUs / tiles > 1 ? kCUs / tiles : 1);
    int best = 1;
    double best_cost = 0.0;
    for (int ks = 1; ks <= max_rounds; ++ks) {
        long wgs = 0;
        int rounds = 0;
        for (int i = 0; i < g.count; ++i) {
            Problem q = g.p[i];
            plan_mfma(q, mt, ks);
            wgs += q.n_blocks;
            if (q.sets_per_split / kMfmaWaves > rounds) rounds = q.sets_per_split / kMfmaWaves;
        }
        const long w = (wgs + kCUs - 1) / kCUs;
        double cost = (double)w * rounds + 0.18 * (double)w + 0.9 * (double)(w > 2 ? w - 2 : 0);
        if (w == 1 && rounds >= 4 && (rows > 8 || wgs * 10 > kCUs * 9)) cost *= 1.12;
        if (ks == 1 || cost < best_cost * 0.999) {
            best = ks;
            best_cost = cost;
        }
    }
    return best;
}

int run_mfma(Problem &p, const Accum &acc)
{
    const int mt = p.M > 16 ? 2 : 1;
    Group one{};
    one.count = 1;
    one.p[0] = p;
    plan_mfma(p, mt, mfma_slices(one, mt));
    if (p.ksplit > 1) {
        int rc = accum_words(acc, (size_t)p.M * p.N, &p.accum);
        if (rc != LUTGEMM_OK) return rc;
    }
    const hipError_t e = launch_mfma(p, mt, false, acc.stream);
    return e == hipSuccess ? LUTGEMM_OK : hip_fail(e);
}

// All problems of a group on the matrix-core kernel in one launch (they share the
// row-tile height: all M <= 16 or all M > 16).
int run_mfma_group(Group &g, const Accum &acc)
{
    const int mt = g.p[0].M > 16 ? 2 : 1;
    size_t words = 0;
    for (int i = 0; i < g.count; ++i) words += (size_t)g.p[i].M * g.p[i].N;
    const int slices = mfma_slices(g, mt);
    int begin = 0;
    bool any_split = false;
    for (int i = 0; i < g.count; ++i) {
        Problem &p = g.p[i];
        plan_mfma(p, mt, slices);
        if (p.n_blocks > begin) begin = p.n_blocks;  // grid.x: the largest problem's workgroups
        any_split = any_split || p.ksplit > 1;
    }
    if (any_split) {
        unsigned long long *base = nullptr;
        int rc = accum_words(acc, words, &base);
        if (rc != LUTGEMM_OK) return rc;
        size_t off = 0;
        for (int i = 0; i < g.count; ++i) {
            g.p[i].accum = base + off;
            off += (size_t)g.p[i].M * g.p[i].N;
        }
    }
    const hipError_t e = g.count == 1 ? launch_mfma_fused(g.p[0], mt, acc.stream) : launch_mfma_group(g, mt, begin, acc.stream);
    return e == hipSuccess ? LUTGEMM_OK : hip_fail(e);
}

// Which kernel a lone problem runs on and how it is cut up (no device work).
enum Kernel : int { kLookup = 0, kMatrixCore = 1 };

int plan_single(Problem &p, int mode, int *kernel, int *mrows)
{
    if (mfma_eligible(p, mode)) {
        const int mt = p.M > 16 ? 2 : 1;
        Group one{};
        one.count = 1;
        one.p[0] = p;
        plan_mfma(p, mt, mfma_slices(one, mt));
        *kernel = kMatrixCore;
        *mrows = 16 * mt;
        return LUTGEMM_OK;
    }
    *kernel = kLookup;
    *mrows = pick_mrows(p.M);
    const long items = (long)((p.N + kTileCols - 1) / kTileCols) * p.nsets;
    const long want = target_blocks((long)p.N * (p.K / 8) * p.nb, items, mode != kRowF16 && mode != kUniformF16);
    int rc = plan_lookup(p, *mrows, want);
    if (rc != LUTGEMM_OK) return rc;
    // One row, per-column alphas and ranges of several items: twin items, i.e. one table build and one
    // barrier per 512 outputs instead of per 256.  A build is about a third of an item's vector
    // instructions at three bit planes, and a launch whose workgroups hold several items each is bound
    // by those; launches of one or two items per workgroup are bound by latencies that twin items would
    // lengthen (half as many ranges to spread over the chip).
    // Measured, plain against twin items (us): 28672x8192x4 27.2 / 24.7-25.1, 28672x8192x3 21.6 / 19.6-20.0;
    // with two bit planes no gain (28672x8192x2 15.0 / 15.2-15.4: bound by the stream), and none where the
    // twin plan has to give up the unequal ranges of the two workgroups of a CU (8192x28672x4 with equal
    // ranges 26.3 / 28.1) or where K is long (the same shape with ranges of 4 and 3 twin items 26.4 / 26.9).
    const int least = option(LUTGEMM_OPTION_TWIN_ITEMS);
    if (least > 0 && *mrows == 1 && (mode == kRowF16 || mode == kUniformF16) && p.nb >= 3 && p.nsets <= 64 &&
        p.short_items >= least && p.items_per_wg >= least) {
        Problem t = p;
        const bool unequal = p.items_per_wg != p.short_items;
        if (plan_lookup(t, 1, want, true) == LUTGEMM_OK && (!unequal || t.items_per_wg != t.short_items) &&
            10 * t.n_blocks >= 9 * p.n_blocks)
            p = t;
    }
    return LUTGEMM_OK;
}

// Block-scaled kernel: a workgroup takes 64 outputs, a chunk of 5, 8 or 16 rows and a K-slice of whole rounds (8 K-steps,
// one per wave); two workgroups fit a CU.  The slice length (rounds) is the one that minimises the
// rounds of the grid times the cost of a workgroup: its rounds plus a constant for its start and end
// (table build, reduction, accumulator words), in units of a round.
void plan_mx(Problem &p)
{
    constexpr long kResident = 2 * 256;
    // (measured: anything from half a round to three rounds plans the same launches for the shapes
    // tried; with no constant at all a slice is a single round and 28672x8192x4 takes 61 us instead of 34)
    constexpr double fixed_rounds = 1.0;
    p.n_tiles = (p.N + kMfmaTileCols - 1) / kMfmaTileCols;
    p.mchunks = (p.M + mx_chunk_rows(p.M) - 1) / mx_chunk_rows(p.M);
    p.nsets = p.K / kMfmaStepK;
    const int rounds = (p.nsets + kMfmaWaves - 1) / kMfmaWaves;
    int best = rounds;
    double best_cost = 0.0;
    for (int r = rounds; r >= 1; --r) {
        const int ks = (rounds + r - 1) / r;
        if (ks > kMaxSlices) break;
        const long wgs = (long)p.n_tiles * p.mchunks * ks;
        const double cost = (double)((wgs + kResident - 1) / kResident) * ((double)r + fixed_rounds);
        if (r == rounds || cost < best_cost * 0.999) {
            best = r;
            best_cost = cost;
        }
    }
    if (const int blocks = mfma_blocks_override()) {
        long want = blocks / ((long)p.n_tiles * p.mchunks);
        if (want < 1) want = 1;
        if (want > kMaxSlices) want = kMaxSlices;
        if (want > rounds) want = rounds;
        best = (rounds + (int)want - 1) / (int)want;
    }
    p.sets_per_split = best * kMfmaWaves;
    p.ksplit = (p.nsets + p.sets_per_split - 1) / p.sets_per_split;
    p.n_blocks = p.n_tiles * p.ksplit * p.mchunks;
}

// Whether a problem that may take the block-scaled kernel should.  It needs one, two or three matrix
// instructions per (bit plane, 16 outputs, 128 inputs) for up to 5, 8 or 16 rows where the fp16 kernel
// needs four (and its sign expansion), but also a launch of its own that splits the activations
// (3 to 4 us with the gap between the launches).  Measured (us, fp16 kernel vs block-scaled):
//   28672x8192x4: 4 rows 50.8 / 33.5, 8 rows 50.1 / 40.2, 16 rows 48.4 / 58.3
//   28672x8192x2: 4 rows 27.1 / 23.5, 8 rows 29.0 / 30.2
//   8192x8192x4:  4 rows 17.0 / 16.4, 8 rows 17.8 / 18.6;  8192x8192x2: 4 rows 11.2 / 13.6
// so: up to 5 rows from 48 MB of sign words on, up to 8 rows from 96 MB on.
bool mx_wanted(const Problem &p)
{
    const int how = option(LUTGEMM_OPTION_BLOCK_SCALED);
    if ((long)p.M * p.K >= (1l << 30)) return false;   // (the split kernel indexes the activations with 32 bits)
    if (how != 1) return how == 2;
    const long sign_bytes = (long)p.N * (p.K / 8) * p.nb;
    return (p.M <= 5 && sign_bytes >= (48l << 20)) || (p.M <= 8 && sign_bytes >= (96l << 20));
}

// Whether a planned fp16 matrix-core launch whose alphas are powers of two should form its sign
// operands through the LDS table and the scaled fp4 -> fp16 conversion (5 vector instructions per
// matrix instruction instead of 10) rather than by shift and bit operation.  The table costs every
// workgroup a 64 KiB build and a barrier (1 to 2 us), which pays from about six rounds of K-steps per
// workgroup on; the 32-row tile would drop to one workgroup per CU with the table and loses.
// Measured (us, shift-and-bit form vs converted form, 16 rows): 28672x8192x4 48.9 / 42.6,
// 8192x28672x4 48.2 / 42.8, 28672x8192x2 30.0 / 28.6 (8 rows 28.4 / 25.0); 8192x8192x4 (2 rounds) 19.6 / 19.4,
// 11008x4096x3 (4 rounds) 15.0 / 15.8, 4096x4096x3 (1 round) 8.8 / 11.0; 32 rows 28672x8192x4 74.1 / 77.6.
// Option POW2_CONVERT: 1 = by this rule, 2 = whenever the promise is given, 0 = never.
bool convert_wanted(const Problem &p, int mt)
{
    const int how = option(LUTGEMM_OPTION_POW2_CONVERT);
    if (how != 1) return how == 2;
    return mt == 1 && p.sets_per_split >= 6 * kMfmaWaves;
}

// Row-wise problem whose alphas are powers of two, with enough rows for the matrix cores: the
// block-scaled kernel (16-row tiles; more rows are further row chunks that stream the same sign
// words side by side).
int run_mx(Problem &p, const Accum &acc)
{
    plan_mx(p);
    if (p.ksplit > 1) {
        int rc = accum_words(acc, (size_t)p.M * p.N, &p.accum);
        if (rc != LUTGEMM_OK) return rc;
    }
    if (acc.fixed) return LUTGEMM_EUNSUP;
    void *buf = nullptr;
    int rc = stream_split_buffer(acc.stream, mx_split_bytes(p.M, p.K), &buf);
    if (rc != LUTGEMM_OK) return rc;
    const hipError_t e = launch_mx(p, buf, acc.stream);
    return e == hipSuccess ? LUTGEMM_OK : hip_fail(e);
}

int run(int mode, const uint32_t *bW, const void *alpha, const void *qbias, const void *x,
        void *out, int N, int K, int nb, int num_groups, int M, const Accum &acc, bool alpha_pow2 = false)
{
    Problem p;
    int rc = fill_problem(p, mode, bW, alpha, qbias, x, out, N, K, nb, num_groups, M);
    if (rc != LUTGEMM_OK) return rc;
    if (alpha_pow2 && mode == kRowF16 && mfma_eligible(p, mode) && p.M >= mfma_min_rows() && mx_wanted(p)) return run_mx(p, acc);
    int kernel = kLookup, mrows = 1;
    rc = plan_single(p, mode, &kernel, &mrows);
    if (rc != LUTGEMM_OK) return rc;
    if (kernel == kMatrixCore ? p.ksplit > 1 : lookup_splits_k(p)) {
        rc = accum_words(acc, (size_t)M * N, &p.accum);
        if (rc != LUTGEMM_OK) return rc;
    }
    hipError_t e;
    if (kernel == kMatrixCore)
        e = launch_mfma(p, mrows / 16, alpha_pow2 && convert_wanted(p, mrows / 16), acc.stream);
    else if (mode == kRowF16 || mode == kUniformF16)
        e = launch_gemv_rowwise(p, mode, mrows, acc.stream);
    else if (p.rows_per_group >= kTileCols)  // a tile spans at most two row groups
        e = launch_gemv_block_staged(p, mode + 4, mrows, acc.stream);
    else
        e = launch_gemv_block(p, mode, mrows, acc.stream);
    return e == hipSuccess ? LUTGEMM_OK : hip_fail(e);
}

// Share a workgroup budget between look-up problems that run side by side so that the longest
// range of every problem takes about the same time.  An item costs a table build plus look-ups in
// proportion to its bit planes (0.45 + 0.13 * nb us measured), whatever the problem; the problems
// end with their slowest workgroup, so the items per workgroup of problem i are floor(T / cost_i)
// for the smallest T whose workgroups fit the budget.  (Sharing in proportion to the sign bytes
// gave q,k,v of 2, 4 and 3 bits 5, 3 and 4 items per workgroup: 3.6, 2.9 and 3.4 us of work.)
// With equal bit widths this is a share in proportion to the items, rounded down: a few
// workgroups more than can be resident run as a second, mostly empty round, and fewer
// workgroups with more items each are the better trade anyway (q,k,v of 4096x4096 as 3 x 64
// workgroups of 4 items 5.31 us per GEMV of the four-launch block, as 3 x 86 of 3 items 5.54).
// *most: the largest workgroup count of a problem (raised only); *any_split: some problem needs
// accumulator words (set only).
int share_workgroups(Problem *const *ps, int count, long budget, int *most, bool *any_split)
{
    long items[kMaxGroup];
    double cost[kMaxGroup];
    double lo = 0.0, hi = 0.0;
    for (int i = 0; i < count; ++i) {
        const Problem &p = *ps[i];
        items[i] = (long)((p.N + kTileCols - 1) / kTileCols) * p.nsets;
        cost[i] = 0.45 + 0.13 * p.nb;
        const double all = (double)items[i] * cost[i];
        if (all > hi) hi = all;
    }
    auto workgroups = [&](double t) {
        long n = 0;
        for (int i = 0; i < count; ++i) {
            long ipw = (long)(t / cost[i]);
            if (ipw < 1) return (long)1 << 40;
            n += ((items[i] + ipw - 1) / ipw) * ps[i]->M;
        }
        return n;
    };
    for (int it = 0; it < 50; ++it) {
        const double mid = 0.5 * (lo + hi);
        if (workgroups(mid) <= budget) hi = mid; else lo = mid;
    }
    for (int i = 0; i < count; ++i) {
        Problem &p = *ps[i];
        long ipw = (long)(hi / cost[i]);
        if (ipw < 1) ipw = 1;
        const long want = ((items[i] + ipw - 1) / ipw) * p.M;
        int rc = plan_lookup(p, 1, want);
        if (rc != LUTGEMM_OK) return rc;
        if (p.n_blocks > *most) *most = p.n_blocks;  // grid.x: the largest problem's workgroups
        *any_split = *any_split || lookup_splits_k(p);
    }
    return LUTGEMM_OK;
}

// Up to kMaxGroup row-wise problems in one launch of the look-up kernel.  Problems
// with enough rows for the matrix-core kernel (and no fused transform) are launched
// on that path instead.
int run_group(int count, const lutgemm_fused_problem *problems, const Accum &acc)
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
        // RMSNorm split over two launches
        if ((q.next_input_f16 != nullptr) != (q.next_norm_weight_f16 != nullptr)) return LUTGEMM_EINVAL;
        if (q.sumsq_out_f32 && q.N % 32 != 0) return LUTGEMM_EINVAL;
        if (q.sumsq_in_f32 && (q.sumsq_in_slots <= 0 || q.norm_weight_f16 || !(q.norm_eps >= 0.0f))) return LUTGEMM_EINVAL;
        if (!q.sumsq_in_f32 && q.sumsq_in_slots != 0) return LUTGEMM_EINVAL;
        // the slots are those a completing problem of K outputs fills (one per 32 columns); the
        // matrix-core kernel reads them four at a time
        if (q.sumsq_in_f32 && (q.K % 32 != 0 || q.sumsq_in_slots != q.K / 32)) return LUTGEMM_EINVAL;
        if (!aligned(q.next_input_f16, 2) || !aligned(q.next_norm_weight_f16, 2) || !aligned(q.sumsq_out_f32, 4) ||
            !aligned(q.sumsq_in_f32, 16))
            return LUTGEMM_EALIGN;
        p.next_w = (const __half *)q.next_norm_weight_f16;
        p.next_in = (__half *)q.next_input_f16;
        p.sumsq_out = q.sumsq_out_f32;
        p.sumsq_in = q.sumsq_in_f32;
        p.sumsq_slots = q.sumsq_in_slots;
        // one kernel instance per transform: the problems of a launch share theirs
        const int mine = p.norm_w ? kXNorm : p.gate ? kXGate : kXNone;
        if (i > 0 && mine != xform) return LUTGEMM_EUNSUP;
        xform = mine;
        plain = plain && !p.norm_w && !p.gate && !p.overwrite && !p.next_in && !p.sumsq_out && !p.sumsq_in;
        all_mfma = all_mfma && mfma_eligible(p, kRowF16);
        words += (size_t)q.M * q.N;
        total_bytes += (long)q.N * (q.K / 8) * q.nb * q.M;
    }
    // Every problem finishes its outputs with a plain read-modify-write, and the outputs are
    // requested early: nothing a problem of the launch writes (out, next_input, sumsq_out) may
    // overlap anything another write or a read of the launch (x, gate) touches.
    {
        struct Span {
            const char *lo, *hi;
            bool written;
        };
        Span spans[6 * kMaxGroup];
        int n = 0;
        auto add = [&](const void *ptr, size_t bytes, bool written) {
            if (ptr) spans[n++] = Span{(const char *)ptr, (const char *)ptr + bytes, written};
        };
        for (int i = 0; i < count; ++i) {
            const Problem &p = g.p[i];
            const size_t mn = (size_t)p.M * p.N, mk = (size_t)p.M * p.K;
            add(p.out, mn * 2, true);
            add(p.next_in, mn * 2, true);
            add(p.sumsq_out, (size_t)p.M * (p.N / 32) * 4, true);
            add(p.x, mk * 2, false);
            add(p.gate, mk * 2, false);
            add(p.sumsq_in, (size_t)p.M * p.sumsq_slots * 4, false);
        }
        for (int i = 0; i < n; ++i)
            for (int j = i + 1; j < n; ++j)
                if ((spans[i].written || spans[j].written) && spans[i].lo < spans[j].hi && spans[j].lo < spans[i].hi)
                    return LUTGEMM_EINVAL;
    }
    // The matrix-core kernel takes plain and (as a group launch) overwriting problems.
    // Input transforms stay with the look-up kernel: there a workgroup transforms only
    // its K-slice of one row, while every 64-output workgroup of the matrix-core kernel
    // would redo the transform of all rows (measured slower than a separate kernel).
    bool same_height = true;
    for (int i = 1; i < count; ++i) same_height = same_height && ((g.p[i].M > 16) == (g.p[0].M > 16));
    if (all_mfma && xform == kXNone && same_height && (count > 1 || !plain)) return run_mfma_group(g, acc);
    if (plain && all_mfma) {
        for (int i = 0; i < count; ++i) {
            int rc = run_mfma(g.p[i], acc);
            if (rc != LUTGEMM_OK) return rc;
        }
        return LUTGEMM_OK;
    }
    Problem *ps[kMaxGroup];
    for (int i = 0; i < count; ++i) ps[i] = &g.p[i];
    int begin = 0;
    bool any_split = false;
    {
        int rc = share_workgroups(ps, count, (long)target_blocks(total_bytes), &begin, &any_split);
        if (rc != LUTGEMM_OK) return rc;
    }
    if (any_split) {
        unsigned long long *base = nullptr;
        int rc = accum_words(acc, words, &base);
        if (rc != LUTGEMM_OK) return rc;
        size_t off = 0;
        for (int i = 0; i < count; ++i) {
            g.p[i].accum = base + off;
            off += (size_t)g.p[i].M * g.p[i].N;
        }
    }
    const hipError_t e = count == 1 ? launch_gemv_fused(g.p[0], xform, acc.stream) : launch_gemv_group(g, xform, begin, acc.stream);
    return e == hipSuccess ? LUTGEMM_OK : hip_fail(e);
}

// Row-wise problems of ONE launch that hand activations to each other through tagged rows.
// The launch's units (one workgroup's range of one problem) are numbered in the order the
// problems are given and taken in that order, so a problem that waits for a tag must come after
// the problem of the call that writes it.  Problems that wait for the same set of producers run
// side by side and share a workgroup budget (a "stage").
// Workgroups of a chained launch: all of them must be resident at once (a unit may wait for a
// unit of another workgroup), so at most what the device holds of this kernel.
int chain_grid(int *out)
{
    int resident = 0;
    const hipError_t e = chain_resident_workgroups(&resident);
    if (e != hipSuccess) return hip_fail(e);
    if (resident < 1) return LUTGEMM_EUNSUP;
    const int v = option(LUTGEMM_OPTION_CHAIN_GRID);
    *out = v > 0 && v < resident ? v : resident;
    return LUTGEMM_OK;
}

// Validate the problems of a chained launch and cut them into units (no device work when
// grid_in > 0).  On return c.g holds the planned problems, c.unit_start the units, depth[] the
// stage of every problem, *grid the workgroups of the launch.
int plan_chain(int count, const lutgemm_chain_problem *problems, int grid_in, Chain &c, int *depth, int *grid_out,
               bool *any_split_out, size_t *words_out)
{
    Group &g = c.g;
    g.count = count;
    size_t words = 0;
    unsigned direct[kMaxGroup], after[kMaxGroup], before_inputs[kMaxGroup];
    for (int i = 0; i < count; ++i) {
        const lutgemm_chain_problem &cq = problems[i];
        const lutgemm_fused_problem &q = cq.p;
        Problem &p = g.p[i];
        int rc = fill_problem(p, kRowF16, q.bW, q.alpha_f16, nullptr, q.x_f16, q.out_f16, q.N, q.K, q.nb, q.num_groups, q.M);
        if (rc != LUTGEMM_OK) return rc;
        if (q.M > LUTGEMM_CHAIN_MAX_ROWS) return LUTGEMM_EUNSUP;   // one row per workgroup: the look-up kernel only
        if (q.norm_weight_f16 && q.gate_f16) return LUTGEMM_EINVAL;
        if (q.overwrite != 0 && q.overwrite != 1) return LUTGEMM_EINVAL;
        if (q.norm_weight_f16 && !(q.norm_eps >= 0.0f)) return LUTGEMM_EINVAL;
        if (!aligned(q.norm_weight_f16, 16) || !aligned(q.gate_f16, 16)) return LUTGEMM_EALIGN;
        if (q.next_norm_weight_f16 || q.next_input_f16 || q.sumsq_out_f32 || q.sumsq_in_f32 || q.sumsq_in_slots)
            return LUTGEMM_EUNSUP;   // the RMSNorm of a chained problem is formed from the (tagged) row itself
        if (cq.x_tag < 0 || cq.x_tag > LUTGEMM_CHAIN_MAX_TAG || cq.gate_tag < 0 || cq.gate_tag > LUTGEMM_CHAIN_MAX_TAG ||
            cq.out_tag < 0 || cq.out_tag > LUTGEMM_CHAIN_MAX_TAG)
            return LUTGEMM_EINVAL;
        if (cq.gate_tag && !q.gate_f16) return LUTGEMM_EINVAL;
        // a thread holds its share of a norm row in two 16-byte registers sets: K <= 8192 when the row is tagged
        if (q.norm_weight_f16 && cq.x_tag && q.K > 8 * 2 * kThreads) return LUTGEMM_EUNSUP;
        p.norm_w = (const __half *)q.norm_weight_f16;
        p.gate = (const __half *)q.gate_f16;
        p.norm_eps = q.norm_eps;
        p.overwrite = q.overwrite;
        p.x_tag = cq.x_tag;
        p.gate_tag = cq.gate_tag;
        p.out_tag = cq.out_tag;
        words += (size_t)q.M * q.N;
        // which problems of the call this one waits for: the writers of the tags it reads
        depth[i] = 0;
        direct[i] = 0;
        auto producer = [&](const void *row, int tag) -> int {
            if (!tag) return LUTGEMM_OK;
            for (int j = 0; j < count; ++j) {
                if (problems[j].p.out_f16 != row || problems[j].out_tag != tag) continue;
                if (j >= i) return LUTGEMM_EINVAL;   // dispatched after its consumer: the wait could starve it
                direct[i] |= 1u << j;
                if (depth[j] + 1 > depth[i]) depth[i] = depth[j] + 1;
            }
            return LUTGEMM_OK;   // (no writer in the call: the row comes from elsewhere, the wait is bounded)
        };
        rc = producer(q.x_f16, cq.x_tag);
        if (rc != LUTGEMM_OK) return rc;
        rc = producer(q.gate_f16, cq.gate_tag);
        if (rc != LUTGEMM_OK) return rc;
        if (i > 0 && depth[i] < depth[i - 1]) return LUTGEMM_EINVAL;   // stages in dispatch order
        // everything this problem waits for, directly or not (after[i]), and through at least one
        // other problem (before_inputs[i])
        after[i] = direct[i];
        before_inputs[i] = 0;
        for (int j = 0; j < i; ++j)
            if (direct[i] >> j & 1u) {
                after[i] |= after[j];
                before_inputs[i] |= after[j];
            }
    }
    // What may overlap.  A problem writes an output only after contributions covering all of K
    // have arrived, each of which has waited for its inputs: when problem i writes anything, every
    // problem in after[i] has finished, and when a workgroup of i has its inputs, every problem in
    // before_inputs[i] has.  So the same tagged row may be written by several problems of a call
    // (a residual row that two GEMVs complete one after the other) and read in between, as long as
    // the waits order them; plain rows may not be shared between a writer and anyone else.
    for (int i = 0; i < count; ++i) {
        const Problem &a = g.p[i];
        const char *a0 = (const char *)a.out, *a1 = a0 + (size_t)a.M * a.N * (a.out_tag ? 4 : 2);
        auto overlaps = [&](const void *ptr, size_t bytes) {
            return ptr && a0 < (const char *)ptr + bytes && (const char *)ptr < a1;
        };
        for (int j = 0; j < count; ++j) {
            if (i == j) continue;
            const Problem &b = g.p[j];
            if (j < i && overlaps(b.out, (size_t)b.M * b.N * (b.out_tag ? 4 : 2))) {
                // an earlier writer of the same row: it must have finished before this one writes,
                // and before this one reads the row when it accumulates into it
                const bool same_row = a.out_tag && b.out_tag && a.out == b.out && a.out_tag != b.out_tag;
                const unsigned need = a.overwrite ? after[i] : before_inputs[i];
                if (!same_row || !(need >> j & 1u)) return LUTGEMM_EINVAL;
            }
            auto read_ok = [&](const __half *row, int tag, size_t bytes) {
                if (!overlaps(row, bytes)) return true;
                if (!(a.out_tag && tag && (const void *)row == (const void *)a.out)) return false;
                if (tag == a.out_tag) return i < j;             // the hand-over itself
                return (after[i] >> j & 1u) || (after[j] >> i & 1u);   // rewritten after the reader, or read after the writer
            };
            if (!read_ok(b.x, b.x_tag, (size_t)b.M * b.K * (b.x_tag ? 4 : 2))) return LUTGEMM_EINVAL;
            if (!read_ok(b.gate, b.gate_tag, (size_t)b.M * b.K * (b.gate_tag ? 4 : 2))) return LUTGEMM_EINVAL;
        }
    }
    // Plan stage by stage: the problems of a stage share one round of the grid (every workgroup
    // takes one unit of the stage) unless LUTGEMM_OPTION_CHAIN_BLOCKS says otherwise.
    int grid = grid_in;
    if (grid <= 0) {
        int rc = chain_grid(&grid);
        if (rc != LUTGEMM_OK) return rc;
    }
    const int stage_blocks = option(LUTGEMM_OPTION_CHAIN_BLOCKS) > 0 ? option(LUTGEMM_OPTION_CHAIN_BLOCKS) : grid;
    int begin = 0;
    bool any_split = false;
    for (int first = 0; first < count;) {
        int last = first;
        long bytes = 0;
        Problem *ps[kMaxGroup];
        while (last < count && depth[last] == depth[first]) {
            ps[last - first] = &g.p[last];
            bytes += (long)g.p[last].N * (g.p[last].K / 8) * g.p[last].nb * g.p[last].M;
            ++last;
        }
        // a range's activations are fetched as one window of sixteen items: a stage whose units
        // would hold more takes further rounds of the grid
        constexpr int kWindowItems = kThreads / kTables;
        for (long rounds = 1;; ++rounds) {
            bool split = false;
            int rc = share_workgroups(ps, last - first, rounds * (long)stage_blocks, &begin, &split);
            if (rc != LUTGEMM_OK) return rc;
            bool fits = true;
            for (int i = first; i < last; ++i) fits = fits && g.p[i].items_per_wg <= kWindowItems;
            if (fits) {
                any_split = any_split || split;
                break;
            }
            if (rounds >= 4096) return LUTGEMM_EUNSUP;
        }
        first = last;
    }
    c.unit_start[0] = 0;
    for (int i = 0; i < count; ++i) c.unit_start[i + 1] = c.unit_start[i] + g.p[i].n_blocks;
    for (int i = count; i < kMaxGroup; ++i) c.unit_start[i + 1] = c.unit_start[count];
    const int total_units = c.unit_start[count];
    *grid_out = total_units < grid ? total_units : grid;
    *any_split_out = any_split;
    *words_out = words;
    (void)begin;
    return LUTGEMM_OK;
}

int run_chain(int count, const lutgemm_chain_problem *problems, const lutgemm_chain_control *ctl, const Accum &acc)
{
    if (!ctl || !ctl->status) return LUTGEMM_EINVAL;
    if (!aligned(ctl->status, 4) || !aligned(ctl->epoch, 4)) return LUTGEMM_EALIGN;
    Chain c{};
    Group &g = c.g;
    int depth[kMaxGroup], grid = 0;
    bool any_split = false;
    size_t words = 0;
    int rc = plan_chain(count, problems, 0, c, depth, &grid, &any_split, &words);
    if (rc != LUTGEMM_OK) return rc;
    if (any_split) {
        unsigned long long *base = nullptr;
        rc = accum_words(acc, words, &base);
        if (rc != LUTGEMM_OK) return rc;
        size_t off = 0;
        for (int i = 0; i < count; ++i) {
            g.p[i].accum = base + off;
            off += (size_t)g.p[i].M * g.p[i].N;
        }
    }
    c.ctl.epoch = ctl->epoch;
    c.ctl.status = ctl->status;
    const unsigned us = ctl->spin_limit_us ? ctl->spin_limit_us : 100000u;
    c.ctl.spin_ticks = (long long)us * 100;   // the wall clock ticks at 100 MHz
    const hipError_t e = launch_gemv_chain(c, grid, acc.stream);
    return e == hipSuccess ? LUTGEMM_OK : hip_fail(e);
}

// ---- tagged rows: conversions and the epoch word ---------------------------------------------
__global__ void __launch_bounds__(256) tag_rows_kernel(uint32_t *dst, const unsigned short *src, size_t n, int tag,
                                                       const uint32_t *epoch)
{
    const uint32_t t = effective_tag(tag, epoch ? *epoch : 0u) << 16;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) dst[i] = t | src[i];
}

__global__ void __launch_bounds__(256) untag_rows_kernel(unsigned short *dst, const uint32_t *src, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
        dst[i] = (unsigned short)src[i];
}

__global__ void advance_epoch_kernel(uint32_t *epoch, uint32_t by)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) *epoch += by;
}

// ---- measurement kernels ------------------------------------------------------------
__global__ void __launch_bounds__(256) copy_kernel(u32x4 *dst, const u32x4 *src, size_t n16)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n16; i += stride) dst[i] = src[i];
}

// Reads `n16` 16-byte units and does nothing with them: what any kernel that has to
// stream that many bytes pays at least.
__global__ void __launch_bounds__(256) stream_read_kernel(const u32x4 *__restrict__ src, size_t n16, uint32_t *sink)
{
    constexpr int kUnroll = 8;
    size_t i = (size_t)blockIdx.x * 256 * kUnroll + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256 * kUnroll;
    u32x4 acc = {0u, 0u, 0u, 0u};
    for (; i + 256 * (kUnroll - 1) < n16; i += stride) {
        u32x4 v[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) v[u] = __builtin_nontemporal_load(src + i + 256 * u);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) acc ^= v[u];
    }
    for (; i < n16; i += 256) acc ^= __builtin_nontemporal_load(src + i);
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u && sink) sink[0] = acc.x;  // (keeps the loads alive)
}

// Same launch geometry and LDS footprint as the look-up kernel, no work.
__global__ void __launch_bounds__(kThreads) empty_kernel(uint32_t *sink)
{
    __shared__ float lds[kLutDwords + kStageDwords];
    if (sink && threadIdx.x == 0xffff) sink[0] = (uint32_t)lds[threadIdx.x];
}

}  // namespace
}  // namespace lutgemm

using namespace lutgemm;

int lutgemm_internal_hip_fail(int hip_error) { return hip_fail((hipError_t)hip_error); }

int lutgemm::option(int which)
{
    load_options();
    return g_option[which].load(std::memory_order_relaxed);
}

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
    case LUTGEMM_ECAPTURE:
        return "the stream is being captured and its workspace would have to grow "
               "(call lutgemm_reserve_workspace before capturing)";
    case LUTGEMM_ETIMEDOUT:
        return "a problem of a chained launch gave up waiting for a tagged row (nothing wrote it within the limit)";
    case LUTGEMM_ETOOBIG:
        return "M * N exceeds LUTGEMM_NOALLOC_MAX_WORDS, the fixed buffer of the entry point that does not allocate";
    default: return "unknown lutgemm error";
    }
}

int lutgemm_last_hip_error(void) { return g_last_hip_error; }

int lutgemm_set_timestamp_buffer(void *readings, size_t count)
{
#ifdef LUTGEMM_TIMESTAMPS
    if (!aligned(readings, 8) || (count > 0 && !readings)) return LUTGEMM_EINVAL;
    g_stamps.store((unsigned long long *)readings);
    g_stamp_slots.store((long long)count);
    return LUTGEMM_OK;
#else
    (void)readings;
    (void)count;
    return LUTGEMM_EUNSUP;   // this build of the library reads no clocks
#endif
}

int lutgemm_set_option(int which, int value)
{
    if (which < 0 || which >= LUTGEMM_OPTION_COUNT) return LUTGEMM_EINVAL;
    load_options();
    g_option[which].store(value < 0 ? env_int(kOptions[which].env, kOptions[which].fallback) : value);
    return LUTGEMM_OK;
}

int lutgemm_get_option(int which)
{
    if (which < 0 || which >= LUTGEMM_OPTION_COUNT) return LUTGEMM_EINVAL;
    return option(which);
}

int lutgemm_gemv_rowwise_f16(const uint32_t *bW, const void *alpha_f16, const void *x_f16,
                             void *out_f16, int N, int K, int nb, int num_groups, int M,
                             void *stream)
{
    return run(kRowF16, bW, alpha_f16, nullptr, x_f16, out_f16, N, K, nb, num_groups, M,
               Accum{(hipStream_t)stream});
}

int lutgemm_gemv_rowwise_pow2_f16(const uint32_t *bW, const void *alpha_f16, const void *x_f16,
                                  void *out_f16, int N, int K, int nb, int num_groups, int M,
                                  void *stream)
{
    return run(kRowF16, bW, alpha_f16, nullptr, x_f16, out_f16, N, K, nb, num_groups, M,
               Accum{(hipStream_t)stream}, true);
}

int lutgemm_gemv_rowwise_f16_noalloc(const uint32_t *bW, const void *alpha_f16, const void *x_f16,
                                     void *out_f16, int N, int K, int nb, int num_groups, int M,
                                     void *stream)
{
    if (N > 0 && M > 0 && (size_t)N * (size_t)M > (size_t)LUTGEMM_NOALLOC_MAX_WORDS) return LUTGEMM_ETOOBIG;
    // set-up on the first call on a device, whether or not this call needs the words
    unsigned long long *unused = nullptr;
    const int rc = scratch_address(&unused);
    if (rc != LUTGEMM_OK) return rc;
    return run(kRowF16, bW, alpha_f16, nullptr, x_f16, out_f16, N, K, nb, num_groups, M,
               Accum{(hipStream_t)stream, true});
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
    return run_group(count, f, Accum{(hipStream_t)stream_v});
}

int lutgemm_gemv_rowwise_f16_fused(int count, const lutgemm_fused_problem *problems, void *stream_v)
{
    if (!problems || count < 1 || count > kMaxGroup) return LUTGEMM_EINVAL;
    return run_group(count, problems, Accum{(hipStream_t)stream_v});
}

int lutgemm_gemv_rowwise_f16_chain(int count, const lutgemm_chain_problem *problems,
                                   const lutgemm_chain_control *control, void *stream_v)
{
    if (!problems || count < 1 || count > kMaxGroup) return LUTGEMM_EINVAL;
    return run_chain(count, problems, control, Accum{(hipStream_t)stream_v});
}

int lutgemm_describe_chain_plan(int count, const lutgemm_chain_problem *problems, int workgroups,
                                lutgemm_chain_plan *plan)
{
    if (!problems || !plan || count < 1 || count > kMaxGroup || workgroups < 0) return LUTGEMM_EINVAL;
    Chain c{};
    int depth[kMaxGroup], grid = 0;
    bool any_split = false;
    size_t words = 0;
    const int rc = plan_chain(count, problems, workgroups, c, depth, &grid, &any_split, &words);
    if (rc != LUTGEMM_OK) return rc;
    *plan = lutgemm_chain_plan{};
    plan->workgroups = grid;
    plan->units = c.unit_start[count];
    plan->needs_workspace = any_split;
    for (int i = 0; i < count; ++i) {
        plan->stage[i] = depth[i];
        plan->first_unit[i] = c.unit_start[i];
        plan->unit_count[i] = c.g.p[i].n_blocks;
        plan->items_per_unit[i] = c.g.p[i].items_per_wg;
    }
    return LUTGEMM_OK;
}

int lutgemm_chain_tag_rows(void *dst_tagged, const void *src_f16, size_t count, int tag, const uint32_t *epoch,
                           void *stream)
{
    if (!dst_tagged || !src_f16 || tag < 1 || tag > LUTGEMM_CHAIN_MAX_TAG) return LUTGEMM_EINVAL;
    if (!aligned(dst_tagged, 4) || !aligned(src_f16, 2) || !aligned(epoch, 4)) return LUTGEMM_EALIGN;
    if (count == 0) return LUTGEMM_OK;
    size_t blocks = (count + 255) / 256;
    if (blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL(tag_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (uint32_t *)dst_tagged,
                       (const unsigned short *)src_f16, count, tag, epoch);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? LUTGEMM_OK : hip_fail(e);
}

int lutgemm_chain_untag_rows(void *dst_f16, const void *src_tagged, size_t count, void *stream)
{
    if (!dst_f16 || !src_tagged) return LUTGEMM_EINVAL;
    if (!aligned(dst_f16, 2) || !aligned(src_tagged, 4)) return LUTGEMM_EALIGN;
    if (count == 0) return LUTGEMM_OK;
    size_t blocks = (count + 255) / 256;
    if (blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL(untag_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (unsigned short *)dst_f16, (const uint32_t *)src_tagged, count);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? LUTGEMM_OK : hip_fail(e);
}

int lutgemm_chain_advance_epoch(uint32_t *epoch, uint32_t by, void *stream)
{
    if (!epoch) return LUTGEMM_EINVAL;
    if (!aligned(epoch, 4)) return LUTGEMM_EALIGN;
    hipLaunchKernelGGL(advance_epoch_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, epoch, by);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? LUTGEMM_OK : hip_fail(e);
}

int lutgemm_chain_status(const uint32_t *status, void *stream)
{
    if (!status) return LUTGEMM_EINVAL;
    uint32_t v = 0;
    hipError_t e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e);
    e = hipMemcpy(&v, status, sizeof(v), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return hip_fail(e);
    return v ? LUTGEMM_ETIMEDOUT : LUTGEMM_OK;
}

int lutgemm_gemv_uniform_f16(const uint32_t *bW, const void *alpha_f16, const void *qbias_f16,
                             const void *x_f16, void *out_f16, int N, int K, int nb,
                             int num_groups, int M, void *stream)
{
    return run(kUniformF16, bW, alpha_f16, qbias_f16, x_f16, out_f16, N, K, nb, num_groups, M,
               Accum{(hipStream_t)stream});
}

int lutgemm_gemv_block_f16(const uint32_t *bW, const void *alpha_f16, const void *x_f16,
                           void *out_f16, int N, int K, int nb, int num_groups, int M,
                           void *stream)
{
    return run(kBlockF16, bW, alpha_f16, nullptr, x_f16, out_f16, N, K, nb, num_groups, M,
               Accum{(hipStream_t)stream});
}

int lutgemm_gemv_block_shift_u16(const uint32_t *bW, const uint16_t *alpha_u16, const void *x_f16,
                                 void *out_f16, int N, int K, int nb, int num_groups,
                                 int num_apot, int M, void *stream)
{
    if (num_apot != 3) return LUTGEMM_EUNSUP;
    return run(kBlockShiftU16, bW, alpha_u16, nullptr, x_f16, out_f16, N, K, nb, num_groups, M,
               Accum{(hipStream_t)stream});
}

int lutgemm_gemv_block_apot_i8(const uint32_t *bW, const int8_t *alpha_i8, const void *x_f16,
                               void *out_f16, int N, int K, int nb, int num_groups, int num_apot,
                               int M, void *stream)
{
    if (num_apot != 3) return LUTGEMM_EUNSUP;
    return run(kBlockApotI8, bW, alpha_i8, nullptr, x_f16, out_f16, N, K, nb, num_groups, M,
               Accum{(hipStream_t)stream});
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

int lutgemm_describe_plan(int format, int N, int K, int nb, int groups, int M, lutgemm_plan *plan)
{
    if (!plan || format < LUTGEMM_FORMAT_ROWWISE_F16 || format > LUTGEMM_FORMAT_UNIFORM_F16) return LUTGEMM_EINVAL;
    // (nothing is dereferenced while planning: any aligned non-null address will do)
    alignas(16) static const uint64_t dummy[2] = {0, 0};
    Problem p;
    int rc = fill_problem(p, format, (const uint32_t *)dummy, dummy, dummy, dummy, (void *)dummy, N, K, nb, groups, M);
    if (rc != LUTGEMM_OK) return rc;
    int kernel = kLookup, mrows = 1;
    rc = plan_single(p, format, &kernel, &mrows);
    if (rc != LUTGEMM_OK) return rc;
    *plan = lutgemm_plan{};
    plan->kernel = kernel;
    plan->workgroups = p.n_blocks;
    plan->rows_per_pass = mrows;
    plan->row_chunks = p.mchunks;
    if (kernel == kMatrixCore) {
        plan->tiles = p.n_tiles;
        plan->tile_columns = kMfmaTileCols;
        plan->k_units = p.nsets;
        plan->k_slices = p.ksplit;
        plan->units_per_slice = p.sets_per_split;
        plan->needs_workspace = p.ksplit > 1;
    } else {
        plan->tiles = p.n_tiles;
        plan->tile_columns = p.twin ? 2 * kTileCols : kTileCols;
        plan->k_units = p.nsets;
        plan->long_ranges = p.long_ranges;
        plan->items_per_long_range = p.items_per_wg;
        plan->items_per_short_range = p.short_items;
        plan->ranges = p.wgs_per_chunk;
        plan->needs_workspace = lookup_splits_k(p);
    }
    return LUTGEMM_OK;
}

int lutgemm_describe_pow2_plan(int N, int K, int nb, int groups, int M, lutgemm_plan *plan)
{
    int rc = lutgemm_describe_plan(LUTGEMM_FORMAT_ROWWISE_F16, N, K, nb, groups, M, plan);
    if (rc != LUTGEMM_OK) return rc;
    alignas(16) static const uint64_t dummy[2] = {0, 0};
    Problem p;
    rc = fill_problem(p, kRowF16, (const uint32_t *)dummy, dummy, dummy, dummy, (void *)dummy, N, K, nb, groups, M);
    if (rc != LUTGEMM_OK) return rc;
    if (!(mfma_eligible(p, kRowF16) && p.M >= mfma_min_rows() && mx_wanted(p))) return LUTGEMM_OK;
    plan_mx(p);
    *plan = lutgemm_plan{};
    plan->kernel = 2;
    plan->workgroups = p.n_blocks;
    plan->rows_per_pass = mx_chunk_rows(p.M);
    plan->row_chunks = p.mchunks;
    plan->tiles = p.n_tiles;
    plan->tile_columns = kMfmaTileCols;
    plan->k_units = p.nsets;
    plan->k_slices = p.ksplit;
    plan->units_per_slice = p.sets_per_split;
    plan->needs_workspace = p.ksplit > 1;
    return LUTGEMM_OK;
}

size_t lutgemm_workspace_words(int N, int M)
{
    if (N <= 0 || M <= 0) return 0;
    return (size_t)N * (size_t)M;
}

int lutgemm_reserve_workspace(void *stream, size_t words)
{
    unsigned long long *unused = nullptr;
    return stream_workspace((hipStream_t)stream, words, &unused);
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

int lutgemm_measure_stream_read(const void *src, size_t bytes, void *sink, void *stream)
{
    if (!src || bytes % 16 != 0) return LUTGEMM_EINVAL;
    if (!aligned(src, 16)) return LUTGEMM_EALIGN;
    if (bytes == 0) return LUTGEMM_OK;
    const size_t n16 = bytes / 16;
    size_t blocks = (n16 + 256 * 8 - 1) / (256 * 8);
    if (blocks > 2048) blocks = 2048;
    hipLaunchKernelGGL(stream_read_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4 *)src, n16, (uint32_t *)sink);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e);
    return LUTGEMM_OK;
}

int lutgemm_measure_empty_launch(int workgroups, void *stream)
{
    if (workgroups < 1 || workgroups > 65535) return LUTGEMM_EINVAL;
    hipLaunchKernelGGL(empty_kernel, dim3((unsigned)workgroups), dim3(kThreads), 0, (hipStream_t)stream,
                       (uint32_t *)nullptr);
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
            if (it->second.split) (void)hipFree(it->second.split);
            for (void *old : it->second.retired_split) (void)hipFree(old);
            it = g_workspaces.erase(it);
        } else {
            ++it;
        }
    }
    return LUTGEMM_OK;
}

}  // extern "C"
