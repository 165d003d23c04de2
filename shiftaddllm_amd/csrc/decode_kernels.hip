// Glue kernels of a single-token decode step around the LUT-GEMV calls, for
// gfx950: RMSNorm (which also clears the next GEMV's accumulate-into outputs),
// rotary embedding + KV-cache append + one-query attention, and SiLU(gate)*up.
//
// A decoder block at one token per sequence is, with these, eight launches:
//   rmsnorm -> {q,k,v} GEMV -> attention -> o_proj GEMV (accumulates into the
//   residual stream) -> rmsnorm -> {gate,up} GEMV -> silu*mul -> down_proj GEMV
//   (accumulates into the residual stream).
// The reference runs the same step through HuggingFace's eager OPT decoder
// (model/opt.py:367-423 of the ShiftAddLLM checkout drives it); it has no fused
// kernels of this kind.  All of them are tiny and latency bound: they exist to
// replace some forty framework kernels per block by four.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "lutgemm_gfx950.h"
#include "lutgemm_internal.h"

namespace {

constexpr int kThreads = 256;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// The value of another lane of the same row of 16, by a data-parallel-primitive move.
template <int CTRL>
__device__ __forceinline__ float dpp_lane(float v)
{
    const int vi = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(vi, vi, CTRL, 0xf, 0xf, false));
}

// Sum / maximum over the 64 lanes of a wave on the vector ALU: xor 1 and 2 inside quads, the
// mirrored quad and the mirrored half of each row of 16, then the four rows by lane reads.
template <bool MAX>
__device__ __forceinline__ float wave_reduce(float v)
{
    auto op = [](float a, float b) { return MAX ? fmaxf(a, b) : a + b; };
    v = op(v, dpp_lane<0xb1>(v));   // quad_perm [1,0,3,2]
    v = op(v, dpp_lane<0x4e>(v));   // quad_perm [2,3,0,1]
    v = op(v, dpp_lane<0x141>(v));  // row_half_mirror
    v = op(v, dpp_lane<0x140>(v));  // row_mirror
    const int vi = __builtin_bit_cast(int, v);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 0));
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 32));
    const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(vi, 48));
    return op(op(r0, r1), op(r2, r3));
}

__device__ __forceinline__ float wave_sum(float v) { return wave_reduce<false>(v); }
__device__ __forceinline__ float wave_max(float v) { return wave_reduce<true>(v); }

// Sum (or max) over the 256 threads of a workgroup; `red` holds 4 floats.
template <bool MAX>
__device__ __forceinline__ float block_reduce(float v, float *red)
{
    v = MAX ? wave_max(v) : wave_sum(v);
    __syncthreads();  // `red` may still be read from a previous reduction
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    const float a = red[0], b = red[1], c = red[2], d = red[3];
    return MAX ? fmaxf(fmaxf(a, b), fmaxf(c, d)) : (a + b) + (c + d);
}

__device__ __forceinline__ void unpack8(const u32x4 &v, float f[8])
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = __half2float(__ushort_as_half((unsigned short)(w[i] & 0xffffu)));
        f[2 * i + 1] = __half2float(__ushort_as_half((unsigned short)(w[i] >> 16)));
    }
}

__device__ __forceinline__ uint32_t pack2(float lo, float hi)
{
    return (uint32_t)__half_as_ushort(__float2half_rn(lo)) |
           ((uint32_t)__half_as_ushort(__float2half_rn(hi)) << 16);
}

// y[r] = fp16(fp16(x[r] * rsqrt(mean(x[r]^2) + eps)) * w); workgroups beyond
// `rows` only help clearing `clear_units` 16-byte units at `clear`.
__global__ void __launch_bounds__(kThreads)
rmsnorm_kernel(const __half *__restrict__ x, const __half *__restrict__ w, __half *__restrict__ y, int rows,
               int hidden, float eps, u32x4 *__restrict__ clear, long clear_units)
{
    __shared__ float red[4];
    const int tid = threadIdx.x;
    for (long u = (long)blockIdx.x * kThreads + tid; u < clear_units; u += (long)gridDim.x * kThreads)
        clear[u] = (u32x4){0u, 0u, 0u, 0u};
    const int r = blockIdx.x;
    if (r >= rows) return;
    const u32x4 *xr = (const u32x4 *)(x + (size_t)r * hidden);
    const u32x4 *wr = (const u32x4 *)w;
    u32x4 *yr = (u32x4 *)(y + (size_t)r * hidden);
    const int chunks = hidden / 8;
    // the first kHeld chunks of a thread stay in registers, with the matching weights,
    // so that rows up to 8192 wide cost one memory round trip
    constexpr int kHeld = 4;
    u32x4 xv[kHeld], wv[kHeld];
#pragma unroll
    for (int u = 0; u < kHeld; ++u) {
        const int c = min(tid + kThreads * u, chunks - 1);
        xv[u] = xr[c];
        wv[u] = wr[c];
    }
    float ss = 0.0f;
#pragma unroll
    for (int u = 0; u < kHeld; ++u) {
        if (tid + kThreads * u < chunks) {
            float f[8];
            unpack8(xv[u], f);
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = fmaf(f[i], f[i], ss);
        }
    }
    for (int c = tid + kThreads * kHeld; c < chunks; c += kThreads) {
        float f[8];
        unpack8(xr[c], f);
#pragma unroll
        for (int i = 0; i < 8; ++i) ss = fmaf(f[i], f[i], ss);
    }
    ss = block_reduce<false>(ss, red);
    const float scale = rsqrtf(ss / (float)hidden + eps);
    auto finish = [&](const u32x4 &xc, const u32x4 &wc) {
        float f[8], g[8];
        unpack8(xc, f);
        unpack8(wc, g);
        u32x4 o;
        uint32_t *ow = (uint32_t *)&o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float a = __half2float(__float2half_rn(f[2 * i] * scale)) * g[2 * i];
            const float b = __half2float(__float2half_rn(f[2 * i + 1] * scale)) * g[2 * i + 1];
            ow[i] = pack2(a, b);
        }
        return o;
    };
#pragma unroll
    for (int u = 0; u < kHeld; ++u)
        if (tid + kThreads * u < chunks) yr[tid + kThreads * u] = finish(xv[u], wv[u]);
    for (int c = tid + kThreads * kHeld; c < chunks; c += kThreads) yr[c] = finish(xr[c], wr[c]);
}

// One workgroup per (sequence b, query head h).  Rotates q and the new k by the
// angle of position *pos, appends k and v to the cache (one writer per kv head),
// and attends over cache positions 0..pos, the newest one taken from LDS.
//   q [B][H*hd], k,v [B][KV*hd], cos,sin [max_pos][hd], caches [B][KV][max_pos][hd],
//   out [B][H*hd].  Dynamic LDS: (3*hd + max_pos + 4 + (256/hd)*hd) floats.
__global__ void __launch_bounds__(kThreads)
attention_kernel(const __half *__restrict__ q, const __half *__restrict__ k, const __half *__restrict__ v,
                 const __half *__restrict__ cos_t, const __half *__restrict__ sin_t, __half *__restrict__ k_cache,
                 __half *__restrict__ v_cache, const long long *__restrict__ pos_ptr, __half *__restrict__ out,
                 int H, int KV, int hd, int max_pos)
{
    extern __shared__ float lds[];
    float *q_s = lds;
    float *k_s = q_s + hd;
    float *v_s = k_s + hd;
    float *score = v_s + hd;
    float *red = score + max_pos;
    float *part = red + 4;

    const int tid = threadIdx.x;
    const int b = blockIdx.x / H, h = blockIdx.x % H;
    const int rep = H / KV, kvh = h / rep;
    int pos = (int)*pos_ptr;
    pos = min(max(pos, 0), max_pos - 1);
    const int half_d = hd / 2;
    const size_t cache_row0 = ((size_t)b * KV + kvh) * max_pos;

    for (int i = tid; i < hd; i += kThreads) {
        const float c = __half2float(cos_t[(size_t)pos * hd + i]);
        const float s = __half2float(sin_t[(size_t)pos * hd + i]);
        const __half *qh = q + ((size_t)b * H + h) * hd;
        const __half *kh = k + ((size_t)b * KV + kvh) * hd;
        const int j = i < half_d ? i + half_d : i - half_d;
        const float sign = i < half_d ? -1.0f : 1.0f;
        const __half qr = __float2half_rn(__half2float(qh[i]) * c + sign * __half2float(qh[j]) * s);
        const __half kr = __float2half_rn(__half2float(kh[i]) * c + sign * __half2float(kh[j]) * s);
        const __half vv = v[((size_t)b * KV + kvh) * hd + i];
        q_s[i] = __half2float(qr);
        k_s[i] = __half2float(kr);
        v_s[i] = __half2float(vv);
        if (h % rep == 0) {
            k_cache[(cache_row0 + pos) * hd + i] = kr;
            v_cache[(cache_row0 + pos) * hd + i] = vv;
        }
    }
    __syncthreads();

    const float scale = rsqrtf((float)hd);
    float local_max = -INFINITY;
    for (int j = tid; j <= pos; j += kThreads) {
        float dot = 0.0f;
        if (j == pos) {
            for (int i = 0; i < hd; ++i) dot = fmaf(q_s[i], k_s[i], dot);
        } else {
            const u32x4 *row = (const u32x4 *)(k_cache + (cache_row0 + j) * hd);
            for (int c = 0; c < hd / 8; ++c) {
                float f[8];
                unpack8(row[c], f);
#pragma unroll
                for (int i = 0; i < 8; ++i) dot = fmaf(q_s[8 * c + i], f[i], dot);
            }
        }
        dot *= scale;
        score[j] = dot;
        local_max = fmaxf(local_max, dot);
    }
    const float mx = block_reduce<true>(local_max, red);
    float local_sum = 0.0f;
    for (int j = tid; j <= pos; j += kThreads) {
        const float e = __expf(score[j] - mx);
        score[j] = e;
        local_sum += e;
    }
    const float inv = 1.0f / block_reduce<false>(local_sum, red);  // its barriers also publish score[]

    const int groups = kThreads / hd;  // >= 1 (hd <= 256)
    const int grp = tid / hd, d = tid % hd;
    if (grp < groups) {
        float acc = 0.0f;
        for (int j = grp; j <= pos; j += groups) {
            const float val = (j == pos) ? v_s[d] : __half2float(v_cache[(cache_row0 + j) * hd + d]);
            acc = fmaf(score[j], val, acc);
        }
        part[grp * hd + d] = acc;
    }
    __syncthreads();
    if (tid < hd) {
        float acc = 0.0f;
        for (int g = 0; g < groups; ++g) acc += part[g * hd + tid];
        out[((size_t)b * H + h) * hd + tid] = __float2half_rn(acc * inv);
    }
}

// The same for head_dim HD in {64, 128}, with the memory latency taken in
// parallel and whole rows per load: thread (jg, ch) holds 16-byte chunk ch of key
// and value rows jg, jg + 256/(HD/8), ... (sixteen of each in registers, requested
// before the first barrier; longer contexts go round in blocks of that size), a
// row's lanes meet by DPP moves for the scores.  Each group of lanes keeps its own
// running maximum, sum of exponentials and weighted value sum (the "online" form of
// softmax), and the groups are merged once at the end: one barrier after the rotary
// step and one before the merge, no pass over the scores in between.
// Dynamic LDS: (3*HD + 2*(256/(HD/8)) + (256/(HD/8))*HD) floats.
template <int HD>
__global__ void __launch_bounds__(kThreads)
attention_hd_kernel(const __half *__restrict__ q, const __half *__restrict__ k, const __half *__restrict__ v,
                    const __half *__restrict__ cos_t, const __half *__restrict__ sin_t,
                    __half *__restrict__ k_cache, __half *__restrict__ v_cache,
                    const long long *__restrict__ pos_ptr, __half *__restrict__ out, int H, int KV, int max_pos)
{
    constexpr int kChunks = HD / 8;             // 16-byte chunks of a row
    constexpr int kPosGroups = kThreads / kChunks;
    extern __shared__ float lds[];
    float *q_s = lds;
    float *k_s = q_s + HD;
    float *v_s = k_s + HD;
    float *grp_max = v_s + HD;
    float *grp_sum = grp_max + kPosGroups;
    float *part = grp_sum + kPosGroups;

    const int tid = threadIdx.x;
    const int b = blockIdx.x / H, h = blockIdx.x % H;
    const int rep = H / KV, kvh = h / rep;
    int pos = (int)*pos_ptr;
    pos = min(max(pos, 0), max_pos - 1);
    const size_t cache_row0 = ((size_t)b * KV + kvh) * max_pos;

    if (tid < HD) {
        const int i = tid;
        const float c = __half2float(cos_t[(size_t)pos * HD + i]);
        const float s = __half2float(sin_t[(size_t)pos * HD + i]);
        const __half *qh = q + ((size_t)b * H + h) * HD;
        const __half *kh = k + ((size_t)b * KV + kvh) * HD;
        const int j = i < HD / 2 ? i + HD / 2 : i - HD / 2;
        const float sign = i < HD / 2 ? -1.0f : 1.0f;
        const __half qr = __float2half_rn(__half2float(qh[i]) * c + sign * __half2float(qh[j]) * s);
        const __half kr = __float2half_rn(__half2float(kh[i]) * c + sign * __half2float(kh[j]) * s);
        const __half vv = v[((size_t)b * KV + kvh) * HD + i];
        q_s[i] = __half2float(qr);
        k_s[i] = __half2float(kr);
        v_s[i] = __half2float(vv);
        if (h % rep == 0) {
            k_cache[(cache_row0 + pos) * HD + i] = kr;
            v_cache[(cache_row0 + pos) * HD + i] = vv;
        }
    }
    // Key and value rows of earlier positions do not depend on the above: the first block
    // of them is fetched before the barrier, so that a step over a short context costs one
    // memory round trip.  Both are walked the same way: thread (jg, ch) takes 16-byte chunk
    // ch of rows jg, jg + kPosGroups, ...: a wave's load covers whole rows (contiguous
    // kilobytes), where a thread fetching "its" row chunk by chunk touches 64 cache lines
    // per instruction.
    constexpr int kRowsInRegs = 16;  // rows per thread and block: a block is 16 * kPosGroups positions
    constexpr int kBlock = kRowsInRegs * kPosGroups;
    const int jg = tid / kChunks, ch = tid % kChunks;
    const u32x4 *kbase = (const u32x4 *)(k_cache + cache_row0 * HD) + ch;
    const u32x4 *vbase = (const u32x4 *)(v_cache + cache_row0 * HD) + ch;
    u32x4 krow[kRowsInRegs], vrow[kRowsInRegs];
    auto fetch_block = [&](int j0) {
#pragma unroll
        for (int u = 0; u < kRowsInRegs; ++u) {
            const int j = j0 + jg + u * kPosGroups;
            krow[u] = (u32x4){0u, 0u, 0u, 0u};
            if (j < pos) krow[u] = kbase[(size_t)j * kChunks];
        }
#pragma unroll
        for (int u = 0; u < kRowsInRegs; ++u) {
            const int j = j0 + jg + u * kPosGroups;
            vrow[u] = (u32x4){0u, 0u, 0u, 0u};
            if (j < pos) vrow[u] = vbase[(size_t)j * kChunks];
        }
    };
    fetch_block(0);
    __syncthreads();

    // a row's kChunks lanes multiply their chunks and are summed inside their row of 16
    // (HD 128) or 8 (HD 64) lanes: every lane of the row ends up with the score
    const float scale = rsqrtf((float)HD);
    float qc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) qc[i] = q_s[8 * ch + i];
    auto row_sum = [](float x) {
        x += dpp_lane<0xb1>(x);   // quad_perm [1,0,3,2]
        x += dpp_lane<0x4e>(x);   // quad_perm [2,3,0,1]
        x += dpp_lane<0x141>(x);  // row_half_mirror: the other quad of the 8
        if (kChunks == 16) x += dpp_lane<0x140>(x);  // row_mirror: the other half of the 16
        return x;
    };
    // running state of this thread's rows: maximum score, sum of exp(score - maximum), and
    // the same weights applied to the value chunks
    float run_max = -INFINITY, run_sum = 0.0f, acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    auto fold = [&](const float *sc, auto &&value_of, auto row_count) {
        constexpr int rows = decltype(row_count)::value;
        float blk_max = run_max;
#pragma unroll
        for (int u = 0; u < rows; ++u) blk_max = fmaxf(blk_max, sc[u]);
        if (blk_max == -INFINITY) return;  // nothing valid so far (uniform over the row's lanes)
        const float keep = __expf(run_max - blk_max);  // 0 when nothing was held before
        run_sum *= keep;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] *= keep;
#pragma unroll
        for (int u = 0; u < rows; ++u) {
            const float pj = __expf(sc[u] - blk_max);  // 0 for a masked row
            run_sum += pj;
            float f[8];
            value_of(u, f);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = fmaf(pj, f[i], acc[i]);
        }
        run_max = blk_max;
    };
    for (int j0 = 0; j0 < pos; j0 += kBlock) {
        if (j0) fetch_block(j0);
        float sc[kRowsInRegs];
#pragma unroll
        for (int u = 0; u < kRowsInRegs; ++u) {
            float f[8];
            unpack8(krow[u], f);
            float dot = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) dot = fmaf(qc[i], f[i], dot);
            dot = row_sum(dot) * scale;
            sc[u] = j0 + jg + u * kPosGroups < pos ? dot : -INFINITY;
        }
        fold(sc, [&](int u, float *f) { unpack8(vrow[u], f); }, std::integral_constant<int, kRowsInRegs>());
    }
    if (jg == 0) {
        // the new position's own key and value, still in LDS
        float dot = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) dot = fmaf(qc[i], k_s[8 * ch + i], dot);
        const float own = row_sum(dot) * scale;
        fold(&own, [&](int, float *f) {
#pragma unroll
            for (int i = 0; i < 8; ++i) f[i] = v_s[8 * ch + i];
        }, std::integral_constant<int, 1>());
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) part[jg * HD + 8 * ch + i] = acc[i];
    if (ch == 0) {
        grp_max[jg] = run_max;
        grp_sum[jg] = run_sum;
    }
    __syncthreads();
    if (tid < HD) {
        // merge the groups: weights exp(group maximum - overall maximum); group 0 always holds
        // the new position, so the overall maximum is finite
        float mx = -INFINITY;
#pragma unroll
        for (int g = 0; g < kPosGroups; ++g) mx = fmaxf(mx, grp_max[g]);
        float sum = 0.0f, total = 0.0f;
#pragma unroll 8
        for (int g = 0; g < kPosGroups; ++g) {
            const float w = __expf(grp_max[g] - mx);  // 0 for a group without rows
            total = fmaf(grp_sum[g], w, total);
            sum = fmaf(part[g * HD + tid], w, sum);
        }
        out[((size_t)b * H + h) * HD + tid] = __float2half_rn(sum / total);
    }
}

// out = fp16(fp16(silu(gate)) * up), 8 values per thread
__global__ void __launch_bounds__(kThreads)
silu_mul_kernel(const u32x4 *__restrict__ gate, const u32x4 *__restrict__ up, u32x4 *__restrict__ out, long units)
{
    const long u = (long)blockIdx.x * kThreads + threadIdx.x;
    if (u >= units) return;
    float g[8], p[8];
    unpack8(gate[u], g);
    unpack8(up[u], p);
    u32x4 o;
    uint32_t *ow = (uint32_t *)&o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float a = __half2float(__float2half_rn(g[2 * i] / (1.0f + __expf(-g[2 * i])))) * p[2 * i];
        const float c = __half2float(__float2half_rn(g[2 * i + 1] / (1.0f + __expf(-g[2 * i + 1])))) * p[2 * i + 1];
        ow[i] = pack2(a, c);
    }
    out[u] = o;
}

bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

int launch_status()
{
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? LUTGEMM_OK : lutgemm_internal_hip_fail((int)e);
}

}  // namespace

extern "C" {

int lutgemm_decode_rmsnorm_f16(const void *x, const void *weight, void *y, int rows, int hidden, float eps,
                               void *clear, size_t clear_bytes, void *stream)
{
    if (!x || !weight || !y || rows < 1 || hidden < 8 || hidden % 8 != 0 || !(eps >= 0.0f)) return LUTGEMM_EINVAL;
    if (clear_bytes % 16 != 0 || (clear_bytes > 0 && !clear)) return LUTGEMM_EINVAL;
    if (!aligned16(x) || !aligned16(weight) || !aligned16(y) || !aligned16(clear)) return LUTGEMM_EALIGN;
    const long units = (long)(clear_bytes / 16);
    long extra = (units + kThreads - 1) / kThreads - rows;
    if (extra < 0) extra = 0;
    if (extra > 256) extra = 256;
    hipLaunchKernelGGL(rmsnorm_kernel, dim3((unsigned)(rows + extra)), dim3(kThreads), 0, (hipStream_t)stream,
                       (const __half *)x, (const __half *)weight, (__half *)y, rows, hidden, eps, (u32x4 *)clear,
                       units);
    return launch_status();
}

int lutgemm_decode_attention_f16(const void *q, const void *k, const void *v, const void *cos_table,
                                 const void *sin_table, void *k_cache, void *v_cache, const int64_t *position,
                                 void *out, int batch, int heads, int kv_heads, int head_dim, int max_positions,
                                 void *stream)
{
    if (!q || !k || !v || !cos_table || !sin_table || !k_cache || !v_cache || !position || !out)
        return LUTGEMM_EINVAL;
    if (batch < 1 || heads < 1 || kv_heads < 1 || heads % kv_heads != 0) return LUTGEMM_EINVAL;
    if (head_dim < 8 || head_dim > kThreads || head_dim % 8 != 0) return LUTGEMM_EINVAL;
    if (max_positions < 1 || max_positions > 8192) return LUTGEMM_EINVAL;
    if (!aligned16(k_cache) || !aligned16(v_cache)) return LUTGEMM_EALIGN;
    if (head_dim == 64 || head_dim == 128) {
        const int pos_groups = kThreads / (head_dim / 8);
        const size_t lds_hd = sizeof(float) * ((size_t)3 * head_dim + 2 * pos_groups + (size_t)pos_groups * head_dim);
        if (head_dim == 128)
            hipLaunchKernelGGL(attention_hd_kernel<128>, dim3((unsigned)(batch * heads)), dim3(kThreads), lds_hd,
                               (hipStream_t)stream, (const __half *)q, (const __half *)k, (const __half *)v,
                               (const __half *)cos_table, (const __half *)sin_table, (__half *)k_cache,
                               (__half *)v_cache, (const long long *)position, (__half *)out, heads, kv_heads,
                               max_positions);
        else
            hipLaunchKernelGGL(attention_hd_kernel<64>, dim3((unsigned)(batch * heads)), dim3(kThreads), lds_hd,
                               (hipStream_t)stream, (const __half *)q, (const __half *)k, (const __half *)v,
                               (const __half *)cos_table, (const __half *)sin_table, (__half *)k_cache,
                               (__half *)v_cache, (const long long *)position, (__half *)out, heads, kv_heads,
                               max_positions);
        return launch_status();
    }
    const int groups = kThreads / head_dim;
    const size_t lds = sizeof(float) * ((size_t)3 * head_dim + max_positions + 4 + (size_t)groups * head_dim);
    hipLaunchKernelGGL(attention_kernel, dim3((unsigned)(batch * heads)), dim3(kThreads), lds, (hipStream_t)stream,
                       (const __half *)q, (const __half *)k, (const __half *)v, (const __half *)cos_table,
                       (const __half *)sin_table, (__half *)k_cache, (__half *)v_cache,
                       (const long long *)position, (__half *)out, heads, kv_heads, head_dim, max_positions);
    return launch_status();
}

int lutgemm_decode_silu_mul_f16(const void *gate, const void *up, void *out, size_t count, void *stream)
{
    if (!gate || !up || !out || count == 0 || count % 8 != 0) return LUTGEMM_EINVAL;
    if (!aligned16(gate) || !aligned16(up) || !aligned16(out)) return LUTGEMM_EALIGN;
    const long units = (long)(count / 8);
    hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)((units + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                       (hipStream_t)stream, (const u32x4 *)gate, (const u32x4 *)up, (u32x4 *)out, units);
    return launch_status();
}

}  // extern "C"
