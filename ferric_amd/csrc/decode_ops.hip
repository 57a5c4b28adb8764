// The steps either side of the quantized matmuls in one decode layer, gfx950: RMSNorm (plain and fused with the residual
// add), rotary embedding, the per-head q/k norm + rotary + KV-cache append of a token's fused qkv row in one launch, the
// KV append on its own, and single-query attention over the cache (split over the keys, all query heads of a KV head
// sharing one pass over its keys and values).
//
// Replaces the reference's WGSL kernels RMSNORM / ADD_RMSNORM / ROPE / FUSED_ATTN / FUSED_ATTN_SPLIT / FUSED_ATTN_COMBINE
// (crates/ferric-tensor/src/lib.rs:2018-2074, 2118-2162, 2675-2726 ff.) and `append2` (lib.rs:1379-1398), as
// `Qwen3::attn` / `apply_layer` compose them (crates/ferric-llama/src/qwen3.rs:861-942, 979-1052).
//
// All of this is f32 arithmetic on small vectors: the kernels are launch- and latency-bound (a decode step has one row),
// except attention, which streams the layer's K and V rows once (HBM-bound: 2 * len * n_kv * head_dim * 4 bytes).
#include "common.hpp"

#include <hip/hip_fp16.h>

#include <math.h>
#include <stdlib.h>

namespace {

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
    int t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xF, false);
    return v + __int_as_float(t);
}
// Sum over the 64 lanes of a wave, returned in every lane (through lane 63 and a scalar register).
__device__ __forceinline__ float wave_sum(float v) {
    v = dpp_add<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
    v = dpp_add<0x141, 0xF>(v);  // row_half_mirror
    v = dpp_add<0x140, 0xF>(v);  // row_mirror: every lane of a 16-lane row holds the row sum
    v = dpp_add<0x142, 0xA>(v);  // row_bcast15 into rows 1 and 3
    v = dpp_add<0x143, 0xC>(v);  // row_bcast31 into rows 2 and 3
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// ---------------------------------------------------------------- RMSNorm, optionally of a + b
// out[r, j] = x[r, j] * (1 / sqrt(mean_j x^2 + eps)) * weight[j]   (lib.rs:2018-2033); with b: x = a + b, and the sum is
// written too (lib.rs:2057-2074). TPR threads share a row (a fixed-shape tree sum, so results do not depend on scheduling).
template <int TPR>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* a, const float* __restrict__ b,
                                                      const float* __restrict__ weight, size_t rows, int d, float eps,
                                                      float* sum_out, float* __restrict__ norm_out) {   // sum_out may be a
    constexpr int RPW = 256 / TPR;   // rows per workgroup
    constexpr int NV = 8;            // float4 per thread held in registers: rows up to 4 * NV * TPR values
    __shared__ float red[4];
    const int tid = threadIdx.x, sub = tid / TPR, t = tid % TPR;
    const size_t row = (size_t)blockIdx.x * RPW + sub;
    const bool live = row < rows;
    const size_t base = (live ? row : 0) * (size_t)d;
    const bool vec = (d & 3) == 0 && d <= 4 * NV * TPR && (((uintptr_t)a | (uintptr_t)b | (uintptr_t)weight | (uintptr_t)sum_out | (uintptr_t)norm_out) & 15) == 0;
    float ms = 0.f;
    if (vec) {
        // every load of the row is issued before the first use, so the row costs one memory round trip, not one per element
        const int nv = d >> 2;
        float4 r[NV];
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int j = t + i * TPR;
            r[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (j < nv) {
                r[i] = ((const float4*)(a + base))[j];
                if (b) { const float4 y = ((const float4*)(b + base))[j]; r[i].x += y.x; r[i].y += y.y; r[i].z += y.z; r[i].w += y.w; }
            }
        }
#pragma unroll
        for (int i = 0; i < NV; i++) ms = fmaf(r[i].x, r[i].x, fmaf(r[i].y, r[i].y, fmaf(r[i].z, r[i].z, fmaf(r[i].w, r[i].w, ms))));
        ms = wave_sum(ms);
        if (TPR == 256) {
            if ((tid & 63) == 0) red[tid >> 6] = ms;
            __syncthreads();
            ms = (red[0] + red[1]) + (red[2] + red[3]);
        }
        const float inv = 1.0f / sqrtf(ms / (float)d + eps);
        if (!live) return;
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int j = t + i * TPR;
            if (j < nv) {
                const float4 w = ((const float4*)weight)[j];
                if (sum_out) ((float4*)(sum_out + base))[j] = r[i];
                ((float4*)(norm_out + base))[j] = make_float4(r[i].x * inv * w.x, r[i].y * inv * w.y, r[i].z * inv * w.z, r[i].w * inv * w.w);
            }
        }
        return;
    }
    const float* xa = a + base;
    const float* xb = b ? b + base : nullptr;
    for (int j = t; j < d; j += TPR) {
        float v = xb ? xa[j] + xb[j] : xa[j];
        if (sum_out && live) sum_out[base + j] = v;
        ms = fmaf(v, v, ms);
    }
    ms = wave_sum(ms);
    if (TPR == 256) {
        if ((tid & 63) == 0) red[tid >> 6] = ms;
        __syncthreads();
        ms = (red[0] + red[1]) + (red[2] + red[3]);
    }
    const float inv = 1.0f / sqrtf(ms / (float)d + eps);
    if (!live) return;
    for (int j = t; j < d; j += TPR) {   // the same thread wrote sum_out[.., j] above, so reading it back is ordered
        float v = sum_out ? sum_out[base + j] : (xb ? xa[j] + xb[j] : xa[j]);
        norm_out[base + j] = v * inv * weight[j];
    }
}

__global__ void u32_add_kernel(uint32_t* w, size_t n, uint32_t delta) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) w[i] += delta;
}

__global__ void add_kernel(const float* a, const float* __restrict__ b, size_t n, float* out) {   // out may be a
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = a[i] + b[i];
}

// out = a * sigmoid(g): the gate of a gated attention layer on the attention output (crates/ferric-llama/src/qwen3.rs:936-938;
// sigmoid as crates/ferric-tensor/src/lib.rs:1915, 1 / (1 + exp(-v)))
__global__ void mul_sigmoid_kernel(const float* a, const float* __restrict__ g, size_t n, float* out) {   // out may be a
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = a[i] * (1.0f / (1.0f + expf(-g[i])));
}

// out[r, j] = gelu_tanh(gu[r, j]) * gu[r, d + j] for rows [gate | up] of 2 d values: the GEGLU of qwen3.rs:953-958 with the
// tanh-approximated GELU of lib.rs:1926, 0.5 v (1 + tanh(clamp(0.79788456 (v + 0.044715 v^3), -15, 15)))
__global__ void geglu_kernel(const float* __restrict__ gu, size_t n, size_t d, float* __restrict__ out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t r = i / d, j = i - r * d;
    const float v = gu[r * 2 * d + j], u = gu[r * 2 * d + d + j];
    float a = 0.7978845608028654f * (v + 0.044715f * v * v * v);
    a = fminf(fmaxf(a, -15.0f), 15.0f);
    out[i] = 0.5f * v * (1.0f + tanhf(a)) * u;
}

// ---------------------------------------------------------------- rotary embedding
// Pair c of a head rotates by angle pos * base^(-2c / n_rot) (times freq_scale[c]); partners are (c, c + n_rot/2) in the
// split-half layout and (2c, 2c + 1) interleaved; dims >= n_rot pass through (lib.rs:2118-2162, 2094-2116). The inverse
// frequency is evaluated in f64 and rounded to f32 once, the angle is the f32 product the reference forms.
__device__ __forceinline__ float rope_inv_freq(int c, int n_rot, float base, const float* freq_scale) {
    float inv = (float)exp(-2.0 * (double)c / (double)n_rot * log((double)base));
    return freq_scale ? inv * freq_scale[c] : inv;
}

__global__ void rope_kernel(const float* __restrict__ x, size_t src_row_stride, int t, int heads, int hd, int n_rot, float base,
                            const uint32_t* __restrict__ pos, uint32_t pos_off, const float* __restrict__ freq_scale, int interleaved,
                            float* __restrict__ out) {
    const int half = n_rot / 2, per_head = hd - half;   // work items per head: the pairs, then the pass-through tail
    size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (size_t)t * heads * per_head) return;
    const int w = (int)(id % per_head), head = (int)((id / per_head) % heads), i = (int)(id / ((size_t)per_head * heads));
    const float* xi = x + (size_t)i * src_row_stride + (size_t)head * hd;
    float* oi = out + ((size_t)i * heads + head) * hd;
    if (w >= half) { const int c = n_rot + (w - half); oi[c] = xi[c]; return; }
    const int c = w;
    const float p = (float)(pos ? pos[i] : pos_off + (uint32_t)i);
    const float ang = p * rope_inv_freq(c, n_rot, base, freq_scale);
    float sn, cs;
    sincosf(ang, &sn, &cs);
    const int p0 = interleaved ? 2 * c : c, p1 = interleaved ? 2 * c + 1 : c + half;
    const float x1 = xi[p0], x2 = xi[p1];
    oi[p0] = x1 * cs - x2 * sn;
    oi[p1] = x2 * cs + x1 * sn;
}

// ---------------------------------------------------------------- qkv row -> q, K cache, V cache
// One wave per head of one token's fused qkv row (n_head query heads, n_kv key heads, n_kv value heads):
//   query / key head: + bias, RMSNorm over the head with q_norm / k_norm (when given), rotary embedding at the token's position;
//   the query goes to q_out[t, n_head * hd], the key to row pos of the K cache; a value head is copied (+ bias) to row pos of
//   the V cache. This is qwen3.rs:861-905 (qn, rope, append2) in one launch.
struct QkvPostParams {
    const float* qkv;        // [t, (n_head + 2 n_kv) * hd]
    const float* bias;       // same width, or null
    const float* q_norm;     // [hd] or null
    const float* k_norm;     // [hd] or null
    const uint32_t* pos;     // [t] absolute positions (device)
    const float* freq_scale; // [n_rot / 2] or null
    float* q_out;            // [t, n_head * hd]
    float* k_cache;          // [cap, n_kv * hd]
    float* v_cache;
    int t, n_head, n_kv, hd, n_rot, interleaved;
    uint32_t cap;
    float eps, base;
    int kv_packed;           // != 0: k_cache / v_cache are packed [t, n_kv * hd] outputs, row i for token i (cap is not looked at)
};

__global__ __launch_bounds__(256) void qkv_post_kernel(QkvPostParams p) {
    const int lane = threadIdx.x & 63;
    const int per_tok = p.n_head + 2 * p.n_kv;
    const size_t wid = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wid >= (size_t)p.t * per_tok) return;
    const int i = (int)(wid / per_tok), h = (int)(wid % per_tok);
    const uint32_t pos = p.pos[i];
    const size_t col = (size_t)h * p.hd;
    const float* x = p.qkv + (size_t)i * per_tok * p.hd + col;
    const float* bias = p.bias ? p.bias + col : nullptr;
    const int kvw = p.n_kv * p.hd;
    float* dst;
    const float* nw;
    bool rotate = true;
    const size_t kv_row = p.kv_packed ? (size_t)i : (size_t)pos;
    if (h < p.n_head) { dst = p.q_out + ((size_t)i * p.n_head + h) * p.hd; nw = p.q_norm; }
    else if (h < p.n_head + p.n_kv) { dst = p.k_cache + kv_row * kvw + (size_t)(h - p.n_head) * p.hd; nw = p.k_norm; }
    else { dst = p.v_cache + kv_row * kvw + (size_t)(h - p.n_head - p.n_kv) * p.hd; nw = nullptr; rotate = false; }
    if (h >= p.n_head && !p.kv_packed && pos >= p.cap) return;   // a position past the cache is dropped, never written out of bounds
    if (!rotate) {
        for (int j = lane; j < p.hd; j += 64) dst[j] = bias ? x[j] + bias[j] : x[j];
        return;
    }
    float inv = 1.f;
    if (nw) {
        float ms = 0.f;
        for (int j = lane; j < p.hd; j += 64) { float v = bias ? x[j] + bias[j] : x[j]; ms = fmaf(v, v, ms); }
        ms = wave_sum(ms);
        inv = 1.0f / sqrtf(ms / (float)p.hd + p.eps);
    }
    auto val = [&](int j) { float v = bias ? x[j] + bias[j] : x[j]; return nw ? v * inv * nw[j] : v; };
    const int half = p.n_rot / 2;
    for (int c = lane; c < half; c += 64) {
        const float ang = (float)pos * rope_inv_freq(c, p.n_rot, p.base, p.freq_scale);
        float sn, cs;
        sincosf(ang, &sn, &cs);
        const int p0 = p.interleaved ? 2 * c : c, p1 = p.interleaved ? 2 * c + 1 : c + half;
        const float x1 = val(p0), x2 = val(p1);
        dst[p0] = x1 * cs - x2 * sn;
        dst[p1] = x2 * cs + x1 * sn;
    }
    for (int j = p.n_rot + lane; j < p.hd; j += 64) dst[j] = val(j);
}

// K and V rows of t tokens into their caches at the tokens' positions, one launch (lib.rs:1379-1398).
__global__ void kv_append_kernel(const float* __restrict__ k, const float* __restrict__ v, int t, int width, const uint32_t* __restrict__ pos,
                                 uint32_t pos_off, uint32_t cap, float* __restrict__ kc, float* __restrict__ vc) {
    size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (size_t)t * width) return;
    const int i = (int)(id / width), j = (int)(id % width);
    const uint32_t r = pos ? pos[i] : pos_off + (uint32_t)i;
    if (r >= cap) return;
    kc[(size_t)r * width + j] = k[id];
    vc[(size_t)r * width + j] = v[id];
}

// ---------------------------------------------------------------- single-query attention over the cache
// out[h] = softmax_j(q[h] . K[j, kv(h)] * scale) @ V[:, kv(h)]   for one query row (nn.rs:140-166, lib.rs:2675-2726).
// Workgroup (kv head, split). A key or value row is read by 16 lanes (DPL = hd / 16 consecutive dims each, 16-byte loads), so a
// wave works on 4 keys at a time and a workgroup is 16 independent key streams, each with its own running (max, sum,
// accumulator) per query head -- the reference's online softmax, lib.rs:2697-2722 -- over keys taken round-robin in pairs.
// Every row is read ONCE for all G = n_head / n_kv query heads of the group. A dot product is reduced inside its 16-lane
// row with 4 DPP adds. The 4 streams of a wave are merged by lane exchange, the 4 waves through LDS, the splits by
// attn_combine_kernel: always the same rescale, exp(m_part - m_all).
constexpr int ATT_KB = 2;         // keys in flight per stream
constexpr int ATT_STREAMS = 16;   // per workgroup of 256 threads

__device__ __forceinline__ float row16_sum(float v) {   // all 16 lanes of a DPP row get the row's sum
    v = dpp_add<0xB1, 0xF>(v);
    v = dpp_add<0x4E, 0xF>(v);
    v = dpp_add<0x141, 0xF>(v);
    v = dpp_add<0x140, 0xF>(v);
    return v;
}

template <int DPL>
__device__ __forceinline__ void load_dims(const float* p, float (&r)[DPL]) {   // p is 16-byte aligned
#pragma unroll
    for (int i = 0; i < DPL; i += 4) {
        float4 v = *(const float4*)(p + i);
        r[i] = v.x; r[i + 1] = v.y; r[i + 2] = v.z; r[i + 3] = v.w;
    }
}

// A block-quantized cache (kvquant.hip's layout) read in place: codes and f16 scales of the keys and of the values.
struct QCache {
    const uint32_t* k_codes; const uint16_t* k_scales;
    const uint32_t* v_codes; const uint16_t* v_scales;
};
// DPL (4 or 8) consecutive dims of one row, starting at column `col` (a multiple of DPL) of block row `key`: the values the
// dequantize kernel would write, by the same single operations (q * d; (q - 8) * d; q * d then + m, not fused), so attention
// over the codes is attention over the dequantized rows, bit for bit.
// What a lane holds of a row between the load and its use: the code words and scale halves as loaded (the next rows are
// requested while the current ones are worked on, and packed they cost a third of the registers of their f32 values).
template <int FMT, int DPL>
struct RawDims {
    uint32_t w[DPL / 4];
    uint16_t d, m;
};
template <int FMT, int DPL>
__device__ __forceinline__ RawDims<FMT, DPL> fetch_dims_q(const uint32_t* __restrict__ codes, const uint16_t* __restrict__ scales, size_t key,
                                                         int nblk, int col) {
    const size_t b = key * (size_t)nblk + (size_t)(col >> 5);
    const int j = col & 31;
    RawDims<FMT, DPL> r;
    r.m = 0;
    if constexpr (FMT == FHIP_KVQ_Q8_0) {
        r.d = scales[b];
#pragma unroll
        for (int w = 0; w < DPL / 4; w++) r.w[w] = codes[b * 8 + (j >> 2) + w];
    } else {
        if constexpr (FMT == FHIP_KVQ_Q4_0) r.d = scales[b];
        else { r.d = scales[2 * b]; r.m = scales[2 * b + 1]; }
#pragma unroll
        for (int w = 0; w < DPL / 4; w++) r.w[w] = codes[b * 4 + ((j & 15) >> 2) + w];
    }
    return r;
}
template <int FMT, int DPL>
__device__ __forceinline__ void expand_dims_q(const RawDims<FMT, DPL>& raw, int col, float (&r)[DPL]) {
#pragma clang fp contract(off)
    const int j = col & 31;
    if constexpr (FMT == FHIP_KVQ_Q8_0) {
        const float d = __half2float(__ushort_as_half(raw.d));
#pragma unroll
        for (int w = 0; w < DPL / 4; w++) {
            const uint32_t word = raw.w[w];
            r[4 * w] = (float)(int8_t)(word & 255u) * d;
            r[4 * w + 1] = (float)(int8_t)((word >> 8) & 255u) * d;
            r[4 * w + 2] = (float)(int8_t)((word >> 16) & 255u) * d;
            r[4 * w + 3] = (float)(int8_t)(word >> 24) * d;
        }
    } else {
        const int shift = j < 16 ? 0 : 4;
        const float d = __half2float(__ushort_as_half(raw.d)), m = __half2float(__ushort_as_half(raw.m));
#pragma unroll
        for (int w = 0; w < DPL / 4; w++) {
            const uint32_t word = raw.w[w] >> shift;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float n = (float)((word >> (8 * i)) & 15u);
                if constexpr (FMT == FHIP_KVQ_Q4_0) r[4 * w + i] = (n - 8.0f) * d;
                else { const float t = n * d; r[4 * w + i] = t + m; }
            }
        }
    }
}

// FUSED: the query heads do not come from memory but are formed here from the raw QKV row of the newest token -- bias, per-head
// RMSNorm, rotation, exactly qkv_post_kernel's arithmetic -- by every workgroup for its own G heads, into LDS; and the
// workgroup whose key range holds the token's position also forms that token's K and V rows for its KV head and appends them
// to the cache before it starts on the keys (a store, a workgroup barrier, then the ordinary loop reads the row back like any
// other: no other workgroup's range holds that row). One launch less per layer than post-processing + attention.
template <bool FUSED> struct CachePtr { typedef const float* __restrict__ type; };
template <> struct CachePtr<true> { typedef const float* type; };   // the fused kernel also writes the cache: no promise of no alias

// QF: -1 for an f32 cache (K, V), else the FHIP_KVQ_* format of the block-quantized cache in qc (K and V are null then).
template <int G, int DPL, bool FUSED, int QF = -1>
__device__ __forceinline__ void attn_split_body(const float* __restrict__ q, typename CachePtr<FUSED>::type K, typename CachePtr<FUSED>::type V,
                                                int n_kv, uint32_t len_host, const uint32_t* __restrict__ len_dev, float scale, int splits,
                                                uint32_t window, float softcap, float* __restrict__ part, float* __restrict__ out,
                                                const QkvPostParams& fp, int gq, const QCache& qc = QCache{}) {
    static_assert(!(FUSED && QF >= 0), "the fused post-processing appends f32 rows");
    constexpr int HD = 16 * DPL;
    __shared__ float sm_m[4][G], sm_l[4][G];
    __shared__ float sm_acc[4][G][HD];
    __shared__ float sm_q[FUSED ? G : 1][FUSED ? HD : 1];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, sub = lane & 15;
    const int sid = wave * 4 + (lane >> 4);
    // Workgroup blockIdx.x takes the G query heads from head0 on; gq = query heads per KV head. gq == G: one workgroup per KV
    // head and split. gq > G (short caches, G = 1): one workgroup per query head, the KV head's rows read by each of them.
    // gq < 0 (G = 1, a one-dimensional grid): one workgroup per (query head, split) for -gq query heads per KV head, dealt so
    // that the workgroups of one KV head and split -- which read the same rows -- are consecutive slots of one XCD (workgroup
    // L runs on XCD L % 8): slot i = L / 8 of XCD x = L % 8 is query head i % g of group (i / g) * 8 + x.
    int head0 = blockIdx.x * G, kvh = gq > 0 ? head0 / gq : 0, split = blockIdx.y;
    if (gq < 0) {
        const int g = -gq, x = blockIdx.x & 7, i = blockIdx.x >> 3;
        const int grp = (i / g) * 8 + x;
        if (grp >= n_kv * splits) return;
        kvh = grp % n_kv; split = grp / n_kv; head0 = kvh * g + i % g;
    }
    // FUSED: the raw values of every head this wave will post-process (job j = wave + 4 r: query head j of the group, then
    // the key and the value row) are requested before anything else, the length word with them, so that one memory round
    // trip covers what used to be three in a row (the length, the first round's rows, the second round's).
    constexpr int ROUNDS = FUSED ? (G + 2 + 3) / 4 : 1, EPL = HD / 64;
    float xr[ROUNDS][EPL];
    if constexpr (FUSED) {
#pragma unroll
        for (int r = 0; r < ROUNDS; r++) {
            const int j = wave + 4 * r;
            if (j < G + 2) {
                const int src = j < G ? head0 + j : (j == G ? fp.n_head + kvh : fp.n_head + n_kv + kvh);
                const float* x = fp.qkv + (size_t)src * HD;
                const float* bias = fp.bias ? fp.bias + (size_t)src * HD : nullptr;
#pragma unroll
                for (int i = 0; i < EPL; i++) xr[r][i] = bias ? x[lane + 64 * i] + bias[lane + 64 * i] : x[lane + 64 * i];
            }
        }
    }
    uint32_t len = len_dev ? *len_dev + 1u : len_host;   // the device word is the newest token's position
    asm volatile("" ::: "memory");                       // keeps the loads above in front of the arithmetic on the length
    if (len > len_host) len = len_host;
    // sliding window (nn.rs:92-111): only the last `window` keys count; 0 or >= len: all of them
    const uint32_t first = (window > 0 && window < len) ? len - window : 0u;
    const uint32_t per = (len - first + splits - 1) / splits;
    const uint32_t k0 = first + (uint32_t)split * per, k1 = min(len, k0 + per);
    const size_t stride = (size_t)n_kv * HD;
    const float* Kb = QF >= 0 ? nullptr : K + (size_t)kvh * HD + sub * DPL;
    const float* Vb = QF >= 0 ? nullptr : V + (size_t)kvh * HD + sub * DPL;

    // The rows of a step are requested one step ahead: a stream's steps depend on one another only through the running
    // maximum, so without this every step paid a memory round trip before its arithmetic (32 in a row for a split of 1024 keys).
    // A step past the split's end re-reads the split's last row (always a row of the cache) and is never used.
    constexpr int QFMT = QF >= 0 ? QF : 0;
    const int qcol = kvh * HD + sub * DPL, qnblk = n_kv * (HD / 32);
    RawDims<QFMT, DPL> kq[QF >= 0 ? ATT_KB : 1], vq[QF >= 0 ? ATT_KB : 1];
    float kf[QF >= 0 ? 1 : ATT_KB][DPL], vf[QF >= 0 ? 1 : ATT_KB][DPL];
    auto request = [&](uint32_t at) {
#pragma unroll
        for (int j = 0; j < ATT_KB; j++) {
            const uint32_t key = min(at + j, k1 - 1);   // a row past the split re-reads its last row and is masked below
            if constexpr (QF >= 0) {
                kq[j] = fetch_dims_q<QFMT, DPL>(qc.k_codes, qc.k_scales, key, qnblk, qcol);
                vq[j] = fetch_dims_q<QFMT, DPL>(qc.v_codes, qc.v_scales, key, qnblk, qcol);
            } else {
                load_dims<DPL>(Kb + key * stride, kf[j]);
                load_dims<DPL>(Vb + key * stride, vf[j]);
            }
        }
    };
    // FUSED: the first step's rows are requested in front of the post-processing, so that their memory round trip runs under it,
    // unless one of them could be the row this workgroup is about to append (then they are requested behind the barrier that
    // follows the store; a step past the split's end re-reads row k1 - 1, which is why that row counts too).
    bool requested = false;
    if constexpr (FUSED) {
        const uint32_t pos = *len_dev;
        if (k0 < k1 && (pos >= k0 + ATT_STREAMS * ATT_KB || pos >= k1)) {
            request(k0 + sid * ATT_KB);
            requested = true;
        }
    }
    if constexpr (FUSED) {
        const uint32_t pos = *len_dev;
        // the rows are appended by the workgroup whose keys include them; a position past the rows attention looks at (but
        // inside the cache) is still appended, by the last split, as the separate post-processing launch would
        const bool owner = pos < fp.cap && (pos < len ? (pos >= k0 && pos < k1) : split == splits - 1);
        const int njobs = G + (owner ? 2 : 0);
        const int kvw = n_kv * HD, half = fp.n_rot / 2;
#pragma unroll
        for (int r = 0; r < ROUNDS; r++) {                 // job j < G: query head j of the group; G: the K row; G + 1: the V row
            const int j = wave + 4 * r;
            if (j >= njobs) continue;
            const int src = j < G ? head0 + j : (j == G ? fp.n_head + kvh : fp.n_head + n_kv + kvh);
            const float* x = fp.qkv + (size_t)src * HD;
            const float* bias = fp.bias ? fp.bias + (size_t)src * HD : nullptr;
            const float* nw = j < G ? fp.q_norm : (j == G ? fp.k_norm : nullptr);
            float* dst = j < G ? &sm_q[FUSED ? j : 0][0] : (j == G ? fp.k_cache : fp.v_cache) + (size_t)pos * kvw + (size_t)kvh * HD;
            if (j == G + 1) {
#pragma unroll
                for (int i = 0; i < EPL; i++) dst[lane + 64 * i] = xr[r][i];
                continue;
            }
            float inv = 1.f;
            if (nw) {
                float ms = 0.f;
#pragma unroll
                for (int i = 0; i < EPL; i++) ms = fmaf(xr[r][i], xr[r][i], ms);
                ms = wave_sum(ms);
                inv = 1.0f / sqrtf(ms / (float)HD + fp.eps);
            }
            auto val = [&](int e) { float v = bias ? x[e] + bias[e] : x[e]; return nw ? v * inv * nw[e] : v; };
            for (int c = lane; c < half; c += 64) {
                const float ang = (float)pos * rope_inv_freq(c, fp.n_rot, fp.base, fp.freq_scale);
                float sn, cs;
                sincosf(ang, &sn, &cs);
                const int p0 = fp.interleaved ? 2 * c : c, p1 = fp.interleaved ? 2 * c + 1 : c + half;
                const float x1 = val(p0), x2 = val(p1);
                dst[p0] = x1 * cs - x2 * sn;
                dst[p1] = x2 * cs + x1 * sn;
            }
            for (int e = fp.n_rot + lane; e < HD; e += 64) dst[e] = val(e);
        }
        __syncthreads();
    }
    float qr[G][DPL], acc[G][DPL], m[G], l[G];
#pragma unroll
    for (int h = 0; h < G; h++) {
        m[h] = -3.0e38f; l[h] = 0.f;
        if constexpr (FUSED) {
#pragma unroll
            for (int i = 0; i < DPL; i++) qr[h][i] = sm_q[FUSED ? h : 0][sub * DPL + i];
        } else {
            load_dims<DPL>(q + ((size_t)head0 + h) * HD + sub * DPL, qr[h]);
        }
#pragma unroll
        for (int i = 0; i < DPL; i++) acc[h][i] = 0.f;
    }
    if (!requested) request(k0 + sid * ATT_KB);
    for (uint32_t kb = k0 + sid * ATT_KB; kb < k1; kb += ATT_STREAMS * ATT_KB) {
        float kr[ATT_KB][DPL], vr[ATT_KB][DPL];
#pragma unroll
        for (int j = 0; j < ATT_KB; j++) {
            if constexpr (QF >= 0) {
                expand_dims_q<QFMT, DPL>(kq[j], qcol, kr[j]);
                expand_dims_q<QFMT, DPL>(vq[j], qcol, vr[j]);
            } else {
#pragma unroll
                for (int i = 0; i < DPL; i++) { kr[j][i] = kf[j][i]; vr[j][i] = vf[j][i]; }
            }
        }
        request(kb + ATT_STREAMS * ATT_KB);
#pragma unroll
        for (int h = 0; h < G; h++) {
            float sc[ATT_KB];
#pragma unroll
            for (int j = 0; j < ATT_KB; j++) {
                float d = 0.f;
#pragma unroll
                for (int i = 0; i < DPL; i++) d = fmaf(qr[h][i], kr[j][i], d);
                d = row16_sum(d) * scale;
                if (softcap > 0.f) d = softcap * tanhf(d / softcap);   // cap * tanh(x / cap), crates/ferric-tensor/src/lib.rs:308
                sc[j] = (kb + j < k1) ? d : -3.0e38f;
            }
            float m_new = m[h];
#pragma unroll
            for (int j = 0; j < ATT_KB; j++) m_new = fmaxf(m_new, sc[j]);
            const float corr = __expf(m[h] - m_new);
            float e[ATT_KB], ps = 0.f;
#pragma unroll
            for (int j = 0; j < ATT_KB; j++) { e[j] = (kb + j < k1) ? __expf(sc[j] - m_new) : 0.f; ps += e[j]; }
            l[h] = fmaf(l[h], corr, ps);
#pragma unroll
            for (int i = 0; i < DPL; i++) {
                float a = acc[h][i] * corr;
#pragma unroll
                for (int j = 0; j < ATT_KB; j++) a = fmaf(e[j], vr[j][i], a);
                acc[h][i] = a;
            }
            m[h] = m_new;
        }
    }
    // merge the wave's four streams (rows of 16 lanes) by exchange with lanes ^16 and ^32
#pragma unroll
    for (int h = 0; h < G; h++) {
        float M = fmaxf(m[h], __shfl_xor(m[h], 16));
        M = fmaxf(M, __shfl_xor(M, 32));
        const float f = __expf(m[h] - M);
        float lv = l[h] * f;
        lv += __shfl_xor(lv, 16);
        lv += __shfl_xor(lv, 32);
#pragma unroll
        for (int i = 0; i < DPL; i++) {
            float a = acc[h][i] * f;
            a += __shfl_xor(a, 16);
            a += __shfl_xor(a, 32);
            if (lane < 16) sm_acc[wave][h][sub * DPL + i] = a;
        }
        if (lane == 0) { sm_m[wave][h] = M; sm_l[wave][h] = lv; }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < G * HD; idx += 256) {
        const int h = idx / HD, d = idx % HD;
        const float M = fmaxf(fmaxf(sm_m[0][h], sm_m[1][h]), fmaxf(sm_m[2][h], sm_m[3][h]));
        float L = 0.f, A = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float f = __expf(sm_m[w][h] - M);
            L = fmaf(sm_l[w][h], f, L);
            A = fmaf(sm_acc[w][h][d], f, A);
        }
        const int head = head0 + h;
        if (splits == 1) {
            out[(size_t)head * HD + d] = A / L;
        } else {
            float* pp = part + ((size_t)head * splits + split) * (HD + 2);
            pp[d] = A;
            if (d == 0) { pp[HD] = M; pp[HD + 1] = L; }
        }
    }
}

template <int G, int DPL>
__global__ __launch_bounds__(256) void attn_split_kernel(const float* __restrict__ q, const float* __restrict__ K, const float* __restrict__ V,
                                                         int n_kv, uint32_t len_host, const uint32_t* __restrict__ len_dev, float scale, int splits,
                                                         uint32_t window, float softcap, float* __restrict__ part, float* __restrict__ out, int gq) {
    attn_split_body<G, DPL, false>(q, K, V, n_kv, len_host, len_dev, scale, splits, window, softcap, part, out, QkvPostParams{}, gq);
}

template <int G, int DPL, int QF>
__global__ __launch_bounds__(256) void attn_split_kvq_kernel(const float* __restrict__ q, QCache qc, int n_kv, uint32_t len_host,
                                                             const uint32_t* __restrict__ len_dev, float scale, int splits, uint32_t window,
                                                             float softcap, float* __restrict__ part, float* __restrict__ out, int gq) {
    attn_split_body<G, DPL, false, QF>(q, nullptr, nullptr, n_kv, len_host, len_dev, scale, splits, window, softcap, part, out, QkvPostParams{}, gq, qc);
}

template <int G, int DPL>
__global__ __launch_bounds__(256) void attn_split_fused_kernel(QkvPostParams fp, int n_kv, uint32_t len_host, const uint32_t* __restrict__ len_dev,
                                                               float scale, int splits, uint32_t window, float softcap, float* __restrict__ part,
                                                               float* __restrict__ out, int gq) {
    attn_split_body<G, DPL, true>(nullptr, fp.k_cache, fp.v_cache, n_kv, len_host, len_dev, scale, splits, window, softcap, part, out, fp, gq);
}

// One workgroup per query head: weights exp(m_s - max m) of the splits once (through LDS), then every output dim is a
// weighted sum of the splits' accumulators over the weighted sum of their sums. splits <= 256. Always launched with
// COMBINE_THREADS threads, whatever the head size: the loops below stride by that constant.
constexpr int COMBINE_THREADS = 128;
__global__ __launch_bounds__(COMBINE_THREADS) void attn_combine_kernel(const float* __restrict__ part, int hd, int splits, float* __restrict__ out) {
    __shared__ float w[256], lw[256];
    const int head = blockIdx.x, tid = threadIdx.x;
    const float* pp = part + (size_t)head * splits * (hd + 2);
    // this thread's output dim of the first splits is requested together with the splits' maxima and sums: one memory round
    // trip instead of two in a row for the short caches, where this kernel is nothing but latency
    constexpr int EARLY = 16;
    float pv[EARLY];
#pragma unroll
    for (int s = 0; s < EARLY; s++) pv[s] = (s < splits && tid < hd) ? pp[(size_t)s * (hd + 2) + tid] : 0.f;
    for (int s = tid; s < splits; s += COMBINE_THREADS) { w[s] = pp[(size_t)s * (hd + 2) + hd]; lw[s] = pp[(size_t)s * (hd + 2) + hd + 1]; }
    __syncthreads();
    float M = -3.0e38f;
    for (int s = 0; s < splits; s++) M = fmaxf(M, w[s]);
    __syncthreads();
    for (int s = tid; s < splits; s += COMBINE_THREADS) { const float f = __expf(w[s] - M); w[s] = f; lw[s] *= f; }
    __syncthreads();
    float L = 0.f;
    for (int s = 0; s < splits; s++) L += lw[s];
    for (int d = tid; d < hd; d += COMBINE_THREADS) {
        float A = 0.f;
        if (d == tid) {
#pragma unroll
            for (int s = 0; s < EARLY; s++)
                if (s < splits) A = fmaf(pv[s], w[s], A);
        }
#pragma unroll 8
        for (int s = d == tid ? EARLY : 0; s < splits; s++) A = fmaf(pp[(size_t)s * (hd + 2) + d], w[s], A);
        out[(size_t)head * hd + d] = A / L;
    }
}

template <int G>
int launch_attn_g(int hd, dim3 grid, hipStream_t s, const float* q, const float* K, const float* V, int n_kv, uint32_t len, const uint32_t* d_len,
                  float scale, int splits, uint32_t window, float softcap, float* part, float* out, int gq = G) {
    switch (hd) {
        case 64: hipLaunchKernelGGL((attn_split_kernel<G, 4>), grid, dim3(256), 0, s, q, K, V, n_kv, len, d_len, scale, splits, window, softcap, part, out, gq); break;
        case 128: hipLaunchKernelGGL((attn_split_kernel<G, 8>), grid, dim3(256), 0, s, q, K, V, n_kv, len, d_len, scale, splits, window, softcap, part, out, gq); break;
        default: return fhip::set_error(FHIP_ERR_SHAPE, "decode_attention: head_dim must be 64 or 128");
    }
    return FHIP_OK;
}

template <int G, int QF>
int launch_attn_kvq_g(int hd, dim3 grid, hipStream_t s, const float* q, const QCache& qc, int n_kv, uint32_t len, const uint32_t* d_len,
                      float scale, int splits, uint32_t window, float softcap, float* part, float* out, int gq = G) {
    switch (hd) {
        case 64: hipLaunchKernelGGL((attn_split_kvq_kernel<G, 4, QF>), grid, dim3(256), 0, s, q, qc, n_kv, len, d_len, scale, splits, window, softcap, part, out, gq); break;
        case 128: hipLaunchKernelGGL((attn_split_kvq_kernel<G, 8, QF>), grid, dim3(256), 0, s, q, qc, n_kv, len, d_len, scale, splits, window, softcap, part, out, gq); break;
        default: return fhip::set_error(FHIP_ERR_SHAPE, "decode_attention: head_dim must be 64 or 128");
    }
    return FHIP_OK;
}
template <int QF>
int launch_attn_kvq(int g, int hd, dim3 grid, hipStream_t s, const float* q, const QCache& qc, int n_kv, uint32_t len, const uint32_t* d_len,
                    float scale, int splits, uint32_t window, float softcap, float* part, float* out) {
    switch (g) {
        case 1: return launch_attn_kvq_g<1, QF>(hd, grid, s, q, qc, n_kv, len, d_len, scale, splits, window, softcap, part, out);
        case 2: return launch_attn_kvq_g<2, QF>(hd, grid, s, q, qc, n_kv, len, d_len, scale, splits, window, softcap, part, out);
        case 3: return launch_attn_kvq_g<3, QF>(hd, grid, s, q, qc, n_kv, len, d_len, scale, splits, window, softcap, part, out);
        case 4: return launch_attn_kvq_g<4, QF>(hd, grid, s, q, qc, n_kv, len, d_len, scale, splits, window, softcap, part, out);
        case 5: return launch_attn_kvq_g<5, QF>(hd, grid, s, q, qc, n_kv, len, d_len, scale, splits, window, softcap, part, out);
        case 6: return launch_attn_kvq_g<6, QF>(hd, grid, s, q, qc, n_kv, len, d_len, scale, splits, window, softcap, part, out);
        case 7: return launch_attn_kvq_g<7, QF>(hd, grid, s, q, qc, n_kv, len, d_len, scale, splits, window, softcap, part, out);
        case 8: return launch_attn_kvq_g<8, QF>(hd, grid, s, q, qc, n_kv, len, d_len, scale, splits, window, softcap, part, out);
        default: return fhip::set_error(FHIP_ERR_SHAPE, "decode_attention: %d query heads per KV head (1..=8 supported)", g);
    }
}

template <int G>
int launch_attn_fused_g(int hd, dim3 grid, hipStream_t s, const QkvPostParams& fp, int n_kv, uint32_t len, const uint32_t* d_len, float scale,
                        int splits, uint32_t window, float softcap, float* part, float* out, int gq = G) {
    switch (hd) {
        case 64: hipLaunchKernelGGL((attn_split_fused_kernel<G, 4>), grid, dim3(256), 0, s, fp, n_kv, len, d_len, scale, splits, window, softcap, part, out, gq); break;
        case 128: hipLaunchKernelGGL((attn_split_fused_kernel<G, 8>), grid, dim3(256), 0, s, fp, n_kv, len, d_len, scale, splits, window, softcap, part, out, gq); break;
        default: return fhip::set_error(FHIP_ERR_SHAPE, "decode_attention: head_dim must be 64 or 128");
    }
    return FHIP_OK;
}

}  // namespace

namespace fhip {

int launch_rmsnorm(const float* a, const float* b, const float* weight, size_t rows, size_t d, float eps, float* sum_out, float* norm_out,
                   hipStream_t s) {
    if (rows == 0 || d == 0) return FHIP_OK;
    if (d > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "rmsnorm: row length exceeds 2^31");
    if (d <= 512) {
        size_t grid = (rows + 3) / 4;
        if (grid > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "rmsnorm: too many rows for one launch");
        hipLaunchKernelGGL((rmsnorm_kernel<64>), dim3((unsigned)grid), dim3(256), 0, s, a, b, weight, rows, (int)d, eps, sum_out, norm_out);
    } else {
        if (rows > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "rmsnorm: too many rows for one launch");
        hipLaunchKernelGGL((rmsnorm_kernel<256>), dim3((unsigned)rows), dim3(256), 0, s, a, b, weight, rows, (int)d, eps, sum_out, norm_out);
    }
    return check_hip(hipGetLastError(), "rmsnorm launch");
}

int launch_u32_add(uint32_t* w, size_t n, uint32_t delta, hipStream_t s) {
    size_t grid = (n + 255) / 256;
    if (grid > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "u32_add: too many words for one launch");
    hipLaunchKernelGGL(u32_add_kernel, dim3((unsigned)grid), dim3(256), 0, s, w, n, delta);
    return check_hip(hipGetLastError(), "u32_add launch");
}

int launch_add(const float* a, const float* b, size_t n, float* out, hipStream_t s) {
    if (n == 0) return FHIP_OK;
    size_t grid = (n + 255) / 256;
    if (grid > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "add: too many elements for one launch");
    hipLaunchKernelGGL(add_kernel, dim3((unsigned)grid), dim3(256), 0, s, a, b, n, out);
    return check_hip(hipGetLastError(), "add launch");
}

int launch_mul_sigmoid(const float* a, const float* g, size_t n, float* out, hipStream_t s) {
    if (n == 0) return FHIP_OK;
    size_t grid = (n + 255) / 256;
    if (grid > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "mul_sigmoid: too many elements for one launch");
    hipLaunchKernelGGL(mul_sigmoid_kernel, dim3((unsigned)grid), dim3(256), 0, s, a, g, n, out);
    return check_hip(hipGetLastError(), "mul_sigmoid launch");
}

int launch_geglu(const float* gu, size_t t, size_t d, float* out, hipStream_t s) {
    const size_t n = t * d;
    if (n == 0) return FHIP_OK;
    size_t grid = (n + 255) / 256;
    if (grid > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "geglu: too many elements for one launch");
    hipLaunchKernelGGL(geglu_kernel, dim3((unsigned)grid), dim3(256), 0, s, gu, n, d, out);
    return check_hip(hipGetLastError(), "geglu launch");
}

int launch_rope(const float* x, size_t src_row_stride, size_t t, int heads, int hd, int n_rot, float base, const uint32_t* d_pos, uint32_t pos_off,
                const float* freq_scale, int interleaved, float* out, hipStream_t s) {
    if (t == 0 || heads == 0 || hd == 0) return FHIP_OK;
    size_t n = t * (size_t)heads * (size_t)(hd - n_rot / 2);
    size_t grid = (n + 255) / 256;
    if (t > 0x7FFFFFFFull || grid > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "rope: too many rows for one launch");
    hipLaunchKernelGGL(rope_kernel, dim3((unsigned)grid), dim3(256), 0, s, x, src_row_stride, (int)t, heads, hd, n_rot, base, d_pos, pos_off,
                       freq_scale, interleaved, out);
    return check_hip(hipGetLastError(), "rope launch");
}

int launch_qkv_post(const float* qkv, const float* bias, const float* q_norm, const float* k_norm, const uint32_t* d_pos, const float* freq_scale,
                    size_t t, int n_head, int n_kv, int hd, int n_rot, int interleaved, float eps, float base, float* q_out, float* k_cache,
                    float* v_cache, size_t cap, hipStream_t s, bool kv_packed) {
    if (t == 0) return FHIP_OK;
    QkvPostParams p;
    p.qkv = qkv; p.bias = bias; p.q_norm = q_norm; p.k_norm = k_norm; p.pos = d_pos; p.freq_scale = freq_scale;
    p.q_out = q_out; p.k_cache = k_cache; p.v_cache = v_cache;
    p.t = (int)t; p.n_head = n_head; p.n_kv = n_kv; p.hd = hd; p.n_rot = n_rot; p.interleaved = interleaved;
    p.cap = (uint32_t)cap; p.eps = eps; p.base = base; p.kv_packed = kv_packed ? 1 : 0;
    size_t waves = t * (size_t)(n_head + 2 * n_kv), grid = (waves + 3) / 4;
    if (t > 0x7FFFFFFFull || grid > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "qkv_post: too many rows for one launch");
    hipLaunchKernelGGL(qkv_post_kernel, dim3((unsigned)grid), dim3(256), 0, s, p);
    return check_hip(hipGetLastError(), "qkv_post launch");
}

int launch_kv_append(const float* k, const float* v, size_t t, size_t width, const uint32_t* d_pos, uint32_t pos_off, size_t cap, float* kc,
                     float* vc, hipStream_t s) {
    if (t == 0 || width == 0) return FHIP_OK;
    size_t n = t * width, grid = (n + 255) / 256;
    if (t > 0x7FFFFFFFull || width > 0x7FFFFFFFull || grid > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "kv_append: too large for one launch");
    hipLaunchKernelGGL(kv_append_kernel, dim3((unsigned)grid), dim3(256), 0, s, k, v, (int)t, (int)width, d_pos, pos_off, (uint32_t)cap, kc, vc);
    return check_hip(hipGetLastError(), "kv_append launch");
}

// Splits of the key range: about two workgroups per CU over all KV heads, at least 64 keys each (two rounds of the
// workgroup's 16 streams x 2 keys; 16 for caches of up to 256 rows), at most 256 (the combine kernel's LDS tables).
// Caches of up to ATT_SHORT rows (a launch sized for that many) with several query heads per KV head: one workgroup per query head over the whole key range, no
// splits, no combine launch. The rows of a KV head are read by each of its query heads' workgroups (a few hundred KB out of the
// L2), which costs less than the second launch and the trip of the partial results through memory.
constexpr size_t ATT_SHORT = 256;   // chained 64-layer step, ms per token, this shape | one workgroup per (query head, split): 180 keys 3.87 | 3.92, 248: 3.96 | 3.99, 300: 4.05 | 3.96, 370: 4.11 | 3.97
bool attn_per_query_head(size_t len, int n_head, int n_kv) { return n_kv > 0 && n_head > n_kv && len <= ATT_SHORT; }

// Between ATT_SHORT and ATT_MID rows under grouped query heads: one workgroup per (query head, split of at least ATT_MID_KEYS
// keys). The kernel that takes all query heads of a KV head at once holds 180 registers a lane (two waves per SIMD) and its
// waves spend their time in the dependent arithmetic of five softmax chains; with one head a workgroup (107 registers, four
// waves per SIMD) the same arithmetic is spread over five times the waves, and the rows they share come out of one XCD's L2
// (see the kernel's workgroup numbering). Chained 64-layer step, ms per token, this shape | all heads of a KV head per
// workgroup: 500 keys 3.99 | 4.24, 1000: 4.06 | 4.28, 2048: 4.22 | 4.56, 4096: 4.63 | 4.77, 6000: 4.97 | 4.90, 8000: 5.41 | 5.08.
constexpr size_t ATT_MID = 5120, ATT_MID_KEYS = 128;
bool attn_per_head_splits(size_t len, int n_head, int n_kv) { return n_kv > 0 && n_head > n_kv && len > ATT_SHORT && len <= ATT_MID; }
// splits of at least ATT_MID_KEYS keys, at most about two and a half workgroups per CU over all query heads
int attn_mid_splits(size_t len, int n_head) {
    const int by_keys = (int)((len + ATT_MID_KEYS - 1) / ATT_MID_KEYS), cap = 5 * device_cus() / 2 / (n_head > 0 ? n_head : 1);
    const int s = by_keys < cap ? by_keys : cap;
    return s < 1 ? 1 : (s > 256 ? 256 : s);
}

int attn_splits(size_t len, int n_kv) {
    if (n_kv <= 0 || len == 0) return 1;
    constexpr int keys = 64;
    int want = (2 * device_cus() + n_kv - 1) / n_kv;
    // up to 256 keys a split of 16 (half of the streams, one round) beat one of 64 by 0.1 ms per token of the chained step;
    // from 512 keys on the larger split count costs more in the combine than it saves
    const size_t per_split = len <= 256 ? 16 : (size_t)keys;
    size_t by_keys = (len + per_split - 1) / per_split;
    int splits = (int)(by_keys < (size_t)want ? by_keys : (size_t)want);
    return splits < 1 ? 1 : (splits > 256 ? 256 : splits);
}

// the most splits any launch shape takes for this cache length: what the workspace has to hold
int attn_ws_splits(size_t len, int n_head, int n_kv) {
    const int a = attn_splits(len, n_kv);
    const int b = attn_per_head_splits(len, n_head, n_kv) ? attn_mid_splits(len, n_head) : 1;
    return a > b ? a : b;
}

int launch_decode_attention(const float* q, const float* K, const float* V, int n_head, int n_kv, int hd, size_t len, const uint32_t* d_len,
                            size_t window, float softcap, float* ws, float* out, hipStream_t s) {
    if (n_head == 0 || hd == 0) return FHIP_OK;
    if (len == 0) return set_error(FHIP_ERR_SHAPE, "decode_attention: empty cache");
    if (n_kv <= 0 || n_head % n_kv != 0) return set_error(FHIP_ERR_SHAPE, "decode_attention: n_heads must be a multiple of n_kv_heads");
    if (hd != 64 && hd != 128) return set_error(FHIP_ERR_SHAPE, "decode_attention: head_dim must be 64 or 128");
    if (len > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "decode_attention: cache length exceeds 2^31");
    const int g = n_head / n_kv;
    const float scale = 1.0f / sqrtf((float)hd);
    const uint32_t win = window > 0x7FFFFFFFull ? 0u : (uint32_t)window;   // a window that large is no window
    if (g > 8) return set_error(FHIP_ERR_SHAPE, "decode_attention: %d query heads per KV head (1..=8 supported)", g);
    if (attn_per_query_head(len, n_head, n_kv)) {
        int rc = launch_attn_g<1>(hd, dim3((unsigned)n_head, 1), s, q, K, V, n_kv, (uint32_t)len, d_len, scale, 1, win, softcap, ws, out, g);
        return rc ? rc : check_hip(hipGetLastError(), "decode_attention launch");
    }
    const bool mid = attn_per_head_splits(len, n_head, n_kv);
    const int splits = mid ? attn_mid_splits(len, n_head) : attn_splits(len, n_kv);
    if (splits > 1 && !ws) return set_error(FHIP_ERR_ARG, "decode_attention: this cache length needs the workspace");
    dim3 grid((unsigned)n_kv, (unsigned)splits);
    int rc;
    if (mid) {
        const unsigned wgs = (unsigned)((n_kv * splits + 7) / 8 * 8 * g);
        rc = launch_attn_g<1>(hd, dim3(wgs, 1), s, q, K, V, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out, -g);
    } else
    switch (g) {
        case 1: rc = launch_attn_g<1>(hd, grid, s, q, K, V, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out); break;
        case 2: rc = launch_attn_g<2>(hd, grid, s, q, K, V, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out); break;
        case 3: rc = launch_attn_g<3>(hd, grid, s, q, K, V, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out); break;
        case 4: rc = launch_attn_g<4>(hd, grid, s, q, K, V, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out); break;
        case 5: rc = launch_attn_g<5>(hd, grid, s, q, K, V, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out); break;
        case 6: rc = launch_attn_g<6>(hd, grid, s, q, K, V, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out); break;
        case 7: rc = launch_attn_g<7>(hd, grid, s, q, K, V, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out); break;
        case 8: rc = launch_attn_g<8>(hd, grid, s, q, K, V, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out); break;
        default: return set_error(FHIP_ERR_SHAPE, "decode_attention: %d query heads per KV head (1..=8 supported)", g);
    }
    if (rc) return rc;
    if ((rc = check_hip(hipGetLastError(), "decode_attention launch"))) return rc;
    if (splits > 1) {
        hipLaunchKernelGGL(attn_combine_kernel, dim3((unsigned)n_head), dim3(COMBINE_THREADS), 0, s, ws, hd, splits, out);
        rc = check_hip(hipGetLastError(), "decode_attention combine launch");
    }
    return rc;
}

int launch_decode_attention_kvq(int fmt, const float* q, const uint32_t* k_codes, const uint16_t* k_scales, const uint32_t* v_codes,
                                const uint16_t* v_scales, int n_head, int n_kv, int hd, size_t len, const uint32_t* d_len, size_t window,
                                float softcap, float* ws, float* out, hipStream_t s) {
    if (n_head == 0 || hd == 0) return FHIP_OK;
    if (len == 0) return set_error(FHIP_ERR_SHAPE, "decode_attention: empty cache");
    if (n_kv <= 0 || n_head % n_kv != 0) return set_error(FHIP_ERR_SHAPE, "decode_attention: n_heads must be a multiple of n_kv_heads");
    if (hd != 64 && hd != 128) return set_error(FHIP_ERR_SHAPE, "decode_attention: head_dim must be 64 or 128");
    if (len > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "decode_attention: cache length exceeds 2^31");
    const int g = n_head / n_kv;
    const float scale = 1.0f / sqrtf((float)hd);
    const uint32_t win = window > 0x7FFFFFFFull ? 0u : (uint32_t)window;
    const QCache qc{k_codes, k_scales, v_codes, v_scales};
    int rc;
    if (g >= 1 && g <= 8 && attn_per_query_head(len, n_head, n_kv)) {   // as the f32 cache's launch: the same sums, the same bits
        const dim3 per_head((unsigned)n_head, 1);
        switch (fmt) {
            case FHIP_KVQ_Q8_0: rc = launch_attn_kvq_g<1, FHIP_KVQ_Q8_0>(hd, per_head, s, q, qc, n_kv, (uint32_t)len, d_len, scale, 1, win, softcap, ws, out, g); break;
            case FHIP_KVQ_Q4_0: rc = launch_attn_kvq_g<1, FHIP_KVQ_Q4_0>(hd, per_head, s, q, qc, n_kv, (uint32_t)len, d_len, scale, 1, win, softcap, ws, out, g); break;
            case FHIP_KVQ_Q4_1: rc = launch_attn_kvq_g<1, FHIP_KVQ_Q4_1>(hd, per_head, s, q, qc, n_kv, (uint32_t)len, d_len, scale, 1, win, softcap, ws, out, g); break;
            default: return set_error(FHIP_ERR_ARG, "decode_attention: unknown KV format %d", fmt);
        }
        return rc ? rc : check_hip(hipGetLastError(), "decode_attention launch");
    }
    const bool mid = g >= 1 && g <= 8 && attn_per_head_splits(len, n_head, n_kv);
    const int splits = mid ? attn_mid_splits(len, n_head) : attn_splits(len, n_kv);
    if (splits > 1 && !ws) return set_error(FHIP_ERR_ARG, "decode_attention: this cache length needs the workspace");
    const dim3 grid((unsigned)n_kv, (unsigned)splits);
    if (mid) {
        const dim3 lin((unsigned)((n_kv * splits + 7) / 8 * 8 * g), 1);
        switch (fmt) {
            case FHIP_KVQ_Q8_0: rc = launch_attn_kvq_g<1, FHIP_KVQ_Q8_0>(hd, lin, s, q, qc, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out, -g); break;
            case FHIP_KVQ_Q4_0: rc = launch_attn_kvq_g<1, FHIP_KVQ_Q4_0>(hd, lin, s, q, qc, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out, -g); break;
            case FHIP_KVQ_Q4_1: rc = launch_attn_kvq_g<1, FHIP_KVQ_Q4_1>(hd, lin, s, q, qc, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out, -g); break;
            default: return set_error(FHIP_ERR_ARG, "decode_attention: unknown KV format %d", fmt);
        }
    } else
    switch (fmt) {
        case FHIP_KVQ_Q8_0: rc = launch_attn_kvq<FHIP_KVQ_Q8_0>(g, hd, grid, s, q, qc, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out); break;
        case FHIP_KVQ_Q4_0: rc = launch_attn_kvq<FHIP_KVQ_Q4_0>(g, hd, grid, s, q, qc, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out); break;
        case FHIP_KVQ_Q4_1: rc = launch_attn_kvq<FHIP_KVQ_Q4_1>(g, hd, grid, s, q, qc, n_kv, (uint32_t)len, d_len, scale, splits, win, softcap, ws, out); break;
        default: return set_error(FHIP_ERR_ARG, "decode_attention: unknown KV format %d", fmt);
    }
    if (rc) return rc;
    if ((rc = check_hip(hipGetLastError(), "decode_attention launch"))) return rc;
    if (splits > 1) {
        hipLaunchKernelGGL(attn_combine_kernel, dim3((unsigned)n_head), dim3(COMBINE_THREADS), 0, s, ws, hd, splits, out);
        rc = check_hip(hipGetLastError(), "decode_attention combine launch");
    }
    return rc;
}

int launch_qkv_post_attention(const float* qkv, const float* bias, const float* q_norm, const float* k_norm, const uint32_t* d_pos,
                              const float* freq_scale, int n_head, int n_kv, int hd, int n_rot, bool interleaved, float eps, float base,
                              float* k_cache, float* v_cache, size_t cap, size_t len, size_t window, float softcap, float* ws, float* out,
                              hipStream_t s) {
    if (n_head == 0 || hd == 0) return FHIP_OK;
    if (len == 0) return set_error(FHIP_ERR_SHAPE, "qkv_post_attention: empty cache");
    if (n_kv <= 0 || n_head % n_kv != 0) return set_error(FHIP_ERR_SHAPE, "qkv_post_attention: n_heads must be a multiple of n_kv_heads");
    if (hd != 64 && hd != 128) return set_error(FHIP_ERR_SHAPE, "qkv_post_attention: head_dim must be 64 or 128");
    if (len > 0x7FFFFFFFull || len > cap) return set_error(FHIP_ERR_SHAPE, "qkv_post_attention: length outside the cache");
    const int g = n_head / n_kv;
    const bool mid = g <= 8 && attn_per_head_splits(len, n_head, n_kv);
    const int splits = attn_per_query_head(len, n_head, n_kv) ? 1 : (mid ? attn_mid_splits(len, n_head) : attn_splits(len, n_kv));
    if (splits > 1 && !ws) return set_error(FHIP_ERR_ARG, "qkv_post_attention: this cache length needs the workspace");
    QkvPostParams fp;
    fp.qkv = qkv; fp.bias = bias; fp.q_norm = q_norm; fp.k_norm = k_norm; fp.pos = d_pos; fp.freq_scale = freq_scale;
    fp.q_out = nullptr; fp.k_cache = k_cache; fp.v_cache = v_cache;
    fp.t = 1; fp.n_head = n_head; fp.n_kv = n_kv; fp.hd = hd; fp.n_rot = n_rot; fp.interleaved = interleaved ? 1 : 0;
    fp.cap = (uint32_t)cap; fp.eps = eps; fp.base = base; fp.kv_packed = 0;
    const float scale = 1.0f / sqrtf((float)hd);
    const uint32_t win = window > 0x7FFFFFFFull ? 0u : (uint32_t)window;
    if (g > 8) return set_error(FHIP_ERR_SHAPE, "qkv_post_attention: %d query heads per KV head (1..=8 supported)", g);
    if (attn_per_query_head(len, n_head, n_kv)) {
        // every workgroup of a KV head forms the new token's K and V rows and stores them (the same bits from each) before
        // it reads them back with the other keys
        int rc = launch_attn_fused_g<1>(hd, dim3((unsigned)n_head, 1), s, fp, n_kv, (uint32_t)len, d_pos, scale, 1, win, softcap, ws, out, g);
        return rc ? rc : check_hip(hipGetLastError(), "qkv_post_attention launch");
    }
    dim3 grid((unsigned)n_kv, (unsigned)splits);
    int rc;
    if (mid) {
        const unsigned wgs = (unsigned)((n_kv * splits + 7) / 8 * 8 * g);
        rc = launch_attn_fused_g<1>(hd, dim3(wgs, 1), s, fp, n_kv, (uint32_t)len, d_pos, scale, splits, win, softcap, ws, out, -g);
    } else
    switch (g) {
        case 1: rc = launch_attn_fused_g<1>(hd, grid, s, fp, n_kv, (uint32_t)len, d_pos, scale, splits, win, softcap, ws, out); break;
        case 2: rc = launch_attn_fused_g<2>(hd, grid, s, fp, n_kv, (uint32_t)len, d_pos, scale, splits, win, softcap, ws, out); break;
        case 3: rc = launch_attn_fused_g<3>(hd, grid, s, fp, n_kv, (uint32_t)len, d_pos, scale, splits, win, softcap, ws, out); break;
        case 4: rc = launch_attn_fused_g<4>(hd, grid, s, fp, n_kv, (uint32_t)len, d_pos, scale, splits, win, softcap, ws, out); break;
        case 5: rc = launch_attn_fused_g<5>(hd, grid, s, fp, n_kv, (uint32_t)len, d_pos, scale, splits, win, softcap, ws, out); break;
        case 6: rc = launch_attn_fused_g<6>(hd, grid, s, fp, n_kv, (uint32_t)len, d_pos, scale, splits, win, softcap, ws, out); break;
        case 7: rc = launch_attn_fused_g<7>(hd, grid, s, fp, n_kv, (uint32_t)len, d_pos, scale, splits, win, softcap, ws, out); break;
        case 8: rc = launch_attn_fused_g<8>(hd, grid, s, fp, n_kv, (uint32_t)len, d_pos, scale, splits, win, softcap, ws, out); break;
        default: return set_error(FHIP_ERR_SHAPE, "qkv_post_attention: %d query heads per KV head (1..=8 supported)", g);
    }
    if (rc) return rc;
    if ((rc = check_hip(hipGetLastError(), "qkv_post_attention launch"))) return rc;
    if (splits > 1) {
        hipLaunchKernelGGL(attn_combine_kernel, dim3((unsigned)n_head), dim3(COMBINE_THREADS), 0, s, ws, hd, splits, out);
        rc = check_hip(hipGetLastError(), "qkv_post_attention combine launch");
    }
    return rc;
}

}  // namespace fhip
