// Mixture-of-experts glue around the "_id" matmuls: the router top-k and the weighted sum of the selected
// experts' down projections.
//
// moe_topk follows crates/ferric-tensor/src/dtype.rs:2415-2461 (MOE_TOPK_WGSL): per token, scores = softmax
// over all experts or sigmoid; the k best by score (+ bias, which never enters the weights) are taken in
// order, ties to the lowest index; their scores, divided by their sum when `norm`, times `scale`, are written
// as [w_0..w_{k-1} | idx_0..idx_{k-1}] with the indices stored as f32. The reference scans with one thread per
// token; here one wave per token holds the scores in registers (n_expert <= 1024 = 16 per lane) and each of
// the k rounds is a wave-wide arg-max with the same ordering rule.
#include "common.hpp"

namespace {

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// All-lanes maximum / sum without LDS traffic: four DPP steps make every lane of a 16-lane row hold its row's
// result, the four rows are then combined through scalar reads of one lane each.
__device__ __forceinline__ float lane_f(float v, int ln) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), ln));
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f<0xB1>(v));    // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_f<0x4E>(v));    // quad_perm [2,3,0,1]
    v = fmaxf(v, dpp_f<0x141>(v));   // row_half_mirror
    v = fmaxf(v, dpp_f<0x140>(v));   // row_mirror
    return fmaxf(fmaxf(lane_f(v, 0), lane_f(v, 16)), fmaxf(lane_f(v, 32), lane_f(v, 48)));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f<0xB1>(v);
    v += dpp_f<0x4E>(v);
    v += dpp_f<0x141>(v);
    v += dpp_f<0x140>(v);
    return (lane_f(v, 0) + lane_f(v, 16)) + (lane_f(v, 32) + lane_f(v, 48));
}

// PL = experts per lane (n_expert <= 64 * PL); expert i lives in lane i % 64, register i / 64
template <int PL>
__global__ void __launch_bounds__(64) moe_topk_kernel(const float* __restrict__ logits, const float* __restrict__ bias, int t, int ne,
                                                       int k, int sigmoid, float scale, int norm, float* __restrict__ out) {
    const int ti = blockIdx.x, lane = threadIdx.x;
    if (ti >= t) return;
    const float* l = logits + (size_t)ti * ne;
    float sc[PL], key[PL];
    float maxl = -3.4e38f;
#pragma unroll
    for (int j = 0; j < PL; j++) {
        const int i = j * 64 + lane;
        sc[j] = i < ne ? l[i] : 0.f;
        if (i < ne && !sigmoid) maxl = fmaxf(maxl, sc[j]);
    }
    float ssum = 0.f;
    if (!sigmoid) {
        maxl = wave_max(maxl);
#pragma unroll
        for (int j = 0; j < PL; j++) {
            const int i = j * 64 + lane;
            sc[j] = i < ne ? expf(sc[j] - maxl) : 0.f;
            ssum += sc[j];
        }
        ssum = wave_sum(ssum);
    }
#pragma unroll
    for (int j = 0; j < PL; j++) {
        const int i = j * 64 + lane;
        if (i < ne) {
            sc[j] = sigmoid ? 1.0f / (1.0f + expf(-sc[j])) : sc[j] / ssum;
            key[j] = bias ? sc[j] + bias[i] : sc[j];
        } else {
            key[j] = -__builtin_inff();   // never beats the reference's starting value
        }
    }
    float wsum = 0.f, myw = 0.f, myi = 0.f;   // lane s keeps slot s
    for (int s = 0; s < k; s++) {
        // best of this lane: larger key first, then lower index; a key must exceed -3.4e38 to count at all
        float bv = -3.4e38f, bs = 0.f;
        int bi = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < PL; j++) {
            if (key[j] > bv) { bv = key[j]; bi = j * 64 + lane; bs = sc[j]; }
        }
        // the wave's best value, then among the lanes that hold it the lowest expert index (usually one lane)
        const float vmax = wave_max(bv);
        unsigned long long m = __ballot(bv == vmax && bi != 0x7fffffff);
        int win = 0, owner = 0;
        float ws = 0.f;
        if (m == 0) {   // nothing selectable (all NaN, or already taken): the reference's scan leaves index 0
            ws = lane_f(sc[0], 0);
        } else {
            win = 0x7fffffff;
            while (m) {
                const int ln = __builtin_ctzll(m);
                const int i = __builtin_amdgcn_readlane(bi, ln);
                if (i < win) { win = i; owner = ln; }
                m &= m - 1;
            }
            ws = lane_f(bs, owner);
            if (lane == owner) {   // retire the winner
#pragma unroll
                for (int j = 0; j < PL; j++)
                    if (j == (win >> 6)) key[j] = -__builtin_inff();
            }
        }
        wsum += ws;
        if (lane == s) { myw = ws; myi = (float)win; }
    }
    const float den = norm ? wsum : 1.0f;
    if (lane < k) {
        out[(size_t)ti * 2 * k + lane] = myw / den * scale;
        out[(size_t)ti * 2 * k + k + lane] = myi;
    }
}

// out[ti, o] = sum_s selw[ti, s] * parts[ti*k + s, o], slots added in order (dtype.rs:2555-2567)
__global__ void __launch_bounds__(256) moe_wsum_kernel(const float* __restrict__ parts, const float* __restrict__ selw, size_t n, int k,
                                                        size_t out_pe, float* __restrict__ y) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t ti = i / out_pe, o = i - ti * out_pe;
    float total = 0.f;
    for (int s = 0; s < k; s++) total = total + selw[ti * 2 * k + s] * parts[(ti * k + s) * out_pe + o];
    y[i] = total;
}

}  // namespace

namespace fhip {

int launch_moe_topk(const float* d_logits, const float* d_bias, size_t t, size_t ne, int k, int sigmoid, float scale, int norm,
                    float* d_out, hipStream_t s) {
    if (t == 0) return FHIP_OK;
    auto go = [&](auto kern) {
        hipLaunchKernelGGL(kern, dim3((unsigned)t), dim3(64), 0, s, d_logits, d_bias, (int)t, (int)ne, k, sigmoid, scale, norm, d_out);
    };
    if (ne <= 64) go(moe_topk_kernel<1>);
    else if (ne <= 128) go(moe_topk_kernel<2>);
    else if (ne <= 256) go(moe_topk_kernel<4>);
    else if (ne <= 512) go(moe_topk_kernel<8>);
    else go(moe_topk_kernel<16>);
    return check_hip(hipGetLastError(), "moe_topk launch");
}

int launch_moe_wsum(const float* d_parts, const float* d_selw, size_t t, int k, size_t out_pe, float* d_y, hipStream_t s) {
    const size_t n = t * out_pe;
    if (n == 0) return FHIP_OK;
    hipLaunchKernelGGL(moe_wsum_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, d_parts, d_selw, n, k, out_pe, d_y);
    return check_hip(hipGetLastError(), "moe_wsum launch");
}

}  // namespace fhip
