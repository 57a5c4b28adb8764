// Block-quantized K / V cache rows: quantize-on-append and dequantize, gfx950.
//
// Replaces the reference's kvquant kernels (crates/ferric-tensor/src/kvquant.rs: QUANT_*_WGSL / DEQUANT_*_WGSL, stated
// operation by operation in its `mod reference`, :943-1186). A row of `width` values is width / 32 blocks; block
// b = row * (width / 32) + col / 32 owns CODE_WORDS u32 of codes and one f16 scale (Q4_1: scale and minimum):
//   Q8_0  d = amax / 127, q = roundf(v * (1 / d)) in [-127, 127]; four int8 per word
//   Q4_0  d = (the value of largest magnitude, the first of equals) / -8, q = floor(v * (1 / d) + 8.5) in [0, 15]
//   Q4_1  d = (max - min) / 15, q = floor((v - min) * (1 / d) + 0.5) in [0, 15]
//   4-bit blocks: byte i = q[i] | q[i + 16] << 4.
// The scale arrays are the reference's bytes (two f16 per u32 word, block b in half b % 2 of word b / 2; Q4_1 d | min << 16)
// but written as 16-bit stores, one thread per block, so no two threads share a word and an append never reads the cache.
//
// Every f32 operation is the reference's, one rounding each: this file is compiled with -ffp-contract=off (no fused
// multiply-add where the reference multiplies and then adds), and divisions are IEEE divisions.
#include "common.hpp"

#include <hip/hip_fp16.h>

namespace {

constexpr int QK = 32;

// f32 -> f16 bits, round to nearest even, overflow to infinity; a NaN keeps its sign and top payload bits and stays quiet
// (kvquant.rs:956-995)
__device__ __forceinline__ uint16_t f16_bits(float x) {
    const uint32_t b = __float_as_uint(x);
    if ((b & 0x7F800000u) == 0x7F800000u && (b & 0x007FFFFFu) != 0)
        return (uint16_t)(((b >> 16) & 0x8000u) | 0x7C00u | 0x0200u | ((b & 0x007FFFFFu) >> 13));
    return __half_as_ushort(__float2half_rn(x));
}
__device__ __forceinline__ float f16_val(uint16_t h) { return __half2float(__ushort_as_half(h)); }

// Rust's `x as i32` behind a clamp: NaN -> 0
__device__ __forceinline__ int clamp_to_int(float r, float lo, float hi) { return r != r ? 0 : (int)fminf(fmaxf(r, lo), hi); }

template <int FMT>
__device__ __forceinline__ void quantize_block(const float (&v)[QK], uint32_t* __restrict__ codes, uint16_t* __restrict__ scales, size_t b) {
    if constexpr (FMT == FHIP_KVQ_Q8_0) {
        float amax = 0.f;
#pragma unroll
        for (int j = 0; j < QK; j++) amax = fmaxf(amax, fabsf(v[j]));      // fmaxf drops a NaN, as f32::max
        const float d = amax / 127.0f;
        const float inv = d > 0.f ? 1.0f / d : 0.f;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            uint32_t word = 0;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float t = v[4 * k + q] * inv;
                const float r = copysignf(floorf(fabsf(t) + 0.5f), t);     // round half away from zero (roundf)
                word |= ((uint32_t)clamp_to_int(r, -127.0f, 127.0f) & 255u) << (8 * q);
            }
            codes[b * 8 + k] = word;
        }
        scales[b] = f16_bits(d);
    } else if constexpr (FMT == FHIP_KVQ_Q4_0) {
        float amax = 0.f, mx = 0.f;
#pragma unroll
        for (int j = 0; j < QK; j++)
            if (amax < fabsf(v[j])) { amax = fabsf(v[j]); mx = v[j]; }
        const float d = mx / -8.0f;
        const float inv = d != 0.f ? 1.0f / d : 0.f;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            uint32_t word = 0;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int j = 4 * k + q;
                const uint32_t lo = (uint32_t)clamp_to_int(floorf(v[j] * inv + 8.5f), 0.f, 15.f);
                const uint32_t hi = (uint32_t)clamp_to_int(floorf(v[j + 16] * inv + 8.5f), 0.f, 15.f);
                word |= (lo | (hi << 4)) << (8 * q);
            }
            codes[b * 4 + k] = word;
        }
        scales[b] = f16_bits(d);
    } else {
        float mn = __builtin_inff(), mx = -__builtin_inff();
#pragma unroll
        for (int j = 0; j < QK; j++) { mn = fminf(mn, v[j]); mx = fmaxf(mx, v[j]); }
        const float d = (mx - mn) / 15.0f;
        const float inv = d != 0.f ? 1.0f / d : 0.f;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            uint32_t word = 0;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int j = 4 * k + q;
                const uint32_t lo = (uint32_t)clamp_to_int(floorf((v[j] - mn) * inv + 0.5f), 0.f, 15.f);
                const uint32_t hi = (uint32_t)clamp_to_int(floorf((v[j + 16] - mn) * inv + 0.5f), 0.f, 15.f);
                word |= (lo | (hi << 4)) << (8 * q);
            }
            codes[b * 4 + k] = word;
        }
        scales[2 * b] = f16_bits(d);
        scales[2 * b + 1] = f16_bits(mn);
    }
}

// One thread per block of t source rows. Row i goes to cache row pos[i] (or pos_off + i); src_at_pos: the source row sits at
// that index too (the newest row of a full-length f32 staging cache), else at i. blockIdx.y picks one of up to two
// (source, cache) pairs, so a token's K and V rows are stored by one launch.
struct KvqTargets {
    const float* src[2];
    uint32_t* codes[2];
    uint16_t* scales[2];
};
template <int FMT>
__global__ __launch_bounds__(256) void kvq_quant_kernel(KvqTargets tg, size_t src_row_stride, int t, int nblk,
                                                       const uint32_t* __restrict__ pos, uint32_t pos_off, int src_at_pos, uint32_t cap) {
    const float* __restrict__ src = tg.src[blockIdx.y];
    uint32_t* __restrict__ codes = tg.codes[blockIdx.y];
    uint16_t* __restrict__ scales = tg.scales[blockIdx.y];
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (size_t)t * nblk) return;
    const int i = (int)(id / nblk), cb = (int)(id % nblk);
    const uint32_t r = pos ? pos[i] : pos_off + (uint32_t)i;
    if (r >= cap) return;
    const float* x = src + (size_t)(src_at_pos ? r : (uint32_t)i) * src_row_stride + (size_t)cb * QK;
    float v[QK];
    if (((uintptr_t)x & 15) == 0) {
#pragma unroll
        for (int j = 0; j < QK; j += 4) {
            const float4 f = *(const float4*)(x + j);
            v[j] = f.x; v[j + 1] = f.y; v[j + 2] = f.z; v[j + 3] = f.w;
        }
    } else {
#pragma unroll
        for (int j = 0; j < QK; j++) v[j] = x[j];
    }
    quantize_block<FMT>(v, codes, scales, (size_t)r * nblk + cb);
}

// Four consecutive values per thread (one code word of a Q8_0 block; four bytes' low or high nibbles of a 4-bit one):
// out row i = cache row row0 + i. last_pos: rows past *last_pos are left alone (a captured step sizes the launch for the
// whole capacity and reads how far the cache is filled on the device).
template <int FMT>
__global__ __launch_bounds__(256) void kvq_dequant_kernel(const uint32_t* __restrict__ codes, const uint16_t* __restrict__ scales, size_t row0,
                                                         size_t rows, int width, const uint32_t* __restrict__ last_pos, float* __restrict__ out) {
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int w4 = width / 4;
    if (id >= rows * (size_t)w4) return;
    const size_t i = id / w4;
    const int col = (int)(id % w4) * 4;
    if (last_pos && row0 + i > (size_t)*last_pos) return;
    const size_t b = (row0 + i) * (size_t)(width / QK) + col / QK;
    const int j = col % QK;
    float4 o;
    if constexpr (FMT == FHIP_KVQ_Q8_0) {
        const float d = f16_val(scales[b]);
        const uint32_t word = codes[b * 8 + j / 4];
        o.x = (float)(int8_t)(word & 255u) * d;
        o.y = (float)(int8_t)((word >> 8) & 255u) * d;
        o.z = (float)(int8_t)((word >> 16) & 255u) * d;
        o.w = (float)(int8_t)(word >> 24) * d;
    } else {
        const uint32_t word = codes[b * 4 + (j % 16) / 4] >> (j < 16 ? 0 : 4);
        const float n0 = (float)(word & 15u), n1 = (float)((word >> 8) & 15u), n2 = (float)((word >> 16) & 15u), n3 = (float)((word >> 24) & 15u);
        if constexpr (FMT == FHIP_KVQ_Q4_0) {
            const float d = f16_val(scales[b]);
            o.x = (n0 - 8.0f) * d; o.y = (n1 - 8.0f) * d; o.z = (n2 - 8.0f) * d; o.w = (n3 - 8.0f) * d;
        } else {
            const float d = f16_val(scales[2 * b]), m = f16_val(scales[2 * b + 1]);
            o.x = n0 * d + m; o.y = n1 * d + m; o.z = n2 * d + m; o.w = n3 * d + m;
        }
    }
    *(float4*)(out + i * (size_t)width + col) = o;
}

}  // namespace

namespace fhip {

// src2 / codes2 / scales2: a second source and cache of the same shape stored by the same launch (null: one only)
int launch_kvq_append(int fmt, const float* src, size_t src_row_stride, size_t t, size_t width, const uint32_t* d_pos, uint32_t pos_off,
                      bool src_at_pos, size_t cap, uint32_t* codes, uint16_t* scales, hipStream_t s, const float* src2, uint32_t* codes2,
                      uint16_t* scales2) {
    if (t == 0 || width == 0) return FHIP_OK;
    const size_t nblk = width / QK, n = t * nblk, grid = (n + 255) / 256;
    if (t > 0x7FFFFFFFull || nblk > 0x7FFFFFFFull || grid > 0x7FFFFFFFull || cap > 0xFFFFFFFFull)
        return set_error(FHIP_ERR_SHAPE, "kvq_append: too large for one launch");
    const dim3 g((unsigned)grid, src2 ? 2u : 1u), wg(256);
    KvqTargets tg;
    tg.src[0] = src; tg.codes[0] = codes; tg.scales[0] = scales;
    tg.src[1] = src2; tg.codes[1] = codes2; tg.scales[1] = scales2;
    const int at = src_at_pos ? 1 : 0;
    switch (fmt) {
        case FHIP_KVQ_Q8_0: hipLaunchKernelGGL((kvq_quant_kernel<FHIP_KVQ_Q8_0>), g, wg, 0, s, tg, src_row_stride, (int)t, (int)nblk, d_pos, pos_off, at, (uint32_t)cap); break;
        case FHIP_KVQ_Q4_0: hipLaunchKernelGGL((kvq_quant_kernel<FHIP_KVQ_Q4_0>), g, wg, 0, s, tg, src_row_stride, (int)t, (int)nblk, d_pos, pos_off, at, (uint32_t)cap); break;
        case FHIP_KVQ_Q4_1: hipLaunchKernelGGL((kvq_quant_kernel<FHIP_KVQ_Q4_1>), g, wg, 0, s, tg, src_row_stride, (int)t, (int)nblk, d_pos, pos_off, at, (uint32_t)cap); break;
        default: return set_error(FHIP_ERR_ARG, "kvq_append: unknown format %d", fmt);
    }
    return check_hip(hipGetLastError(), "kvq_append launch");
}

int launch_kvq_dequantize(int fmt, const uint32_t* codes, const uint16_t* scales, size_t row0, size_t rows, size_t width, const uint32_t* d_last_pos,
                          float* out, hipStream_t s) {
    if (rows == 0 || width == 0) return FHIP_OK;
    const size_t n = rows * (width / 4), grid = (n + 255) / 256;
    if (width > 0x7FFFFFFFull || grid > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "kvq_dequantize: too large for one launch");
    const dim3 g((unsigned)grid), wg(256);
    switch (fmt) {
        case FHIP_KVQ_Q8_0: hipLaunchKernelGGL((kvq_dequant_kernel<FHIP_KVQ_Q8_0>), g, wg, 0, s, codes, scales, row0, rows, (int)width, d_last_pos, out); break;
        case FHIP_KVQ_Q4_0: hipLaunchKernelGGL((kvq_dequant_kernel<FHIP_KVQ_Q4_0>), g, wg, 0, s, codes, scales, row0, rows, (int)width, d_last_pos, out); break;
        case FHIP_KVQ_Q4_1: hipLaunchKernelGGL((kvq_dequant_kernel<FHIP_KVQ_Q4_1>), g, wg, 0, s, codes, scales, row0, rows, (int)width, d_last_pos, out); break;
        default: return set_error(FHIP_ERR_ARG, "kvq_dequantize: unknown format %d", fmt);
    }
    return check_hip(hipGetLastError(), "kvq_dequantize launch");
}

}  // namespace fhip
