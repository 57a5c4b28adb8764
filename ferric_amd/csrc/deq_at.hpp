// Random-access dequantisation of ONE weight: element `col` of a row of raw GGUF blocks, with exactly the operations and
// roundings of the reference's block dequantisers (crates/ferric-gguf/src/lib.rs:608-615 Q8_0, :618-684 Q4_0 / Q4_1 / Q5_0 /
// Q5_1, :692-716 Q5_K, :721-746 Q6_K, :751-791 IQ4_NL / IQ4_XS, :793-825 Q4_K, :857-908 MXFP4). Byte loads only, so it works at
// any alignment. Slow by design: it serves the element-by-element branch the mat-vec kernels take for activation runs that
// block fixed point cannot represent (NaN, +-inf, magnitudes near the bottom of the f32 range).
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ferric_hip.h"

namespace fhip {

__device__ __forceinline__ float da_f16(const uint8_t* p) {
    return __half2float(__ushort_as_half((unsigned short)((uint32_t)p[0] | ((uint32_t)p[1] << 8))));
}

// 6-bit (scale, min) of sub-block j of a Q4_K / Q5_K block: get_sc_min, crates/ferric-gguf/src/lib.rs:795-804
__device__ __forceinline__ void da_sc_min(const uint8_t* s, int j, uint32_t& sc, uint32_t& m) {
    if (j < 4) {
        sc = s[j] & 63u;
        m = s[j + 4] & 63u;
    } else {
        sc = (s[j + 4] & 0x0Fu) | ((uint32_t)(s[j - 4] >> 6) << 4);
        m = (uint32_t)(s[j + 4] >> 4) | ((uint32_t)(s[j] >> 6) << 4);
    }
}

template <uint32_t TYPE>
__device__ inline float deq_at(const uint8_t* row, int col) {
    if constexpr (TYPE == FHIP_Q8_0) {
        const uint8_t* b = row + (size_t)(col >> 5) * 34;
        return __fmul_rn((float)(int8_t)b[2 + (col & 31)], da_f16(b));
    } else if constexpr (TYPE == FHIP_Q4_K || TYPE == FHIP_Q5_K) {
        constexpr int BYTES = TYPE == FHIP_Q4_K ? 144 : 176, QS = TYPE == FHIP_Q4_K ? 16 : 48;
        const uint8_t* b = row + (size_t)(col >> 8) * BYTES;
        const int v = col & 255, sb = v >> 5, l = v & 31;
        uint32_t sc, m;
        da_sc_min(b + 4, sb, sc, m);
        uint32_t q = b[QS + 32 * (sb >> 1) + l];
        q = (sb & 1) ? q >> 4 : q & 15u;
        if constexpr (TYPE == FHIP_Q5_K) q |= ((uint32_t)(b[16 + l] >> sb) & 1u) << 4;
        const float d1 = __fmul_rn(da_f16(b), (float)sc), mm = __fmul_rn(da_f16(b + 2), (float)m);
        return __fsub_rn(__fmul_rn(d1, (float)q), mm);
    } else if constexpr (TYPE == FHIP_Q6_K) {
        const uint8_t* b = row + (size_t)(col >> 8) * 210;
        const int v = col & 255, hf = v >> 7, w = v & 127, g = w >> 5, l = w & 31, is = l >> 4;
        const float sc = (float)(int8_t)b[192 + 8 * hf + is + 2 * g];
        const uint32_t ql = b[64 * hf + 32 * (g & 1) + l], qh = b[128 + 32 * hf + l];
        const uint32_t nib = g >= 2 ? ql >> 4 : ql & 15u;
        const int q = (int)(nib | (((qh >> (2 * g)) & 3u) << 4)) - 32;
        return __fmul_rn(__fmul_rn(da_f16(b + 208), sc), (float)q);
    } else if constexpr (TYPE == FHIP_Q4_0 || TYPE == FHIP_Q4_1 || TYPE == FHIP_Q5_0 || TYPE == FHIP_Q5_1) {
        constexpr bool HAS_M = TYPE == FHIP_Q4_1 || TYPE == FHIP_Q5_1, HAS_QH = TYPE == FHIP_Q5_0 || TYPE == FHIP_Q5_1;
        constexpr int QH = HAS_M ? 4 : 2, QS = QH + (HAS_QH ? 4 : 0), BYTES = QS + 16;
        constexpr int OFF = TYPE == FHIP_Q4_0 ? 8 : TYPE == FHIP_Q5_0 ? 16 : 0;
        const uint8_t* b = row + (size_t)(col >> 5) * BYTES;
        const int v = col & 31;
        uint32_t q = b[QS + (v & 15)];
        q = v >= 16 ? q >> 4 : q & 15u;
        if constexpr (HAS_QH) {
            const uint32_t qh = (uint32_t)b[QH] | ((uint32_t)b[QH + 1] << 8) | ((uint32_t)b[QH + 2] << 16) | ((uint32_t)b[QH + 3] << 24);
            q |= ((qh >> v) & 1u) << 4;
        }
        const float f = (float)((int)q - OFF), d = da_f16(b);
        if constexpr (HAS_M) return __fadd_rn(__fmul_rn(f, d), da_f16(b + 2));
        return __fmul_rn(f, d);
    } else if constexpr (TYPE == FHIP_IQ4_NL || TYPE == FHIP_IQ4_XS) {
        const float kv[16] = {-127.f, -104.f, -83.f, -65.f, -49.f, -35.f, -22.f, -10.f, 1.f, 13.f, 25.f, 38.f, 53.f, 69.f, 89.f, 113.f};
        float dl;
        uint32_t q;
        int v;
        if constexpr (TYPE == FHIP_IQ4_XS) {
            const uint8_t* b = row + (size_t)(col >> 8) * 136;
            const int ib = (col & 255) >> 5;
            v = col & 31;
            const uint32_t sh = (uint32_t)b[2] | ((uint32_t)b[3] << 8);
            const uint32_t sl = (uint32_t)b[4] | ((uint32_t)b[5] << 8) | ((uint32_t)b[6] << 16) | ((uint32_t)b[7] << 24);
            const int ls = (int)(((sl >> (4 * ib)) & 0xFu) | (((sh >> (2 * ib)) & 3u) << 4));
            dl = __fmul_rn(da_f16(b), (float)(ls - 32));
            q = b[8 + 16 * ib + (v & 15)];
        } else {
            const uint8_t* b = row + (size_t)(col >> 5) * 18;
            v = col & 31;
            dl = da_f16(b);
            q = b[2 + (v & 15)];
        }
        q = v >= 16 ? q >> 4 : q & 15u;
        return __fmul_rn(dl, kv[q]);
    } else {
        static_assert(TYPE == FHIP_MXFP4, "deq_at: format without a random-access dequantiser");
        const float kv[16] = {0.f, 1.f, 2.f, 3.f, 4.f, 6.f, 8.f, 12.f, 0.f, -1.f, -2.f, -3.f, -4.f, -6.f, -8.f, -12.f};
        const uint8_t* b = row + (size_t)(col >> 5) * 17;
        const int v = col & 31;
        const uint32_t e = b[0];
        const float d = __uint_as_float(e == 0 ? (1u << 21) : e == 1 ? (1u << 22) : (e - 1u) << 23);
        uint32_t q = b[1 + (v & 15)];
        q = v >= 16 ? q >> 4 : q & 15u;
        return __fmul_rn(kv[q], d);
    }
}

}  // namespace fhip
