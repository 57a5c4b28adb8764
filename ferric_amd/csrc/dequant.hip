// Bit-exact block unpackers for Q8_0 / Q4_K / Q6_K (and Q4_0 / Q4_1 / Q5_0 / Q5_1 / Q5_K) on gfx950.
//
// The reference CPU dequantizers round every f32 operation separately (Rust never fuses a*b+c):
//   Q8_0  y = f32(q) * d                       crates/ferric-gguf/src/lib.rs:608-615
//   Q4_K  y = (d*sc)*q - (dmin*m)              crates/ferric-gguf/src/lib.rs:793-825
//   Q6_K  y = (d*sc)*q                         crates/ferric-gguf/src/lib.rs:721-746
// so this file is compiled with -ffp-contract=off AND spells every operation with the
// round-to-nearest intrinsics, which the compiler never contracts.
//
// These kernels are write-bound (4 B out per 0.53-1.06 B in): one lane produces 4 consecutive
// outputs and stores them as one 16-byte vector, so a wave writes 1 KiB contiguous per store.
#include "common.hpp"

#include <hip/hip_fp16.h>

namespace {

__device__ __forceinline__ float f16_bits(uint32_t b) {
    // v_cvt_f32_f16: exact for every finite / subnormal / infinite pattern.
    return __half2float(__ushort_as_half((unsigned short)b));
}

// 4 bytes from a 2-byte-aligned address (Q8_0 and Q6_K blocks are only 2-byte aligned).
__device__ __forceinline__ uint32_t ld4_a2(const uint8_t* p) {
    const uint16_t* h = (const uint16_t*)p;
    return (uint32_t)h[0] | ((uint32_t)h[1] << 16);
}

__global__ void f16_to_f32_kernel(const uint16_t* __restrict__ in, size_t n, float* __restrict__ out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = f16_bits(in[i]);
}

// crates/ferric-gguf/src/lib.rs:501: a bf16 pattern is the top half of the f32 pattern
__global__ void bf16_to_f32_kernel(const uint16_t* __restrict__ in, size_t n, float* __restrict__ out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = __uint_as_float((uint32_t)in[i] << 16);
}

// ---- Q8_0: 34 B = [f16 d][i8 q[32]] ------------------------------------------------------------
__global__ void deq_q8_0_kernel(const uint8_t* __restrict__ raw, size_t nquads, float* __restrict__ out) {
    size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // one lane = 4 values
    if (t >= nquads) return;
    size_t blk = t >> 3;
    int j = (int)(t & 7) * 4;
    const uint8_t* b = raw + blk * 34;
    float d = f16_bits(*(const uint16_t*)b);
    uint32_t q = ld4_a2(b + 2 + j);
    float4 o;
    o.x = __fmul_rn((float)(int8_t)(q & 0xFF), d);
    o.y = __fmul_rn((float)(int8_t)((q >> 8) & 0xFF), d);
    o.z = __fmul_rn((float)(int8_t)((q >> 16) & 0xFF), d);
    o.w = __fmul_rn((float)(int8_t)(q >> 24), d);
    *(float4*)(out + t * 4) = o;
}

// ---- Q4_K: 144 B = [f16 d][f16 dmin][u8 s[12]][u8 qs[128]] --------------------------------------
// 6-bit (scale, min) of sub-block j -- get_sc_min, crates/ferric-gguf/src/lib.rs:795-804.
__device__ __forceinline__ void q4k_sc_min(const uint8_t* s, int j, uint32_t& sc, uint32_t& m) {
    if (j < 4) {
        sc = s[j] & 63u;
        m = s[j + 4] & 63u;
    } else {
        sc = (s[j + 4] & 0x0Fu) | ((uint32_t)(s[j - 4] >> 6) << 4);
        m = (uint32_t)(s[j + 4] >> 4) | ((uint32_t)(s[j] >> 6) << 4);
    }
}

__global__ void deq_q4_k_kernel(const uint8_t* __restrict__ raw, size_t nquads, float* __restrict__ out) {
    size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // one lane = 4 values, 64 lanes = one block
    if (t >= nquads) return;
    size_t blk = t >> 6;
    int v = (int)(t & 63) * 4;
    int sb = v >> 5, l = v & 31;
    const uint8_t* b = raw + blk * 144;  // 16-byte aligned
    uint32_t hd = *(const uint32_t*)b;
    float d = f16_bits(hd & 0xFFFFu), dmin = f16_bits(hd >> 16);
    uint32_t sc, m;
    q4k_sc_min(b + 4, sb, sc, m);
    uint32_t q = *(const uint32_t*)(b + 16 + 32 * (sb >> 1) + l);
    if (sb & 1) q >>= 4;
    q &= 0x0F0F0F0Fu;
    float d1 = __fmul_rn(d, (float)sc), mm = __fmul_rn(dmin, (float)m);
    float4 o;
    o.x = __fsub_rn(__fmul_rn(d1, (float)(q & 0xFF)), mm);
    o.y = __fsub_rn(__fmul_rn(d1, (float)((q >> 8) & 0xFF)), mm);
    o.z = __fsub_rn(__fmul_rn(d1, (float)((q >> 16) & 0xFF)), mm);
    o.w = __fsub_rn(__fmul_rn(d1, (float)(q >> 24)), mm);
    *(float4*)(out + t * 4) = o;
}

// ---- Q6_K: 210 B = [u8 ql[128]][u8 qh[64]][i8 sc[16]][f16 d] ------------------------------------
__global__ void deq_q6_k_kernel(const uint8_t* __restrict__ raw, size_t nquads, float* __restrict__ out) {
    size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= nquads) return;
    size_t blk = t >> 6;
    int v = (int)(t & 63) * 4;
    int hf = v >> 7, w = v & 127, g = w >> 5, l = w & 31, is = l >> 4;
    const uint8_t* b = raw + blk * 210;  // 2-byte aligned
    float d = f16_bits(*(const uint16_t*)(b + 208));
    float sc = (float)(int8_t)b[192 + 8 * hf + is + 2 * g];
    uint32_t ql = ld4_a2(b + 64 * hf + 32 * (g & 1) + l);
    uint32_t qh = ld4_a2(b + 128 + 32 * hf + l);
    uint32_t nib = (g >= 2 ? (ql >> 4) : ql) & 0x0F0F0F0Fu;
    uint32_t q = nib | (((qh >> (2 * g)) & 0x03030303u) << 4);
    float ds = __fmul_rn(d, sc);
    float4 o;
    o.x = __fmul_rn(ds, (float)((int)(q & 0xFF) - 32));
    o.y = __fmul_rn(ds, (float)((int)((q >> 8) & 0xFF) - 32));
    o.z = __fmul_rn(ds, (float)((int)((q >> 16) & 0xFF) - 32));
    o.w = __fmul_rn(ds, (float)((int)(q >> 24) - 32));
    *(float4*)(out + t * 4) = o;
}

// ---- the 32-value formats: [f16 d][f16 m]?[u32 qh]?[u8 qs[16]], blocks 2-byte aligned ----------------------
// value i < 16 is the low nibble of qs[i], value 16 + i the high one; the fifth bit of value v is bit v of qh.
//   Q4_0 y = f32(n - 8) * d            lib.rs:618-629      Q4_1 y = f32(n) * d + m            lib.rs:633-645
//   Q5_0 y = f32((n | b<<4) - 16) * d  lib.rs:650-665      Q5_1 y = f32(n | b<<4) * d + m     lib.rs:669-684
template <int BYTES, bool HAS_M, bool HAS_QH, int OFF>
__global__ void deq_legacy_kernel(const uint8_t* __restrict__ raw, size_t nquads, float* __restrict__ out) {
    size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // one lane = 4 values, 8 lanes = one block
    if (t >= nquads) return;
    size_t blk = t >> 3;
    int v = (int)(t & 7) * 4;
    const uint8_t* b = raw + blk * BYTES;
    constexpr int QH = HAS_M ? 4 : 2, QS = QH + (HAS_QH ? 4 : 0);
    float d = f16_bits(*(const uint16_t*)b);
    float m = HAS_M ? f16_bits(*(const uint16_t*)(b + 2)) : 0.f;
    uint32_t q = ld4_a2(b + QS + (v & 15));
    if (v >= 16) q >>= 4;
    q &= 0x0F0F0F0Fu;
    if (HAS_QH) {
        uint32_t hb = (ld4_a2(b + QH) >> v) & 0xFu;
        q |= ((hb * 0x00204081u) & 0x01010101u) << 4;   // bit j of hb -> bit 4 of byte j
    }
    float o[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float f = (float)((int)((q >> (8 * k)) & 0xFF) - OFF);
        o[k] = HAS_M ? __fadd_rn(__fmul_rn(f, d), m) : __fmul_rn(f, d);
    }
    *(float4*)(out + t * 4) = make_float4(o[0], o[1], o[2], o[3]);
}

// ---- Q5_K: 176 B = [f16 d][f16 dmin][u8 s[12]][u8 qh[32]][u8 qs[128]]; y = (d*sc)*(n + 16*bit) - dmin*m, lib.rs:692-716
__global__ void deq_q5_k_kernel(const uint8_t* __restrict__ raw, size_t nquads, float* __restrict__ out) {
    size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= nquads) return;
    size_t blk = t >> 6;
    int v = (int)(t & 63) * 4;
    int sb = v >> 5, l = v & 31;
    const uint8_t* b = raw + blk * 176;  // 16-byte aligned
    uint32_t hd = *(const uint32_t*)b;
    float d = f16_bits(hd & 0xFFFFu), dmin = f16_bits(hd >> 16);
    uint32_t sc, m;
    q4k_sc_min(b + 4, sb, sc, m);
    uint32_t q = *(const uint32_t*)(b + 48 + 32 * (sb >> 1) + l);
    if (sb & 1) q >>= 4;
    q &= 0x0F0F0F0Fu;
    q |= ((*(const uint32_t*)(b + 16 + l) >> sb) & 0x01010101u) << 4;   // bit sb of qh[l + k]
    float d1 = __fmul_rn(d, (float)sc), mm = __fmul_rn(dmin, (float)m);
    float4 o;
    o.x = __fsub_rn(__fmul_rn(d1, (float)(q & 0xFF)), mm);
    o.y = __fsub_rn(__fmul_rn(d1, (float)((q >> 8) & 0xFF)), mm);
    o.z = __fsub_rn(__fmul_rn(d1, (float)((q >> 16) & 0xFF)), mm);
    o.w = __fsub_rn(__fmul_rn(d1, (float)(q >> 24)), mm);
    *(float4*)(out + t * 4) = o;
}

// ---- IQ4_NL / IQ4_XS: 4-bit indices into a 16-level non-linear codebook (lib.rs:751), value = scale * level.
//   IQ4_NL 18 B = [f16 d][qs[16]]                                  y = d * kv[idx]                  lib.rs:755-767
//   IQ4_XS 136 B = [f16 d][u16 scales_h][scales_l[4]][qs[128]]     y = (d * (ls - 32)) * kv[idx]    lib.rs:772-791
// element j of a 32-value (sub-)block is the low nibble of its qs[j], element 16 + j the high nibble. Every product is exact
// in f32 (11-bit d x 6-bit ls x 7-bit level), so the order of the two multiplies cannot change a bit.
__device__ const float KV_IQ4NL[16] = {-127.f, -104.f, -83.f, -65.f, -49.f, -35.f, -22.f, -10.f, 1.f, 13.f, 25.f, 38.f, 53.f, 69.f, 89.f, 113.f};

template <bool XS>
__global__ void deq_iq4_kernel(const uint8_t* __restrict__ raw, size_t nquads, float* __restrict__ out) {
    size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // one lane = 4 values
    if (t >= nquads) return;
    uint32_t q;
    float dl;
    bool high;
    if (XS) {
        size_t blk = t >> 6;
        int v = (int)(t & 63) * 4, ib = v >> 5, l = v & 31;
        const uint8_t* b = raw + blk * 136;  // 8-byte aligned
        uint32_t hd = *(const uint32_t*)b, sl = *(const uint32_t*)(b + 4);
        int ls = (int)(((sl >> (4 * ib)) & 0xFu) | ((((hd >> 16) >> (2 * ib)) & 3u) << 4));
        dl = __fmul_rn(f16_bits(hd & 0xFFFFu), (float)(ls - 32));
        q = *(const uint32_t*)(b + 8 + 16 * ib + (l & 15));
        high = l >= 16;
    } else {
        size_t blk = t >> 3;
        int v = (int)(t & 7) * 4;
        const uint8_t* b = raw + blk * 18;
        dl = f16_bits(*(const uint16_t*)b);
        q = ld4_a2(b + 2 + (v & 15));
        high = v >= 16;
    }
    if (high) q >>= 4;
    float o[4];
#pragma unroll
    for (int k = 0; k < 4; k++) o[k] = __fmul_rn(dl, KV_IQ4NL[(q >> (8 * k)) & 0xFu]);
    *(float4*)(out + t * 4) = make_float4(o[0], o[1], o[2], o[3]);
}

// ---- MXFP4: 17 B = [u8 e][qs[16]]; y = (2 * E2M1[code]) * 2^(e - 128), lib.rs:857-908. The doubled table with the halved
// scale keeps (e = 255, code = 1) at the finite 2^127; e = 0 and 1 give subnormal scales, built from their bit patterns.
// One IEEE multiply per value: it rounds only where the result is subnormal or overflows, exactly as the reference's does.
__device__ const float KV_MXFP4_2X[16] = {0.f, 1.f, 2.f, 3.f, 4.f, 6.f, 8.f, 12.f, 0.f, -1.f, -2.f, -3.f, -4.f, -6.f, -8.f, -12.f};

__global__ void deq_mxfp4_kernel(const uint8_t* __restrict__ raw, size_t nquads, float* __restrict__ out) {
    size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= nquads) return;
    size_t blk = t >> 3;
    int v = (int)(t & 7) * 4;
    const uint8_t* b = raw + blk * 17;  // no alignment at all: byte loads
    uint32_t e = b[0];
    float d = __uint_as_float(e == 0 ? (1u << 21) : e == 1 ? (1u << 22) : (e - 1u) << 23);
    const uint8_t* qs = b + 1 + (v & 15);
    int sh = v >= 16 ? 4 : 0;
    float o[4];
#pragma unroll
    for (int k = 0; k < 4; k++) o[k] = __fmul_rn(KV_MXFP4_2X[(qs[k] >> sh) & 0xFu], d);
    *(float4*)(out + t * 4) = make_float4(o[0], o[1], o[2], o[3]);
}

}  // namespace

namespace fhip {

int launch_f16_to_f32(const uint16_t* d_bits, size_t n, float* d_out, hipStream_t s) {
    if (n == 0) return FHIP_OK;
    unsigned grid = (unsigned)((n + 255) / 256);
    hipLaunchKernelGGL(f16_to_f32_kernel, dim3(grid), dim3(256), 0, s, d_bits, n, d_out);
    return check_hip(hipGetLastError(), "f16_to_f32 launch");
}

int launch_bf16_to_f32(const uint16_t* d_bits, size_t n, float* d_out, hipStream_t s) {
    if (n == 0) return FHIP_OK;
    unsigned grid = (unsigned)((n + 255) / 256);
    hipLaunchKernelGGL(bf16_to_f32_kernel, dim3(grid), dim3(256), 0, s, d_bits, n, d_out);
    return check_hip(hipGetLastError(), "bf16_to_f32 launch");
}

int launch_dequant(uint32_t type, const uint8_t* d_raw, size_t nblocks, float* d_out, hipStream_t s) {
    if (nblocks == 0) return FHIP_OK;
    size_t vals = (type == FHIP_Q4_K || type == FHIP_Q5_K || type == FHIP_Q6_K || type == FHIP_IQ4_XS) ? 256 : 32;
    size_t nquads = nblocks * vals / 4;
    size_t grid = (nquads + 255) / 256;
    if (grid > 0x7FFFFFFFull) return set_error(FHIP_ERR_ARG, "dequant: %zu blocks exceed one launch", nblocks);
    switch (type) {
        case FHIP_Q8_0: hipLaunchKernelGGL(deq_q8_0_kernel, dim3((unsigned)grid), dim3(256), 0, s, d_raw, nquads, d_out); break;
        case FHIP_Q4_K: hipLaunchKernelGGL(deq_q4_k_kernel, dim3((unsigned)grid), dim3(256), 0, s, d_raw, nquads, d_out); break;
        case FHIP_Q6_K: hipLaunchKernelGGL(deq_q6_k_kernel, dim3((unsigned)grid), dim3(256), 0, s, d_raw, nquads, d_out); break;
        case FHIP_Q5_K: hipLaunchKernelGGL(deq_q5_k_kernel, dim3((unsigned)grid), dim3(256), 0, s, d_raw, nquads, d_out); break;
        case FHIP_Q4_0: hipLaunchKernelGGL((deq_legacy_kernel<18, false, false, 8>), dim3((unsigned)grid), dim3(256), 0, s, d_raw, nquads, d_out); break;
        case FHIP_Q4_1: hipLaunchKernelGGL((deq_legacy_kernel<20, true, false, 0>), dim3((unsigned)grid), dim3(256), 0, s, d_raw, nquads, d_out); break;
        case FHIP_Q5_0: hipLaunchKernelGGL((deq_legacy_kernel<22, false, true, 16>), dim3((unsigned)grid), dim3(256), 0, s, d_raw, nquads, d_out); break;
        case FHIP_Q5_1: hipLaunchKernelGGL((deq_legacy_kernel<24, true, true, 0>), dim3((unsigned)grid), dim3(256), 0, s, d_raw, nquads, d_out); break;
        case FHIP_IQ4_NL: hipLaunchKernelGGL((deq_iq4_kernel<false>), dim3((unsigned)grid), dim3(256), 0, s, d_raw, nquads, d_out); break;
        case FHIP_IQ4_XS: hipLaunchKernelGGL((deq_iq4_kernel<true>), dim3((unsigned)grid), dim3(256), 0, s, d_raw, nquads, d_out); break;
        case FHIP_MXFP4: hipLaunchKernelGGL(deq_mxfp4_kernel, dim3((unsigned)grid), dim3(256), 0, s, d_raw, nquads, d_out); break;
        default: return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "unsupported ggml type %u", type);
    }
    return check_hip(hipGetLastError(), "dequant launch");
}

}  // namespace fhip
