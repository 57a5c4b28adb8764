// General-shape mat-vec (and small-batch mat-mat) on the raw GGUF block stream, gfx950: covers every
// cols the formats allow (any multiple of 256, or of 32 for the 32-value formats), with plain f32 multiply-adds,
// and every block format of the path (Q8_0, Q4_K, Q6_K, and Q4_0 / Q4_1 / Q5_0 / Q5_1 / Q5_K / IQ4_NL / IQ4_XS / MXFP4).
// The streaming kernel in gemv.hip takes over for row lengths it tiles exactly; this one is the
// shape-complete path behind it.
//
//   y[m, o] = sum_k x[m, k] * dequant(W[o, k])        f32 activations, f32 accumulate
//
// Replaces the reference's split-K / flat WGSL kernels (crates/ferric-tensor/src/dtype.rs:2995-3051
// Q4_K, :3423-3469 Q6_K, :3473-3529 Q8_0) and the fused gate/up SwiGLU kernels (:2372-2410, :2734-2775).
//
// Work decomposition (memory-bound design, one pass over the weight bytes):
//   * The unit of lane work is 32 weights of one row ("unit"): a 16-byte quant chunk of a Q4_K
//     block, an (8+8+8)-byte ql/ql/qh triple of a Q6_K block, or one whole 34-byte Q8_0 block.
//     A row has cols/32 units, for every format.
//   * A wave owns 64 consecutive units of the row (a K-slice) and keeps the matching 32 activation
//     values per lane in REGISTERS for its whole life: the lane -> column mapping is the same for
//     every row, so x is read once per wave (staged through LDS once per workgroup) and never again.
//   * S = ceil(units/64) waves cover one row (K split across waves); G such wave-sets ("row groups")
//     share a workgroup and walk disjoint contiguous row spans, streaming the weight bytes with
//     16-/8-byte loads straight from the GGUF layout, U rows in flight per wave.
//   * Per row each wave reduces its 64 partial sums with DPP (no LDS traffic) and parks one float
//     in LDS; after one barrier the S partials of each row are added in a fixed order, so the result
//     does not depend on scheduling.
#include "common.hpp"

#include <hip/hip_fp16.h>
#include <stdlib.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
// Q6_K / Q8_0 blocks are only 2-byte aligned in the GGUF stream; gfx950 global loads accept that.
struct __attribute__((packed, aligned(2))) U4A2 { u32x4 v; };
struct __attribute__((packed, aligned(2))) U2A2 { u32x2 v; };

__device__ __forceinline__ float f16_bits(uint32_t b) { return __half2float(__ushort_as_half((unsigned short)b)); }
__device__ __forceinline__ float ub(uint32_t v, int k) { return (float)((v >> (8 * k)) & 0xFFu); }  // v_cvt_f32_ubyteK
__device__ __forceinline__ float sb(uint32_t v, int k) { return (float)(int8_t)((v >> (8 * k)) & 0xFFu); }

// Pins a loaded dword in a VGPR at the point of use. Without it the optimizer unpacks the bytes of
// a prefetched row the moment the load returns and carries 32 unpacked values per row in flight,
// which spills; with it the rows in flight stay as the packed dwords that were loaded.
__device__ __forceinline__ void pin(uint32_t& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void pin(u32x2& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void pin(u32x4& v) { asm volatile("" : "+v"(v)); }

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
    int t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xF, false);
    return v + __int_as_float(t);
}
// Sum over the 64 lanes of a wave; the total lands in lane 63.
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
    v = dpp_add<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
    v = dpp_add<0x141, 0xF>(v);  // row_half_mirror
    v = dpp_add<0x140, 0xF>(v);  // row_mirror: every lane of a 16-lane row holds the row sum
    v = dpp_add<0x142, 0xA>(v);  // row_bcast15 into rows 1 and 3
    v = dpp_add<0x143, 0xC>(v);  // row_bcast31 into rows 2 and 3
    return v;
}

// ------------------------------------------------------------------------------------------------
// Per-format lane work. `setup` maps unit u of a row to byte offsets inside the row and to the four
// runs of 8 activation columns the lane needs (x[m][8*j + i] = x[m, xo[j] + i]). `dot` returns the
// lane's share of the dot product for M activation rows. sx[m][j] = sum_i x[m][8*j+i].
// ------------------------------------------------------------------------------------------------

struct Q4K {
    // 144 B = [f16 d][f16 dmin][12 B packed 6-bit scales/mins][128 B nibbles]; every piece 16-byte aligned.
    struct Lane { uint32_t off_h, off_q, sh; bool high; };
    struct Data { u32x4 h, q; __device__ __forceinline__ void pin_all() { pin(h); pin(q); } };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&xo)[4]) {
        int b = u >> 3, p = u & 7, g = p >> 1, hf = p & 1;
        L.off_h = b * 144;
        L.off_q = b * 144 + 16 + 16 * p;  // qs[16p, 16p+16): group g, l in [16hf, 16hf+16)
        L.sh = 16 * (g & 1);
        L.high = g >= 2;
        int base = 256 * b + 64 * g + 16 * hf;
        xo[0] = base; xo[1] = base + 8; xo[2] = base + 32; xo[3] = base + 40;  // low nibbles, then high nibbles
    }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L) {
        Data d;
        d.h = *(const u32x4*)(row + L.off_h);
        d.q = *(const u32x4*)(row + L.off_q);
        return d;
    }
    template <int M>
    static __device__ __forceinline__ void dot(const Data& D, const Lane& L, const float (&x)[M][32], const float (&sx)[M][4],
                                               float (&out)[M]) {
        // (sc, m) of sub-blocks 2g and 2g+1 as two packed bytes each -- get_sc_min,
        // crates/ferric-gguf/src/lib.rs:795-804, evaluated for a byte pair at once.
        uint32_t a = D.h[1] >> L.sh, b = D.h[2] >> L.sh, c = D.h[3] >> L.sh;
        uint32_t scp = L.high ? ((c & 0x0F0Fu) | ((a >> 2) & 0x3030u)) : (a & 0x3F3Fu);
        uint32_t mp = L.high ? (((c >> 4) & 0x0F0Fu) | ((b >> 2) & 0x3030u)) : (b & 0x3F3Fu);
        float d = f16_bits(D.h[0] & 0xFFFFu), dmin = f16_bits(D.h[0] >> 16);
        float d0 = d * ub(scp, 0), d1 = d * ub(scp, 1) * 0.0625f;  // high nibbles are used as 16*n
        float m0 = dmin * ub(mp, 0), m1 = dmin * ub(mp, 1);
        float lo[M], hi[M];
#pragma unroll
        for (int m = 0; m < M; m++) { lo[m] = 0.f; hi[m] = 0.f; }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t ql = D.q[i] & 0x0F0F0F0Fu, qh = D.q[i] & 0xF0F0F0F0u;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float fl = ub(ql, k), fh = ub(qh, k);
#pragma unroll
                for (int m = 0; m < M; m++) {
                    lo[m] = fmaf(x[m][4 * i + k], fl, lo[m]);
                    hi[m] = fmaf(x[m][16 + 4 * i + k], fh, hi[m]);
                }
            }
        }
#pragma unroll
        for (int m = 0; m < M; m++)
            out[m] = d0 * lo[m] - m0 * (sx[m][0] + sx[m][1]) + (d1 * hi[m] - m1 * (sx[m][2] + sx[m][3]));
    }
};

struct Q6K {
    // 210 B = [ql 128][qh 64][i8 sc 16][f16 d]; unit (hf, t): l in [8t, 8t+8) of half hf.
    struct Lane { uint32_t off_a, off_h, off_s, off_d, ssh; };
    struct Data { u32x2 a, b, h, s; uint32_t d; __device__ __forceinline__ void pin_all() { pin(a); pin(b); pin(h); pin(s); pin(d); } };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&xo)[4]) {
        int b = u >> 3, r = u & 7, hf = r >> 2, t = r & 3;
        L.off_a = b * 210 + 64 * hf + 8 * t;
        L.off_h = b * 210 + 128 + 32 * hf + 8 * t;
        L.off_s = b * 210 + 192 + 8 * hf;
        L.off_d = b * 210 + 208;
        L.ssh = 8 * (t >> 1);  // is = l / 16
        int base = 256 * b + 128 * hf + 8 * t;
        xo[0] = base; xo[1] = base + 32; xo[2] = base + 64; xo[3] = base + 96;
    }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L) {
        Data d;
        d.a = ((const U2A2*)(row + L.off_a))->v;
        d.b = ((const U2A2*)(row + L.off_a + 32))->v;
        d.h = ((const U2A2*)(row + L.off_h))->v;
        d.s = ((const U2A2*)(row + L.off_s))->v;
        d.d = *(const uint16_t*)(row + L.off_d);
        return d;
    }
    template <int M>
    static __device__ __forceinline__ void dot(const Data& D, const Lane& L, const float (&x)[M][32], const float (&sx)[M][4],
                                               float (&out)[M]) {
        float acc[M][4];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[m][j] = 0.f;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            uint32_t A = D.a[i], B = D.b[i], H = D.h[i];
            // the four 6-bit quants that share byte l -- crates/ferric-gguf/src/lib.rs:733-736, four bytes at a time
            uint32_t q[4];
            q[0] = (A & 0x0F0F0F0Fu) | ((H & 0x03030303u) << 4);
            q[1] = (B & 0x0F0F0F0Fu) | ((H & 0x0C0C0C0Cu) << 2);
            q[2] = ((A >> 4) & 0x0F0F0F0Fu) | (H & 0x30303030u);
            q[3] = ((B >> 4) & 0x0F0F0F0Fu) | ((H >> 2) & 0x30303030u);
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    float f = ub(q[j], k);
#pragma unroll
                    for (int m = 0; m < M; m++) acc[m][j] = fmaf(x[m][8 * j + 4 * i + k], f, acc[m][j]);
                }
        }
        uint32_t s0 = D.s[0] >> L.ssh, s1 = D.s[1] >> L.ssh;  // sc[is], sc[is+2] | sc[is+4], sc[is+6]
        float c0 = sb(s0, 0), c1 = sb(s0, 2), c2 = sb(s1, 0), c3 = sb(s1, 2);
        float d = f16_bits(D.d);
#pragma unroll
        for (int m = 0; m < M; m++) {
            // sum_l x*(q-32) = sum_l x*q - 32*sum_l x
            float t = c0 * fmaf(-32.f, sx[m][0], acc[m][0]);
            t = fmaf(c1, fmaf(-32.f, sx[m][1], acc[m][1]), t);
            t = fmaf(c2, fmaf(-32.f, sx[m][2], acc[m][2]), t);
            t = fmaf(c3, fmaf(-32.f, sx[m][3], acc[m][3]), t);
            out[m] = d * t;
        }
    }
};

struct Q80 {
    // 34 B = [f16 d][i8 q[32]]; one unit = one block.
    struct Lane { uint32_t off; };
    struct Data { u32x4 q0, q1; uint32_t d; __device__ __forceinline__ void pin_all() { pin(q0); pin(q1); pin(d); } };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&xo)[4]) {
        L.off = u * 34;
        xo[0] = 32 * u; xo[1] = 32 * u + 8; xo[2] = 32 * u + 16; xo[3] = 32 * u + 24;
    }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L) {
        Data d;
        d.d = *(const uint16_t*)(row + L.off);
        d.q0 = ((const U4A2*)(row + L.off + 2))->v;
        d.q1 = ((const U4A2*)(row + L.off + 18))->v;
        return d;
    }
    template <int M>
    static __device__ __forceinline__ void dot(const Data& D, const Lane&, const float (&x)[M][32], const float (&)[M][4],
                                               float (&out)[M]) {
        float acc[M];
#pragma unroll
        for (int m = 0; m < M; m++) acc[m] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t w = i < 4 ? D.q0[i] : D.q1[i - 4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float f = sb(w, k);
#pragma unroll
                for (int m = 0; m < M; m++) acc[m] = fmaf(x[m][4 * i + k], f, acc[m]);
            }
        }
        float d = f16_bits(D.d);
        // per block: part = sum x*q, then part*d -- crates/ferric-tensor/src/cpu_simd.rs:66-70
#pragma unroll
        for (int m = 0; m < M; m++) out[m] = acc[m] * d;
    }
};

// The four 32-value formats: [f16 d][f16 m]?[u32 qh]?[u8 qs[16]], one unit = one block; value i < 16 is the low nibble
// of qs[i], value 16 + i the high one, the fifth bit of value v is bit v of qh (crates/ferric-gguf/src/lib.rs:618-684).
//   Q4_0 (n - 8) d      Q4_1 n d + m      Q5_0 ((n | b<<4) - 16) d      Q5_1 (n | b<<4) d + m
template <int BYTES, bool HAS_M, bool HAS_QH, int OFF>
struct Legacy {
    static constexpr int QH = HAS_M ? 4 : 2, QS = QH + (HAS_QH ? 4 : 0);
    struct Lane { uint32_t off; };
    struct Data { u32x4 q; uint32_t dm, qh; __device__ __forceinline__ void pin_all() { pin(q); pin(dm); pin(qh); } };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&xo)[4]) {
        L.off = u * BYTES;
        xo[0] = 32 * u; xo[1] = 32 * u + 8; xo[2] = 32 * u + 16; xo[3] = 32 * u + 24;
    }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L) {
        Data d;
        const uint16_t* h = (const uint16_t*)(row + L.off);
        d.dm = HAS_M ? ((uint32_t)h[0] | ((uint32_t)h[1] << 16)) : (uint32_t)h[0];
        d.qh = HAS_QH ? ((uint32_t)h[QH / 2] | ((uint32_t)h[QH / 2 + 1] << 16)) : 0u;
        d.q = ((const U4A2*)(row + L.off + QS))->v;
        return d;
    }
    template <int M>
    static __device__ __forceinline__ void dot(const Data& D, const Lane&, const float (&x)[M][32], const float (&sx)[M][4],
                                               float (&out)[M]) {
        float acc[M];
#pragma unroll
        for (int m = 0; m < M; m++) acc[m] = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t lo = D.q[i] & 0x0F0F0F0Fu, hi = (D.q[i] >> 4) & 0x0F0F0F0Fu;
            if (HAS_QH) {   // bit j of a 4-bit field -> bit 4 of byte j
                lo |= ((((D.qh >> (4 * i)) & 0xFu) * 0x00204081u) & 0x01010101u) << 4;
                hi |= ((((D.qh >> (16 + 4 * i)) & 0xFu) * 0x00204081u) & 0x01010101u) << 4;
            }
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float fl = ub(lo, k), fh = ub(hi, k);
#pragma unroll
                for (int m = 0; m < M; m++) {
                    acc[m] = fmaf(x[m][4 * i + k], fl, acc[m]);
                    acc[m] = fmaf(x[m][16 + 4 * i + k], fh, acc[m]);
                }
            }
        }
        const float d = f16_bits(D.dm & 0xFFFFu), mn = HAS_M ? f16_bits(D.dm >> 16) : 0.f;
#pragma unroll
        for (int m = 0; m < M; m++) {
            const float s = (sx[m][0] + sx[m][1]) + (sx[m][2] + sx[m][3]);
            // sum x (q - OFF) d + m sum x
            out[m] = fmaf(d, fmaf(-(float)OFF, s, acc[m]), mn * s);
        }
    }
};
typedef Legacy<18, false, false, 8> Q40;
typedef Legacy<20, true, false, 0> Q41;
typedef Legacy<22, false, true, 16> Q50;
typedef Legacy<24, true, true, 0> Q51;

struct Q5K {
    // 176 B = [f16 d][f16 dmin][12 B packed 6-bit scales/mins][32 B high bits][128 B nibbles]: Q4_K plus bit s of qh[l] as
    // the fifth bit of element l of sub-block s (crates/ferric-gguf/src/lib.rs:692-716); every piece 16-byte aligned.
    struct Lane { uint32_t off_h, off_q, off_b, sh, g2; bool high; };
    struct Data { u32x4 h, q, b; __device__ __forceinline__ void pin_all() { pin(h); pin(q); pin(b); } };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&xo)[4]) {
        int b = u >> 3, p = u & 7, g = p >> 1, hf = p & 1;
        L.off_h = b * 176;
        L.off_b = b * 176 + 16 + 16 * hf;   // qh[16hf, 16hf+16)
        L.off_q = b * 176 + 48 + 16 * p;    // qs[16p, 16p+16): group g, l in [16hf, 16hf+16)
        L.sh = 16 * (g & 1);
        L.g2 = 2 * g;
        L.high = g >= 2;
        int base = 256 * b + 64 * g + 16 * hf;
        xo[0] = base; xo[1] = base + 8; xo[2] = base + 32; xo[3] = base + 40;  // sub-block 2g, then 2g+1
    }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L) {
        Data d;
        d.h = *(const u32x4*)(row + L.off_h);
        d.q = *(const u32x4*)(row + L.off_q);
        d.b = *(const u32x4*)(row + L.off_b);
        return d;
    }
    template <int M>
    static __device__ __forceinline__ void dot(const Data& D, const Lane& L, const float (&x)[M][32], const float (&sx)[M][4],
                                               float (&out)[M]) {
        uint32_t a = D.h[1] >> L.sh, b = D.h[2] >> L.sh, c = D.h[3] >> L.sh;
        uint32_t scp = L.high ? ((c & 0x0F0Fu) | ((a >> 2) & 0x3030u)) : (a & 0x3F3Fu);
        uint32_t mp = L.high ? (((c >> 4) & 0x0F0Fu) | ((b >> 2) & 0x3030u)) : (b & 0x3F3Fu);
        float d = f16_bits(D.h[0] & 0xFFFFu), dmin = f16_bits(D.h[0] >> 16);
        float d0 = d * ub(scp, 0), d1 = d * ub(scp, 1);
        float m0 = dmin * ub(mp, 0), m1 = dmin * ub(mp, 1);
        float lo[M], hi[M];
#pragma unroll
        for (int m = 0; m < M; m++) { lo[m] = 0.f; hi[m] = 0.f; }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t hb = D.b[i] >> L.g2;
            uint32_t ql = (D.q[i] & 0x0F0F0F0Fu) | ((hb & 0x01010101u) << 4);
            uint32_t qh = ((D.q[i] >> 4) & 0x0F0F0F0Fu) | ((hb & 0x02020202u) << 3);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float fl = ub(ql, k), fh = ub(qh, k);
#pragma unroll
                for (int m = 0; m < M; m++) {
                    lo[m] = fmaf(x[m][4 * i + k], fl, lo[m]);
                    hi[m] = fmaf(x[m][16 + 4 * i + k], fh, hi[m]);
                }
            }
        }
#pragma unroll
        for (int m = 0; m < M; m++)
            out[m] = d0 * lo[m] - m0 * (sx[m][0] + sx[m][1]) + (d1 * hi[m] - m1 * (sx[m][2] + sx[m][3]));
    }
};

// Four 4-bit indices (one per byte of idx, the upper nibbles clear) looked up in a 16-entry byte table held in t0..t3.
__device__ __forceinline__ uint32_t lut16x4(uint32_t idx, uint32_t t0, uint32_t t1, uint32_t t2, uint32_t t3) {
    uint32_t sel = idx & 0x07070707u;
    uint32_t lo = __builtin_amdgcn_perm(t1, t0, sel);   // selector 0..3: bytes of t0, 4..7: bytes of t1
    uint32_t hi = __builtin_amdgcn_perm(t3, t2, sel);
    uint32_t m = ((idx >> 3) & 0x01010101u) * 0xFFu;
    return (hi & m) | (lo & ~m);
}
struct __attribute__((packed, aligned(8))) U4A8 { u32x4 v; };
struct __attribute__((packed, aligned(1))) U4A1 { u32x4 v; };

// IQ4_NL (18 B = [f16 d][qs[16]]) and IQ4_XS (136 B = [f16 d][u16 scales_h][scales_l[4]][qs[128]]): 4-bit indices into the
// codebook {-127 .. 113} (crates/ferric-gguf/src/lib.rs:751-791); one unit = one 32-value (sub-)block, element j the low
// nibble of its qs[j], element 16 + j the high one. The table is held biased by +128 so that a lookup result converts as an
// unsigned byte; the bias leaves as 128 * sum(x): out = dl * (sum x (kv + 128) - 128 sum x), dl = d or d * (ls - 32).
template <bool XS>
struct IQ4 {
    struct Lane { uint32_t off_h, off_q, ib; };
    struct Data { u32x4 q; uint32_t h0, h1; __device__ __forceinline__ void pin_all() { pin(q); pin(h0); pin(h1); } };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&xo)[4]) {
        if (XS) { L.ib = u & 7; L.off_h = (u >> 3) * 136; L.off_q = L.off_h + 8 + 16 * L.ib; }
        else { L.ib = 0; L.off_h = u * 18; L.off_q = L.off_h + 2; }
        xo[0] = 32 * u; xo[1] = 32 * u + 8; xo[2] = 32 * u + 16; xo[3] = 32 * u + 24;
    }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L) {
        Data d;
        if (XS) {
            d.h0 = *(const uint32_t*)(row + L.off_h);
            d.h1 = *(const uint32_t*)(row + L.off_h + 4);
            d.q = ((const U4A8*)(row + L.off_q))->v;
        } else {
            d.h0 = *(const uint16_t*)(row + L.off_h);
            d.h1 = 0;
            d.q = ((const U4A2*)(row + L.off_q))->v;
        }
        return d;
    }
    template <int M>
    static __device__ __forceinline__ void dot(const Data& D, const Lane& L, const float (&x)[M][32], const float (&sx)[M][4],
                                               float (&out)[M]) {
        float acc[M];
#pragma unroll
        for (int m = 0; m < M; m++) acc[m] = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t lo = lut16x4(D.q[i] & 0x0F0F0F0Fu, 0x3F2D1801u, 0x766A5D4Fu, 0xA6998D81u, 0xF1D9C5B5u);
            uint32_t hi = lut16x4((D.q[i] >> 4) & 0x0F0F0F0Fu, 0x3F2D1801u, 0x766A5D4Fu, 0xA6998D81u, 0xF1D9C5B5u);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float fl = ub(lo, k), fh = ub(hi, k);
#pragma unroll
                for (int m = 0; m < M; m++) {
                    acc[m] = fmaf(x[m][4 * i + k], fl, acc[m]);
                    acc[m] = fmaf(x[m][16 + 4 * i + k], fh, acc[m]);
                }
            }
        }
        float dl = f16_bits(D.h0 & 0xFFFFu);
        if (XS) {
            int ls = (int)(((D.h1 >> (4 * L.ib)) & 0xFu) | ((((D.h0 >> 16) >> (2 * L.ib)) & 3u) << 4));
            dl *= (float)(ls - 32);
        }
#pragma unroll
        for (int m = 0; m < M; m++) {
            const float s = (sx[m][0] + sx[m][1]) + (sx[m][2] + sx[m][3]);
            out[m] = dl * fmaf(-128.f, s, acc[m]);
        }
    }
};
typedef IQ4<false> IQ4NL;
typedef IQ4<true> IQ4XS;

// MXFP4 (17 B = [u8 e][qs[16]], crates/ferric-gguf/src/lib.rs:857-908): weight = (2 * E2M1[code]) * 2^(e - 128), formed BEFORE
// it meets the activation as the reference's kernel does (crates/ferric-tensor/src/dtype.rs:3331-3344): a block whose scale
// saturates contributes inf whatever x is. Magnitudes {0,1,2,3,4,6,8,12} by byte permute on the low three bits of a code, the
// fourth bit is the sign. Blocks have no alignment; the hardware's unaligned global loads take them.
struct MXF4 {
    struct Lane { uint32_t off; };
    struct Data { u32x4 q; uint32_t e; __device__ __forceinline__ void pin_all() { pin(q); pin(e); } };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&xo)[4]) {
        L.off = u * 17;
        xo[0] = 32 * u; xo[1] = 32 * u + 8; xo[2] = 32 * u + 16; xo[3] = 32 * u + 24;
    }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L) {
        Data d;
        d.e = row[L.off];
        d.q = ((const U4A1*)(row + L.off + 1))->v;
        return d;
    }
    template <int M>
    static __device__ __forceinline__ void dot(const Data& D, const Lane&, const float (&x)[M][32], const float (&)[M][4],
                                               float (&out)[M]) {
        const float d = __uint_as_float(D.e == 0 ? (1u << 21) : D.e == 1 ? (1u << 22) : (D.e - 1u) << 23);
        float acc[M];
#pragma unroll
        for (int m = 0; m < M; m++) acc[m] = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t q = D.q[i];
            uint32_t lo = __builtin_amdgcn_perm(0x0C080604u, 0x03020100u, q & 0x07070707u);
            uint32_t hi = __builtin_amdgcn_perm(0x0C080604u, 0x03020100u, (q >> 4) & 0x07070707u);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float wl = __uint_as_float(__float_as_uint(ub(lo, k) * d) | ((q << (28 - 8 * k)) & 0x80000000u));
                float wh = __uint_as_float(__float_as_uint(ub(hi, k) * d) | ((q << (24 - 8 * k)) & 0x80000000u));
#pragma unroll
                for (int m = 0; m < M; m++) {
                    acc[m] = fmaf(x[m][4 * i + k], wl, acc[m]);
                    acc[m] = fmaf(x[m][16 + 4 * i + k], wh, acc[m]);
                }
            }
        }
#pragma unroll
        for (int m = 0; m < M; m++) out[m] = acc[m];
    }
};

struct GemvParams {
    const uint8_t* W;
    const float* x;      // [M, cols]
    float* y;            // [M, out_rows]
    int out_rows;        // rows of y (n_ff when fused SwiGLU)
    int cols;
    size_t row_bytes;
    size_t pair_bytes;   // fused SwiGLU: byte distance from gate row r to up row r (= n_ff * row_bytes)
    int S, G, rpg;       // waves per row, row groups per workgroup, output rows per row group
    int stage;           // 1: x staged through LDS once per workgroup
    fhip::SelParams sel; // expert selection (selw == nullptr: none)
};

// Threads per workgroup allowed for M activation rows: the 32*M resident activation registers per
// lane must fit the VGPR budget the launch bound implies (1024 threads -> 128, 768 -> 168, 512 -> 256).
constexpr int max_threads(int M) { return M == 1 ? 1024 : M == 2 ? 768 : 512; }
// Rows in flight per wave: 4 at batch 1, 2 when the batch already fills the register file.
constexpr int rows_in_flight(int M) { return M == 1 ? 4 : 2; }

template <class F, int M, int U, bool SWIGLU>
__global__ void __launch_bounds__(max_threads(M)) gemv_kernel(GemvParams p) {
    extern __shared__ float smem[];
    fhip::apply_selection(p);
    constexpr int VPR = SWIGLU ? 2 : 1;  // weight rows walked per output row
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps row pointers and loop control scalar
    const int ks = wave % p.S, rg = wave / p.S;
    float* part = smem + (p.stage ? M * p.cols : 0);  // [G][rpg*VPR][S][M]

    const int units = p.cols >> 5;
    const int u = ks * 64 + lane;
    const bool valid = u < units;
    typename F::Lane L;
    int xo[4];
    F::setup(valid ? u : 0, L, xo);

    // ---- activations: 32 columns per lane, resident in registers for the life of the wave
    float x[M][32], sx[M][4];
    if (p.stage) {
        for (int i = tid * 4; i < M * p.cols; i += blockDim.x * 4) *(float4*)(smem + i) = *(const float4*)(p.x + i);
        __syncthreads();
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float4 a = *(const float4*)(smem + m * p.cols + xo[j]), b = *(const float4*)(smem + m * p.cols + xo[j] + 4);
                x[m][8 * j + 0] = a.x; x[m][8 * j + 1] = a.y; x[m][8 * j + 2] = a.z; x[m][8 * j + 3] = a.w;
                x[m][8 * j + 4] = b.x; x[m][8 * j + 5] = b.y; x[m][8 * j + 6] = b.z; x[m][8 * j + 7] = b.w;
            }
    } else {
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float4 a = *(const float4*)(p.x + (size_t)m * p.cols + xo[j]), b = *(const float4*)(p.x + (size_t)m * p.cols + xo[j] + 4);
                x[m][8 * j + 0] = a.x; x[m][8 * j + 1] = a.y; x[m][8 * j + 2] = a.z; x[m][8 * j + 3] = a.w;
                x[m][8 * j + 4] = b.x; x[m][8 * j + 5] = b.y; x[m][8 * j + 6] = b.z; x[m][8 * j + 7] = b.w;
            }
    }
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) s += x[m][8 * j + i];
            sx[m][j] = s;
        }

    // ---- stream the rows of this row group: virtual row v -> weight row r0 + v/VPR (+ pair for odd v)
    const int r0 = (blockIdx.x * p.G + rg) * p.rpg;
    int nrows = p.out_rows - r0;
    nrows = nrows < 0 ? 0 : (nrows > p.rpg ? p.rpg : nrows);
    const int nv = nrows * VPR;
    const uint8_t* base = p.W + (size_t)r0 * p.row_bytes;
    auto row_ptr = [&](int v) -> const uint8_t* {
        return SWIGLU ? base + (size_t)(v >> 1) * p.row_bytes + (size_t)(v & 1) * p.pair_bytes : base + (size_t)v * p.row_bytes;
    };
    float* mypart = part + ((size_t)rg * p.rpg * VPR * p.S + ks) * M;

    typename F::Data buf[U];
#pragma unroll
    for (int j = 0; j < U; j++)
        if (j < nv) buf[j] = F::load(row_ptr(j), L);
#pragma unroll 1
    for (int v = 0; v < nv; v += U) {
#pragma unroll
        for (int j = 0; j < U; j++) {
            if (v + j < nv) {
                typename F::Data cur = buf[j];
                if (v + j + U < nv) buf[j] = F::load(row_ptr(v + j + U), L);
                cur.pin_all();
                float acc[M];
                F::template dot<M>(cur, L, x, sx, acc);
#pragma unroll
                for (int m = 0; m < M; m++) {
                    float t = wave_sum_to_lane63(valid ? acc[m] : 0.f);
                    if (lane == 63) mypart[(size_t)(v + j) * p.S * M + m] = t;
                }
            }
        }
    }
    __syncthreads();

    // ---- combine the S partials of each output in a fixed order, apply SwiGLU, store
    const int per_wg = p.G * p.rpg;
    for (int i = tid; i < per_wg * M; i += blockDim.x) {
        int m = i / per_wg, rr = i % per_wg;  // consecutive threads -> consecutive output rows
        int g = rr / p.rpg, rl = rr % p.rpg;
        int r = (blockIdx.x * p.G + g) * p.rpg + rl;
        if (r >= p.out_rows) continue;
        const float* q = part + (((size_t)g * p.rpg + rl) * VPR * p.S) * M + m;
        float a = 0.f;
        for (int s = 0; s < p.S; s++) a += q[s * M];
        if (SWIGLU) {
            float b = 0.f;
            for (int s = 0; s < p.S; s++) b += q[(p.S + s) * M];
            // silu(g) * u, crates/ferric-tensor/src/dtype.rs:2408
            a = (a / (1.0f + expf(-a))) * b;
        }
        if (p.sel.relu2) { a = fmaxf(a, 0.f); a *= a; }   // max(v, 0)^2, crates/ferric-tensor/src/dtype.rs:3755-3756
        p.y[(size_t)m * p.out_rows + r] = a;
    }
}

template <class F, int M, bool SWIGLU>
int launch_one(const fhip_weight* w, const float* d_x, float* d_y, size_t out_rows, hipStream_t s, const fhip::SelParams* sel = nullptr) {
    GemvParams p;
    p.W = w->d_raw; p.x = d_x; p.y = d_y;
    p.out_rows = (int)out_rows; p.cols = (int)w->cols; p.row_bytes = w->row_bytes;
    p.pair_bytes = SWIGLU ? out_rows * w->row_bytes : 0;
    p.sel = sel ? *sel : fhip::SelParams{nullptr, 0, 0, 0, 0, 0, 1, 0};
    const int units = (int)(w->cols / 32);
    p.S = (units + 63) / 64;
    constexpr int MAXW = max_threads(M) / 64;
    if (p.S > MAXW) return fhip::set_error(FHIP_ERR_SHAPE, "matmul_q: cols %zu exceeds the %d this kernel covers", w->cols, MAXW * 2048);
    // Row groups per workgroup: fill the workgroup with waves.
    int G = MAXW / p.S;
    if (G < 1) G = 1;
    while (G > 1 && p.S * G > MAXW) G--;
    p.stage = (size_t)M * w->cols * 4 <= 48 * 1024 ? 1 : 0;
    p.G = G;
    // Rows per row group: enough workgroups to spread over every CU several times, but at least a
    // few rows per wave so the one-time activation load is amortised.
    int cus = fhip::device_cus() > 0 ? fhip::device_cus() : 256;
    if (p.sel.npairs > 1) cus = cus / p.sel.npairs > 0 ? cus / p.sel.npairs : 1;   // the pairs of an "_id" launch share the chip
    int rpg = (int)((out_rows + (size_t)cus * G - 1) / ((size_t)cus * G));
    if (rpg > 32) rpg = 32;
    if (rpg < 1) rpg = 1;
    p.rpg = rpg;
    const size_t per_wg = (size_t)G * rpg;
    const size_t grid = (out_rows + per_wg - 1) / per_wg;
    const size_t lds = ((p.stage ? (size_t)M * w->cols : 0) + per_wg * (SWIGLU ? 2 : 1) * p.S * M) * sizeof(float);
    if (lds > 64 * 1024) return fhip::set_error(FHIP_ERR_SHAPE, "matmul_q: LDS budget exceeded (%zu B)", lds);
    dim3 block(64 * p.S * G);
    constexpr int U = rows_in_flight(M);
    const dim3 g3 = fhip::sel_grid((unsigned)grid, p.sel);
    hipLaunchKernelGGL((gemv_kernel<F, M, U, SWIGLU>), g3, block, lds, s, p);
    return fhip::check_hip(hipGetLastError(), "gemv launch");
}

template <class F, bool SWIGLU>
int launch_fmt(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, size_t out_rows, hipStream_t s) {
    size_t m0 = 0;
    while (m0 < rows_x) {
        size_t left = rows_x - m0;
        const float* x = d_x + m0 * w->cols;
        float* y = d_y + m0 * out_rows;
        int rc;
        const size_t waves_per_row = (w->cols / 32 + 63) / 64;
        if (left >= 4 && waves_per_row * 64 <= (size_t)max_threads(4)) { rc = launch_one<F, 4, SWIGLU>(w, x, y, out_rows, s); m0 += 4; }
        else if (left >= 2 && waves_per_row * 64 <= (size_t)max_threads(2)) { rc = launch_one<F, 2, SWIGLU>(w, x, y, out_rows, s); m0 += 2; }
        else { rc = launch_one<F, 1, SWIGLU>(w, x, y, out_rows, s); m0 += 1; }
        if (rc != FHIP_OK) return rc;
    }
    return FHIP_OK;
}

}  // namespace

namespace fhip {

int launch_gemv_generic(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, size_t n_ff, hipStream_t s) {
    const size_t out_rows = n_ff ? n_ff : w->rows;
    // y is [rows_x, out_rows]: a batch slice starting at m0 is contiguous, so slicing by pointer is exact.
    switch (w->type) {
        case FHIP_Q4_K: return n_ff ? launch_fmt<Q4K, true>(w, d_x, rows_x, d_y, out_rows, s) : launch_fmt<Q4K, false>(w, d_x, rows_x, d_y, out_rows, s);
        case FHIP_Q6_K: return n_ff ? launch_fmt<Q6K, true>(w, d_x, rows_x, d_y, out_rows, s) : launch_fmt<Q6K, false>(w, d_x, rows_x, d_y, out_rows, s);
        case FHIP_Q8_0:
            if (n_ff) return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "matmul_q_swiglu: no fused kernel for Q8_0");
            return launch_fmt<Q80, false>(w, d_x, rows_x, d_y, out_rows, s);
        case FHIP_Q5_K: return n_ff ? launch_fmt<Q5K, true>(w, d_x, rows_x, d_y, out_rows, s) : launch_fmt<Q5K, false>(w, d_x, rows_x, d_y, out_rows, s);
        case FHIP_Q4_0: case FHIP_Q4_1: case FHIP_Q5_0: case FHIP_Q5_1: case FHIP_IQ4_NL: case FHIP_IQ4_XS: case FHIP_MXFP4:
            // the reference fuses gate/up + SwiGLU for the K-quants only (crates/ferric-tensor/src/dtype.rs:949-959)
            if (n_ff) return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "matmul_q_swiglu: no fused kernel for ggml type %u", w->type);
            if (w->type == FHIP_Q4_0) return launch_fmt<Q40, false>(w, d_x, rows_x, d_y, out_rows, s);
            if (w->type == FHIP_Q4_1) return launch_fmt<Q41, false>(w, d_x, rows_x, d_y, out_rows, s);
            if (w->type == FHIP_Q5_0) return launch_fmt<Q50, false>(w, d_x, rows_x, d_y, out_rows, s);
            if (w->type == FHIP_Q5_1) return launch_fmt<Q51, false>(w, d_x, rows_x, d_y, out_rows, s);
            if (w->type == FHIP_IQ4_NL) return launch_fmt<IQ4NL, false>(w, d_x, rows_x, d_y, out_rows, s);
            if (w->type == FHIP_IQ4_XS) return launch_fmt<IQ4XS, false>(w, d_x, rows_x, d_y, out_rows, s);
            return launch_fmt<MXF4, false>(w, d_x, rows_x, d_y, out_rows, s);
        default: return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "QMatrix: no native matmul for ggml type %u", w->type);
    }
}

int launch_gemv_generic_sel(const fhip_weight* w, const float* d_x, float* d_y, size_t out_rows, bool swiglu,
                            const SelParams& sel, hipStream_t s) {
    if (sel.npairs == 0 || out_rows == 0) return FHIP_OK;
    switch (w->type) {
        case FHIP_Q4_K: return swiglu ? launch_one<Q4K, 1, true>(w, d_x, d_y, out_rows, s, &sel) : launch_one<Q4K, 1, false>(w, d_x, d_y, out_rows, s, &sel);
        case FHIP_Q6_K: return swiglu ? launch_one<Q6K, 1, true>(w, d_x, d_y, out_rows, s, &sel) : launch_one<Q6K, 1, false>(w, d_x, d_y, out_rows, s, &sel);
        case FHIP_Q8_0: return swiglu ? launch_one<Q80, 1, true>(w, d_x, d_y, out_rows, s, &sel) : launch_one<Q80, 1, false>(w, d_x, d_y, out_rows, s, &sel);
        case FHIP_Q5_K: return swiglu ? launch_one<Q5K, 1, true>(w, d_x, d_y, out_rows, s, &sel) : launch_one<Q5K, 1, false>(w, d_x, d_y, out_rows, s, &sel);
        case FHIP_Q4_0: return swiglu ? launch_one<Q40, 1, true>(w, d_x, d_y, out_rows, s, &sel) : launch_one<Q40, 1, false>(w, d_x, d_y, out_rows, s, &sel);
        case FHIP_Q4_1: return swiglu ? launch_one<Q41, 1, true>(w, d_x, d_y, out_rows, s, &sel) : launch_one<Q41, 1, false>(w, d_x, d_y, out_rows, s, &sel);
        case FHIP_Q5_0: return swiglu ? launch_one<Q50, 1, true>(w, d_x, d_y, out_rows, s, &sel) : launch_one<Q50, 1, false>(w, d_x, d_y, out_rows, s, &sel);
        case FHIP_Q5_1: return swiglu ? launch_one<Q51, 1, true>(w, d_x, d_y, out_rows, s, &sel) : launch_one<Q51, 1, false>(w, d_x, d_y, out_rows, s, &sel);
        case FHIP_IQ4_NL: return swiglu ? launch_one<IQ4NL, 1, true>(w, d_x, d_y, out_rows, s, &sel) : launch_one<IQ4NL, 1, false>(w, d_x, d_y, out_rows, s, &sel);
        case FHIP_IQ4_XS: return swiglu ? launch_one<IQ4XS, 1, true>(w, d_x, d_y, out_rows, s, &sel) : launch_one<IQ4XS, 1, false>(w, d_x, d_y, out_rows, s, &sel);
        case FHIP_MXFP4: return swiglu ? launch_one<MXF4, 1, true>(w, d_x, d_y, out_rows, s, &sel) : launch_one<MXF4, 1, false>(w, d_x, d_y, out_rows, s, &sel);
        default: return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "QMatrix: no native matmul for ggml type %u", w->type);
    }
}

}  // namespace fhip
