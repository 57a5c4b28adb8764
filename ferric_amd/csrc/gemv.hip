// Decode mat-vec (and batch <= 4 per pass) streaming the raw GGUF block bytes once, gfx950.
//
//   y[m, o] = sum_k x[m, k] * dequant(W[o, k])
//
// Replaces the reference's split-K / flat WGSL kernels (crates/ferric-tensor/src/dtype.rs:2995-3051
// Q4_K, :3423-3469 Q6_K, :3473-3529 Q8_0) and the fused gate/up SwiGLU kernels (:2372-2410, :2734-2775);
// the same skeleton takes Q5_K, Q4_0 / Q4_1 / Q5_0 / Q5_1, IQ4_NL / IQ4_XS and MXFP4 (:1049, :1838-1904, :3185-3420)
// as further per-format structs.
//
// Why it looks the way it does. At 8 TB/s a CU gets ~13 weight bytes per clock, i.e. ~23 Q4_K weights,
// while it can issue 64 lane-instructions per clock: under 3 instructions per weight all-in, and in
// practice far fewer, because a wave that spends its cycles issuing cannot keep loads in flight. A plain
// "unpack nibble, convert, f32 multiply-add" loop costs ~4.7. This kernel gets to ~1.4 by
//   * holding the activations as block fixed point: per run of 32 or 16 columns (the format's own
//     sub-block) NP signed byte planes ("balanced digits", each in [-128, 127]) and one f32 scale, so
//     the inner products are v_dot4_i32_i8 -- four weights per instruction and plane, exact integer
//     sums, converted to f32 once per sub-block and from there on accumulated in f32. NP = 2 is a
//     16-bit significand at the run maximum (dot products to ~2e-5 of ||w|| ||x|| / sqrt(K)), NP = 3
//     a 24-bit one (the f32 significand);
//   * taking a Q4_K byte's high nibble where it stands: (w ^ 0x80808080) & 0xF0F0F0F0 is one
//     v_bitop3 and reads, as a signed byte, 16 * (nibble - 8); the 16 goes into the sub-block scale and
//     the 8 into the term that already multiplies the run's sum of activations;
//   * giving a lane 64 weights that share one scale header (two nibble chunks of one Q4_K group, one
//     ql/ql/qh triple of a Q6_K half), so the 6-bit scale decode is paid once per 64 weights;
//   * keeping the lane -> column mapping fixed for the life of a wave, so the activation planes sit in
//     registers (quantised once per workgroup through LDS) and are never re-read;
//   * reducing the rows of a pipeline step together: U rows' lane partials go through one transposing
//     butterfly (11 DPP/select operations for 4 rows instead of 16) and leave in one LDS store.
//
// Tiling. 16 lanes ("slot") cover 16 units = 1024 weights (512 for the 32-value formats) of one row; a row
// is NG slots. Waves 0..NG/4-1 of a row group take 4 consecutive slots of the same row; the NG%4 left-over
// slots go to one tail wave that works on 4 (or 2) rows at once, so no lane idles for K = 5120 or 17408.
// After one barrier the NG partials of a row are added in a fixed order (results do not depend on
// scheduling or on how rows are partitioned over workgroups). Row groups walk contiguous row spans with U
// rows of 16-byte loads in flight per wave; weight loads for the first rows are issued before the
// activations are touched, so the two latencies overlap.
//
// Activations that block fixed point cannot hold (a run with a NaN or an infinity, a run whose largest magnitude is
// above 2^96 or below 2^-100) are marked by a NaN run scale; a lane that owns such a run
// computes its share of every row element by element in f32 from the raw activations and the exactly
// dequantised weights, which is what the reference's CPU path does (crates/ferric-tensor/src/cpu_simd.rs:57-72,
// crates/ferric-gguf/src/lib.rs:497 then a dense dot): NaN stays NaN, inf * w is +-inf, inf * 0 is NaN.
#include "common.hpp"
#include "deq_at.hpp"

#include <hip/hip_fp16.h>

#include <cstddef>
#include <type_traits>

// This file is compiled twice, once per activation precision (FHIP_GEMV_PLANES = 2 and 3); the two copies export their
// launchers under different names and the precision of the weight handle picks between them at every launch. The kernel
// carries the suffix too, so that a profiler's trace says which copy ran.
#ifndef FHIP_GEMV_PLANES
#define FHIP_GEMV_PLANES 2
#endif
#if FHIP_GEMV_PLANES == 2
#define GEMV_EXPORT(name) name##_p2
#else
#define GEMV_EXPORT(name) name##_p3
#endif
#define gemv_stream_kernel GEMV_EXPORT(gemv_stream_kernel)

namespace {

constexpr int NP = FHIP_GEMV_PLANES;   // byte planes per activation run
static_assert(NP == 2 || NP == 3, "two or three activation planes");
// Largest quantised magnitude: every digit at 127; the run's largest activation maps onto it. With two planes the rounding
// of the reciprocal and of the product moves that by at most 0.02, never to the next integer; with three (8.4e6 * 2^-22 = 2)
// the quantiser clamps.
constexpr float QMAX = NP == 2 ? 32639.0f : 8355711.0f;
constexpr float TINY_RUN = 7.888609052210118e-31f;   // 2^-100: below this QMAX / amax leaves the f32 range's comfortable part
constexpr float HUGE_RUN = 7.922816251426434e28f;    // 2^96

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
struct __attribute__((packed, aligned(2))) U4A2 { u32x4 v; };
struct __attribute__((packed, aligned(2))) U2A2 { u32x2 v; };

__device__ __forceinline__ float f16_bits(uint32_t b) { return __half2float(__ushort_as_half((unsigned short)b)); }
__device__ __forceinline__ float ub(uint32_t v, int k) { return (float)((v >> (8 * k)) & 0xFFu); }
__device__ __forceinline__ float sb(uint32_t v, int k) { return (float)(int8_t)((v >> (8 * k)) & 0xFFu); }
__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) { return __builtin_amdgcn_sdot4((int)a, (int)b, c, false); }

// Keeps a prefetched row as the packed dwords that were loaded (otherwise the optimizer unpacks
// bytes as soon as a load returns and carries the unpacked values across the pipeline, which spills).
__device__ __forceinline__ void pin(uint32_t& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void pin(u32x2& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void pin(u32x4& v) { asm volatile("" : "+v"(v)); }

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true); }
constexpr int DPP_XOR1 = 0xB1, DPP_XOR2 = 0x4E, DPP_HALF_MIRROR = 0x141, DPP_MIRROR = 0x140;   // quad_perm [1,0,3,2], [2,3,0,1]; row_*
constexpr int DPP_ROR4 = 0x124, DPP_ROR8 = 0x128;   // rotate within the 16-lane row: lane l reads lane l - 4 / l - 8, so l & 3 is kept
// All-reduce over the 16 lanes of a DPP row.
__device__ __forceinline__ float slot_sum(float v) {
    v += dpp_f<DPP_XOR1>(v);
    v += dpp_f<DPP_XOR2>(v);
    v += dpp_f<DPP_HALF_MIRROR>(v);
    v += dpp_f<DPP_MIRROR>(v);
    return v;
}

// Sums U (<= 4) values over the 16 lanes of a DPP row at once. Afterwards lane l of the row holds the row sum of value
// slot_of(l & 3), with slot_of = {0, 2, 1, 3}: each of the first two butterfly steps halves the number of values a lane
// carries instead of repeating the whole sum for every value.
template <int U>
__device__ __forceinline__ float slot_sum_many(const float (&v)[U], bool bit0, bool bit1) {
    static_assert(U >= 1 && U <= 4, "one to four values");
    if constexpr (U == 1) {   // the same tree of additions as below, so that a row's bits do not depend on U
        float r = v[0] + dpp_f<DPP_XOR1>(v[0]);
        r += dpp_f<DPP_XOR2>(r);
        r += dpp_f<DPP_ROR4>(r);
        r += dpp_f<DPP_ROR8>(r);
        return r;
    }
    float a, b;
    if constexpr (U == 2) {
        a = v[0] + dpp_f<DPP_XOR1>(v[0]);
        b = v[1] + dpp_f<DPP_XOR1>(v[1]);
    } else {
        const float v3 = U == 4 ? v[U - 1] : 0.f;
        const float keep_a = bit0 ? v[2] : v[0], send_a = bit0 ? v[0] : v[2];
        const float keep_b = bit0 ? v3 : v[1], send_b = bit0 ? v[1] : v3;
        a = keep_a + dpp_f<DPP_XOR1>(send_a);
        b = keep_b + dpp_f<DPP_XOR1>(send_b);
    }
    const float keep = bit1 ? b : a, send = bit1 ? a : b;
    float r = keep + dpp_f<DPP_XOR2>(send);   // the quad's sum of this lane's value
    r += dpp_f<DPP_ROR4>(r);                  // the four quads of the row (the mirrors would pair lanes that hold different values)
    r += dpp_f<DPP_ROR8>(r);
    return r;
}
// value index held by lane l (l & 3) after slot_sum_many<U>
template <int U>
__device__ __forceinline__ int slot_of(int l) {
    if constexpr (U == 1) return 0;
    if constexpr (U == 2) return (l >> 1) & 1;
    return ((l & 1) << 1) | ((l >> 1) & 1);
}

// exact integer plane sums -> f32 (one rounding, at most 2^-24 relative)
__device__ __forceinline__ float planes_f32(const int (&a)[NP]) {
    if constexpr (NP == 2) return (float)((a[0] << 8) + a[1]);
    else return fmaf((float)a[0], 65536.0f, (float)((a[1] << 8) + a[NP - 1]));
}

// ------------------------------------------------------------------------------------------------
// Per-format lane work. A unit is WPL weights of one row; RUN is the activation run that shares one
// fixed-point scale (the format's own sub-block length); a lane needs NRUN runs, and run j of the lane is
// columns [run[j] * RUN, run[j] * RUN + RUN) of the row.
//   setup(u)  -> byte offsets of unit u inside a row and the indices of its activation runs
//   load      -> the raw bytes of the unit for one row (16-/8-byte loads, 2-byte aligned where the
//                GGUF layout is)
//   dot<M>    -> the lane's share of the M dot products
// xp[m][j][p][i]: plane p (most significant first), dword i of run j;  xs[m][j]: scale of run j;
// xq[m][j]: scale * (sum of the run's quantised activations), i.e. the sum of x over the run as the planes hold it.
// ------------------------------------------------------------------------------------------------

struct Q4K {
    static constexpr uint32_t TYPE = FHIP_Q4_K;
    static constexpr int WPL = 64, RUN = 32, NRUN = 2, U1 = 2;
    static constexpr bool RR = true, RR_ONE_ROW = true;      // round-robin row dealing of large weights
    struct Lane { uint32_t off_h, off_q, sh, m1, m2, m3; };
    struct Data {
        u32x4 h, q0, q1;
        __device__ __forceinline__ void pin_all() { pin(h); pin(q0); pin(q1); }
    };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&run)[NRUN]) {
        int b = u >> 2, g = u & 3;             // unit = group g of block b: qs[32g, 32g+32)
        L.off_h = b * 144;
        L.off_q = b * 144 + 16 + 32 * g;
        L.sh = 16 * (g & 1);
        // get_sc_min (crates/ferric-gguf/src/lib.rs:795-804) for the byte pair (2g, 2g+1), as masks so both
        // branches are one expression: g < 2 -> s & 63; g >= 2 -> (s' & 15) | ((s >> 6) << 4)
        L.m1 = g >= 2 ? 0u : 0x3F3Fu;
        L.m2 = g >= 2 ? 0x0F0Fu : 0u;
        L.m3 = g >= 2 ? 0x3030u : 0u;
        run[0] = 2 * u;                        // low nibbles  -> sub-block 2g   = columns [64u, 64u+32)
        run[1] = 2 * u + 1;                    // high nibbles -> sub-block 2g+1 = columns [64u+32, 64u+64)
    }
    // the unit that uses run r of a row, and which of that unit's runs it is (the inverse of `run` above)
    static __device__ __forceinline__ void owner(int r, int& u, int& j) { u = r >> 1; j = r & 1; }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L, uint32_t eo) {
        Data d;
        d.h = *(const u32x4*)(row + (L.off_h + eo));
        d.q0 = *(const u32x4*)(row + (L.off_q + eo));
        d.q1 = *(const u32x4*)(row + (L.off_q + eo) + 16);
        return d;
    }
    template <int M>
    static __device__ __forceinline__ void dot(const Data& D, const Lane& L, const uint32_t (&xp)[M][NRUN][NP][RUN / 4],
                                               const float (&xs)[M][NRUN], const float (&xq)[M][NRUN], float (&out)[M]) {
        // 6-bit (scale, min) of sub-blocks 2g and 2g+1, two packed bytes each
        uint32_t a = D.h[1] >> L.sh, b = D.h[2] >> L.sh, c = D.h[3] >> L.sh;
        uint32_t scp = (a & L.m1) | (c & L.m2) | ((a >> 2) & L.m3);
        uint32_t mp = (b & L.m1) | ((c >> 4) & L.m2) | ((b >> 2) & L.m3);
        const float d = f16_bits(D.h[0] & 0xFFFFu), dmin = f16_bits(D.h[0] >> 16);
        const float s0 = ub(scp, 0), s1 = ub(scp, 1), n0 = ub(mp, 0), n1 = ub(mp, 1);
        int acc[M][2][NP];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int p = 0; p < NP; p++) acc[m][j][p] = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t w = i < 4 ? D.q0[i] : D.q1[i - 4];
            const uint32_t lo = w & 0x0F0F0F0Fu;
            const uint32_t hi = (w ^ 0x80808080u) & 0xF0F0F0F0u;   // as signed bytes: 16 * (high nibble - 8)
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int p = 0; p < NP; p++) {
                    acc[m][0][p] = dot4(xp[m][0][p][i], lo, acc[m][0][p]);
                    acc[m][1][p] = dot4(xp[m][1][p][i], hi, acc[m][1][p]);
                }
        }
#pragma unroll
        for (int m = 0; m < M; m++) {
            const float f0 = xs[m][0] * planes_f32(acc[m][0]);
            // sum x * nibble = (sum x * 16 (nibble - 8)) / 16 + 8 sum x
            const float f1 = fmaf(xs[m][1] * 0.0625f, planes_f32(acc[m][1]), 8.0f * xq[m][1]);
            // sum_l x_l (d*sc*q_l - dmin*m) = d * (sc0 f0 + sc1 f1) - dmin * (m0 sum0 + m1 sum1)
            out[m] = d * fmaf(s1, f1, s0 * f0) - dmin * fmaf(n1, xq[m][1], n0 * xq[m][0]);
        }
    }
};

struct Q6K {
    static constexpr uint32_t TYPE = FHIP_Q6_K;
    static constexpr int WPL = 64, RUN = 16, NRUN = 4, U1 = 2;
    // round-robin row dealing: with three planes and two rows in flight its index arithmetic spills 8 registers (the vocabulary head
    // 151936 x 5120 at 24 bits 118.7 -> 122.6 us dealt); with one row in flight it fits (down 5120 x 17408: 17.86 -> 17.39 us)
    static constexpr bool RR = NP == 2, RR_ONE_ROW = true;
    struct Lane { uint32_t off_a, off_h, off_s, off_d, ssh; };
    struct Data {
        u32x4 a, b, h; u32x2 s; uint32_t d;
        __device__ __forceinline__ void pin_all() { pin(a); pin(b); pin(h); pin(s); pin(d); }
    };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&run)[NRUN]) {
        int b = u >> 2, hf = (u >> 1) & 1, t = u & 1;   // unit: l in [16t, 16t+16) of half hf of block b
        L.off_a = b * 210 + 64 * hf + 16 * t;           // ql[l], and ql[l+32] at +32
        L.off_h = b * 210 + 128 + 32 * hf + 16 * t;
        L.off_s = b * 210 + 192 + 8 * hf;
        L.off_d = b * 210 + 208;
        L.ssh = 8 * t;                                  // is = l / 16 = t
#pragma unroll
        for (int g = 0; g < 4; g++) run[g] = 16 * b + 8 * hf + t + 2 * g;   // columns 256b + 128hf + 32g + 16t + [0,16)
    }
    static __device__ __forceinline__ void owner(int r, int& u, int& j) {
        u = ((r >> 4) << 2) | (((r >> 3) & 1) << 1) | (r & 1);
        j = (r >> 1) & 3;
    }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L, uint32_t eo) {
        Data d;
        d.a = ((const U4A2*)(row + (L.off_a + eo)))->v;
        d.b = ((const U4A2*)(row + (L.off_a + eo) + 32))->v;
        d.h = ((const U4A2*)(row + (L.off_h + eo)))->v;
        d.s = ((const U2A2*)(row + (L.off_s + eo)))->v;
        d.d = *(const uint16_t*)(row + (L.off_d + eo));
        return d;
    }
    template <int M>
    static __device__ __forceinline__ void dot(const Data& D, const Lane& L, const uint32_t (&xp)[M][NRUN][NP][RUN / 4],
                                               const float (&xs)[M][NRUN], const float (&xq)[M][NRUN], float (&out)[M]) {
        int acc[M][4][NP];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
                for (int p = 0; p < NP; p++) acc[m][g][p] = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t A = D.a[i], B = D.b[i], H = D.h[i];
            // the four 6-bit quants that share byte l (crates/ferric-gguf/src/lib.rs:733-736), 4 bytes at a time, as 0..63
            uint32_t q[4];
            q[0] = (A & 0x0F0F0F0Fu) | ((H & 0x03030303u) << 4);
            q[1] = (B & 0x0F0F0F0Fu) | ((H & 0x0C0C0C0Cu) << 2);
            q[2] = ((A >> 4) & 0x0F0F0F0Fu) | (H & 0x30303030u);
            q[3] = ((B >> 4) & 0x0F0F0F0Fu) | ((H >> 2) & 0x30303030u);
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int g = 0; g < 4; g++)
#pragma unroll
                    for (int p = 0; p < NP; p++) acc[m][g][p] = dot4(xp[m][g][p][i], q[g], acc[m][g][p]);
        }
        uint32_t s0 = D.s[0] >> L.ssh, s1 = D.s[1] >> L.ssh;  // sc[is], sc[is+2] | sc[is+4], sc[is+6]
        float c[4] = {sb(s0, 0), sb(s0, 2), sb(s1, 0), sb(s1, 2)};
        float d = f16_bits(D.d);
#pragma unroll
        for (int m = 0; m < M; m++) {
            float t = 0.f;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const float f = fmaf(xs[m][g], planes_f32(acc[m][g]), -32.f * xq[m][g]);   // sum x*(q-32) = sum x*q - 32*sum x
                t = fmaf(c[g], f, t);
            }
            out[m] = d * t;
        }
    }
};

struct Q80 {
    static constexpr uint32_t TYPE = FHIP_Q8_0;
    static constexpr int WPL = 32, RUN = 32, NRUN = 1, U1 = 2;   // two rows in flight: 4096 x 4096 6.89 -> 6.57 us against four
    static constexpr bool RR = true, RR_ONE_ROW = true;      // round-robin row dealing of large weights
    struct Lane { uint32_t off; };
    struct Data {
        u32x4 q0, q1; uint32_t d;
        __device__ __forceinline__ void pin_all() { pin(q0); pin(q1); pin(d); }
    };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&run)[NRUN]) {
        L.off = u * 34;
        run[0] = u;
    }
    static __device__ __forceinline__ void owner(int r, int& u, int& j) { u = r; j = 0; }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L, uint32_t eo) {
        Data d;
        d.d = *(const uint16_t*)(row + (L.off + eo));
        d.q0 = ((const U4A2*)(row + (L.off + eo) + 2))->v;
        d.q1 = ((const U4A2*)(row + (L.off + eo) + 18))->v;
        return d;
    }
    template <int M>
    static __device__ __forceinline__ void dot(const Data& D, const Lane&, const uint32_t (&xp)[M][NRUN][NP][RUN / 4],
                                               const float (&xs)[M][NRUN], const float (&)[M][NRUN], float (&out)[M]) {
        int acc[M][NP];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int p = 0; p < NP; p++) acc[m][p] = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t w = i < 4 ? D.q0[i] : D.q1[i - 4];
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int p = 0; p < NP; p++) acc[m][p] = dot4(xp[m][0][p][i], w, acc[m][p]);
        }
        float d = f16_bits(D.d);
        // per block: part = sum x*q, then part*d -- crates/ferric-tensor/src/cpu_simd.rs:66-70
#pragma unroll
        for (int m = 0; m < M; m++) out[m] = (xs[m][0] * planes_f32(acc[m])) * d;
    }
};

// Q5_K: 176 B = [f16 d][f16 dmin][12 B 6-bit scales/mins][qh 32 B][qs 128 B] -- Q4_K plus bit s of qh[l] as the fifth bit of
// element l of sub-block s (crates/ferric-gguf/src/lib.rs:692-716). Unit = group g of block b (sub-blocks 2g, 2g+1): its 32
// quant bytes and the whole 32 bytes of high bits; codes 0..31.
struct Q5K {
    static constexpr uint32_t TYPE = FHIP_Q5_K;
    static constexpr int WPL = 64, RUN = 32, NRUN = 2, U1 = 2;
    static constexpr bool RR = NP == 2, RR_ONE_ROW = NP == 2;   // (three planes: the index arithmetic spills)
    struct Lane { uint32_t off_h, off_q, sh, g2, m1, m2, m3; };
    struct Data {
        u32x4 h, b0, b1, q0, q1;
        __device__ __forceinline__ void pin_all() { pin(h); pin(b0); pin(b1); pin(q0); pin(q1); }
    };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&run)[NRUN]) {
        int b = u >> 2, g = u & 3;
        L.off_h = b * 176;
        L.off_q = b * 176 + 48 + 32 * g;
        L.sh = 16 * (g & 1);
        L.g2 = 2 * g;
        L.m1 = g >= 2 ? 0u : 0x3F3Fu;
        L.m2 = g >= 2 ? 0x0F0Fu : 0u;
        L.m3 = g >= 2 ? 0x3030u : 0u;
        run[0] = 2 * u;
        run[1] = 2 * u + 1;
    }
    static __device__ __forceinline__ void owner(int r, int& u, int& j) { u = r >> 1; j = r & 1; }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L, uint32_t eo) {
        Data d;
        d.h = *(const u32x4*)(row + (L.off_h + eo));
        d.b0 = *(const u32x4*)(row + (L.off_h + eo) + 16);
        d.b1 = *(const u32x4*)(row + (L.off_h + eo) + 32);
        d.q0 = *(const u32x4*)(row + (L.off_q + eo));
        d.q1 = *(const u32x4*)(row + (L.off_q + eo) + 16);
        return d;
    }
    template <int M>
    static __device__ __forceinline__ void dot(const Data& D, const Lane& L, const uint32_t (&xp)[M][NRUN][NP][RUN / 4],
                                               const float (&xs)[M][NRUN], const float (&xq)[M][NRUN], float (&out)[M]) {
        uint32_t a = D.h[1] >> L.sh, b = D.h[2] >> L.sh, c = D.h[3] >> L.sh;
        uint32_t scp = (a & L.m1) | (c & L.m2) | ((a >> 2) & L.m3);
        uint32_t mp = (b & L.m1) | ((c >> 4) & L.m2) | ((b >> 2) & L.m3);
        const float d = f16_bits(D.h[0] & 0xFFFFu), dmin = f16_bits(D.h[0] >> 16);
        const float s0 = ub(scp, 0), s1 = ub(scp, 1), n0 = ub(mp, 0), n1 = ub(mp, 1);
        int acc[M][2][NP];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int p = 0; p < NP; p++) acc[m][j][p] = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t w = i < 4 ? D.q0[i] : D.q1[i - 4];
            uint32_t hb = (i < 4 ? D.b0[i] : D.b1[i - 4]) >> L.g2;      // bit 0: sub-block 2g, bit 1: sub-block 2g+1
            uint32_t lo = (w & 0x0F0F0F0Fu) | ((hb & 0x01010101u) << 4);
            uint32_t hi = ((w >> 4) & 0x0F0F0F0Fu) | ((hb & 0x02020202u) << 3);
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int p = 0; p < NP; p++) {
                    acc[m][0][p] = dot4(xp[m][0][p][i], lo, acc[m][0][p]);
                    acc[m][1][p] = dot4(xp[m][1][p][i], hi, acc[m][1][p]);
                }
        }
#pragma unroll
        for (int m = 0; m < M; m++) {
            const float f0 = xs[m][0] * planes_f32(acc[m][0]);
            const float f1 = xs[m][1] * planes_f32(acc[m][1]);
            out[m] = d * fmaf(s1, f1, s0 * f0) - dmin * fmaf(n1, xq[m][1], n0 * xq[m][0]);
        }
    }
};

// The four 32-value formats, [f16 d][f16 m]?[u32 qh]?[qs 16 B] (crates/ferric-gguf/src/lib.rs:618-684): value i < 16 is the low
// nibble of qs[i], value 16 + i the high one, the fifth bit of value v is bit v of qh; (n - OFF) d or n d + m. Unit = one block;
// the offset leaves as OFF * sum(x), the affine term as m * sum(x).
template <uint32_t TY, int BYTES, bool HAS_M, bool HAS_QH, int OFF>
struct LegS {
    static constexpr uint32_t TYPE = TY;
    static constexpr int WPL = 32, RUN = 32, NRUN = 1, U1 = 4;
    static constexpr bool RR = true, RR_ONE_ROW = true;      // round-robin row dealing of large weights
    static constexpr int QH = HAS_M ? 4 : 2, QS = QH + (HAS_QH ? 4 : 0);
    struct Lane { uint32_t off; };
    struct Data {
        u32x4 q; uint32_t dm, qh;
        __device__ __forceinline__ void pin_all() { pin(q); pin(dm); pin(qh); }
    };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&run)[NRUN]) {
        L.off = u * BYTES;
        run[0] = u;
    }
    static __device__ __forceinline__ void owner(int r, int& u, int& j) { u = r; j = 0; }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L, uint32_t eo) {
        Data d;
        const uint16_t* h = (const uint16_t*)(row + (L.off + eo));
        d.dm = HAS_M ? ((uint32_t)h[0] | ((uint32_t)h[1] << 16)) : (uint32_t)h[0];
        d.qh = HAS_QH ? ((uint32_t)h[QH / 2] | ((uint32_t)h[QH / 2 + 1] << 16)) : 0u;
        d.q = ((const U4A2*)(row + (L.off + eo) + QS))->v;
        return d;
    }
    template <int M>
    static __device__ __forceinline__ void dot(const Data& D, const Lane&, const uint32_t (&xp)[M][NRUN][NP][RUN / 4],
                                               const float (&xs)[M][NRUN], const float (&xq)[M][NRUN], float (&out)[M]) {
        int acc[M][NP];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int p = 0; p < NP; p++) acc[m][p] = 0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint32_t lo = D.q[j] & 0x0F0F0F0Fu, hi = (D.q[j] >> 4) & 0x0F0F0F0Fu;
            if (HAS_QH) {   // bit k of a 4-bit field -> bit 4 of byte k
                lo |= ((((D.qh >> (4 * j)) & 0xFu) * 0x00204081u) & 0x01010101u) << 4;
                hi |= ((((D.qh >> (16 + 4 * j)) & 0xFu) * 0x00204081u) & 0x01010101u) << 4;
            }
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int p = 0; p < NP; p++) {
                    acc[m][p] = dot4(xp[m][0][p][j], lo, acc[m][p]);
                    acc[m][p] = dot4(xp[m][0][p][4 + j], hi, acc[m][p]);
                }
        }
        const float d = f16_bits(D.dm & 0xFFFFu), mn = HAS_M ? f16_bits(D.dm >> 16) : 0.f;
#pragma unroll
        for (int m = 0; m < M; m++)
            out[m] = fmaf(d, fmaf(-(float)OFF, xq[m][0], xs[m][0] * planes_f32(acc[m])), mn * xq[m][0]);
    }
};
typedef LegS<FHIP_Q4_0, 18, false, false, 8> Q40;
typedef LegS<FHIP_Q4_1, 20, true, false, 0> Q41;
typedef LegS<FHIP_Q5_0, 22, false, true, 16> Q50;
typedef LegS<FHIP_Q5_1, 24, true, true, 0> Q51;

// IQ4_NL (18 B = [f16 d][qs 16 B]) and IQ4_XS (136 B = [f16 d][u16 scales_h][scales_l 4 B][qs 128 B]): 4-bit indices into the
// 16-level codebook {-127 .. 113} (crates/ferric-gguf/src/lib.rs:751-791), looked up four at a time by byte permute into int8
// levels. Unit = one 32-value (sub-)block.
__device__ __forceinline__ uint32_t lut16x4(uint32_t idx, uint32_t t0, uint32_t t1, uint32_t t2, uint32_t t3) {
    uint32_t sel = idx & 0x07070707u;
    uint32_t lo = __builtin_amdgcn_perm(t1, t0, sel);   // selector 0..3: bytes of t0, 4..7: bytes of t1
    uint32_t hi = __builtin_amdgcn_perm(t3, t2, sel);
    uint32_t m = ((idx >> 3) & 0x01010101u) * 0xFFu;
    return (hi & m) | (lo & ~m);
}
struct __attribute__((packed, aligned(8))) U4A8 { u32x4 v; };

template <bool XS>
struct IQ4S {
    static constexpr uint32_t TYPE = XS ? FHIP_IQ4_XS : FHIP_IQ4_NL;
    static constexpr int WPL = 32, RUN = 32, NRUN = 1, U1 = 4;
    static constexpr bool RR = true, RR_ONE_ROW = true;      // round-robin row dealing of large weights
    struct Lane { uint32_t off_h, off_q, ib; };
    struct Data {
        u32x4 q; uint32_t h0, h1;
        __device__ __forceinline__ void pin_all() { pin(q); pin(h0); pin(h1); }
    };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&run)[NRUN]) {
        if (XS) { L.ib = u & 7; L.off_h = (u >> 3) * 136; L.off_q = L.off_h + 8 + 16 * L.ib; }
        else { L.ib = 0; L.off_h = u * 18; L.off_q = L.off_h + 2; }
        run[0] = u;
    }
    static __device__ __forceinline__ void owner(int r, int& u, int& j) { u = r; j = 0; }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L, uint32_t eo) {
        Data d;
        if (XS) {
            d.h0 = *(const uint32_t*)(row + (L.off_h + eo));
            d.h1 = *(const uint32_t*)(row + (L.off_h + eo) + 4);
            d.q = ((const U4A8*)(row + (L.off_q + eo)))->v;
        } else {
            d.h0 = *(const uint16_t*)(row + (L.off_h + eo));
            d.h1 = 0;
            d.q = ((const U4A2*)(row + (L.off_q + eo)))->v;
        }
        return d;
    }
    template <int M>
    static __device__ __forceinline__ void dot(const Data& D, const Lane& L, const uint32_t (&xp)[M][NRUN][NP][RUN / 4],
                                               const float (&xs)[M][NRUN], const float (&)[M][NRUN], float (&out)[M]) {
        // the codebook as int8 bytes, four levels per word
        constexpr uint32_t T0 = 0xBFAD9881u, T1 = 0xF6EADDCFu, T2 = 0x26190D01u, T3 = 0x71594535u;
        int acc[M][NP];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int p = 0; p < NP; p++) acc[m][p] = 0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint32_t lo = lut16x4(D.q[j] & 0x0F0F0F0Fu, T0, T1, T2, T3), hi = lut16x4((D.q[j] >> 4) & 0x0F0F0F0Fu, T0, T1, T2, T3);
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int p = 0; p < NP; p++) {
                    acc[m][p] = dot4(xp[m][0][p][j], lo, acc[m][p]);
                    acc[m][p] = dot4(xp[m][0][p][4 + j], hi, acc[m][p]);
                }
        }
        float dl = f16_bits(D.h0 & 0xFFFFu);
        if (XS) {
            int ls = (int)(((D.h1 >> (4 * L.ib)) & 0xFu) | ((((D.h0 >> 16) >> (2 * L.ib)) & 3u) << 4));
            dl *= (float)(ls - 32);
        }
#pragma unroll
        for (int m = 0; m < M; m++) out[m] = (xs[m][0] * planes_f32(acc[m])) * dl;
    }
};
typedef IQ4S<false> IQ4NL;
typedef IQ4S<true> IQ4XS;

// MXFP4 (17 B = [u8 e][qs 16 B], crates/ferric-gguf/src/lib.rs:857-908): weight = k * 2^(e - 128) with k the doubled E2M1 value,
// an integer in {0, +-1, +-2, +-3, +-4, +-6, +-8, +-12}: int8 codes, the power of two applied to the block's integer dot
// product. The reference forms k * scale per element BEFORE it meets the activation
// (crates/ferric-tensor/src/dtype.rs:3331-3344), which only differs where that product overflows (e >= 252): such a block takes
// the element-by-element branch below, on the activations as the planes hold them (zeros stay zeros, so inf * 0 is still NaN).
struct __attribute__((packed, aligned(1))) U4A1 { u32x4 v; };
struct MXF4S {
    static constexpr uint32_t TYPE = FHIP_MXFP4;
    static constexpr int WPL = 32, RUN = 32, NRUN = 1, U1 = 4;
    static constexpr bool RR = true, RR_ONE_ROW = true;      // round-robin row dealing of large weights
    struct Lane { uint32_t off; };
    struct Data {
        u32x4 q; uint32_t e;
        __device__ __forceinline__ void pin_all() { pin(q); pin(e); }
    };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&run)[NRUN]) {
        L.off = u * 17;
        run[0] = u;
    }
    static __device__ __forceinline__ void owner(int r, int& u, int& j) { u = r; j = 0; }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L, uint32_t eo) {
        Data d;
        d.e = row[L.off + eo];
        d.q = ((const U4A1*)(row + (L.off + eo) + 1))->v;
        return d;
    }
    template <int M>
    static __device__ __forceinline__ void dot(const Data& D, const Lane&, const uint32_t (&xp)[M][NRUN][NP][RUN / 4],
                                               const float (&xs)[M][NRUN], const float (&)[M][NRUN], float (&out)[M]) {
        constexpr uint32_t T0 = 0x03020100u, T1 = 0x0C080604u, T2 = 0xFDFEFF00u, T3 = 0xF4F8FAFCu;
        const float d = __uint_as_float(D.e == 0 ? (1u << 21) : D.e == 1 ? (1u << 22) : (D.e - 1u) << 23);
        uint32_t lo[4], hi[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            lo[j] = lut16x4(D.q[j] & 0x0F0F0F0Fu, T0, T1, T2, T3);
            hi[j] = lut16x4((D.q[j] >> 4) & 0x0F0F0F0Fu, T0, T1, T2, T3);
        }
        if (D.e >= 252u) {   // a weight of this block may be +-inf: the reference's per-element products
#pragma unroll 1
            for (int m = 0; m < M; m++) {
                float a = 0.f;
#pragma unroll 1
                for (int el = 0; el < 32; el++) {
                    const int i = el >> 2, sh = 8 * (el & 3);
                    int v = 0;
#pragma unroll
                    for (int p = 0; p < NP; p++) v = v * 256 + (int)(int8_t)(xp[m][0][p][i] >> sh);
                    const uint32_t kw = el < 16 ? lo[el >> 2] : hi[(el - 16) >> 2];
                    const float w = (float)(int)(int8_t)(kw >> sh) * d;
                    a = fmaf(xs[m][0] * (float)v, w, a);
                }
                out[m] = a;
            }
            return;
        }
        int acc[M][NP];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int p = 0; p < NP; p++) acc[m][p] = 0;
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int p = 0; p < NP; p++) {
                    acc[m][p] = dot4(xp[m][0][p][j], lo[j], acc[m][p]);
                    acc[m][p] = dot4(xp[m][0][p][4 + j], hi[j], acc[m][p]);
                }
#pragma unroll
        for (int m = 0; m < M; m++) out[m] = (xs[m][0] * planes_f32(acc[m])) * d;
    }
};

struct GemvParams {
    const uint8_t* W;
    const float* x;      // [M, cols]
    float* y;            // [M, out_rows]
    int out_rows;        // rows of y (n_ff when fused SwiGLU)
    int cols;
    uint32_t row_bytes;  // below 2^32 (rows of at most ~40 000 columns): a row's address is one 32 x 32 -> 64 bit product
    size_t pair_bytes;   // fused SwiGLU: byte distance from gate row r to up row r (= n_ff * row_bytes)
    int NG;              // 16-lane slots per row = ceil(units / 16)
    int units;           // units per row = cols / WPL; the last slot may be partly filled
    int RF;              // replicas of the full-wave set, each taking every RF-th row (balances them against the tail wave)
    int G;               // row groups per workgroup
    int S;               // waves that stage the activations (all of them when the input norm is fused)
    int rpg;             // output rows per row group
    // ceil(2^32 / d) for the three divisors of the kernel's index arithmetic (waves per row group, full waves per row, RF), 0
    // for d = 1: floor(n / d) = mulhi(n, magic) for n < 65 536, 2 <= d <= 1024; a hardware-less integer division costs ~35
    // dependent instructions, and four of them stood in front of the first load
    uint32_t m_rf, m_rpg;
    // What wave w of a workgroup is, worked out by the launcher once instead of by every wave in front of its first load
    // (wave_word): bits 0-3 its row group in the workgroup, 4-7 the first virtual row it takes, 8 set for the tail wave of a
    // row group, 9-10 the slots the tail holds (NG % 4), 11-18 the first slot of its four, 19-20 log2 of the rows a tail wave
    // works on at once. (The table sits here, among the fields every wave loads at its start: at the end of the struct, two
    // cache lines further, its load missed the scalar cache and the launch was 0.14 us slower.)
    uint32_t wtab[16];
    // Dealing of rows to row groups. rr == 0: row group g owns the rpg consecutive rows from g * rpg. rr == 1 (large weights):
    // the rows are dealt in chunks of 4, chunk c to row group c % nrg, so that at any moment the whole chip reads one dense
    // window of the weight that moves through it (measured 3 - 5 % faster than 768 separate streams on the FFN shapes);
    // kfull = rounds in which every row group gets a whole chunk, rem = rows left for the last round.
    int rr, nrg, kfull, rem;
    fhip::SelParams sel; // expert selection (selw == nullptr: none)
    // Fused input norm (norm_w != nullptr; M = 1, cols <= 8 * threads): the activation row is rmsnorm(x [+ resid]) * norm_w,
    // formed by every workgroup while it stages the row; one workgroup also stores x + resid to x_out (never x itself).
    const float* norm_w;
    const float* resid;
    float* x_out;
    float eps;
    uint32_t red_off;    // byte offset in LDS of 64 floats: four partial sums of squares per wave
    int row_wgs;         // workgroups that own rows; the launch may hold one more, which only stores x + resid
};

// Threads per workgroup allowed for M activation rows (register budget: 1024 -> 128 VGPRs, 640 -> 168, 512 -> 256).
// Two Q4_K activation rows fit 168 registers, ten waves (5120 columns: two row groups per workgroup; cold, two rows: 5120 x 5120
// 8.9 -> 8.0 us, fused gate|up 27.7 -> 23.2); Q6_K fits them with one weight row in flight per wave instead of two (156
// registers; with two it spills: 5120 x 17408 at two rows 23.0 us in eight waves, 28.9 in ten with spills, 20.2 in ten with one
// row in flight; 151936 x 5120 133 -> 120).
// (With three activation planes both spill at 168 registers, 152 and 64 bytes a lane: that build keeps eight waves.)
template <class F> constexpr int max_threads(int M) {
    return M == 1 ? 1024 : (NP == 2 && (F::TYPE == FHIP_Q4_K || F::TYPE == FHIP_Q6_K) ? 640 : 512);
}
// Rows in flight per wave, sized so the prefetched rows plus the resident activation planes fit 128 VGPRs
// at batch 1 (16 waves per CU).
template <class F> constexpr int rows_in_flight(int M) { return M == 1 ? F::U1 : (NP == 2 && F::TYPE == FHIP_Q6_K ? 1 : 2); }
// Activation rows one pass can hold in registers.
template <class F> constexpr int max_m() { return F::WPL == 64 ? 2 : 4; }

__device__ __forceinline__ uint32_t div_magic(uint32_t n, uint32_t magic) { return magic ? __umulhi(n, magic) : n; }

// Eight consecutive activations of one run -> NP plane dword pairs, the run's scale and the run's quantised sum.
// The 2 (RUN 16) or 4 (RUN 32) lanes of a run sit in one quad and agree on amax, the scale and the sum afterwards.
template <int RUN>
__device__ __forceinline__ void quantize8(const float (&v)[8], uint32_t (&pl)[NP][2], float& scale_out, float& sum_out) {
    float amax = fmaxf(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))),
                       fmaxf(fmaxf(fabsf(v[4]), fabsf(v[5])), fmaxf(fabsf(v[6]), fabsf(v[7]))));
    float sum = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));   // NaN / inf detector (fmaxf drops NaNs)
    amax = fmaxf(amax, dpp_f<DPP_XOR1>(amax));
    sum += dpp_f<DPP_XOR1>(sum);
    if (RUN == 32) {
        amax = fmaxf(amax, dpp_f<DPP_XOR2>(amax));
        sum += dpp_f<DPP_XOR2>(sum);
    }
    // not representable in block fixed point: non-finite members (their sum is not finite either), a run so large that a
    // format's offset term (up to 128 times the run's sum) could leave the f32 range where the element-wise products do not,
    // or a run so small that QMAX / amax would overflow
    const bool special = !(fabsf(sum) <= 3.4028234663852886e38f) || amax > HUGE_RUN || (amax < TINY_RUN && amax > 0.f);
    const float inv = amax > 0.f ? QMAX * __builtin_amdgcn_rcpf(amax) : 0.f;
    uint32_t t[8];
    if constexpr (NP == 2) {
        // round to nearest by adding 1.5 * 2^23; the 128 makes the low byte an offset-binary digit
#pragma unroll
        for (int i = 0; i < 8; i++) t[i] = __float_as_uint(fmaf(v[i], inv, 12582912.0f + 128.0f));
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            int q = __float2int_rn(v[i] * inv);
            q = q > (int)QMAX ? (int)QMAX : (q < -(int)QMAX ? -(int)QMAX : q);
            t[i] = (uint32_t)(q + 0x8080);
        }
    }
#pragma unroll
    for (int hh = 0; hh < 2; hh++) {
        const uint32_t t0 = t[4 * hh], t1 = t[4 * hh + 1], t2 = t[4 * hh + 2], t3 = t[4 * hh + 3];
        const uint32_t p01 = __builtin_amdgcn_perm(t1, t0, 0x05010400u), p23 = __builtin_amdgcn_perm(t3, t2, 0x05010400u);
        pl[NP - 1][hh] = __builtin_amdgcn_perm(p23, p01, 0x05040100u) ^ 0x80808080u;   // bytes 0, back to signed digits
        if constexpr (NP == 2) {
            pl[0][hh] = __builtin_amdgcn_perm(p23, p01, 0x07060302u);                  // bytes 1: the signed top digit
        } else {
            pl[1][hh] = __builtin_amdgcn_perm(p23, p01, 0x07060302u) ^ 0x80808080u;
            const uint32_t u01 = __builtin_amdgcn_perm(t1, t0, 0x00000602u), u23 = __builtin_amdgcn_perm(t3, t2, 0x00000602u);
            pl[0][hh] = __builtin_amdgcn_perm(u23, u01, 0x05040100u);                  // bytes 2
        }
    }
    int qs[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) qs[p] = dot4(pl[p][1], 0x01010101u, dot4(pl[p][0], 0x01010101u, 0));
    int qsum = qs[0];
#pragma unroll
    for (int p = 1; p < NP; p++) qsum = (qsum << 8) + qs[p];
    qsum += dpp_i<DPP_XOR1>(qsum);
    if (RUN == 32) qsum += dpp_i<DPP_XOR2>(qsum);
    const float scale = amax * (1.0f / QMAX);
    scale_out = special ? __uint_as_float(0x7FC00000u) : scale;
    sum_out = scale * (float)qsum;
}

template <class F, int M, int U, bool SWIGLU, bool NORM, bool LATE>
__global__ void __launch_bounds__(max_threads<F>(M)) gemv_stream_kernel(GemvParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    fhip::apply_selection(p);
    constexpr int VPR = SWIGLU ? 2 : 1;       // weight rows walked per output row
    constexpr int RUN = F::RUN, NRUN = F::NRUN, RD = RUN / 4;
    const int tid = threadIdx.x, lane = tid & 63;
    // The activation loads go out before anything else: they need the thread index only, and the index arithmetic below
    // (a few hundred scalar instructions, which the four waves of a SIMD get through one after the other, oldest first)
    // then runs under their latency instead of in front of it.
    // The activations are staged by the first p.S waves of the workgroup only (the oldest, so the first to be scheduled in
    // every phase): up to four 8-value pieces per thread, all requested here so that they arrive under one memory round
    // trip. The other waves go straight to their weight rows and meet the stagers at the barrier.
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // What this wave is (wtab), wave-uniform: one scalar load straight from the kernel-argument segment (the struct is the kernel's only argument, so
    // its fields lie at their offsets there; indexing the by-value copy with a run-time index would move all of it to scratch)
    typedef const uint32_t __attribute__((address_space(4))) karg_word;
    const uint32_t ww = ((karg_word*)__builtin_amdgcn_kernarg_segment_ptr())[offsetof(GemvParams, wtab) / 4 + wave];
    const bool stager = wave < p.S;
    const int e0 = stager ? tid * 8 : M * p.cols, e_step = p.S * 512;
    // A staging wave asks for its pieces unconditionally, from a clamped address: a piece past the end is loaded from a
    // place inside the row instead and never used (under a condition each piece cost eight register clears and a branch
    // in front of the wave's first weight request). A wave that does not stage skips them in one branch and leaves the
    // registers as they are: nothing reads them (every wave re-reading the one last line: 5120 x 5120 5.37 -> 5.94 us).
    constexpr bool fused_norm = NORM && M == 1;   // a separate instantiation: the plain kernel carries none of this
    constexpr int XR = 3;
    float4 xa0, xb0, xar[XR], xbr[XR];
    if (stager) {
        const int e_last = M * p.cols - 8, e_own = e0 < e_last ? e0 : e_last;
        // (a later piece past the end re-reads the thread's own first piece, not the row's last: many threads on one line wait)
        auto piece = [&](int e) { return p.x + (e <= e_last ? e : e_own); };
        xa0 = *(const float4*)(p.x + e_own); xb0 = *(const float4*)(p.x + e_own + 4);
        if constexpr (!fused_norm) {               // under the fused norm a thread holds at most one piece of the row
#pragma unroll
            for (int k = 0; k < XR; k++) {
                const float* src = piece(e0 + (k + 1) * e_step);
                xar[k] = *(const float4*)src; xbr[k] = *(const float4*)(src + 4);
            }
        }
    }
    float4 nwa = {1, 1, 1, 1}, nwb = {1, 1, 1, 1}, rsa = {0, 0, 0, 0}, rsb = {0, 0, 0, 0};
    if (fused_norm && e0 < p.cols) {              // the norm's weights and the residual ride with the activations
        nwa = *(const float4*)(p.norm_w + e0); nwb = *(const float4*)(p.norm_w + e0 + 4);
        if (p.resid) { rsa = *(const float4*)(p.resid + e0); rsb = *(const float4*)(p.resid + e0 + 4); }
    }
    asm volatile("" ::: "memory");   // keeps the loads here
    if (fused_norm && (int)blockIdx.x >= p.row_wgs) {
        // A workgroup past the ones that own rows, launched when a CU is free for it: it stores x + resid and is done. Stored
        // by a workgroup that streams rows, the sum costs that workgroup the store's acknowledgement (1.4 us measured on the
        // gate|up shape): its later waits for weight rows count the store too.
        if (p.x_out && e0 < p.cols) {
            xa0.x += rsa.x; xa0.y += rsa.y; xa0.z += rsa.z; xa0.w += rsa.w;
            xb0.x += rsb.x; xb0.y += rsb.y; xb0.z += rsb.z; xb0.w += rsb.w;
            *(float4*)(p.x_out + e0) = xa0; *(float4*)(p.x_out + e0 + 4) = xb0;
        }
        return;
    }
    const int rg = (int)(ww & 15u);                       // row group within the workgroup
    const bool tail = ((ww >> 8) & 1u) != 0;
    const int NT = (int)((ww >> 9) & 3u), gbase = (int)((ww >> 11) & 255u);
    const int RTL = (int)((ww >> 19) & 3u);               // log2 of the rows this wave works on at once (0 unless tail)
    const int RT = 1 << RTL;
    // iteration i of this wave works on virtual row v_start + i * v_step (+ row_off per lane in a tail wave)
    const int v_start = (int)((ww >> 4) & 15u), v_step = tail ? RT : p.RF;

    // LDS: activation planes | scales [M][NRUN][units] | sums [M][NRUN][units] | partials. The planes are laid out for the
    // readers: the 16-byte piece c of plane pp of run j of unit u (of activation row m) sits at
    // ((((m NRUN + j) NP + pp) RD/4 + c) units + u) * 16, so the lanes of a wave (consecutive units) read consecutive pieces
    // and a 16-byte read of 64 lanes touches every bank once (run-major storage put the lanes 128 bytes apart: 8 banks).
    const int nrun = p.cols / RUN;
    constexpr int RC = RD / 4;                           // 16-byte pieces per plane of a run
    uint8_t* planes = smem;
    float* scales = (float*)(smem + (size_t)M * p.cols * NP);
    float* sums = scales + (size_t)M * nrun;
    float* part = sums + (size_t)M * nrun;               // [G][rpg*VPR][NG][M]

    // ---- which unit of which row this lane works on
    const int slot = lane >> 4, l16 = lane & 15;
    int group, row_off;
    bool lane_ok = true;
    if (!tail) { group = gbase + slot; row_off = 0; }
    else if (NT == 3) { lane_ok = slot < 3; group = gbase + (lane_ok ? slot : 0); row_off = 0; }
    else { group = gbase + (NT == 2 ? (slot & 1) : 0); row_off = NT == 2 ? (slot >> 1) : slot; }
    typename F::Lane L;
    int run[NRUN];
    // a lane past the row's last unit (rows whose length does not fill the last slot) works on unit 0 and contributes 0
    const bool unit_ok = group * 16 + l16 < p.units;
    const int my_unit = unit_ok ? group * 16 + l16 : 0;
    F::setup(my_unit, L, run);

    const bool dealt = (F::RR || (F::RR_ONE_ROW && U == 1)) && p.rr != 0;   // rows dealt round-robin in chunks of 4
    // Dealt, the row groups are numbered across the workgroups (row group rg of workgroup b is number rg * row_wgs + b): the chunks
    // of a last, partly filled round then go to the workgroups in turn. Numbered b * G + rg, the first workgroups got a chunk more
    // in every one of their row groups and the last ones none (fused gate|up 34816 x 5120, two row groups a workgroup: 72 rows
    // in workgroups 0 - 127, 64 in the others, whose row loops ended 1.3 us sooner).
    const int rgid = dealt ? rg * p.row_wgs + (int)blockIdx.x : (int)blockIdx.x * p.G + rg;
    // Address of iteration `it`: a wave-uniform row base (scalar registers) plus a 32-bit lane offset. A tail
    // wave's lanes sit row_off rows further (v_start + it*v_step is a multiple of RT there, so with fused
    // SwiGLU the gate/up split of row_off is fixed); lanes past the last row read the uniform row instead
    // and are masked when the partial is written.
    const uint32_t lane_extra = SWIGLU ? (uint32_t)((size_t)(row_off >> 1) * p.row_bytes + (size_t)(row_off & 1) * p.pair_bytes)
                                       : (uint32_t)((size_t)row_off * p.row_bytes);
    // row l of the row group is row l of its span, or, dealt (rr): row l % 4 of the row group's chunk l / 4, which is chunk
    // (l / 4) * nrg + rgid of the weight. A tail wave's RT rows start at a multiple of RT <= 4, so they lie in one chunk and
    // lane_extra holds as it stands.
    auto weight_row = [&](int l) { return dealt ? ((((l >> 2) * p.nrg + rgid) << 2) + (l & 3)) : rgid * p.rpg + l; };

    // ---- The activation loads went out first; now the weight bytes of the wave's first row, UNCONDITIONALLY and from an
    // address that needs as little arithmetic as possible: the row the wave would start on, clamped to the weight's last
    // row (a wave or a lane without a share loads a row that exists and drops it). How many rows the wave owns, how many
    // iterations that makes and where the later rows lie is worked out behind this load, under its latency: a CU has one
    // scalar unit, a SIMD's four waves get one scalar instruction in 16 cycles each while they all run this prologue, and
    // every instruction in front of the first weight request is paid by the whole launch (5120 x 5120: with the
    // launch geometry as compile-time constants, 95 instructions fewer in front of the load, 5.51 -> 5.26 us).
    // Loads return in issue order, so the wait for the activations is a counted one only if the compiler knows how many
    // loads follow them; behind a conditional load it has to drain the queue, and the quantisation below then waits for
    // every prefetched row of the wave. The rest of the prefetch goes out behind the quantisation.
    typename F::Data buf[U];
    // One row in flight per wave (the long Q6_K rows, whose staging takes four passes and is what the launch waits for): the
    // first row is requested behind the share arithmetic as before, so that it does not stand in front of the younger
    // workgroups' activation loads any earlier (5120 x 17408: 16.5 us; requested early 16.7).
    constexpr bool EARLY = U > 1;
    if constexpr (EARLY) {
        const int l0 = SWIGLU ? v_start >> 1 : v_start;
        const int last = p.out_rows - 1;
        int row = weight_row(l0);
        const bool lane_row_ok = row + (SWIGLU ? row_off >> 1 : row_off) <= last;
        row = row < last ? row : last;
        const uint8_t* first = p.W + (size_t)(uint32_t)row * p.row_bytes + (SWIGLU && (v_start & 1) ? p.pair_bytes : (size_t)0);
        buf[0] = F::load(first, L, lane_row_ok ? lane_extra : 0u);
    }
    asm volatile("" ::: "memory");

    const int r0 = dealt ? 0 : rgid * p.rpg;              // rr: the row group's rows are spread over the weight, see weight_row
    int nrows = p.out_rows - r0;
    if (dealt) {                                         // kfull whole chunks and what the last round leaves this row group
        int last = p.rem - rgid * 4;
        last = last < 0 ? 0 : (last > 4 ? 4 : last);
        nrows = p.kfull * 4 + last;
    }
    nrows = nrows < 0 ? 0 : (nrows > p.rpg ? p.rpg : nrows);
    const int nv = nrows * VPR;                          // virtual rows: v -> the row group's row v/VPR (+ pair for odd v)
    // (nv - v_start + v_step - 1) / v_step with v_step = 4, 2, 1 (tail wave) or RF
    const uint32_t n_num = (uint32_t)(nv - v_start + v_step - 1);
    const int n_it = nv > v_start ? (int)(tail ? n_num >> RTL : div_magic(n_num, p.m_rf)) : 0;
    // iterations all of whose rows exist (a tail wave's last iteration may hold fewer than RT)
    const int n_full = tail ? nv >> RTL : n_it;
    const uint8_t* base = p.W + (size_t)(uint32_t)(nrows > 0 ? r0 : 0) * p.row_bytes;   // a row group past the end points at row 0
    auto row_base = [&](int it) -> const uint8_t* {
        const int v = v_start + it * v_step;             // wave-uniform
        int l = SWIGLU ? v >> 1 : v;                     // row of the row group
        if (dealt) l = (((l >> 2) * p.nrg + rgid) << 2) + (l & 3);   // as weight_row, from row 0 (r0 = 0)
        return SWIGLU ? base + (size_t)(uint32_t)l * p.row_bytes + (size_t)(v & 1) * p.pair_bytes : base + (size_t)(uint32_t)l * p.row_bytes;
    };
    auto lane_eo = [&](int it) { return (v_start + it * v_step + row_off < nv) ? lane_extra : 0u; };
    auto fetch = [&](int it) { return F::load(row_base(it), L, lane_eo(it)); };
    auto fetch_full = [&](int it) { return F::load(row_base(it), L, lane_extra); };   // it < n_full: every lane's row exists
    if constexpr (!EARLY) {
        buf[0] = F::load(n_it > 0 ? row_base(0) : p.W, L, n_it > 0 ? lane_eo(0) : 0u);
        asm volatile("" ::: "memory");
    }

    if (fused_norm) {
        // x <- rmsnorm(x + resid) * norm_w (crates/ferric-tensor/src/lib.rs:2057-2074): each thread holds at most one
        // 8-value piece of the row (cols <= 8 * threads). The row's scale 1 / rms is one number and the mat-vec is linear in
        // x, so the row is staged as (x + resid) * norm_w, the waves leave their sums of squares in LDS on the way (the
        // barrier behind the staging publishes them), and the scale meets the finished dot products at the end: no
        // barrier of its own in front of the staging.
        xa0.x += rsa.x; xa0.y += rsa.y; xa0.z += rsa.z; xa0.w += rsa.w;
        xb0.x += rsb.x; xb0.y += rsb.y; xb0.z += rsb.z; xb0.w += rsb.w;
        // with no CU to spare, the last workgroup that owns rows stores the sum
        if (p.x_out && (int)gridDim.x == p.row_wgs && (int)blockIdx.x == p.row_wgs - 1 && e0 < p.cols) {
            *(float4*)(p.x_out + e0) = xa0; *(float4*)(p.x_out + e0 + 4) = xb0;
        }
        float ss = fmaf(xa0.x, xa0.x, fmaf(xa0.y, xa0.y, fmaf(xa0.z, xa0.z, xa0.w * xa0.w)))
                 + fmaf(xb0.x, xb0.x, fmaf(xb0.y, xb0.y, fmaf(xb0.z, xb0.z, xb0.w * xb0.w)));
        if (e0 >= p.cols) ss = 0.f;                           // a thread past the row holds a copy of the last piece
        ss = slot_sum(ss);                                    // four 16-lane sums per wave, no trip through LDS to combine them
        float* red = (float*)(smem + p.red_off);
        if ((lane & 15) == 0) red[wave * 4 + (lane >> 4)] = ss;
        xa0.x *= nwa.x; xa0.y *= nwa.y; xa0.z *= nwa.z; xa0.w *= nwa.w;
        xb0.x *= nwb.x; xb0.y *= nwb.y; xb0.z *= nwb.z; xb0.w *= nwb.w;
    }

    // ---- activations -> block fixed point, once per workgroup, through LDS
    if (!fused_norm && stager) __builtin_amdgcn_s_setprio(3);   // the whole workgroup waits for this
    auto stage = [&](int e, const float4& a, const float4& b) {
        const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        uint32_t pl[NP][2];
        float scale, qsum;
        quantize8<RUN>(v, pl, scale, qsum);
        const int m = M == 1 ? 0 : e / p.cols, col = M == 1 ? e : e - m * p.cols;
        const int within = col % RUN;
        int u, j;
        F::owner(col / RUN, u, j);
        const int mj = m * NRUN + j;
#pragma unroll
        for (int pp = 0; pp < NP; pp++)
            *(u32x2*)(planes + ((size_t)((mj * NP + pp) * RC + (within >> 4)) * p.units + u) * 16 + (within & 15)) = u32x2{pl[pp][0], pl[pp][1]};
        if (within == 0) { scales[mj * p.units + u] = scale; sums[mj * p.units + u] = qsum; }
    };
    if (e0 < M * p.cols) stage(e0, xa0, xb0);
    if constexpr (!fused_norm) {
#pragma unroll
        for (int k = 0; k < XR; k++) {
            const int e = e0 + (k + 1) * e_step;
            if (e < M * p.cols) stage(e, xar[k], xbr[k]);
        }
        for (int e = e0 + (XR + 1) * e_step; e < M * p.cols; e += e_step)      // rows beyond four passes
            stage(e, *(const float4*)(p.x + e), *(const float4*)(p.x + e + 4));
    }
    if (!fused_norm && stager) __builtin_amdgcn_s_setprio(0);
    // The rest of the prefetch. Early: in flight while the workgroup meets at the barrier and copies its planes out of LDS
    // (rows so long that the staging takes several passes, and the large weights, whose row loop should find its pipeline
    // full). Late, behind the barrier: what is requested in front of the barrier stands in the memory pipe in front of the
    // younger workgroups' activation loads, and a small weight is all latency: with one row per wave there instead of two
    // the staged activations are ready sooner and the launch ends sooner (Q4_K 5120 x 5120 5.96 -> 5.53 us, 7168 x 5120
    // 7.20 -> 6.96, Q6_K 5120 x 5120 7.84 -> 7.08 on cold weights; no row at all in front of the barrier: 6.59).
    if constexpr (!LATE) {
#pragma unroll
        for (int j = 1; j < U; j++)
            if (j < n_it) buf[j] = fetch(j);
    }
    __syncthreads();

    // The row scale the staged activations went without, for the threads that will write outputs: worked out here, under
    // the wait for the first weight rows, and not behind the last barrier where every cycle is on the critical path.
    const int per_wg = p.G * p.rpg;
    float ninv = 1.0f;
    if (fused_norm && tid < per_wg) {
        const float4* red = (const float4*)(smem + p.red_off);
        const int nwaves = (int)(blockDim.x >> 6);
        float tot = 0.f;
#pragma unroll
        for (int wv = 0; wv < 16; wv++) {
            const float4 r4 = red[wv < nwaves ? wv : 0];
            tot += wv < nwaves ? (r4.x + r4.y) + (r4.z + r4.w) : 0.f;
        }
        ninv = 1.0f / sqrtf(tot / (float)p.cols + p.eps);
    }

    uint32_t xp[M][NRUN][NP][RD];
    float xs[M][NRUN], xq[M][NRUN];
    bool special = false;                                // one of this lane's runs needs the element-by-element branch
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int j = 0; j < NRUN; j++) {
            const int mj = m * NRUN + j;
            xs[m][j] = scales[mj * p.units + my_unit];
            xq[m][j] = sums[mj * p.units + my_unit];
            special = special || xs[m][j] != xs[m][j];
#pragma unroll
            for (int pp = 0; pp < NP; pp++)
#pragma unroll
                for (int i = 0; i < RD; i += 4) {
                    u32x4 t = *(const u32x4*)(planes + ((size_t)((mj * NP + pp) * RC + (i >> 2)) * p.units + my_unit) * 16);
                    xp[m][j][pp][i] = t[0]; xp[m][j][pp][i + 1] = t[1]; xp[m][j][pp][i + 2] = t[2]; xp[m][j][pp][i + 3] = t[3];
                }
        }
    special = special && unit_ok;

    // ---- stream the rows. Software pipeline over the U row buffers, written so that the steady-state
    // loop has no conditional reload: a reload under a condition makes the loop-carried buffers phi
    // nodes whose copies wait for every outstanding load at the back edge, which serialises the stream.
    float* mypart = part + (size_t)rg * p.rpg * VPR * p.NG * M;
    // The U rows of a pipeline step are summed over the slot together; lane l < 4 of a slot then holds the sum for the
    // step's row slot_of(l) and stores it.
    const bool bit0 = (lane & 1) != 0, bit1 = (lane & 2) != 0;
    const int my_j = slot_of<U>(l16);
    const bool store_lane = lane_ok && l16 < (U == 1 ? 1 : U == 2 ? 4 : 4) && my_j < U && (U != 2 || (l16 & 1) == 0);
    auto store_step = [&](const float (&outs)[M][U], int it0) {
        const int v = v_start + (it0 + my_j) * v_step + row_off;
#pragma unroll
        for (int m = 0; m < M; m++) {
            const float t = slot_sum_many<U>(outs[m], bit0, bit1);
            if (store_lane && v < nv) mypart[((size_t)v * p.NG + group) * M + m] = t;
        }
    };
    const bool contributes = unit_ok && !special;        // a special lane's share is added by the pass behind the loop
    auto consume = [&](typename F::Data& cur, int it, float (&outs)[M][U], int j) {
        cur.pin_all();
        float acc[M];
        F::template dot<M>(cur, L, xp, xs, xq, acc);
#pragma unroll
        for (int m = 0; m < M; m++) outs[m][j] = contributes ? acc[m] : 0.f;
    };
    int i0 = 0;
    float outs[M][U];
    // All prologue loads have landed by now (they overlapped the activation quantisation). Saying so
    // explicitly gives the compiler's wait-count tracking a clean state at the loop head; without it the
    // merge of the prologue's load order with the loop's makes every iteration wait for vmcnt(0).
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), expcnt/lgkmcnt untouched
    if constexpr (LATE) {
#pragma unroll
        for (int j = 1; j < U; j++)
            if (j < n_it) buf[j] = fetch(j);
    }
#pragma unroll 1
    for (; i0 + 2 * U <= n_full; i0 += U) {      // every row of this step and of the next one exists
#pragma unroll
        for (int j = 0; j < U; j++) {
            // consume, then refill the same registers: the old bytes are dead when the new load is issued,
            // so the loop-carried buffer needs no copy (and no wait) at the back edge
            consume(buf[j], i0 + j, outs, j);
            buf[j] = fetch_full(i0 + j + U);
        }
        store_step(outs, i0);
    }
    // drain, step A: iterations [i0, i0+U) that exist, reloading what is left of the step after it
#pragma unroll
    for (int j = 0; j < U; j++) {
        const int it = i0 + j;
        if (it < n_it) {
            consume(buf[j], it, outs, j);
            if (it + U < n_it) buf[j] = fetch(it + U);
        } else {
#pragma unroll
            for (int m = 0; m < M; m++) outs[m][j] = 0.f;
        }
    }
    if (i0 < n_it) store_step(outs, i0);
    // drain, step B: iterations [i0+U, n_it)
#pragma unroll
    for (int j = 0; j < U; j++) {
        const int it = i0 + U + j;
        if (it < n_it) consume(buf[j], it, outs, j);
        else {
#pragma unroll
            for (int m = 0; m < M; m++) outs[m][j] = 0.f;
        }
    }
    if (i0 + U < n_it) store_step(outs, i0 + U);

    // ---- the element-by-element pass of the lanes whose activations block fixed point cannot hold (rare: only waves
    // that own such a run enter): the unit's columns from the raw activations (for the fused norm: as staged,
    // (x + resid) * norm_w) times the exactly dequantised weights, summed over the slot and added to what the slot's
    // other lanes left in LDS for the row.
    if (__builtin_amdgcn_ballot_w64(special) != 0) {
#pragma unroll 1
        for (int it = 0; it < n_it; it++) {
            const uint8_t* rowp = row_base(it) + lane_eo(it);
            const int v = v_start + it * v_step + row_off;
#pragma unroll 1
            for (int m = 0; m < M; m++) {
                float a = 0.f;
                if (special) {
#pragma unroll 1
                    for (int j = 0; j < NRUN; j++)
#pragma unroll 1
                        for (int i = 0; i < RUN; i++) {
                            const int col = run[j] * RUN + i;
                            float xv = p.x[(size_t)m * p.cols + col];
                            if (fused_norm) xv = (xv + (p.resid ? p.resid[col] : 0.f)) * p.norm_w[col];
                            a += xv * fhip::deq_at<F::TYPE>(rowp, col);
                        }
                }
                a = slot_sum(a);
                if (lane_ok && l16 == 0 && v < nv) mypart[((size_t)v * p.NG + group) * M + m] += a;
            }
        }
    }
    __syncthreads();

    // ---- add the NG slot partials of each output in a fixed order, apply SwiGLU, store.
    // Local row rr = g*rpg + rl is output row blockIdx.x*G*rpg + rr, and its partials start at rr*VPR*NG.
    const int row0 = blockIdx.x * per_wg;
#pragma unroll
    for (int m = 0; m < M; m++)
        for (int rr = tid; rr < per_wg; rr += blockDim.x) {   // consecutive threads -> consecutive output rows
            int r = row0 + rr;
            if (dealt) {                                 // local row -> (row group, row in it) -> row of the weight
                const int g = (int)div_magic((uint32_t)rr, p.m_rpg), l = rr - g * p.rpg;
                r = (((l >> 2) * p.nrg + g * p.row_wgs + (int)blockIdx.x) << 2) + (l & 3);
                if (r >= p.out_rows) continue;
            } else if (r >= p.out_rows) break;
            const float* q = part + ((size_t)rr * VPR * p.NG) * M + m;
            float a = 0.f;
            for (int s = 0; s < p.NG; s++) a += q[s * M];
            if (fused_norm) a *= ninv;
            if (SWIGLU) {
                float b = 0.f;
                for (int s = 0; s < p.NG; s++) b += q[(p.NG + s) * M];
                if (fused_norm) b *= ninv;
                a = (a / (1.0f + expf(-a))) * b;             // silu(gate) * up, crates/ferric-tensor/src/dtype.rs:2408
            }
            if (p.sel.relu2) { a = fmaxf(a, 0.f); a *= a; }  // max(v, 0)^2, crates/ferric-tensor/src/dtype.rs:3755-3756
            p.y[(size_t)m * p.out_rows + r] = a;
        }
}

// Un-fused SwiGLU, crates/ferric-tensor/src/lib.rs:2603-2618: gu [t, 2d] = [gate | up] per row.
__global__ void swiglu_kernel(const float* __restrict__ gu, size_t n, size_t d, float* __restrict__ out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    size_t row = i / d, col = i % d;
    float g = gu[row * 2 * d + col], u = gu[row * 2 * d + d + col];
    out[i] = (g / (1.0f + expf(-g))) * u;
}

__global__ void zero_kernel(float* __restrict__ out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = 0.f;
}

bool g_force_generic = false;   // tests: send every shape to the shape-complete f32 kernel

// The tail wave of a row group works on 4 (NG%4 == 1) or 2 (NG%4 == 2) rows per iteration while a full
// wave works on one; replicating the full-wave set RF times, each replica taking every RF-th row, evens
// the iteration counts out (K = 5120: 4 full waves + 1 tail wave, one iteration each per 4 rows).
int full_wave_replicas(int NG, int maxw) {
    const int NGF = NG / 4, NT = NG % 4;
    if (NGF == 0 || NT == 0 || NT == 3) return 1;
    int rf = NT == 1 ? 4 : 2;
    while (rf > 1 && NGF * rf + 1 > maxw) rf /= 2;
    return rf;
}
// What wave `wave` of a workgroup is (GemvParams::wtab): a row group is NG / 4 full waves (four slots of one row each),
// replicated RF times with replica q taking every RF-th row from row q, and, when NG % 4 slots are left over, a tail wave that
// holds them for 4 (one slot), 2 (two) or 1 (three) rows at once.
uint32_t wave_word(int wave, int NG, int RF, int WPR) {
    const int NGF = NG >> 2, NT = NG & 3, NFW = NGF * RF;
    const int rg = wave / WPR, wr = wave - rg * WPR;
    const bool tail = wr == NFW;
    const int wq = NGF ? wr / NGF : 0, wm = NGF ? wr - wq * NGF : 0;
    const int rtl = tail ? (NT == 1 ? 2 : NT == 2 ? 1 : 0) : 0;
    const int v_start = tail ? 0 : wq, gbase = tail ? 4 * NGF : 4 * wm;
    return (uint32_t)rg | (uint32_t)v_start << 4 | (tail ? 1u : 0u) << 8 | (uint32_t)NT << 9 | (uint32_t)gbase << 11 | (uint32_t)rtl << 19;
}
int waves_per_row_group(int NG, int maxw) { return (NG / 4) * full_wave_replicas(NG, maxw) + (NG % 4 ? 1 : 0); }

template <class F, int M, bool SWIGLU>
size_t lds_bytes(size_t cols, int NG, int G, int rpg) {
    return M * cols * NP + 2 * M * (cols / F::RUN) * sizeof(float) + (size_t)G * rpg * (SWIGLU ? 2 : 1) * NG * M * sizeof(float);
}

template <class F, int M, bool SWIGLU, int U>
int launch_one_u(const fhip_weight* w, const float* d_x, float* d_y, size_t out_rows, hipStream_t s, const fhip::SelParams* sel,
                 const fhip::NormParams* norm) {
    // The prefetch of a wave's later rows waits behind the staging barrier for the small weights of the formats the
    // decode layers are made of (see the kernel; also Q5_K 5120 x 5120 7.20 -> 6.47 us, Q8_0 4096 x 4096 6.78 -> 6.57);
    // measured level or worse elsewhere: rows of 14336 columns and more, whose staging takes several passes (Q6_K
    // 5120 x 17408 16.7 -> 17.3 us), Q4_K from 28 MB on (10240 x 5120 8.13 -> 8.30), the other 32-value formats.
    constexpr bool HAS_LATE = M == 1 && U > 1 && (F::TYPE == FHIP_Q4_K || F::TYPE == FHIP_Q6_K || F::TYPE == FHIP_Q5_K || F::TYPE == FHIP_Q8_0);
    const size_t wbytes = out_rows * (SWIGLU ? 2 : 1) * w->row_bytes;   // of the rows this launch walks (one expert's, behind a selection)
    const bool small = wbytes < ((size_t)28 << 20);
    bool late = HAS_LATE && w->cols <= 8192 && (F::TYPE == FHIP_Q6_K || small);
    GemvParams p;
    p.W = w->d_raw; p.x = d_x; p.y = d_y;
    p.out_rows = (int)out_rows; p.cols = (int)w->cols; p.row_bytes = (uint32_t)w->row_bytes;
    p.pair_bytes = SWIGLU ? out_rows * w->row_bytes : 0;
    p.sel = sel ? *sel : fhip::SelParams{nullptr, 0, 0, 0, 0, 0, 1, 0};
    p.units = (int)(w->cols / F::WPL);
    p.NG = (p.units + 15) / 16;
    constexpr int MAXW = max_threads<F>(M) / 64;
    p.RF = full_wave_replicas(p.NG, MAXW);
    int WPR = waves_per_row_group(p.NG, MAXW);
    // Rows per row group (rpg) and row groups per workgroup (G). A CU holds Gcap row groups at once (one
    // workgroup of MAXW waves). Every workgroup pays a fixed few microseconds (activation quantisation,
    // pipeline fill and drain), so the rows are dealt out in as few rounds as possible: one workgroup per
    // CU with up to RPG_MAX rows per row group, more rounds of equal size only beyond that. With a
    // partly filled single round the row groups are spread over all CUs.
    // A small late-prefetch weight whose rows leave one slot over (5120 columns: four full waves' worth and a tail slot) runs
    // two replicas of the full-wave set per row group instead of four: row groups of three waves, five of them per workgroup,
    // four rows each where 5120 rows meet 256 CUs -- every full wave gets exactly two rows and no CU stays empty (5120 x 5120
    // Q4_K 5.53 -> 5.50 us, QKV 6.96 -> 6.86, Q6_K 5120 x 5120 7.09 -> 6.83, Q5_K 6.48 -> 6.33; the large weights lose 5 - 8 %
    // that way and keep four).
    if (late && small && M == 1 && p.RF == 4 && (p.NG & 3) == 1) {
        p.RF = 2;
        WPR = (p.NG >> 2) * 2 + 1;
    }
    int RPG_MAX = 256;
    int cus = fhip::device_cus() > 0 ? fhip::device_cus() : 256;
    if (p.sel.npairs > 1) cus = cus / p.sel.npairs > 0 ? cus / p.sel.npairs : 1;   // the pairs of an "_id" launch share the chip
    int Gcap = MAXW / WPR;
    if (Gcap < 1) Gcap = 1;
    // Fewer waves per CU for the launches that live off the memory system's queue depth rather than off latency hiding.
    // About 10 MB in flight fill this device's HBM pipe (6.5 TB/s times ~1.5 us), 40 KB per CU; 15 waves with two rows each
    // hold 90 - 100 KB, and what is queued beyond the pipe's depth only reaches the DRAM pages in a worse order. Measured on
    // cold weights, one activation row: Q6_K is fastest with 5 - 7 waves per workgroup at every size (5120 columns, 5120 /
    // 20480 / 151936 rows: 8.65 -> 7.83, 19.7 -> 18.5, 118.5 -> 107.0 us; 128256 x 4096: 82.1 -> 73.7 us with six row groups),
    // Q4_K with the fewest whole row groups that make 8 waves (8 - 14) once the weight has 28 MB or more (20480 x 5120 13.9 -> 12.6 us, fused gate|up 34816 x 5120
    // 20.9 -> 20.2, 28672 x 4096 15.3 -> 14.6) and with all 15 - 16 below that (5120 x 5120: 5.95 us against 6.39). A small
    // Q6_K weight whose later rows are requested behind the barrier keeps all its waves (5120 x 5120: 7.08 us against 7.98;
    // twelve of the sixteen one-wave row groups of 4096 columns: 4096 x 4096 5.49 us against 5.98).
    if (M == 1 && p.sel.npairs <= 1) {
        int want = Gcap;
        if (F::TYPE == FHIP_Q6_K) want = late && small ? (WPR == 1 ? 12 : Gcap) : 6 / WPR;
        else if (F::TYPE == FHIP_Q4_K && !small) want = (8 + WPR - 1) / WPR;
        if (want < 1) want = 1;
        // the fused norm holds one 8-value piece of the row per thread
        if (norm) {
            const int need = (int)((w->cols + (size_t)512 * WPR - 1) / ((size_t)512 * WPR));
            // a weight of 128 MB and more loses more to the extra waves than a norm launch of its own costs (vocabulary head
            // 151936 x 5120: 119.2 us fused in two row groups, 107.7 + 3 apart): nothing is launched, the caller norms first
            if (want < need && wbytes >= ((size_t)128 << 20)) return fhip::NORM_NOT_FUSED;
            if (want < need) want = need;
        }
        if (want < Gcap) {
            // rows per CU after rounding up to whole row groups: one or two row groups fewer where that leaves a twentieth or
            // more of the chip less idle (8192 rows on 256 CUs: five row groups of 7 rows fill 234 CUs, four of 8 fill all;
            // 8192 x 8192 Q4_K 10.4 -> 9.4 us). More row groups for the same reason measured slower (22016 x 4096: 12.2 -> 12.6).
            const int need = norm ? (int)((w->cols + (size_t)512 * WPR - 1) / ((size_t)512 * WPR)) : 1;
            auto rows_per_cu = [&](int g) { return (size_t)g * ((out_rows + (size_t)cus * g - 1) / ((size_t)cus * g)); };
            int best = want;
            for (int g = want - 1; g >= want - 2 && g >= 1 && g >= need; g--)
                if (rows_per_cu(g) * 20 <= rows_per_cu(best) * 19) best = g;
            want = best;
            Gcap = want;
            // one round for up to 1024 rows per row group where the partial sums still fit beside the staged row
            if (lds_bytes<F, M, SWIGLU>(w->cols, p.NG, Gcap, 1024) + 512 <= fhip::device_lds_bytes()) RPG_MAX = 1024;
        }
    }
    const size_t slots = (size_t)cus * Gcap;
    const size_t rounds = (out_rows + slots * (size_t)RPG_MAX - 1) / (slots * (size_t)RPG_MAX);
    int rpg = (int)((out_rows + slots * rounds - 1) / (slots * rounds));
    if (rpg < 1) rpg = 1;
    const size_t nrg = (out_rows + rpg - 1) / rpg;
    int G = nrg >= slots ? Gcap : (int)((nrg + cus - 1) / cus);
    // Large weights (16 rows per row group and more, one round): rows dealt round-robin in chunks of 4 over the row groups of
    // all CUs (one CU is left to the workgroup that stores x + resid when the fused norm asks for that).
    p.rr = 0; p.nrg = 0; p.kfull = 0; p.rem = 0;
    const bool spare = norm && norm->x_out && cus > 1;
    if ((F::RR || (F::RR_ONE_ROW && U == 1)) && rpg >= 16 && rounds == 1 && p.sel.npairs <= 1) {
        const size_t nrg_all = (size_t)(cus - (spare ? 1 : 0)) * G, S = nrg_all * 4;
        const size_t kfull = out_rows / S, rem = out_rows % S;
        const size_t rr_rpg = (kfull + (rem ? 1 : 0)) * 4;
        if (rr_rpg <= (size_t)RPG_MAX) { p.rr = 1; p.nrg = (int)nrg_all; p.kfull = (int)kfull; p.rem = (int)rem; rpg = (int)rr_rpg; }
    }
    p.G = G; p.rpg = rpg;
    // With one row per wave there is no later row to hold back and the two kernels do the same work; which of the two
    // compilations is the faster one then was measured per format (Q4_K 4096 x 4096: 4.71 us early, 4.82 late; Q6_K
    // 4096 x 4096: 6.38 early, 5.49 late).
    if (F::TYPE != FHIP_Q6_K && rpg * (SWIGLU ? 2 : 1) <= p.RF) late = false;
    void (*kernel)(GemvParams) = gemv_stream_kernel<F, M, U, SWIGLU, false, false>;
    if constexpr (M == 1) {
        if (norm) kernel = gemv_stream_kernel<F, M, U, SWIGLU, true, false>;
    }
    if constexpr (HAS_LATE) {
        if (late) kernel = norm ? gemv_stream_kernel<F, M, U, SWIGLU, true, true> : gemv_stream_kernel<F, M, U, SWIGLU, false, true>;
    }
    static bool lds_raised[4] = {false, false, false, false};
    const int variant = (norm ? 1 : 0) + (late ? 2 : 0);
    if (!lds_raised[variant]) {  // workgroups may use more than the default 64 KiB of the CU's 160 KiB
        (void)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)fhip::device_lds_bytes());
        (void)hipGetLastError();
        lds_raised[variant] = true;
    }
    auto magic = [](int d) { return d > 1 ? (uint32_t)(((1ull << 32) + (unsigned)d - 1) / (unsigned)d) : 0u; };
    p.m_rf = magic(p.RF); p.m_rpg = magic(rpg);
    for (int wv = 0; wv < 16; wv++) p.wtab[wv] = wv < WPR * G ? wave_word(wv, p.NG, p.RF, WPR) : 0u;
    const size_t per_wg = (size_t)G * rpg;
    const size_t grid = p.rr ? (size_t)p.nrg / G : (out_rows + per_wg - 1) / per_wg;
    size_t lds = lds_bytes<F, M, SWIGLU>(w->cols, p.NG, G, rpg);
    p.norm_w = nullptr; p.resid = nullptr; p.x_out = nullptr; p.eps = 0.f; p.red_off = 0;
    if (norm) {
        if (M != 1 || w->cols > (size_t)8 * 64 * WPR * G) return fhip::NORM_NOT_FUSED;   // nothing launched
        p.norm_w = norm->norm_w; p.resid = norm->resid; p.x_out = norm->x_out; p.eps = norm->eps;
        lds = (lds + 15) & ~(size_t)15;
        p.red_off = (uint32_t)lds;
        lds += 256;
        if (lds > fhip::device_lds_bytes()) return fhip::NORM_NOT_FUSED;   // no room left beside the staged row
    }
    p.row_wgs = (int)grid;
    {   // staging waves: enough for at most four 8-value pieces per thread, at least four (one per SIMD)
        const int nwaves = WPR * G;
        int S = (int)((M * w->cols + 2047) / 2048);
        S = S < 4 ? 4 : S;
        p.S = norm || S > nwaves ? nwaves : S;
    }
    const size_t launch_wgs = grid + ((norm && norm->x_out && grid < (size_t)cus) ? 1 : 0);
    hipLaunchKernelGGL(kernel, fhip::sel_grid((unsigned)launch_wgs, p.sel), dim3(64 * WPR * G), lds, s, p);
    return fhip::check_hip(hipGetLastError(), "gemv launch");
}

template <class F, int M, bool SWIGLU>
int launch_one(const fhip_weight* w, const float* d_x, float* d_y, size_t out_rows, hipStream_t s, const fhip::SelParams* sel = nullptr,
               const fhip::NormParams* norm = nullptr) {
    // Q6_K rows of more than 8192 columns (the down projection: nine waves per workgroup, early prefetch) stream with one row in
    // flight per wave instead of two: 5120 x 17408 16.7 -> 16.35 us, 4096 x 14336 12.56 -> 12.41 on cold weights (Q4_K rows of
    // that length lose 6 % the same way and keep two). The slot sums are the same tree of additions for every U, so the row's
    // bits stay those of the batched launches.
    if constexpr (M == 1 && F::TYPE == FHIP_Q6_K) {
        if (w->cols > 8192 && !sel && !norm) return launch_one_u<F, M, SWIGLU, 1>(w, d_x, d_y, out_rows, s, sel, norm);
    }
    return launch_one_u<F, M, SWIGLU, rows_in_flight<F>(M)>(w, d_x, d_y, out_rows, s, sel, norm);
}

// Largest batch width (4, 2, 1, or 0 = shape not covered) whose workgroup fits the wave and LDS limits.
template <class F, bool SWIGLU>
int max_batch(const fhip_weight* w, size_t left) {
    if (w->cols % F::WPL != 0 || g_force_generic) return 0;
    const int NG = (int)((w->cols / F::WPL + 15) / 16);
    auto WPRm = [&](int m) { return waves_per_row_group(NG, max_threads<F>(m) / 64); };
    const size_t cap = fhip::device_lds_bytes();
    if (left >= 4 && max_m<F>() >= 4 && WPRm(4) * 64 <= max_threads<F>(4) && lds_bytes<F, 4, SWIGLU>(w->cols, NG, max_threads<F>(4) / 64 / WPRm(4), 256) <= cap) return 4;
    if (left >= 2 && WPRm(2) * 64 <= max_threads<F>(2) && lds_bytes<F, 2, SWIGLU>(w->cols, NG, max_threads<F>(2) / 64 / WPRm(2), 256) <= cap) return 2;
    if (WPRm(1) * 64 <= max_threads<F>(1) && lds_bytes<F, 1, SWIGLU>(w->cols, NG, max_threads<F>(1) / 64 / WPRm(1), 256) <= cap) return 1;
    return 0;
}

template <class F, bool SWIGLU>
int launch_fmt(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, size_t out_rows, size_t n_ff, hipStream_t s) {
    // The kernel choice depends on the weight's shape only, never on the batch, so a row of a batch
    // result is bit-identical to the same row computed alone.
    if (max_batch<F, SWIGLU>(w, 1) == 0) return fhip::launch_gemv_generic(w, d_x, rows_x, d_y, n_ff, s);
    size_t m0 = 0;
    while (m0 < rows_x) {
        const float* x = d_x + m0 * w->cols;
        float* y = d_y + m0 * out_rows;
        int mb = max_batch<F, SWIGLU>(w, rows_x - m0), rc;
        if constexpr (max_m<F>() >= 4) {
            if (mb == 4) { rc = launch_one<F, 4, SWIGLU>(w, x, y, out_rows, s); if (rc != FHIP_OK) return rc; m0 += 4; continue; }
        }
        if (mb == 2) rc = launch_one<F, 2, SWIGLU>(w, x, y, out_rows, s);
        else rc = launch_one<F, 1, SWIGLU>(w, x, y, out_rows, s);
        if (rc != FHIP_OK) return rc;
        m0 += mb;
    }
    return FHIP_OK;
}

}  // namespace

namespace fhip {

int GEMV_EXPORT(launch_gemv)(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, size_t n_ff, hipStream_t s) {
    if (w->rows == 0 || rows_x == 0) return FHIP_OK;
    const size_t out_rows = n_ff ? n_ff : w->rows;
    if (w->cols == 0) {  // empty inner dimension: every dot product is 0 (and silu(0)*0 = 0)
        size_t n = rows_x * out_rows;
        hipLaunchKernelGGL(zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, d_y, n);
        return check_hip(hipGetLastError(), "zero launch");
    }
    // y is [rows_x, out_rows]: a batch slice starting at row m0 is contiguous, so slicing by pointer is exact.
    switch (w->type) {
        case FHIP_Q4_K: return n_ff ? launch_fmt<Q4K, true>(w, d_x, rows_x, d_y, out_rows, n_ff, s) : launch_fmt<Q4K, false>(w, d_x, rows_x, d_y, out_rows, n_ff, s);
        case FHIP_Q6_K: return n_ff ? launch_fmt<Q6K, true>(w, d_x, rows_x, d_y, out_rows, n_ff, s) : launch_fmt<Q6K, false>(w, d_x, rows_x, d_y, out_rows, n_ff, s);
        case FHIP_Q8_0:
            if (n_ff) return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "matmul_q_swiglu: no fused kernel for Q8_0");
            return launch_fmt<Q80, false>(w, d_x, rows_x, d_y, out_rows, n_ff, s);
        case FHIP_Q5_K: return n_ff ? launch_fmt<Q5K, true>(w, d_x, rows_x, d_y, out_rows, n_ff, s) : launch_fmt<Q5K, false>(w, d_x, rows_x, d_y, out_rows, n_ff, s);
        case FHIP_Q4_0: case FHIP_Q4_1: case FHIP_Q5_0: case FHIP_Q5_1:
            if (n_ff) return launch_gemv_generic(w, d_x, rows_x, d_y, n_ff, s);   // reports that these formats have no fused SwiGLU
            if (w->type == FHIP_Q4_0) return launch_fmt<Q40, false>(w, d_x, rows_x, d_y, out_rows, n_ff, s);
            if (w->type == FHIP_Q4_1) return launch_fmt<Q41, false>(w, d_x, rows_x, d_y, out_rows, n_ff, s);
            if (w->type == FHIP_Q5_0) return launch_fmt<Q50, false>(w, d_x, rows_x, d_y, out_rows, n_ff, s);
            return launch_fmt<Q51, false>(w, d_x, rows_x, d_y, out_rows, n_ff, s);
        case FHIP_IQ4_NL: case FHIP_IQ4_XS:
            if (n_ff) return launch_gemv_generic(w, d_x, rows_x, d_y, n_ff, s);
            return w->type == FHIP_IQ4_NL ? launch_fmt<IQ4NL, false>(w, d_x, rows_x, d_y, out_rows, n_ff, s)
                                          : launch_fmt<IQ4XS, false>(w, d_x, rows_x, d_y, out_rows, n_ff, s);
        case FHIP_MXFP4:
            return n_ff ? launch_gemv_generic(w, d_x, rows_x, d_y, n_ff, s) : launch_fmt<MXF4S, false>(w, d_x, rows_x, d_y, out_rows, n_ff, s);
        default: return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "QMatrix: no native matmul for ggml type %u", w->type);
    }
}

// Whether launch_gemv runs this Q4_K / Q5_K / Q6_K / Q8_0 weight on the streaming kernel (and not on the shape-complete f32 kernel, whose
// sums round differently): the four-row mat-vec, which promises the streaming kernel's bits, takes a weight only then.
bool GEMV_EXPORT(gemv_streams)(const fhip_weight* w, size_t n_ff) {
    if (w->type == FHIP_Q4_K) return (n_ff ? max_batch<Q4K, true>(w, 1) : max_batch<Q4K, false>(w, 1)) > 0;
    if (w->type == FHIP_Q6_K) return (n_ff ? max_batch<Q6K, true>(w, 1) : max_batch<Q6K, false>(w, 1)) > 0;
    if (w->type == FHIP_Q5_K) return (n_ff ? max_batch<Q5K, true>(w, 1) : max_batch<Q5K, false>(w, 1)) > 0;
    if (w->type == FHIP_Q8_0) return !n_ff && max_batch<Q80, false>(w, 1) > 0;
    return false;
}

// One activation row with the input norm fused into its staging; NORM_NOT_FUSED (nothing launched) when this weight's
// shape goes to the generic kernel or its row is longer than one pass of the workgroup.
template <class F>
int launch_norm_fmt(const fhip_weight* w, const float* d_x, float* d_y, size_t out_rows, bool swiglu, const NormParams& norm, hipStream_t s) {
    const bool covered = swiglu ? max_batch<F, true>(w, 1) != 0 : max_batch<F, false>(w, 1) != 0;
    if (!covered) return NORM_NOT_FUSED;
    return swiglu ? launch_one<F, 1, true>(w, d_x, d_y, out_rows, s, nullptr, &norm) : launch_one<F, 1, false>(w, d_x, d_y, out_rows, s, nullptr, &norm);
}

int GEMV_EXPORT(launch_gemv_norm)(const fhip_weight* w, const float* d_x, float* d_y, size_t n_ff, const NormParams& norm, hipStream_t s) {
    if (w->rows == 0 || w->cols == 0) return NORM_NOT_FUSED;
    const size_t out_rows = n_ff ? n_ff : w->rows;
    switch (w->type) {
        case FHIP_Q4_K: return launch_norm_fmt<Q4K>(w, d_x, d_y, out_rows, n_ff != 0, norm, s);
        case FHIP_Q6_K: return launch_norm_fmt<Q6K>(w, d_x, d_y, out_rows, n_ff != 0, norm, s);
        case FHIP_Q8_0: return n_ff ? NORM_NOT_FUSED : launch_norm_fmt<Q80>(w, d_x, d_y, out_rows, false, norm, s);
        case FHIP_Q5_K: return launch_norm_fmt<Q5K>(w, d_x, d_y, out_rows, n_ff != 0, norm, s);
        default: return NORM_NOT_FUSED;
    }
}

// the same without the fused-SwiGLU instantiation (formats the reference has no fused gate/up kernel for)
template <class F>
int launch_sel_plain(const fhip_weight* w, const float* d_x, float* d_y, size_t out_rows, const SelParams& sel, hipStream_t s) {
    if (max_batch<F, false>(w, 1) == 0) return launch_gemv_generic_sel(w, d_x, d_y, out_rows, false, sel, s);
    return launch_one<F, 1, false>(w, d_x, d_y, out_rows, s, &sel);
}

template <class F>
int launch_sel_fmt(const fhip_weight* w, const float* d_x, float* d_y, size_t out_rows, bool swiglu, const SelParams& sel, hipStream_t s) {
    const bool covered = swiglu ? max_batch<F, true>(w, 1) != 0 : max_batch<F, false>(w, 1) != 0;
    if (!covered) return launch_gemv_generic_sel(w, d_x, d_y, out_rows, swiglu, sel, s);
    return swiglu ? launch_one<F, 1, true>(w, d_x, d_y, out_rows, s, &sel) : launch_one<F, 1, false>(w, d_x, d_y, out_rows, s, &sel);
}

int GEMV_EXPORT(launch_gemv_sel)(const fhip_weight* w, const float* d_x, float* d_y, size_t out_rows, bool swiglu, const SelParams& sel,
                    hipStream_t s) {
    if (sel.npairs == 0 || out_rows == 0) return FHIP_OK;
    switch (w->type) {
        case FHIP_Q4_K: return launch_sel_fmt<Q4K>(w, d_x, d_y, out_rows, swiglu, sel, s);
        case FHIP_Q6_K: return launch_sel_fmt<Q6K>(w, d_x, d_y, out_rows, swiglu, sel, s);
        case FHIP_Q8_0: return launch_sel_fmt<Q80>(w, d_x, d_y, out_rows, swiglu, sel, s);
        case FHIP_Q5_K: return launch_sel_fmt<Q5K>(w, d_x, d_y, out_rows, swiglu, sel, s);
        case FHIP_Q4_0: case FHIP_Q4_1: case FHIP_Q5_0: case FHIP_Q5_1:
            if (swiglu) return launch_gemv_generic_sel(w, d_x, d_y, out_rows, swiglu, sel, s);
            if (w->type == FHIP_Q4_0) return launch_sel_plain<Q40>(w, d_x, d_y, out_rows, sel, s);
            if (w->type == FHIP_Q4_1) return launch_sel_plain<Q41>(w, d_x, d_y, out_rows, sel, s);
            if (w->type == FHIP_Q5_0) return launch_sel_plain<Q50>(w, d_x, d_y, out_rows, sel, s);
            return launch_sel_plain<Q51>(w, d_x, d_y, out_rows, sel, s);
        case FHIP_IQ4_NL: case FHIP_IQ4_XS:
            if (swiglu) return launch_gemv_generic_sel(w, d_x, d_y, out_rows, swiglu, sel, s);
            return w->type == FHIP_IQ4_NL ? launch_sel_plain<IQ4NL>(w, d_x, d_y, out_rows, sel, s) : launch_sel_plain<IQ4XS>(w, d_x, d_y, out_rows, sel, s);
        case FHIP_MXFP4:
            return swiglu ? launch_gemv_generic_sel(w, d_x, d_y, out_rows, swiglu, sel, s) : launch_sel_plain<MXF4S>(w, d_x, d_y, out_rows, sel, s);
        default: return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "QMatrix: no native matmul for ggml type %u", w->type);
    }
}

void GEMV_EXPORT(gemv_force_generic)(bool on) { g_force_generic = on; }

#if FHIP_GEMV_PLANES == 2
int launch_swiglu(const float* d_gu, size_t t, size_t d, float* d_out, hipStream_t s) {
    size_t n = t * d;
    if (n == 0) return FHIP_OK;
    hipLaunchKernelGGL(swiglu_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, d_gu, n, d, d_out);
    return check_hip(hipGetLastError(), "swiglu launch");
}
#endif

}  // namespace fhip
