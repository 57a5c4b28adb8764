// Mat-vec for three or four activation rows in one pass over a Q4_K, Q5_K, Q6_K or Q8_0 weight (the reference's matmul_q4_k /
// matmul_q6_k / matmul_q4_k_swiglu at small M, crates/ferric-tensor/src/dtype.rs:954-1003, and the CPU row loop
// crates/ferric-tensor/src/cpu_simd.rs:175-200 whose result for a row does not depend on the rows beside it).
//
// The arithmetic is the streaming mat-vec's (gemv.hip), bit for bit: activations as block fixed point (a scale per run of 16
// or 32 columns, two or three signed byte planes), exact integer dot products per run, the same f32 operations in the same
// order above them, the same trees for the sums over a row's units. What differs is who multiplies. Here the integer
// products go through v_mfma_i32_4x4x4_16b_i8: sixteen independent 4 x 4 x 4 products per wave. A wave's lane l = 4 u + r
// holds unit u (64 weights; a block of 32 for Q8_0) of WEIGHT row r of a quad of four rows as the B operand (four bytes of it
// are four consecutive columns: one column of B) and the planes of unit u of ACTIVATION row r as the A operand (one row of A). Block u of the
// instruction then gives all 16 (activation row, weight row) dot products of the unit's four columns, and lane 4 u + r ends
// up with its own weight row's sums against the four activation rows in its four accumulator registers -- next to that
// row's scales, which the same lane unpacked. No transposition, no LDS between the weight stream and the instruction: the
// layout the weights arrive in (one unit per lane) is the layout the instruction wants.
//
// A wave owns one 16-unit group of the row for a pass (its lanes' activation planes stay in registers) and takes quads of the
// workgroup's rows from a counter it shares with the other waves of its group; rows longer than ten groups are covered in
// passes (a row's partial sums are kept per group, so the order of the visits does not matter). The activations of a pass
// are quantised once per workgroup through LDS, as in the streaming mat-vec.
//
// What it costs: a quad of rows x one group is 48 matrix instructions (32 with two planes) at 4.1 ns a SIMD, which do not
// overlap with vector instructions of other waves on this chip (measured: 1 MFMA + 4 VALU = 9.4 ns, 4.1 + 4 x 1.35), beside
// some 200 vector instructions: about 0.5 us a SIMD, and a CU's 170 of them on the fused gate|up weight 34816 x 5120 take
// 23 us; the staging of four activation rows takes the first 5 us of the launch (one row: 2.3). Four rows, cold, at three
// planes (two): gate|up + SwiGLU 31 us (28), O 5120 x 5120 12.2 (10.8), down 5120 x 17408, two passes, 42 (39), against 20.1 /
// 5.9 / 17.2 for one row and twice 28 / 8 / 29 for four rows as two passes of the dot-product kernel. Against the one-pass f16
// kernels (gemm_f16x2.hip) with their split and sum launches it wins wherever it needs one pass and loses where it needs
// two, which is how the entry points choose (api.hip).
//
// Built once per activation precision like gemv.hip (FHIP_GEMV_PLANES = 2 or 3).
#include "common.hpp"
#include "deq_at.hpp"

#include <hip/hip_fp16.h>

#ifndef FHIP_GEMV_PLANES
#define FHIP_GEMV_PLANES 2
#endif
#if FHIP_GEMV_PLANES == 2
#define QUAD_EXPORT(name) name##_p2
#else
#define QUAD_EXPORT(name) name##_p3
#endif
#define gemv_quad_kernel QUAD_EXPORT(gemv_quad_kernel)

namespace {

constexpr int NP = FHIP_GEMV_PLANES;
static_assert(NP == 2 || NP == 3, "two or three activation planes");
// the quantiser's constants: those of gemv.hip, or the two kernels' bits part
constexpr float QMAX = NP == 2 ? 32639.0f : 8355711.0f;
constexpr float TINY_RUN = 7.888609052210118e-31f;   // 2^-100
constexpr float HUGE_RUN = 7.922816251426434e28f;    // 2^96

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
struct __attribute__((packed, aligned(2))) U4A2 { u32x4 v; };
struct __attribute__((packed, aligned(2))) U2A2 { u32x2 v; };

__device__ __forceinline__ float f16_bits(uint32_t b) { return __half2float(__ushort_as_half((unsigned short)b)); }
__device__ __forceinline__ float ub(uint32_t v, int k) { return (float)((v >> (8 * k)) & 0xFFu); }
__device__ __forceinline__ float sb(uint32_t v, int k) { return (float)(int8_t)((v >> (8 * k)) & 0xFFu); }
__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) { return __builtin_amdgcn_sdot4((int)a, (int)b, c, false); }
__device__ __forceinline__ void pin(uint32_t& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void pin(u32x2& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void pin(u32x4& v) { asm volatile("" : "+v"(v)); }

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true); }
constexpr int DPP_XOR1 = 0xB1, DPP_XOR2 = 0x4E;   // quad_perm [1,0,3,2], [2,3,0,1]
constexpr int DPP_ROR4 = 0x124, DPP_ROR8 = 0x128;   // lane l of a 16-lane row reads lane l - 4 / l - 8 of the row
// the value lane `src` holds
__device__ __forceinline__ float lane_read(float v, int src) {
    return __int_as_float(__builtin_amdgcn_ds_bpermute(src << 2, __float_as_int(v)));
}

// exact integer plane sums -> f32 (one rounding), as gemv.hip
__device__ __forceinline__ float planes_f32(const int (&a)[NP]) {
    if constexpr (NP == 2) return (float)((a[0] << 8) + a[1]);
    else return fmaf((float)a[0], 65536.0f, (float)((a[1] << 8) + a[NP - 1]));
}

__device__ __forceinline__ i32x4 mma(uint32_t a, uint32_t b, i32x4 c) { return __builtin_amdgcn_mfma_i32_4x4x4i8((int)a, (int)b, c, 0, 0, 0); }

// ------------------------------------------------------------------------------------------------
// Per-format lane work. A unit is WPL weights of one row, read as the streaming mat-vec reads it; a lane needs NRUN activation
// runs of RUN columns, run j being columns [run[j] * RUN, run[j] * RUN + RUN).
//   products() : the unit's integer products with the lane's activation planes, one accumulator quad per (run, plane);
//                element m of a quad is the lane's weight row against activation row m
//   scales()   : the NS numbers of the lane's weight row that the sums of a unit are scaled with
//   unit_sums(): the four (weight row, activation row) sums of the unit from those, the accumulators and the activation rows'
//                run scales xs(m, j) and run sums xq(m, j) -- gemv.hip's expression, term for term
// ------------------------------------------------------------------------------------------------
struct Q4K {
    static constexpr uint32_t TYPE = FHIP_Q4_K;
    static constexpr int WPL = 64, RUN = 32, NRUN = 2, NS = 6, DEPTH = 2;
    struct Lane { uint32_t off_h, off_q, sh, m1, m2, m3; };
    struct Data {
        u32x4 h, q0, q1;
        __device__ __forceinline__ void pin_all() { pin(h); pin(q0); pin(q1); }
    };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&run)[NRUN]) {
        const int b = u >> 2, g = u & 3;       // unit = group g of block b: qs[32g, 32g+32)
        L.off_h = b * 144;
        L.off_q = b * 144 + 16 + 32 * g;
        L.sh = 16 * (g & 1);
        // get_sc_min (crates/ferric-gguf/src/lib.rs:795-804) for the byte pair (2g, 2g+1) as masks
        L.m1 = g >= 2 ? 0u : 0x3F3Fu;
        L.m2 = g >= 2 ? 0x0F0Fu : 0u;
        L.m3 = g >= 2 ? 0x3030u : 0u;
        run[0] = 2 * u;
        run[1] = 2 * u + 1;
    }
    // the unit that uses run r of a row, and which of that unit's runs it is (the inverse of `run` above)
    static __device__ __forceinline__ void owner(int r, int& u, int& j) { u = r >> 1; j = r & 1; }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L) {
        Data d;
        d.h = *(const u32x4*)(row + L.off_h);
        d.q0 = *(const u32x4*)(row + L.off_q);
        d.q1 = *(const u32x4*)(row + L.off_q + 16);
        return d;
    }
    static constexpr uint32_t GROUP_BYTES = 576;   // sixteen units further along a row: four blocks
    // plane(j, p, c): dwords 4c .. 4c+3 of plane p of the lane's run j
    template <class PL>
    static __device__ __forceinline__ void products(const Data& D, PL plane, i32x4 (&acc)[NRUN][NP]) {
#pragma unroll
        for (int c = 0; c < 2; c++) {
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t w = c == 0 ? D.q0[k] : D.q1[k];
                lo[k] = w & 0x0F0F0F0Fu;
                hi[k] = (w ^ 0x80808080u) & 0xF0F0F0F0u;   // as signed bytes: 16 * (high nibble - 8)
            }
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const u32x4 x0 = plane(0, p, c), x1 = plane(1, p, c);
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    acc[0][p] = mma(x0[k], lo[k], acc[0][p]);
                    acc[1][p] = mma(x1[k], hi[k], acc[1][p]);
                }
            }
        }
    }
    static __device__ __forceinline__ void scales(const Data& D, const Lane& L, float (&sv)[NS]) {
        const uint32_t a = D.h[1] >> L.sh, b = D.h[2] >> L.sh, c = D.h[3] >> L.sh;
        const uint32_t scp = (a & L.m1) | (c & L.m2) | ((a >> 2) & L.m3);
        const uint32_t mp = (b & L.m1) | ((c >> 4) & L.m2) | ((b >> 2) & L.m3);
        sv[0] = f16_bits(D.h[0] & 0xFFFFu); sv[1] = ub(scp, 0); sv[2] = ub(scp, 1);
        sv[3] = f16_bits(D.h[0] >> 16); sv[4] = ub(mp, 0); sv[5] = ub(mp, 1);
    }
    // outs[m]: this lane's weight row against activation row m over the unit -- gemv.hip's expression, term for term
    template <class PL, class XS, class XQ>
    static __device__ __forceinline__ void unit_sums(const Data& D, const Lane& L, PL plane, XS xs, XQ xq, float (&outs)[4]) {
        i32x4 acc[NRUN][NP];
#pragma unroll
        for (int j = 0; j < NRUN; j++)
#pragma unroll
            for (int p = 0; p < NP; p++) acc[j][p] = i32x4{0, 0, 0, 0};
        products(D, plane, acc);
        float sv[NS];
        scales(D, L, sv);
        const float d = sv[0], s0 = sv[1], s1 = sv[2], dmin = sv[3], n0 = sv[4], n1 = sv[5];
#pragma unroll
        for (int m = 0; m < 4; m++) {
            int a0[NP], a1[NP];
#pragma unroll
            for (int p = 0; p < NP; p++) { a0[p] = acc[0][p][m]; a1[p] = acc[1][p][m]; }
            const float xq0 = xq(m, 0), xq1 = xq(m, 1);
            const float f0 = xs(m, 0) * planes_f32(a0);
            // sum x * nibble = (sum x * 16 (nibble - 8)) / 16 + 8 sum x
            const float f1 = fmaf(xs(m, 1) * 0.0625f, planes_f32(a1), 8.0f * xq1);
            // sum_l x_l (d*sc*q_l - dmin*m) = d * (sc0 f0 + sc1 f1) - dmin * (m0 sum0 + m1 sum1)
            outs[m] = d * fmaf(s1, f1, s0 * f0) - dmin * fmaf(n1, xq1, n0 * xq0);
        }
    }
};

// Q5_K: 176 B = [f16 d][f16 dmin][12 B 6-bit scales/mins][qh 32 B][qs 128 B] -- Q4_K plus bit s of qh[l] as the fifth bit of
// element l of sub-block s (crates/ferric-gguf/src/lib.rs:692-716). Unit = group g of block b (sub-blocks 2g, 2g+1): its 32
// quant bytes and the whole 32 bytes of high bits; codes 0..31.
struct Q5K {
    static constexpr uint32_t TYPE = FHIP_Q5_K;
    // (weight quads in flight: a unit is 20 registers, and with three activation planes two of them spill)
    static constexpr int WPL = 64, RUN = 32, NRUN = 2, NS = 6, DEPTH = NP == 3 ? 1 : 2;
    struct Lane { uint32_t off_h, off_q, sh, g2, m1, m2, m3; };
    struct Data {
        u32x4 h, b0, b1, q0, q1;
        __device__ __forceinline__ void pin_all() { pin(h); pin(b0); pin(b1); pin(q0); pin(q1); }
    };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&run)[NRUN]) {
        const int b = u >> 2, g = u & 3;
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
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L) {
        Data d;
        d.h = *(const u32x4*)(row + L.off_h);
        d.b0 = *(const u32x4*)(row + L.off_h + 16);
        d.b1 = *(const u32x4*)(row + L.off_h + 32);
        d.q0 = *(const u32x4*)(row + L.off_q);
        d.q1 = *(const u32x4*)(row + L.off_q + 16);
        return d;
    }
    template <class PL, class XS, class XQ>
    static __device__ __forceinline__ void unit_sums(const Data& D, const Lane& L, PL plane, XS xs, XQ xq, float (&outs)[4]) {
        i32x4 acc[NRUN][NP];
#pragma unroll
        for (int j = 0; j < NRUN; j++)
#pragma unroll
            for (int p = 0; p < NP; p++) acc[j][p] = i32x4{0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < 2; c++) {
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t w = c == 0 ? D.q0[k] : D.q1[k];
                const uint32_t hb = (c == 0 ? D.b0[k] : D.b1[k]) >> L.g2;   // bit 0: sub-block 2g, bit 1: sub-block 2g+1
                lo[k] = (w & 0x0F0F0F0Fu) | ((hb & 0x01010101u) << 4);
                hi[k] = ((w >> 4) & 0x0F0F0F0Fu) | ((hb & 0x02020202u) << 3);
            }
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const u32x4 x0 = plane(0, p, c), x1 = plane(1, p, c);
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    acc[0][p] = mma(x0[k], lo[k], acc[0][p]);
                    acc[1][p] = mma(x1[k], hi[k], acc[1][p]);
                }
            }
        }
        const uint32_t a = D.h[1] >> L.sh, b = D.h[2] >> L.sh, c = D.h[3] >> L.sh;
        const uint32_t scp = (a & L.m1) | (c & L.m2) | ((a >> 2) & L.m3);
        const uint32_t mp = (b & L.m1) | ((c >> 4) & L.m2) | ((b >> 2) & L.m3);
        const float d = f16_bits(D.h[0] & 0xFFFFu), dmin = f16_bits(D.h[0] >> 16);
        const float s0 = ub(scp, 0), s1 = ub(scp, 1), n0 = ub(mp, 0), n1 = ub(mp, 1);
#pragma unroll
        for (int m = 0; m < 4; m++) {
            int a0[NP], a1[NP];
#pragma unroll
            for (int p = 0; p < NP; p++) { a0[p] = acc[0][p][m]; a1[p] = acc[1][p][m]; }
            const float xq0 = xq(m, 0), xq1 = xq(m, 1);
            const float f0 = xs(m, 0) * planes_f32(a0);
            const float f1 = xs(m, 1) * planes_f32(a1);
            outs[m] = d * fmaf(s1, f1, s0 * f0) - dmin * fmaf(n1, xq1, n0 * xq0);
        }
    }
};

struct Q6K {
    static constexpr uint32_t TYPE = FHIP_Q6_K;
    // (weight quads a wave has in flight: with three activation planes a second one spills 20 registers, and the down
    // projection 5120 x 17408 at four rows takes 58 us with it against 44 without)
    static constexpr int WPL = 64, RUN = 16, NRUN = 4, NS = 5, DEPTH = NP == 3 ? 1 : 2;
    struct Lane { uint32_t off_a, off_h, off_s, off_d, ssh; };
    struct Data {
        u32x4 a, b, h; u32x2 s; uint32_t d;
        __device__ __forceinline__ void pin_all() { pin(a); pin(b); pin(h); pin(s); pin(d); }
    };
    static __device__ __forceinline__ void setup(int u, Lane& L, int (&run)[NRUN]) {
        const int b = u >> 2, hf = (u >> 1) & 1, t = u & 1;   // unit: l in [16t, 16t+16) of half hf of block b
        L.off_a = b * 210 + 64 * hf + 16 * t;                 // ql[l], and ql[l+32] at +32
        L.off_h = b * 210 + 128 + 32 * hf + 16 * t;
        L.off_s = b * 210 + 192 + 8 * hf;
        L.off_d = b * 210 + 208;
        L.ssh = 8 * t;
#pragma unroll
        for (int g = 0; g < 4; g++) run[g] = 16 * b + 8 * hf + t + 2 * g;   // columns 256b + 128hf + 32g + 16t + [0,16)
    }
    static __device__ __forceinline__ void owner(int r, int& u, int& j) {
        u = ((r >> 4) << 2) | (((r >> 3) & 1) << 1) | (r & 1);
        j = (r >> 1) & 3;
    }
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L) {
        Data d;
        d.a = ((const U4A2*)(row + L.off_a))->v;
        d.b = ((const U4A2*)(row + L.off_a + 32))->v;
        d.h = ((const U4A2*)(row + L.off_h))->v;
        d.s = ((const U2A2*)(row + L.off_s))->v;
        d.d = *(const uint16_t*)(row + L.off_d);
        return d;
    }
    static constexpr uint32_t GROUP_BYTES = 840;   // sixteen units further along a row: four blocks
    // plane(j, p, c): dwords 4c .. 4c+3 of plane p of the lane's run j (c = 0: a run is four dwords).
    // The products of runs 2 HF and 2 HF + 1 (low nibbles for HF = 0, high nibbles for HF = 1): two accumulator quads per plane
    // live at a time instead of four
    template <int HF, class PL>
    static __device__ __forceinline__ void products_half(const Data& D, PL plane, i32x4 (&acc)[2][NP]) {
        // the four 6-bit quants that share byte l (crates/ferric-gguf/src/lib.rs:733-736), 4 bytes at a time, as 0..63
        uint32_t q[2][4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t A = D.a[i], B = D.b[i], H = D.h[i];
            if constexpr (HF == 0) {
                q[0][i] = (A & 0x0F0F0F0Fu) | ((H & 0x03030303u) << 4);
                q[1][i] = (B & 0x0F0F0F0Fu) | ((H & 0x0C0C0C0Cu) << 2);
            } else {
                q[0][i] = ((A >> 4) & 0x0F0F0F0Fu) | (H & 0x30303030u);
                q[1][i] = ((B >> 4) & 0x0F0F0F0Fu) | ((H >> 2) & 0x30303030u);
            }
        }
#pragma unroll
        for (int g = 0; g < 2; g++)
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const u32x4 x = plane(2 * HF + g, p, 0);
#pragma unroll
                for (int i = 0; i < 4; i++) acc[g][p] = mma(x[i], q[g][i], acc[g][p]);
            }
    }
    static __device__ __forceinline__ void scales(const Data& D, const Lane& L, float (&sv)[NS]) {
        const uint32_t s0 = D.s[0] >> L.ssh, s1 = D.s[1] >> L.ssh;  // sc[is], sc[is+2] | sc[is+4], sc[is+6]
        sv[0] = sb(s0, 0); sv[1] = sb(s0, 2); sv[2] = sb(s1, 0); sv[3] = sb(s1, 2);
        sv[4] = f16_bits(D.d);
    }
    // outs[m]: this lane's weight row against activation row m over the unit -- gemv.hip's expression, term for term
    template <class PL, class XS, class XQ>
    static __device__ __forceinline__ void unit_sums(const Data& D, const Lane& L, PL plane, XS xs, XQ xq, float (&outs)[4]) {
        float sv[NS];
        scales(D, L, sv);
        float f[4][NRUN];
        auto half = [&](auto Hc) {
            constexpr int HF = decltype(Hc)::value;
            i32x4 acc[2][NP];
#pragma unroll
            for (int g = 0; g < 2; g++)
#pragma unroll
                for (int p = 0; p < NP; p++) acc[g][p] = i32x4{0, 0, 0, 0};
            products_half<HF>(D, plane, acc);
#pragma unroll
            for (int m = 0; m < 4; m++)
#pragma unroll
                for (int g = 0; g < 2; g++) {
                    int a[NP];
#pragma unroll
                    for (int p = 0; p < NP; p++) a[p] = acc[g][p][m];
                    f[m][2 * HF + g] = fmaf(xs(m, 2 * HF + g), planes_f32(a), -32.f * xq(m, 2 * HF + g));   // sum x*(q-32) = sum x*q - 32*sum x
                }
        };
        half(std::integral_constant<int, 0>{});
        half(std::integral_constant<int, 1>{});
#pragma unroll
        for (int m = 0; m < 4; m++) {
            float t = 0.f;
#pragma unroll
            for (int g = 0; g < 4; g++) t = fmaf(sv[g], f[m][g], t);
            outs[m] = sv[4] * t;
        }
    }
};

// Eight consecutive activations of one run -> NP plane dword pairs, the run's scale and the run's quantised sum: the
// streaming mat-vec's quantiser (gemv.hip), operation for operation. The 2 (RUN 16) or 4 (RUN 32) lanes of a run sit in one
// quad and agree on the maximum, the scale and the sum afterwards.
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
    const bool special = !(fabsf(sum) <= 3.4028234663852886e38f) || amax > HUGE_RUN || (amax < TINY_RUN && amax > 0.f);
    const float inv = amax > 0.f ? QMAX * __builtin_amdgcn_rcpf(amax) : 0.f;
    uint32_t t[8];
    if constexpr (NP == 2) {
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
        pl[NP - 1][hh] = __builtin_amdgcn_perm(p23, p01, 0x05040100u) ^ 0x80808080u;
        if constexpr (NP == 2) {
            pl[0][hh] = __builtin_amdgcn_perm(p23, p01, 0x07060302u);
        } else {
            pl[1][hh] = __builtin_amdgcn_perm(p23, p01, 0x07060302u) ^ 0x80808080u;
            const uint32_t u01 = __builtin_amdgcn_perm(t1, t0, 0x00000602u), u23 = __builtin_amdgcn_perm(t3, t2, 0x00000602u);
            pl[0][hh] = __builtin_amdgcn_perm(u23, u01, 0x05040100u);
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

// Q8_0: 34 B = [f16 d][32 int8] (crates/ferric-gguf/src/lib.rs:608-615). Unit = one block: the quants are the B operand as they
// lie in memory.
struct Q80 {
    static constexpr uint32_t TYPE = FHIP_Q8_0;
    static constexpr int WPL = 32, RUN = 32, NRUN = 1, NS = 1, DEPTH = 2;
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
    static __device__ __forceinline__ Data load(const uint8_t* row, const Lane& L) {
        Data d;
        d.d = *(const uint16_t*)(row + L.off);
        d.q0 = ((const U4A2*)(row + L.off + 2))->v;
        d.q1 = ((const U4A2*)(row + L.off + 18))->v;
        return d;
    }
    template <class PL, class XS, class XQ>
    static __device__ __forceinline__ void unit_sums(const Data& D, const Lane&, PL plane, XS xs, XQ, float (&outs)[4]) {
        i32x4 acc[NP];
#pragma unroll
        for (int p = 0; p < NP; p++) acc[p] = i32x4{0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < 2; c++)
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const u32x4 x = plane(0, p, c);
#pragma unroll
                for (int k = 0; k < 4; k++) acc[p] = mma(x[k], c == 0 ? D.q0[k] : D.q1[k], acc[p]);
            }
        const float d = f16_bits(D.d);
        // per block: part = sum x*q, then part*d -- crates/ferric-tensor/src/cpu_simd.rs:66-70
#pragma unroll
        for (int m = 0; m < 4; m++) {
            int a[NP];
#pragma unroll
            for (int p = 0; p < NP; p++) a[p] = acc[p][m];
            outs[m] = (xs(m, 0) * planes_f32(a)) * d;
        }
    }
};

struct QuadParams {
    const uint8_t* W;
    const float* x;      // [rows_x, cols]
    float* y;            // [rows_x, out_rows]
    int rows_x;          // 1 .. 4
    int out_rows;        // rows of y (n_ff when fused SwiGLU)
    int cols;
    uint32_t row_bytes;
    uint32_t pair_bytes; // fused SwiGLU: byte distance from gate row r to up row r
    int units, NG;       // units (F::WPL weights) per row; 16-unit groups per row
    int WPS, QS, GPW;    // waves that share a quad of rows (one group each per pass); quads in flight per workgroup; passes
    int rows_wg;         // output rows per workgroup (rows_wg * VPR is a multiple of 4)
    int pieces;          // 8-column pieces of a pass's activations a thread stages
    uint32_t magic_S;    // ceil(2^32 / S), S = 2 WPL WPS the pieces of one activation row of a pass: thread index -> activation row of its first piece
    int step_m, step_slot;   // threads / S, threads % S: from one piece of a thread to its next
    uint32_t scales_off, sums_off, ctr_off, part_off;   // byte offsets in LDS: run scales, run sums, quad counters, group sums [virtual row][NG][4]
};

constexpr int QUAD_PIECES = 4;   // activation pieces a thread requests at once while it stages a pass

// LDS of a pass over UP = 16 WPS units (the groups the workgroup's waves hold in that pass), the streaming mat-vec's layout
// with the pass's units in place of the row's: planes -- the 16-byte piece c of plane pp of run j of unit u of activation row m
// at ((((m NRUN + j) NP + pp) RC + c) UP + u) * 16 -- then the run scales [UP][4][NRUN] and the run sums [UP][4][NRUN] (a
// unit's 4 NRUN numbers side by side).
template <class F, bool SWIGLU>
__global__ void __launch_bounds__(640) gemv_quad_kernel(QuadParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int VPR = SWIGLU ? 2 : 1;                              // weight rows walked per output row
    constexpr int RUN = F::RUN, NRUN = F::NRUN, RD = RUN / 4, RC = RD / 4;
    constexpr int U = F::DEPTH;                                      // weight quads a wave has in flight
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int u16 = lane >> 2, r = lane & 3;   // unit of the group; weight row of the quad (B operand) and activation row (A operand)
    const int qs = wave / p.WPS, kw = wave - qs * p.WPS;
    const int row0 = blockIdx.x * p.rows_wg;
    int nrows = p.out_rows - row0;
    nrows = nrows > p.rows_wg ? p.rows_wg : nrows;
    if (nrows <= 0) return;                                          // (the launcher sends no such workgroup)
    const int nv = nrows * VPR, nq = (nv + 3) >> 2;
    const uint8_t* base = p.W + (size_t)row0 * p.row_bytes;
    // virtual row v of the workgroup: output row v / VPR, and with fused SwiGLU the up row of the pair for odd v
    auto row_ptr = [&](int v) -> const uint8_t* {
        return SWIGLU ? base + ((uint32_t)(v >> 1) * p.row_bytes + (uint32_t)(v & 1) * p.pair_bytes) : base + (uint32_t)v * p.row_bytes;
    };
    const int UP = 16 * p.WPS;
    uint8_t* planes = smem;
    float* scales = (float*)(smem + p.scales_off);
    float* sums = (float*)(smem + p.sums_off);
    float* part = (float*)(smem + p.part_off);

    for (int pass = 0; pass < p.GPW; pass++) {
        const int group = kw + pass * p.WPS;                         // wave-uniform
        const bool has_group = group < p.NG;
        const int u_lo = pass * UP;                                  // first unit of the pass
        const int unit = group * 16 + u16;
        const bool unit_ok = has_group && unit < p.units;
        typename F::Lane L;
        int run[NRUN];
        F::setup(unit_ok ? unit : 0, L, run);
        // the lane's weight row of quad q; a quad or a row past the end reads the workgroup's first row and is dropped
        auto fetch = [&](int q) {
            const int v = 4 * q + r;
            return F::load(row_ptr(v < nv ? v : 0), L);
        };
        // The waves that hold the same group share its quads through a counter in LDS: each takes the next quad when it is
        // ready for one. (Dealt out in fixed shares, the waves on a SIMD that carries three of the workgroup's ten finished
        // half as late again as those on a SIMD with two: 24 us against 16 on the fused gate|up weight.) Which wave adds a
        // quad's sums up does not change them.
        int* next_quad = (int*)(smem + p.ctr_off);
        auto grab = [&]() {
            int q = 0;
            if (lane == 0) q = atomicAdd(&next_quad[kw], 1);
            return __builtin_amdgcn_readfirstlane(q);
        };

        // ---- the pass's activations -> block fixed point, once per workgroup, through LDS: thread t takes the eight columns
        // from 8 t of the pass's 4 x (WPL UP) values, then 8 (t + threads), ...; all of a thread's pieces are requested before the
        // first is used, so that they cost one trip to memory, and the first weight quads go out right behind them. A piece
        // past the row's end or of an activation row the batch does not have is staged as zeros (its lanes take part in the
        // quantiser's lane exchanges all the same).
        if (pass > 0) __syncthreads();                               // the planes of the pass before are still being read
        if (tid < p.WPS) next_quad[tid] = p.QS;                      // quads 0 .. QS-1 are the waves' first; the others are taken as the waves go
        // Piece id of a thread's k-th piece: tid + k * threads; id -> activation row m = id / S and 8-column slot id % S of the
        // pass's columns, S = 2 WPL WPS. Worked out once by a multiplication and carried along by additions (a division and the
        // address products per piece were as many instructions as the quantiser itself).
        const int col_lo = F::WPL * u_lo, S = (F::WPL / 8) * 16 * p.WPS;
        const uint32_t UP16 = (uint32_t)UP * 16u, row_stride = (uint32_t)(NRUN * NP * RC) * UP16;
        int pm = (int)__umulhi((uint32_t)tid, p.magic_S), pslot = tid - pm * S;
        typename F::Data buf[U];
#pragma unroll 1
        for (int k0 = 0; k0 < p.pieces; k0 += QUAD_PIECES) {         // rounds of QUAD_PIECES pieces a thread: one trip to memory each
            float4 xa[QUAD_PIECES], xb[QUAD_PIECES];
            int ms[QUAD_PIECES], slots[QUAD_PIECES];
#pragma unroll
            for (int k = 0; k < QUAD_PIECES; k++) {
                ms[k] = pm; slots[k] = pslot;
                const int col = col_lo + 8 * pslot;
                xa[k] = float4{0.f, 0.f, 0.f, 0.f}; xb[k] = xa[k];
                if (k0 + k < p.pieces && pm < p.rows_x && col < p.cols) {
                    const float* src = p.x + ((uint32_t)__umul24(pm, p.cols) + (uint32_t)col);
                    xa[k] = *(const float4*)src; xb[k] = *(const float4*)(src + 4);
                }
                pm += p.step_m; pslot += p.step_slot;
                if (pslot >= S) { pslot -= S; pm++; }
            }
            if (k0 == 0) {                                           // the wave's first quad goes out behind the first activations
                asm volatile("" ::: "memory");
                buf[0] = fetch(qs);
                asm volatile("" ::: "memory");
            }
#pragma unroll
            for (int k = 0; k < QUAD_PIECES; k++) {
                if (k0 + k < p.pieces && ms[k] < 4) {                // whole waves: an activation row's S pieces are a multiple of 64
                    const int m = ms[k], cl = 8 * slots[k], col = col_lo + cl;
                    const float v[8] = {xa[k].x, xa[k].y, xa[k].z, xa[k].w, xb[k].x, xb[k].y, xb[k].z, xb[k].w};
                    uint32_t pl[NP][2];
                    float scale, qsum;
                    quantize8<RUN>(v, pl, scale, qsum);
                    const int within = cl & (RUN - 1);
                    int gu, j;                                       // the unit that uses the run, and which of its runs it is
                    F::owner(col / RUN, gu, j);
                    const int ul = gu - u_lo;
                    uint8_t* dst = planes + (__umul24(m, row_stride) + __umul24(j * (NP * RC) + (within >> 4), UP16) + (uint32_t)(ul * 16 + (within & 15)));
#pragma unroll
                    for (int pp = 0; pp < NP; pp++) *(u32x2*)(dst + pp * (RC * UP16)) = u32x2{pl[pp][0], pl[pp][1]};
                    if (within == 0) { scales[ul * (4 * NRUN) + m * NRUN + j] = scale; sums[ul * (4 * NRUN) + m * NRUN + j] = qsum; }
                }
            }
        }
        __syncthreads();
        if (!has_group) continue;                                    // (a wave without a group in this pass still staged and met the barriers)

        // ---- the lane's operands: the planes of its own activation row for its unit; every activation row's run scales and
        // run sums stay in LDS, side by side per unit
        const int ul = (unit_ok ? unit : group * 16) - u_lo;
        uint32_t xp[NRUN][NP][RD];
        const float* my_scales = scales + ul * (4 * NRUN);
        const float* my_sums = sums + ul * (4 * NRUN);
        bool special[4] = {false, false, false, false};
#pragma unroll
        for (int j = 0; j < NRUN; j++) {
            const int mj = r * NRUN + j;
#pragma unroll
            for (int pp = 0; pp < NP; pp++)
#pragma unroll
                for (int i = 0; i < RD; i += 4) {
                    const u32x4 t = *(const u32x4*)(planes + ((size_t)((mj * NP + pp) * RC + (i >> 2)) * UP + ul) * 16);
                    xp[j][pp][i] = t[0]; xp[j][pp][i + 1] = t[1]; xp[j][pp][i + 2] = t[2]; xp[j][pp][i + 3] = t[3];
                }
#pragma unroll
            for (int m = 0; m < 4; m++) {
                const float sc = my_scales[m * NRUN + j];
                special[m] = special[m] || sc != sc;
            }
        }
        bool any_special = false;
#pragma unroll
        for (int m = 0; m < 4; m++) {
            special[m] = special[m] && unit_ok;
            any_special = any_special || special[m];
        }
        auto plane = [&](int j, int pp, int c) { return u32x4{xp[j][pp][4 * c], xp[j][pp][4 * c + 1], xp[j][pp][4 * c + 2], xp[j][pp][4 * c + 3]}; };

        auto consume = [&](typename F::Data& cur, int q) {
            cur.pin_all();
            float outs[4];
            F::unit_sums(cur, L, plane, [&](int m, int j) { return my_scales[m * NRUN + j]; }, [&](int m, int j) { return my_sums[m * NRUN + j]; }, outs);
#pragma unroll
            for (int m = 0; m < 4; m++) outs[m] = (unit_ok && !special[m]) ? outs[m] : 0.f;
            // Sum over the group's 16 units, for each activation row, in the streaming mat-vec's tree: with Q(k) = (v[4k] +
            // v[4k+1]) + (v[4k+2] + v[4k+3]) over the units, (Q0 + Q3) + (Q2 + Q1). Units 4k .. 4k+3 are the four quads of
            // 16-lane row k here, so Q(k) forms in that row's last quad, and the rows meet through two lane reads.
            float tot[4];
#pragma unroll
            for (int m = 0; m < 4; m++) {
                float t = outs[m];
                t += dpp_f<DPP_ROR4>(t);                    // units 4k+1, 4k+3: v[u] + v[u-1]
                t += dpp_f<DPP_ROR8>(t);                    // unit 4k+3: (v3 + v2) + (v1 + v0) = Q(k)
                t += lane_read(t, (lane + 48) & 63);        // row 0: Q0 + Q3; row 2: Q2 + Q1
                t += lane_read(t, (lane + 32) & 63);        // row 0: (Q0 + Q3) + (Q2 + Q1)
                tot[m] = t;
            }
            const int v = 4 * q + r;
            // The element-by-element share of the lanes whose unit holds an activation run block fixed point cannot hold
            // (non-finite members, magnitudes at the ends of the f32 range): the unit's columns of that activation row from the
            // raw activations times the exactly dequantised weights of the lane's row, summed over the group in the tree the
            // streaming mat-vec uses there, (Q0 + Q1) + (Q3 + Q2), and added to what the group's other lanes gave the row.
            if (__builtin_amdgcn_ballot_w64(any_special) != 0) {
                const uint8_t* rowp = row_ptr(v < nv ? v : 0);
#pragma unroll 1
                for (int m = 0; m < 4; m++) {
                    float a = 0.f;
                    if (special[m]) {
#pragma unroll 1
                        for (int j = 0; j < NRUN; j++)
#pragma unroll 1
                            for (int i = 0; i < RUN; i++) {
                                const int col = run[j] * RUN + i;
                                a += p.x[(size_t)m * p.cols + col] * fhip::deq_at<F::TYPE>(rowp, col);
                            }
                    }
                    a += dpp_f<DPP_ROR4>(a);
                    a += dpp_f<DPP_ROR8>(a);
                    a += lane_read(a, lane ^ 16);           // row 0: Q0 + Q1; row 3: Q3 + Q2
                    a += lane_read(a, lane ^ 48);           // row 0: (Q0 + Q1) + (Q3 + Q2)
                    tot[m] += a;
                }
            }
            if (lane >= 12 && lane < 16 && v < nv) *(float4*)(part + ((size_t)v * p.NG + group) * 4) = float4{tot[0], tot[1], tot[2], tot[3]};
        };

        // U quads in flight; a quad past the last is fetched from the first row and dropped, so the loop body has no condition
        int qi[U];
        qi[0] = qs;
#pragma unroll
        for (int k = 1; k < U; k++) { qi[k] = grab(); buf[k] = fetch(qi[k]); }
#pragma unroll 1
        while (qi[0] < nq) {
#pragma unroll
            for (int j = 0; j < U; j++) {
                const int nxt = grab();
                consume(buf[j], qi[j]);
                qi[j] = nxt;
                buf[j] = fetch(nxt);
            }
        }
    }
    __syncthreads();

    // add the NG group sums of each output in a fixed order, apply SwiGLU, store: the streaming mat-vec's last step
    for (int m = 0; m < p.rows_x; m++)
        for (int rr = tid; rr < nrows; rr += blockDim.x) {
            const float* q = part + ((size_t)rr * VPR * p.NG) * 4 + m;
            float a = 0.f;
            for (int s = 0; s < p.NG; s++) a += q[s * 4];
            if (SWIGLU) {
                float b = 0.f;
                for (int s = 0; s < p.NG; s++) b += q[(p.NG + s) * 4];
                a = (a / (1.0f + expf(-a))) * b;             // silu(gate) * up, crates/ferric-tensor/src/dtype.rs:2408
            }
            p.y[(size_t)m * p.out_rows + row0 + rr] = a;
        }
}

template <class F, bool SWIGLU>
int launch_quad(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, size_t out_rows, hipStream_t s) {
    constexpr int VPR = SWIGLU ? 2 : 1, MAXW = 10;
    QuadParams p;
    p.W = w->d_raw; p.x = d_x; p.y = d_y;
    p.rows_x = (int)rows_x; p.out_rows = (int)out_rows; p.cols = (int)w->cols;
    p.row_bytes = (uint32_t)w->row_bytes;
    p.pair_bytes = (uint32_t)(out_rows * w->row_bytes);
    p.units = (int)(w->cols / F::WPL);
    p.NG = (p.units + 15) / 16;
    p.GPW = (p.NG + MAXW - 1) / MAXW;
    p.WPS = (p.NG + p.GPW - 1) / p.GPW;
    p.QS = MAXW / p.WPS;
    const long long cus = fhip::device_cus() > 0 ? fhip::device_cus() : 256;
    // LDS: a pass's staged activations (4 rows x 16 WPL WPS columns: planes, run scales, run sums), then the group sums
    const size_t plane_bytes = (size_t)4 * (16 * F::WPL) * p.WPS * NP, sc_bytes = (size_t)16 * p.WPS * 4 * F::NRUN * sizeof(float);
    p.scales_off = (uint32_t)plane_bytes;
    p.sums_off = p.scales_off + (uint32_t)sc_bytes;
    p.ctr_off = p.sums_off + (uint32_t)sc_bytes;
    p.part_off = p.ctr_off + 64;
    const size_t stage = p.part_off;
    const size_t lds_max = fhip::device_lds_bytes() > 0 ? fhip::device_lds_bytes() : 65536;
    if (stage + 4096 > lds_max) return fhip::set_error(FHIP_ERR_SHAPE, "gemv_quad: %zu bytes of staged activations do not fit the workgroup's LDS", stage);
    // rows per workgroup: the chip's workgroups share the rows evenly, in whole quads, and a workgroup's group sums fit what is left
    const int step = 4 / VPR;
    long long rows_wg = ((long long)out_rows + cus - 1) / cus;
    rows_wg = (rows_wg + step - 1) / step * step;
    const long long max_rows = (long long)((lds_max - stage) / ((size_t)VPR * p.NG * 16)) / step * step;
    if (max_rows < step) return fhip::set_error(FHIP_ERR_SHAPE, "gemv_quad: rows of %zu columns are too long", w->cols);
    if (rows_wg > max_rows) rows_wg = max_rows;
    p.rows_wg = (int)rows_wg;
    const int quads = (int)(rows_wg * VPR / 4);
    if (p.QS > quads) p.QS = quads;                      // no wave without a quad
    const unsigned grid = (unsigned)((out_rows + rows_wg - 1) / rows_wg);
    const unsigned threads = 64u * (unsigned)(p.WPS * p.QS);
    // 8-column pieces of a pass (4 rows x 16 WPL WPS columns) per thread
    const unsigned S = (unsigned)(F::WPL / 8) * 16u * (unsigned)p.WPS;
    p.pieces = (int)((4 * (size_t)S + threads - 1) / threads);
    p.magic_S = (uint32_t)(((1ull << 32) + S - 1) / S);
    p.step_m = (int)(threads / S); p.step_slot = (int)(threads % S);
    const size_t lds = stage + (size_t)rows_wg * VPR * p.NG * 16;
    static bool lds_raised = false;
    if (!lds_raised) {  // workgroups may use more than the default 64 KiB of the CU's 160 KiB
        (void)hipFuncSetAttribute((const void*)gemv_quad_kernel<F, SWIGLU>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_max);
        (void)hipGetLastError();
        lds_raised = true;
    }
    hipLaunchKernelGGL((gemv_quad_kernel<F, SWIGLU>), dim3(grid), dim3(threads), lds, s, p);
    return fhip::check_hip(hipGetLastError(), "gemv_quad launch");
}

}  // namespace

namespace fhip {

bool QUAD_EXPORT(gemv_quad_supports)(const fhip_weight* w, size_t rows_x, size_t n_ff) {
    if (!w || (w->type != FHIP_Q4_K && w->type != FHIP_Q5_K && w->type != FHIP_Q6_K && w->type != FHIP_Q8_0)) return false;
    if (rows_x < 1 || rows_x > 4 || w->cols == 0 || w->rows == 0) return false;
    // Q8_0: no fused SwiGLU (the reference has none), and rows the kernel covers in one pass (ten groups of 16 blocks): longer
    // rows have the four-row dot-product kernel, one pass whatever their length
    if (w->type == FHIP_Q8_0 ? (n_ff != 0 || w->cols % 32 != 0 || w->cols > 5120) : w->cols % 256 != 0) return false;
    if (n_ff ? w->rows != 2 * n_ff : false) return false;
    const size_t out_rows = n_ff ? n_ff : w->rows;
    // 32-bit byte offsets inside a workgroup's span and to the up row of a pair
    if (w->row_bytes > 0xFFFFu * 4 || out_rows * w->row_bytes > 0xF0000000ull) return false;
    // only where one or two rows would take the streaming kernel: its bits are what this kernel promises (the longest rows go to
    // the shape-complete f32 kernel instead)
    return w->cols <= 32768 && ((uintptr_t)w->d_raw & 15) == 0 && QUAD_EXPORT(gemv_streams)(w, n_ff);
}

// y [rows_x, out_rows] = x [rows_x, cols] W^T (n_ff != 0: silu(gate) * up over the fused [gate | up] rows), rows_x <= 4
int QUAD_EXPORT(launch_gemv_quad)(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, size_t n_ff, hipStream_t s) {
    if (!QUAD_EXPORT(gemv_quad_supports)(w, rows_x, n_ff)) return set_error(FHIP_ERR_ARG, "gemv_quad: unsupported weight or batch");
    const size_t out_rows = n_ff ? n_ff : w->rows;
    if (w->type == FHIP_Q4_K) return n_ff ? launch_quad<Q4K, true>(w, d_x, rows_x, d_y, out_rows, s) : launch_quad<Q4K, false>(w, d_x, rows_x, d_y, out_rows, s);
    if (w->type == FHIP_Q8_0) return launch_quad<Q80, false>(w, d_x, rows_x, d_y, out_rows, s);
    if (w->type == FHIP_Q5_K) return n_ff ? launch_quad<Q5K, true>(w, d_x, rows_x, d_y, out_rows, s) : launch_quad<Q5K, false>(w, d_x, rows_x, d_y, out_rows, s);
    return n_ff ? launch_quad<Q6K, true>(w, d_x, rows_x, d_y, out_rows, s) : launch_quad<Q6K, false>(w, d_x, rows_x, d_y, out_rows, s);
}

}  // namespace fhip
