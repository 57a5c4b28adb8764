// Small-batch (1..32 activation rows) quantized matmul on the f16 matrix cores with f32-grade results, gfx950:
//     Y[t, n] = sum_k X[t, k] * dequant(W[n, k]),   X f32 [T, K], W raw GGUF blocks [N, K], Y f32 [T, N]
//
// Stands for Tensor::matmul_q with a few activation rows (crates/ferric-tensor/src/dtype.rs:935-944; kernels
// :2995-3051 Q4_K, :3423-3469 Q6_K), which the reference runs as one thread per output walking the weight row: the
// weights are re-read per activation row there. Here one pass over the weights serves every row.
//
// How the matrix cores give f32-grade results from 16-bit operands:
//   * Weights. A K-quant weight is (super-block scale d) x (small integer): d * (sc * q) - dmin * (m) for Q4_K with
//     sc, m < 64 and q < 16, d * (sc * (q - 32)) for Q6_K. The integer factor sc*q <= 945 is exact in f16, so the B
//     operand holds sc*q as f16 and the f32 factor d is applied to the f32 accumulator once per super-block. The Q4_K
//     minima are one more MFMA per super-block: sum_sb m[n, sb] * (sum of the activations of sub-block sb). (Q6_K:
//     |sc*(q-32)| can reach 4096; products above 2048 are rounded to even, a relative 2^-12 on those weights.)
//     Q8_0 (:2948-2990) is d * (int8): the B operand holds the quant, the f32 result of every 32-wide slice takes its
//     block's d.
//   * Activations. The 256 columns of a chunk of a row are scaled by a power of two so that their largest magnitude
//     lies in [2^14, 2^15), then split into hi = f16(x) and lo = f16(x - hi): two operand rows per activation row, 22
//     significant bits at the chunk's maximum. The 16 rows of a v_mfma_f32_16x16x32_f16 hold hi and lo of 8 activation
//     rows; a chunk's f32 result takes the chunk's scale out again as it joins the total, and the two partial results
//     are added in f32 at the end. (A scale per chunk, not per row: the preparation needs no pass over the whole row in
//     front of it -- one launch less per matmul -- and a chunk of small values keeps its bits beside a large one.)
//   * Unpack cost. A lane turns a dword of 8 nibbles into 8 f16 with 1 shift, 4 and-or (the nibble lands in the
//     mantissa of the f16 constant 1024 or, for the high nibble, 16 positions up) and 4 packed f16 fma that remove the
//     constant and apply the sub-block scale: 9 VALU for 8 weights, against ~30 for the bf16 path's f32 arithmetic.
//     The k order inside an MFMA is free as long as both operands agree, so the activations are laid out in the
//     order the nibbles come out (xsplit_f16_kernel does that once per call).
//
// Lane (g4 = lane / 16, c = lane % 16) of a wave works on weight row c of a 16-row set and on k-group g4 of each
// 32-wide MFMA slice; a wave carries two row sets (32 weight rows), a workgroup four waves (128 rows; the row-streaming
// kernel for up to 8 activation rows: eight waves, 256 rows). The (row group, 256-column chunk) units are dealt to the workgroups in equal contiguous runs; a run that covers its
// group's whole K stores, any other adds atomically into a Y cleared beforehand (or, when the caller asks for ordered sums, stores
// into a slot of its own that sum_split_kernel adds in contributor order).
#include "common.hpp"
#include <algorithm>
#include "loads.hpp"

#include <hip/hip_fp16.h>

#include <cmath>
#include <type_traits>

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float f16_bits(uint32_t b) { return __half2float(__ushort_as_half((unsigned short)b)); }
__device__ __forceinline__ uint32_t hfma2(uint32_t v, uint32_t s, uint32_t c) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(f16x2, v), __builtin_bit_cast(f16x2, s),
                                                                  __builtin_bit_cast(f16x2, c)));
}
__device__ __forceinline__ uint32_t hmul2(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, a) * __builtin_bit_cast(f16x2, b));
}
__device__ __forceinline__ uint32_t hadd2(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, a) + __builtin_bit_cast(f16x2, b));
}
__device__ __forceinline__ uint32_t splat_h(_Float16 h) { return __builtin_bit_cast(uint32_t, (f16x2){h, h}); }
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t m, uint32_t o) { return (a & m) | o; }

constexpr uint32_t H1024 = 0x64006400u;      // f16 pair (1024, 1024): mantissa step 1
constexpr uint32_t H64 = 0x54005400u;        // f16 pair (64, 64): mantissa step 1/16
constexpr uint32_t HNEG1024 = 0xE400E400u;   // (-1024, -1024)
constexpr uint32_t HNEG64 = 0xD400D400u;     // (-64, -64)
constexpr uint32_t HNEG96 = 0xD600D600u;     // (-96, -96)
constexpr uint32_t H16TH = 0x2C002C00u;      // (1/16, 1/16)

struct __attribute__((packed, aligned(2))) U4A2 { u32x4 v; };   // 16 bytes at an address that is only 2-byte aligned

constexpr int CHUNK = 256;   // columns per chunk: one K-quant super-block
// f16 per staged operand row of a chunk: 256 activations, 8 sub-block sums, 8 zeros, then the f32 factor that takes the
// chunk's scale out again (two f16 places) and 6 of padding (row stride 35 x 16 bytes: the 16 rows a 16-byte read
// instruction touches fall into different bank groups)
constexpr int XR = 280;
constexpr int XSCALE = 272;   // column of the f32 factor

__host__ __device__ constexpr int p4(int j) { return ((j & 1) << 1) | (j >> 1); }   // 0, 2, 1, 3: byte pairs (b0,b2), (b1,b3)

template <int I, int N, class Fn>
__device__ __forceinline__ void static_for(Fn&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// ------------------------------------------------------------------------------------------------
// Per-format weight streams. `Raw` is the register image of the bytes of one chunk of one weight row that lane
// k-group g4 unpacks; pre<I>() derives the scales slice I is the first to need; frag<I>() is the B operand of slice I (8 per chunk): the
// 8 weights this lane contributes, as integers times their sub-block scale; src_k(pos) is the column (inside the chunk)
// whose activation belongs at operand position pos = (I * 4 + g4) * 8 + j.
// ------------------------------------------------------------------------------------------------

struct Q4K {
    static constexpr int BLOCK = 144;
    static constexpr bool HAS_MIN = true;
    static __host__ __device__ constexpr int occupancy(int nt) { return nt == 1 ? 4 : (nt == 2 ? 3 : 2); }   // workgroups per CU the registers allow
    // lane g4 owns bytes qs[32 g4, +32): the low nibbles are sub-block 2 g4, the high nibbles 2 g4 + 1
    // (crates/ferric-gguf/src/lib.rs:805-823); slice I is dword I of those, j < 4 its low, j >= 4 its high nibbles.
    static __host__ __device__ constexpr int src_k(int pos) {
        const int j = pos & 7, g4 = (pos >> 3) & 3, i = pos >> 5;
        return 64 * g4 + 32 * (j >> 2) + 4 * i + p4(j & 3);
    }
    static __host__ __device__ constexpr int pos_of(int k) {   // inverse of src_k
        return (((k >> 2) & 7) * 4 + (k >> 6)) * 8 + 4 * ((k >> 5) & 1) + p4(k & 3);
    }
    struct Raw { u32x4 hd, q0, q1; };
    struct Head { u32x4 hd; };
    struct Ctx { uint32_t s0, c0, s1, c1; float d, dm; int sh; };   // sh: Q5_K's shift to its fifth-bit planes
    static __device__ __forceinline__ void prime(Raw& r, const uint8_t* row, int c, int g4) {
        const uint8_t* blk = row + (size_t)c * BLOCK;
        r.hd = *(const u32x4*)blk;
        r.q0 = *(const u32x4*)(blk + 16 + 32 * g4);
        r.q1 = *(const u32x4*)(blk + 32 + 32 * g4);
    }
    static __device__ __forceinline__ void head(Head& h, const uint8_t* row, int c) { h.hd = *(const u32x4*)(row + (size_t)c * BLOCK); }
    // row-streaming kernel: a block is PARTS 16-byte pieces in global memory and a row of LROW bytes in the wave's LDS image
    static constexpr int PARTS = 9, LROW = 144, TAILS = 0, ROWS_OCCUPANCY = 3;   // (workgroups of the four-wave row-streaming kernel per CU)
    static constexpr bool ROWS_AT_16 = false;   // 9..16 rows, cold weights: 44.9 us against 42.0 us for the one-row-per-lane kernel
    static constexpr bool ROW_PER_LANE = true, SLICE_SCALE = false;
    static __device__ __forceinline__ u32x4 ldg(const uint8_t* p) { return *(const u32x4*)p; }
    // where 16-byte piece `part` of chunk ck starts in the weight row / in the LDS row (tails: 2-byte pieces)
    static __device__ __forceinline__ uint32_t piece_off(int ck, int part, int) { return (uint32_t)(ck * BLOCK + 16 * part); }
    static __device__ __forceinline__ int piece_lds(int part) { return 16 * part; }
    static __device__ __forceinline__ uint32_t tail_off(int, int, int, bool& live) { live = false; return 0; }
    static __device__ __forceinline__ int tail_lds(int) { return 0; }
    static __device__ __forceinline__ void from_lds(Raw& r, const uint8_t* row, int g4) {
        r.hd = *(const u32x4*)row;
        r.q0 = *(const u32x4*)(row + 16 + 32 * g4);
        r.q1 = *(const u32x4*)(row + 32 + 32 * g4);
    }
    static __device__ __forceinline__ void take(Raw& r, const Head& h) { r.hd = h.hd; }
    // after slice I the registers it was the last to read are reloaded with the same bytes of chunk nc
    template <int I>
    static __device__ __forceinline__ void refill(Raw& r, const uint8_t* row, int nc, int g4) {
        const uint8_t* blk = row + (size_t)nc * BLOCK;
        if (I == 3) r.q0 = *(const u32x4*)(blk + 16 + 32 * g4);
        if (I == 7) r.q1 = *(const u32x4*)(blk + 32 + 32 * g4);
    }
    // get_sc_min (crates/ferric-gguf/src/lib.rs:795-804) as bytes: scales 0..3 / 4..7 and minima 0..3 / 4..7
    static __device__ __forceinline__ uint32_t sc_bytes(const u32x4& hd, bool upper) {
        return upper ? ((hd[3] & 0x0F0F0F0Fu) | ((hd[1] >> 2) & 0x30303030u)) : (hd[1] & 0x3F3F3F3Fu);
    }
    static __device__ __forceinline__ uint32_t min_bytes(const u32x4& hd, bool upper) {
        return upper ? (((hd[3] >> 4) & 0x0F0F0F0Fu) | ((hd[2] >> 2) & 0x30303030u)) : (hd[2] & 0x3F3F3F3Fu);
    }
    template <int I>
    static __device__ __forceinline__ void pre(const Raw& r, int g4, Ctx& x) {
        if (I != 0) return;
        const uint32_t scw = sc_bytes(r.hd, g4 >= 2) >> (16 * (g4 & 1));
        const uint32_t s0 = splat_h((_Float16)(unsigned short)(scw & 0xFFu)), s1 = splat_h((_Float16)(unsigned short)((scw >> 8) & 0xFFu));
        // low nibble: (1024 + q) * sc - 1024 sc; high nibble in place: (1024 + 16 q) * (sc / 16) - 64 sc. All exact in f16.
        x.s0 = s0; x.c0 = hmul2(s0, HNEG1024);
        x.s1 = hmul2(s1, H16TH); x.c1 = hmul2(s1, HNEG64);
        x.d = f16_bits(r.hd[0] & 0xFFFFu);
        x.dm = -64.0f * f16_bits(r.hd[0] >> 16);   // the sub-block sums are staged divided by 64
    }
    template <int I>
    static __device__ __forceinline__ f16x8 frag(const Raw& r, const Ctx& x) {
        const uint32_t w = I < 4 ? r.q0[I & 3] : r.q1[I & 3], w8 = w >> 8;
        u32x4 o;
        o[0] = hfma2(and_or(w, 0x000F000Fu, H1024), x.s0, x.c0);
        o[1] = hfma2(and_or(w8, 0x000F000Fu, H1024), x.s0, x.c0);
        o[2] = hfma2(and_or(w, 0x00F000F0u, H1024), x.s1, x.c1);
        o[3] = hfma2(and_or(w8, 0x00F000F0u, H1024), x.s1, x.c1);
        return __builtin_bit_cast(f16x8, o);
    }
    // B operand of the minima MFMA: m[0..7] of this row as f16 in k-group 0, zeros in the others
    static __device__ __forceinline__ f16x8 mins(const Raw& r, int g4) {
        const uint32_t lo = min_bytes(r.hd, false), hi = min_bytes(r.hd, true);
        u32x4 o;
        o[0] = hadd2(__builtin_amdgcn_perm(0x64646464u, lo, 0x04010400u), HNEG1024);
        o[1] = hadd2(__builtin_amdgcn_perm(0x64646464u, lo, 0x04030402u), HNEG1024);
        o[2] = hadd2(__builtin_amdgcn_perm(0x64646464u, hi, 0x04010400u), HNEG1024);
        o[3] = hadd2(__builtin_amdgcn_perm(0x64646464u, hi, 0x04030402u), HNEG1024);
        if (g4 != 0) o = (u32x4){0u, 0u, 0u, 0u};
        return __builtin_bit_cast(f16x8, o);
    }
};

// Q5_K (crates/ferric-gguf/src/lib.rs:687-716): Q4_K's header and nibbles with 32 bytes in between that hold a fifth bit
// for every weight: bit 2 g4 of qh[l] belongs to the low nibble of qs[32 g4 + l], bit 2 g4 + 1 to its high nibble. The
// operand order, the scales and the minima are Q4_K's; codes up to 31 times scales up to 63 are still exact in f16.
struct Q5K {
    static constexpr int BLOCK = 176;
    static constexpr bool HAS_MIN = true;
    static __host__ __device__ constexpr int occupancy(int nt) { return nt == 1 ? 3 : 2; }
    static __host__ __device__ constexpr int src_k(int pos) { return Q4K::src_k(pos); }
    static __host__ __device__ constexpr int pos_of(int k) { return Q4K::pos_of(k); }
    struct Raw { u32x4 hd, h0, h1, q0, q1; };
    struct Head { u32x4 hd; };
    typedef Q4K::Ctx Ctx;
    static __device__ __forceinline__ void prime(Raw& r, const uint8_t* row, int c, int g4) {
        const uint8_t* blk = row + (size_t)c * BLOCK;
        r.hd = *(const u32x4*)blk;
        r.h0 = *(const u32x4*)(blk + 16);
        r.h1 = *(const u32x4*)(blk + 32);
        r.q0 = *(const u32x4*)(blk + 48 + 32 * g4);
        r.q1 = *(const u32x4*)(blk + 64 + 32 * g4);
    }
    static __device__ __forceinline__ void head(Head& h, const uint8_t* row, int c) { h.hd = *(const u32x4*)(row + (size_t)c * BLOCK); }
    static constexpr int PARTS = 11, LROW = 176, TAILS = 0, ROWS_OCCUPANCY = 3;   // (workgroups of the four-wave row-streaming kernel per CU)
    static constexpr bool ROWS_AT_16 = false;
    static constexpr bool ROW_PER_LANE = true, SLICE_SCALE = false;
    static __device__ __forceinline__ u32x4 ldg(const uint8_t* p) { return *(const u32x4*)p; }
    static __device__ __forceinline__ uint32_t piece_off(int ck, int part, int) { return (uint32_t)(ck * BLOCK + 16 * part); }
    static __device__ __forceinline__ int piece_lds(int part) { return 16 * part; }
    static __device__ __forceinline__ uint32_t tail_off(int, int, int, bool& live) { live = false; return 0; }
    static __device__ __forceinline__ int tail_lds(int) { return 0; }
    static __device__ __forceinline__ void from_lds(Raw& r, const uint8_t* row, int g4) {
        r.hd = *(const u32x4*)row;
        r.h0 = *(const u32x4*)(row + 16);
        r.h1 = *(const u32x4*)(row + 32);
        r.q0 = *(const u32x4*)(row + 48 + 32 * g4);
        r.q1 = *(const u32x4*)(row + 64 + 32 * g4);
    }
    static __device__ __forceinline__ void take(Raw& r, const Head& h) { r.hd = h.hd; }
    template <int I>
    static __device__ __forceinline__ void refill(Raw& r, const uint8_t* row, int nc, int g4) {
        const uint8_t* blk = row + (size_t)nc * BLOCK;
        if (I == 3) { r.h0 = *(const u32x4*)(blk + 16); r.q0 = *(const u32x4*)(blk + 48 + 32 * g4); }
        if (I == 7) { r.h1 = *(const u32x4*)(blk + 32); r.q1 = *(const u32x4*)(blk + 64 + 32 * g4); }
    }
    template <int I>
    static __device__ __forceinline__ void pre(const Raw& r, int g4, Ctx& x) {
        if (I != 0) return;
        const uint32_t scw = Q4K::sc_bytes(r.hd, g4 >= 2) >> (16 * (g4 & 1));
        const uint32_t s0 = splat_h((_Float16)(unsigned short)(scw & 0xFFu)), s1 = splat_h((_Float16)(unsigned short)((scw >> 8) & 0xFFu));
        x.s0 = s0; x.c0 = hmul2(s0, HNEG1024);
        x.s1 = hmul2(s1, H16TH); x.c1 = hmul2(s1, HNEG64);
        x.d = f16_bits(r.hd[0] & 0xFFFFu);
        x.dm = -64.0f * f16_bits(r.hd[0] >> 16);
        // the two fifth-bit planes of this lane's sub-blocks, moved to bits 0 and 1 of every byte once for the chunk
        x.sh = 2 * g4;
    }
    // the fifth bit is worth 16: mantissa bit 4 beside a low nibble (step 1), bit 8 beside a high nibble in place (step 1/16)
    template <int I>
    static __device__ __forceinline__ f16x8 frag(const Raw& r, const Ctx& x) {
        const uint32_t w = I < 4 ? r.q0[I & 3] : r.q1[I & 3], w8 = w >> 8;
        const uint32_t hb = (I < 4 ? r.h0[I & 3] : r.h1[I & 3]) >> x.sh;
        u32x4 o;
        o[0] = hfma2(and_or(w, 0x000F000Fu, H1024) | ((hb << 4) & 0x00100010u), x.s0, x.c0);
        o[1] = hfma2(and_or(w8, 0x000F000Fu, H1024) | ((hb >> 4) & 0x00100010u), x.s0, x.c0);
        o[2] = hfma2(and_or(w, 0x00F000F0u, H1024) | ((hb << 7) & 0x01000100u), x.s1, x.c1);
        o[3] = hfma2(and_or(w8, 0x00F000F0u, H1024) | ((hb >> 1) & 0x01000100u), x.s1, x.c1);
        return __builtin_bit_cast(f16x8, o);
    }
    static __device__ __forceinline__ f16x8 mins(const Raw& r, int g4) {
        Q4K::Raw q;
        q.hd = r.hd;
        return Q4K::mins(q, g4);
    }
};

struct Q6K {
    static constexpr int BLOCK = 210;
    static constexpr bool HAS_MIN = false;
    static __host__ __device__ constexpr int occupancy(int nt) { return nt == 1 ? 3 : (nt == 2 ? 2 : 1); }
    // lane g4 = (hf, lh) owns l in [16 lh, 16 lh + 16) of half hf (crates/ferric-gguf/src/lib.rs:833-851): slice I = (par, dd) is
    // dword dd of ql[64 hf + 32 par + 16 lh ..] and of qh[32 hf + 16 lh ..]; j < 4 are the low nibbles (quarter par of the
    // half, high bits in field par of the qh byte), j >= 4 the high nibbles (quarter par + 2, field par + 2). All of a
    // lane's l share l / 16 = lh, so it needs four scales a chunk: sc[8 hf + 2 qt + lh].
    static __host__ __device__ constexpr int src_k(int pos) {
        const int j = pos & 7, g4 = (pos >> 3) & 3, i = pos >> 5;
        const int hf = g4 >> 1, lh = g4 & 1, par = i >> 2, dd = i & 3;
        return 128 * hf + 32 * (par + 2 * (j >> 2)) + 16 * lh + 4 * dd + p4(j & 3);
    }
    static __host__ __device__ constexpr int pos_of(int k) {   // inverse of src_k
        const int hf = k >> 7, qt = (k >> 5) & 3, lh = (k >> 4) & 1, dd = (k >> 2) & 3;
        return ((4 * (qt & 1) + dd) * 4 + 2 * hf + lh) * 8 + 4 * (qt >> 1) + p4(k & 3);
    }
    struct Raw { u32x4 ql[2], qh, sc; uint32_t d; };
    struct Head { u32x4 sc; uint32_t d; };
    struct Ctx { uint32_t s[4]; float d, dm; };
    static __device__ __forceinline__ u32x4 ld16(const uint8_t* p) { return fhip::load16_a2(p); }   // blocks of 210 bytes
    static __device__ __forceinline__ void head(Head& h, const uint8_t* row, int c) {
        const uint8_t* blk = row + (size_t)c * BLOCK;
        h.sc = ld16(blk + 192);
        h.d = *(const uint16_t*)(blk + 208);
    }
    static __device__ __forceinline__ void take(Raw& r, const Head& h) { r.sc = h.sc; r.d = h.d; }
    // row-streaming kernel: 13 16-byte pieces + the 2-byte d; LDS rows of 240 bytes (a multiple of 16 whose dword count,
    // 60, puts the 16 rows of a read instruction into different banks). Contiguous lanes read contiguous bytes here, which
    // the 2-byte alignment of the blocks does not slow down.
    static constexpr int PARTS = 13, LROW = 240, TAILS = 1, ROWS_OCCUPANCY = 3;   // (workgroups of the four-wave row-streaming kernel per CU)
    static constexpr bool ROWS_AT_16 = true;    // 9..16 rows, cold weights: 33.2 us against 41.2 us
    static constexpr bool ROW_PER_LANE = true, SLICE_SCALE = false;
    static __device__ __forceinline__ u32x4 ldg(const uint8_t* p) { return ((const U4A2*)p)->v; }
    static __device__ __forceinline__ uint32_t piece_off(int ck, int part, int) { return (uint32_t)(ck * BLOCK + 16 * part); }
    static __device__ __forceinline__ int piece_lds(int part) { return 16 * part; }
    static __device__ __forceinline__ uint32_t tail_off(int ck, int, int, bool& live) { live = true; return (uint32_t)(ck * BLOCK + 208); }
    static __device__ __forceinline__ int tail_lds(int) { return 208; }
    static __device__ __forceinline__ void from_lds(Raw& r, const uint8_t* row, int g4) {
        const int hf = g4 >> 1, lh = g4 & 1;
        r.ql[0] = *(const u32x4*)(row + 64 * hf + 16 * lh);
        r.ql[1] = *(const u32x4*)(row + 64 * hf + 32 + 16 * lh);
        r.qh = *(const u32x4*)(row + 128 + 32 * hf + 16 * lh);
        r.sc = *(const u32x4*)(row + 192);
        r.d = *(const uint16_t*)(row + 208);
    }
    static __device__ __forceinline__ void prime(Raw& r, const uint8_t* row, int c, int g4) {
        const uint8_t* blk = row + (size_t)c * BLOCK;
        const int hf = g4 >> 1, lh = g4 & 1;
        r.ql[0] = ld16(blk + 64 * hf + 16 * lh);
        r.ql[1] = ld16(blk + 64 * hf + 32 + 16 * lh);
        r.qh = ld16(blk + 128 + 32 * hf + 16 * lh);
        r.sc = ld16(blk + 192);
        r.d = *(const uint16_t*)(blk + 208);
    }
    // after slice I the registers it was the last to read are reloaded with the same bytes of chunk nc
    template <int I>
    static __device__ __forceinline__ void refill(Raw& r, const uint8_t* row, int nc, int g4) {
        const uint8_t* blk = row + (size_t)nc * BLOCK;
        const int hf = g4 >> 1, lh = g4 & 1;
        if (I == 3) r.ql[0] = ld16(blk + 64 * hf + 16 * lh);
        if (I == 7) {
            r.ql[1] = ld16(blk + 64 * hf + 32 + 16 * lh);
            r.qh = ld16(blk + 128 + 32 * hf + 16 * lh);
        }
    }
    template <int I>
    static __device__ __forceinline__ void pre(const Raw& r, int g4, Ctx& x) {
        if (I != 0) return;
        const int hf = g4 >> 1, lh = g4 & 1;
        const uint32_t w0 = (hf ? r.sc[2] : r.sc[0]) >> (8 * lh), w1 = (hf ? r.sc[3] : r.sc[1]) >> (8 * lh);
#pragma unroll
        for (int qt = 0; qt < 4; qt++) {
            const uint32_t w = qt < 2 ? w0 : w1;
            const int v = (int)(int8_t)((w >> (16 * (qt & 1))) & 0xFFu);
            const uint32_t sp = splat_h((_Float16)(short)v);
            x.s[qt] = sp;
        }
        x.d = f16_bits(r.d);
        x.dm = 0.f;
    }
    template <int I>
    static __device__ __forceinline__ f16x8 frag(const Raw& r, const Ctx& x) {
        constexpr int par = I >> 2, dd = I & 3, flo = par, fhi = par + 2;
        const uint32_t ql = r.ql[par][dd], qh = r.qh[dd];
        constexpr uint32_t NM = 0x00F000F0u, HM = 0x03000300u;
        // a 6-bit q lands in mantissa bits 4..9 of the f16 constant 64 (step 1/16): the value is 64 + q
        const uint32_t p0 = and_or(qh << (8 - 2 * flo), HM, and_or(ql << 4, NM, H64));
        const uint32_t p1 = and_or(qh >> (2 * flo), HM, and_or(ql >> 4, NM, H64));
        const uint32_t p2 = and_or(qh << (8 - 2 * fhi), HM, and_or(ql, NM, H64));
        const uint32_t p3 = and_or(qh >> (2 * fhi), HM, and_or(ql >> 8, NM, H64));
        u32x4 o;
        const uint32_t clo = hmul2(x.s[flo], HNEG96), chi = hmul2(x.s[fhi], HNEG96);   // (64 + q) * sc - 96 sc = (q - 32) * sc
        o[0] = hfma2(p0, x.s[flo], clo);
        o[1] = hfma2(p1, x.s[flo], clo);
        o[2] = hfma2(p2, x.s[fhi], chi);
        o[3] = hfma2(p3, x.s[fhi], chi);
        return __builtin_bit_cast(f16x8, o);
    }
    static __device__ __forceinline__ f16x8 mins(const Raw&, int) { return (f16x8){0, 0, 0, 0, 0, 0, 0, 0}; }
};


// Q8_0: 34-byte blocks of 32 int8 under one f16 scale (crates/ferric-gguf/src/lib.rs:855-872), eight blocks to a chunk.
// Only the row-streaming kernel reads it. A weight enters the B operand as the exact integer q; the block's scale is
// applied to the f32 result of each 32-wide slice, which is one block. The LDS row is the chunk's 256 quants followed
// by its 8 scales: 272 bytes, 68 dwords, so the 8-byte reads of a half wave (16 rows x 2 k-groups) cover all 64 banks.
struct Q80 {
    static constexpr int BLOCK = 34;
    static constexpr bool HAS_MIN = false;
    static __host__ __device__ constexpr int occupancy(int) { return 2; }
    static __host__ __device__ constexpr int src_k(int pos) { return pos; }   // slice I is block I, in order
    static __host__ __device__ constexpr int pos_of(int k) { return k; }
    static constexpr int PARTS = 16, LROW = 272, TAILS = 8, ROWS_OCCUPANCY = 3;   // (workgroups of the four-wave row-streaming kernel per CU)
    static constexpr bool ROWS_AT_16 = true;
    static constexpr bool ROW_PER_LANE = false, SLICE_SCALE = true;
    static __device__ __forceinline__ u32x4 ldg(const uint8_t* p) { return ((const U4A2*)p)->v; }
    // a row that ends inside its last chunk: the blocks past the end re-read the last real block and get scale 0
    static __device__ __forceinline__ uint32_t piece_off(int ck, int part, int nblk) {
        const int b = 8 * ck + (part >> 1);
        return (uint32_t)(BLOCK * (b < nblk ? b : nblk - 1) + 2 + 16 * (part & 1));
    }
    static __device__ __forceinline__ int piece_lds(int part) { return 16 * part; }
    static __device__ __forceinline__ uint32_t tail_off(int ck, int t, int nblk, bool& live) {
        const int b = 8 * ck + t;
        live = b < nblk;
        return (uint32_t)(BLOCK * (live ? b : nblk - 1));
    }
    static __device__ __forceinline__ int tail_lds(int t) { return 256 + 2 * t; }
    struct Raw { const uint8_t* row; };
    struct Ctx { float d, dm; };
    static __device__ __forceinline__ void from_lds(Raw& r, const uint8_t* row, int g4) { r.row = row + 8 * g4; }
    template <int I>
    static __device__ __forceinline__ void pre(const Raw& r, int g4, Ctx& x) {
        x.d = f16_bits(*(const uint16_t*)(r.row - 8 * g4 + 256 + 2 * I));
        x.dm = 0.f;
    }
    template <int I>
    static __device__ __forceinline__ f16x8 frag(const Raw& r, const Ctx&) {
        const u32x2 q = *(const u32x2*)(r.row + 32 * I);
        // int8 q -> the byte q + 128 in the mantissa of the f16 constant 1024 -> minus 1152
        const uint32_t a = q[0] ^ 0x80808080u, b = q[1] ^ 0x80808080u;
        constexpr uint32_t HNEG1152 = 0xE480E480u;
        u32x4 o;
        o[0] = hadd2(__builtin_amdgcn_perm(0x64646464u, a, 0x04010400u), HNEG1152);
        o[1] = hadd2(__builtin_amdgcn_perm(0x64646464u, a, 0x04030402u), HNEG1152);
        o[2] = hadd2(__builtin_amdgcn_perm(0x64646464u, b, 0x04010400u), HNEG1152);
        o[3] = hadd2(__builtin_amdgcn_perm(0x64646464u, b, 0x04030402u), HNEG1152);
        return __builtin_bit_cast(f16x8, o);
    }
    static __device__ __forceinline__ f16x8 mins(const Raw&, int) { return (f16x8){0, 0, 0, 0, 0, 0, 0, 0}; }
};

// ------------------------------------------------------------------------------------------------
// Activation preparation, one short kernel. Output per chunk: 16 NT operand rows of XR f16 (rows 16 q + i, i < 8: hi of
// activation row 8 q + i; rows 16 q + 8 + i: its lo), columns in operand order (F::pos_of), followed by the 8 sub-block
// sums / 64 (formats with minima), zeros, and the f32 factor that takes the chunk's power-of-two scale out again.
// SWIGLU: the row is silu(gate) * up of a [T, 2d] = [gate | up] matrix (crates/ferric-tensor/src/lib.rs:2603-2618).
// ------------------------------------------------------------------------------------------------
constexpr int MAXW = 64;   // rows of up to 65 536 columns

// Workgroup b of G takes units [b U / G, (b + 1) U / G): the workgroup that holds unit u
__device__ __host__ __forceinline__ int holder_of(long long u, long long G, long long U) { return (int)(((u + 1) * G - 1) / U); }

// element n of row t of the matrix the split reads: as stored, or, where the producing matmul left a K-split group's
// partial sums to this launch, slot 0 + slot 1 + ... of that group (the order sum_split_kernel adds them in)
__device__ __forceinline__ float x_at(const float* __restrict__ x, int t, size_t n, const fhip::F16Parts& src) {
    if (src.part) {
        const int gsh = src.group == 256 ? 8 : 7;   // (groups of 128 or 256 outputs)
        const int grp = (int)(n >> gsh);
        const int first = holder_of((long long)grp * src.nchunks, src.grid, src.units);
        const int nk = holder_of((long long)(grp + 1) * src.nchunks - 1, src.grid, src.units) - first + 1;
        if (nk > 1) {
            // (eight slots requested at a time: one trip to memory for the usual three or four contributors instead of one each)
            const float* q = src.part + ((size_t)grp * src.kmax * 32 + t) * src.group + (n & (size_t)(src.group - 1));
            float a = q[0];
            for (int k0 = 1; k0 < nk; k0 += 8) {
                float v[8];
#pragma unroll
                for (int j = 0; j < 8; j++) v[j] = q[(size_t)(k0 + j < nk ? k0 + j : 0) * (32 * (size_t)src.group)];
#pragma unroll
                for (int j = 0; j < 8; j++)
                    if (k0 + j < nk) a += v[j];
            }
            return a;
        }
    }
    return x[n];
}

template <bool SWIGLU>
__device__ __forceinline__ float act(const float* __restrict__ x, int t, int K, int k, const fhip::F16Parts& src) {
    if (SWIGLU) {
        const float g = x_at(x, t, k, src), u = x_at(x, t, (size_t)K + k, src);
        return (g / (1.0f + expf(-g))) * u;
    }
    return x_at(x, t, k, src);
}

// one workgroup per (chunk, operand row of a group of 8): thread k of it converts column k of the chunk
template <class F, bool SWIGLU>
__global__ void __launch_bounds__(256) xsplit_f16_kernel(const float* __restrict__ X, int T, int K, int NT, uint16_t* __restrict__ Xp,
                                                       float* __restrict__ zero, size_t zero_n, fhip::F16Parts src) {
    __shared__ float red[4];
    const int tid = threadIdx.x, lane = tid & 63;
    const size_t nwg = (size_t)gridDim.x * gridDim.y;
    for (size_t k = ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 256 + tid; k < zero_n; k += nwg * 256) zero[k] = 0.f;
    const int ck = blockIdx.x, t = blockIdx.y;
    const bool live = t < T;
    const int k = ck * CHUNK + tid;
    const float* x = X + (size_t)(live ? t : 0) * (SWIGLU ? 2 * (size_t)K : (size_t)K);
    const float raw = (live && k < K) ? act<SWIGLU>(x, live ? t : 0, K, k, src) : 0.f;
    // the chunk's largest magnitude (a NaN is not one: it reaches the operands as it is and makes the output row NaN)
    float m = fabsf(raw);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
    if (lane == 0) red[tid >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float sc = 1.0f, inv = 1.0f;
    if (m > 0.f && m < INFINITY) {
        int ex;
        (void)frexpf(m, &ex);            // m < 2^ex
        ex = ex < -111 ? -111 : ex;      // the scale stays a finite f32; chunks below 2^-111 keep fewer bits
        sc = ldexpf(1.0f, 15 - ex);      // scaled maximum in [2^14, 2^15)
        inv = ldexpf(1.0f, ex - 15);
    }
    const size_t row = ((size_t)(ck * NT + (t >> 3)) * 16 + (t & 7)) * XR;
    auto put = [&](int col, float v) {
        const _Float16 h = (_Float16)v;
        const _Float16 l = (_Float16)(v - (float)h);
        Xp[row + col] = __builtin_bit_cast(uint16_t, h);
        Xp[row + 8 * XR + col] = __builtin_bit_cast(uint16_t, l);
    };
    const float v = raw * sc;
    put(F::pos_of(tid), v);
    // columns 256..263: sub-block sums / 64 (|sum| <= 32 * 2^15, so the quotient stays below 2^14); 264..271: zeros
    float s = F::HAS_MIN ? v : 0.f;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) s += __shfl_xor(s, o);
    if ((tid & 31) == 0) put(CHUNK + (tid >> 5), s * 0.015625f);
    if (tid < 8) put(CHUNK + 8 + tid, 0.f);
    // columns 272, 273 of the hi and the lo row: the factor as f32; 274..279: zeros
    if (tid >= 8 && tid < 16) {
        const uint32_t bits = __float_as_uint(inv);
        const uint16_t w = tid == 8 ? (uint16_t)(bits & 0xFFFFu) : tid == 9 ? (uint16_t)(bits >> 16) : (uint16_t)0;
        Xp[row + XSCALE + (tid - 8)] = w;
        Xp[row + 8 * XR + XSCALE + (tid - 8)] = w;
    }
}

struct F16Params {
    const uint8_t* W;
    const uint16_t* Xp;   // prepared activations: [nchunks][16 NT][XR] f16
    float* Y;             // [T, N]
    int T, N, nchunks;
    int nblk;             // Q8_0: blocks in a weight row (the last chunk may hold fewer than 8)
    size_t row_bytes;
    long long units;      // row groups * nchunks, chunk fastest
    int group;            // rows of a group: 128, or 256 for the eight-wave row-streaming kernel
    float* part;          // null: a run that holds part of a group's K adds into Y atomically. Else it stores its partial sums
                          // into slot (group, contributor) of [groups][kmax][32][group] floats, and sum_split_kernel adds them in order
    int kmax;
};

// where a partial output (activation row t, output n of group grp) goes in ordered mode
__device__ __forceinline__ float* part_slot(const F16Params& p, int grp, int t, int n) {
    const int k = (int)blockIdx.x - holder_of((long long)grp * p.nchunks, gridDim.x, p.units);
    return p.part + (((size_t)grp * p.kmax + k) * 32 + t) * p.group + (n - grp * p.group);
}

template <class F, int NT>
__global__ void __launch_bounds__(256, F::occupancy(NT)) gemm_q_f16x2_kernel(F16Params p) {
    constexpr int ROWS = 16 * NT, PIECES = ROWS * XR / 8, NP = (PIECES + 255) / 256;
    __shared__ __attribute__((aligned(16))) uint16_t Xs[2][ROWS * XR];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g4 = lane >> 4, c = lane & 15;
    const int nchunks = p.nchunks;
    // the units are dealt evenly: workgroup b takes [b U / G, (b + 1) U / G), so every CU carries the same number of them
    long long u = (long long)blockIdx.x * p.units / gridDim.x;
    const long long u_end = (long long)(blockIdx.x + 1) * p.units / gridDim.x;

    u32x4 stage[NP];
    auto load_x = [&](int ck) {
        const u32x4* src = (const u32x4*)(p.Xp + (size_t)ck * ROWS * XR);
#pragma unroll
        for (int q = 0; q < NP; q++)
            if (tid + 256 * q < PIECES) stage[q] = src[tid + 256 * q];
    };
    auto store_x = [&](int buf) {
#pragma unroll
        for (int q = 0; q < NP; q++)
            if (tid + 256 * q < PIECES) ((u32x4*)Xs[buf])[tid + 256 * q] = stage[q];
    };
    const int a_rd = c * XR + 8 * g4;                     // + 16 q XR + 32 I
    const int m_rd = c * XR + CHUNK + (g4 ? 8 : 0);       // sub-block sums for k-group 0, zeros for the others

    for (int seg = 0; u < u_end; seg++) {
        const int grp = (int)(u / nchunks);
        const int c_begin = (int)(u - (long long)grp * nchunks);
        const int c_end = (long long)(nchunks - c_begin) < u_end - u ? nchunks : c_begin + (int)(u_end - u);
        u += c_end - c_begin;
        const bool whole = c_begin == 0 && c_end == nchunks;
        int n[2];
        const uint8_t* wrow[2];
#pragma unroll
        for (int s = 0; s < 2; s++) {
            n[s] = grp * 128 + wave * 32 + 16 * s + c;
            wrow[s] = p.W + (size_t)(n[s] < p.N ? n[s] : p.N - 1) * p.row_bytes;
        }
        f32x4 total[2][NT];
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
            for (int q = 0; q < NT; q++) total[s][q] = (f32x4){0.f, 0.f, 0.f, 0.f};
        // Weight bytes: the quant registers of a chunk are reloaded with the next chunk's bytes as soon as their last slice
        // has read them (half a chunk to a chunk ahead of their use); the few header bytes go through `hd` a chunk ahead.
        typename F::Raw raw[2];
        typename F::Head hd[2];
#pragma unroll
        for (int s = 0; s < 2; s++) F::prime(raw[s], wrow[s], c_begin, g4);
        load_x(c_begin);
        if (seg > 0) __syncthreads();   // the previous segment's last reads of buffer 0 are done
        store_x(0);
        __syncthreads();

        for (int ck = c_begin; ck < c_end; ck++) {
            const int buf = (ck - c_begin) & 1;
            const int cn = ck + 1 < c_end ? ck + 1 : ck;
#pragma unroll
            for (int s = 0; s < 2; s++) F::head(hd[s], wrow[s], cn);
            load_x(cn);
            typename F::Ctx x[2];
            f32x4 acc[2][NT];
#pragma unroll
            for (int s = 0; s < 2; s++)
#pragma unroll
                for (int q = 0; q < NT; q++) acc[s][q] = (f32x4){0.f, 0.f, 0.f, 0.f};
            static_for<0, 8>([&](auto Ic) {
                constexpr int I = decltype(Ic)::value;
                f16x8 a[NT];
#pragma unroll
                for (int q = 0; q < NT; q++) a[q] = *(const f16x8*)(&Xs[buf][a_rd + 16 * q * XR + 32 * I]);
#pragma unroll
                for (int s = 0; s < 2; s++) {
                    F::template pre<I>(raw[s], g4, x[s]);
                    const f16x8 b = F::template frag<I>(raw[s], x[s]);
#pragma unroll
                    for (int q = 0; q < NT; q++) acc[s][q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[q], b, acc[s][q], 0, 0, 0);
                    F::template refill<I>(raw[s], wrow[s], cn, g4);
                }
            });
            // the chunk's f32 result: super-block scale times the integer-weight products (and the minima's term), then the
            // factor that takes the activation scale of the chunk's operand rows 4 g4 + r out again
            float e[NT][4];
#pragma unroll
            for (int q = 0; q < NT; q++)
#pragma unroll
                for (int r = 0; r < 4; r++) e[q][r] = *(const float*)(&Xs[buf][(16 * q + 4 * g4 + r) * XR + XSCALE]);
#pragma unroll
            for (int s = 0; s < 2; s++)
#pragma unroll
                for (int q = 0; q < NT; q++)
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[s][q][r] *= x[s].d;
            if constexpr (F::HAS_MIN) {
                f16x8 am[NT];
#pragma unroll
                for (int q = 0; q < NT; q++) am[q] = *(const f16x8*)(&Xs[buf][m_rd + 16 * q * XR]);
#pragma unroll
                for (int s = 0; s < 2; s++) {
                    const f16x8 bm = F::mins(raw[s], g4);
#pragma unroll
                    for (int q = 0; q < NT; q++) {
                        const f32x4 z = {0.f, 0.f, 0.f, 0.f};
                        const f32x4 accm = __builtin_amdgcn_mfma_f32_16x16x32_f16(am[q], bm, z, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 4; r++) acc[s][q][r] = fmaf(x[s].dm, accm[r], acc[s][q][r]);
                    }
                }
            }
#pragma unroll
            for (int s = 0; s < 2; s++)
#pragma unroll
                for (int q = 0; q < NT; q++)
#pragma unroll
                    for (int r = 0; r < 4; r++) total[s][q][r] = fmaf(e[q][r], acc[s][q][r], total[s][q][r]);
            store_x(buf ^ 1);
            __syncthreads();
#pragma unroll
            for (int s = 0; s < 2; s++) F::take(raw[s], hd[s]);
        }

        // D layout of the 16x16 MFMA: register r of lane (g4, c) is operand row 4 g4 + r, column c. Operand rows 0..7
        // are the hi parts of activation rows 8 q + [0, 8), rows 8..15 their lo parts: lanes g4 and g4 ^ 2 hold the
        // two parts of the same output.
        float* const slot0 = (!whole && p.part) ? part_slot(p, grp, 0, grp * 128) : nullptr;   // (its division once, not per store; p.group = 128 here)
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
            for (int q = 0; q < NT; q++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int t = 8 * q + 4 * (g4 & 1) + r;
                    float v = total[s][q][r];
                    v += __shfl_xor(v, 32);
                    if (g4 < 2 && t < p.T && n[s] < p.N) {
                        float* y = p.Y + (size_t)t * p.N + n[s];
                        if (whole) *y = v;
                        else if (p.part) slot0[t * 128 + (n[s] - grp * 128)] = v;
                        else unsafeAtomicAdd(y, v);
                    }
                }
    }
}

// ------------------------------------------------------------------------------------------------
// Up to 8 activation rows, the same arithmetic with the weight bytes streamed the way the mat-vec kernel streams them: a
// wave fetches the chunk blocks of its 32 rows with contiguous lanes on contiguous bytes (9 lanes per 144-byte Q4_K block,
// 13 + a 2-byte tail per 210-byte Q6_K block), parks them in its own LDS image and reads them back one row per lane. A
// block is requested once, as one run of bytes, and the registers that wait for memory (the next chunk in flight) are not
// the registers in use, so loads are outstanding through all of a chunk's arithmetic. On weights no cache holds (each launch
// on bytes it has not seen) this takes 34 us for a 34816 x 5120 Q4_K weight and 27 us for 5120 x 17408 Q6_K, the kernel
// above 39 and 35.5 us: its one-row-per-lane loads ask for every cache line two or three times, 16 bytes at a time.
// ------------------------------------------------------------------------------------------------
template <class F, int NT, int WAVES>
__global__ void __launch_bounds__(64 * WAVES, WAVES == 8 ? 1 : (NT == 1 ? F::ROWS_OCCUPANCY : 2)) gemm_q_f16x2_rows_kernel(F16Params p) {
    // WAVES = 8 (up to 8 activation rows on the large K-split weights of the FFN block): ONE workgroup of eight waves (256 weight
    // rows) per CU. Three workgroups of four waves, each with its own staged activations, ended far apart -- the younger a workgroup on its CU the later (ends of the first / second / third
    // a CU received 24.2 / 26.0 / 28.8 us on the fused gate|up weight, 17.5 / 21.3 / 24.3 on the down projection), the last
    // one at 32.5 / 27.6 us; eight waves of one age share one staging and one barrier: whole calls 37.4 -> 35.2 and 31.6 -> 30.0 us
    // (twelve waves 35.7 - 36.8 / 30.7, ten 36.4 / 31.2, six 45.3 / 32.0, two workgroups of eight 36.2 / 35.0, of six 37.9 / 35.1).
    // Small weights and weights whose groups are not cut along K keep the four-wave workgroups (at 8 rows, ordered sums, eight waves
    // against four: 4096 x 4096 14.6 against 14.0 us, Q8_0 12288 x 4096 29.0 / 26.6, the vocabulary head 199 / 177).
    constexpr int NTHR = 64 * WAVES, GROUP = 32 * WAVES;
    constexpr int PIECES = 16 * NT * XR / 8, NP = (PIECES + NTHR - 1) / NTHR;
    constexpr int WP = 32 * F::PARTS, NW = (WP + 63) / 64;
    __shared__ __attribute__((aligned(16))) uint16_t Xs[2][16 * NT * XR];
    __shared__ __attribute__((aligned(16))) uint8_t Wl[WAVES][32 * F::LROW];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g4 = lane >> 4, c = lane & 15;
    const int nchunks = p.nchunks;
    // the units are dealt evenly: workgroup b takes [b U / G, (b + 1) U / G), so every CU carries the same number of them
    long long u = (long long)blockIdx.x * p.units / gridDim.x;
    const long long u_end = (long long)(blockIdx.x + 1) * p.units / gridDim.x;

    u32x4 stage[NP];
    auto load_x = [&](int ck) {
        const u32x4* src = (const u32x4*)(p.Xp + (size_t)ck * 16 * NT * XR);
#pragma unroll
        for (int q = 0; q < NP; q++)
            if (tid + NTHR * q < PIECES) stage[q] = src[tid + NTHR * q];
    };
    auto store_x = [&](int buf) {
#pragma unroll
        for (int q = 0; q < NP; q++)
            if (tid + NTHR * q < PIECES) ((u32x4*)Xs[buf])[tid + NTHR * q] = stage[q];
    };
    const int a_rd = c * XR + 8 * g4;
    const int m_rd = c * XR + CHUNK + (g4 ? 8 : 0);

    // piece i * 64 + lane of the wave's chunk image is 16-byte part (piece % PARTS) of row (piece / PARTS)
    uint8_t* const wl = Wl[wave];
    u32x4 G[NW];
    constexpr int NTL = (32 * F::TAILS + 63) / 64;   // 2-byte tail pieces per lane
    uint32_t gt[NTL ? NTL : 1];
    // requests the bytes of unit (row group, chunk); rows past the end of the weight repeat its last row
    auto load_w = [&](int grp, int ck) {
        const int row0 = grp * GROUP + wave * 32 < p.N ? grp * GROUP + wave * 32 : p.N - 1;
        const int rmax = p.N - 1 - row0;
        const uint8_t* b = p.W + (size_t)row0 * p.row_bytes;
#pragma unroll
        for (int i = 0; i < NW; i++) {
            const int pc = i * 64 + lane, row = pc / F::PARTS;
            const uint32_t off = (uint32_t)(row < rmax ? row : rmax) * (uint32_t)p.row_bytes + F::piece_off(ck, pc - row * F::PARTS, p.nblk);
            if (pc < WP) G[i] = F::ldg(b + off);
        }
#pragma unroll
        for (int i = 0; i < NTL; i++) {
            const int tc = i * 64 + lane, row = tc / (F::TAILS ? F::TAILS : 1);
            bool live;
            const uint32_t off = (uint32_t)(row < rmax ? row : rmax) * (uint32_t)p.row_bytes + F::tail_off(ck, tc - row * F::TAILS, p.nblk, live);
            if (tc < 32 * F::TAILS) {
                gt[i] = *(const uint16_t*)(b + off);
                if (!live) gt[i] = 0;
            }
        }
    };
    auto park_w = [&]() {
#pragma unroll
        for (int i = 0; i < NW; i++) {
            const int pc = i * 64 + lane, row = pc / F::PARTS;
            if (pc < WP) *(u32x4*)(wl + row * F::LROW + F::piece_lds(pc - row * F::PARTS)) = G[i];
        }
#pragma unroll
        for (int i = 0; i < NTL; i++) {
            const int tc = i * 64 + lane, row = tc / (F::TAILS ? F::TAILS : 1);
            if (tc < 32 * F::TAILS) *(uint16_t*)(wl + row * F::LROW + F::tail_lds(tc - row * F::TAILS)) = (uint16_t)gt[i];
        }
    };
    if (u >= u_end) return;

    // The workgroup's run of units is one stream: the chunk after a group's last is the next group's first, fetched and
    // parked like any other, so a run that crosses a group boundary pays no second start-up.
    // (group, chunk) of the unit being worked on and of the next one to request: carried along by additions -- a 64-bit
    // division per unit is some hundred scalar instructions, as many cycles of a wave as the unit's arithmetic
    const long long u_begin = u;
    int grp = (int)(u / nchunks), ck = (int)(u - (long long)grp * nchunks);
    int lgrp = grp, lck = ck;
    auto request_next = [&]() {
        load_w(lgrp, lck);
        if (++lck == nchunks) { lck = 0; lgrp++; }
    };
    request_next();
    load_x(ck);
    store_x(0);
    park_w();
    if (u + 1 < u_end) request_next();
    __syncthreads();

    f32x4 total[2][NT];
    for (int it = 0; u < u_end; u++, it++) {
        const int buf = it & 1;
        const bool more = u + 1 < u_end;
        if (more) load_x(ck + 1 < nchunks ? ck + 1 : 0);
        if (u == u_begin || ck == 0) {
#pragma unroll
            for (int s = 0; s < 2; s++)
#pragma unroll
                for (int q = 0; q < NT; q++) total[s][q] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }
        // the factor that takes the activation scale of this chunk's operand rows 4 g4 + r out again
        float e[NT][4];
#pragma unroll
        for (int q = 0; q < NT; q++)
#pragma unroll
            for (int r = 0; r < 4; r++) e[q][r] = *(const float*)(&Xs[buf][(16 * q + 4 * g4 + r) * XR + XSCALE]);
#pragma unroll
        for (int s = 0; s < 2; s++) {
            typename F::Raw raw;
            F::from_lds(raw, wl + (16 * s + c) * F::LROW, g4);
            typename F::Ctx x;
            f32x4 acc[NT], ct[NT];     // the running MFMA result; the chunk's f32 result before the activation scale is taken out
            float dprev = 0.f;
#pragma unroll
            for (int q = 0; q < NT; q++) { acc[q] = (f32x4){0.f, 0.f, 0.f, 0.f}; ct[q] = (f32x4){0.f, 0.f, 0.f, 0.f}; }
            static_for<0, 8>([&](auto Ic) {
                constexpr int I = decltype(Ic)::value;
                F::template pre<I>(raw, g4, x);
                const f16x8 b = F::template frag<I>(raw, x);
                if constexpr (F::SLICE_SCALE) {
                    // every slice has a scale of its own: its product starts from zero, and joins the total while the next
                    // slice's MFMA runs
                    f32x4 cur[NT];
#pragma unroll
                    for (int q = 0; q < NT; q++) {
                        const f16x8 a = *(const f16x8*)(&Xs[buf][a_rd + 16 * q * XR + 32 * I]);
                        const f32x4 z = {0.f, 0.f, 0.f, 0.f};
                        cur[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, z, 0, 0, 0);
                        asm volatile("" : "+v"(cur[q]));
                    }
                    if constexpr (I > 0) {
#pragma unroll
                        for (int q = 0; q < NT; q++) {
#pragma unroll
                            for (int r = 0; r < 4; r++) ct[q][r] = fmaf(dprev, acc[q][r], ct[q][r]);
                            asm volatile("" : "+v"(ct[q]));
                        }
                    }
#pragma unroll
                    for (int q = 0; q < NT; q++) acc[q] = cur[q];
                    dprev = x.d;
                } else {
#pragma unroll
                    for (int q = 0; q < NT; q++) {
                        const f16x8 a = *(const f16x8*)(&Xs[buf][a_rd + 16 * q * XR + 32 * I]);
                        acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[q], 0, 0, 0);
                        // keeps the MFMA here: left alone, the optimiser sinks the whole chain below the last fragment and holds
                        // all eight fragments and operand rows in registers meanwhile
                        asm volatile("" : "+v"(acc[q]));
                    }
                }
            });
            if constexpr (F::HAS_MIN) {
                const f16x8 bm = F::mins(raw, g4);
#pragma unroll
                for (int q = 0; q < NT; q++) {
                    const f16x8 am = *(const f16x8*)(&Xs[buf][m_rd + 16 * q * XR]);
                    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
                    const f32x4 accm = __builtin_amdgcn_mfma_f32_16x16x32_f16(am, bm, z, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; r++) ct[q][r] = fmaf(x.dm, accm[r], ct[q][r]);
                }
            }
            // the chunk's product (the last slice's, where every slice has its own scale), then out with the activation scale
#pragma unroll
            for (int q = 0; q < NT; q++)
#pragma unroll
                for (int r = 0; r < 4; r++) total[s][q][r] = fmaf(e[q][r], fmaf(x.d, acc[q][r], ct[q][r]), total[s][q][r]);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (more) {
            park_w();                             // unit u + 1 over unit u, which this wave has finished reading
            if (u + 2 < u_end) request_next();    // in flight through all of the next unit's arithmetic
            store_x(buf ^ 1);
        }
        if (!more || ck == nchunks - 1) {
            // this group's share is complete: whole iff the run held all of its chunks
            const bool whole = (long long)grp * nchunks >= u_begin && (long long)(grp + 1) * nchunks <= u_end;
            float* const slot0 = (!whole && p.part) ? part_slot(p, grp, 0, grp * GROUP) : nullptr;   // (one division, once per group share)
#pragma unroll
            for (int s = 0; s < 2; s++)
#pragma unroll
              for (int q = 0; q < NT; q++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int t = 8 * q + 4 * (g4 & 1) + r, n = grp * GROUP + wave * 32 + 16 * s + c;
                    float v = total[s][q][r];
                    v += __shfl_xor(v, 32);
                    if (g4 < 2 && t < p.T && n < p.N) {
                        float* y = p.Y + (size_t)t * p.N + n;
                        if (whole) *y = v;
                        else if (p.part) slot0[t * GROUP + (n - grp * GROUP)] = v;
                        else unsafeAtomicAdd(y, v);
                    }
                }
        }
        __syncthreads();
        if (++ck == nchunks) { ck = 0; grp++; }
    }
}

// Ordered mode: group `blockIdx.x` of `group` (128 or 256) outputs, if more than one workgroup held part of its K: Y = slot 0 + slot 1 + ...
// in that order. Thread = output column (threadIdx.x & 127) of activation row 2 * blockIdx.y + (threadIdx.x >> 7).
__global__ void __launch_bounds__(256) sum_split_kernel(float* __restrict__ Y, const float* __restrict__ part, int T, int N, int nchunks,
                                                      long long units, int grid, int kmax, int group) {
    const int grp = blockIdx.x;
    const int first = holder_of((long long)grp * nchunks, grid, units), last = holder_of((long long)(grp + 1) * nchunks - 1, grid, units);
    const int nk = last - first + 1;
    if (nk == 1) return;
    const int per = 256 / group, trow = (int)threadIdx.x / group, col = (int)threadIdx.x - trow * group, n = grp * group + col, t = per * blockIdx.y + trow;
    if (n >= N || t >= T) return;
    const size_t slot = 32 * (size_t)group;
    const float* q = part + (size_t)grp * kmax * slot + t * group + col;
    // (24 slots requested at a time: the down projection's 19 - 20 contributors in one trip to memory instead of three)
    float a = q[0];
    for (int k0 = 1; k0 < nk; k0 += 24) {
        float v[24];
#pragma unroll
        for (int j = 0; j < 24; j++) v[j] = q[(size_t)(k0 + j < nk ? k0 + j : 0) * slot];
#pragma unroll
        for (int j = 0; j < 24; j++)
            if (k0 + j < nk) a += v[j];
    }
    Y[(size_t)t * N + n] = a;
}

__global__ void zero_f32_kernel(float* __restrict__ out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = 0.f;
}

struct Plan {
    int nt, nchunks;
    long long units, groups;
    unsigned grid;
    bool split;
    int kmax;             // most workgroups that hold part of one group's K
    int group;            // rows of a group: 256 for up to 8 activation rows (the eight-wave kernel), else 128
};

// workgroups of the kernel that serves `nt` operand row sets that fit on a CU together
template <class F>
constexpr int slots(int nt) { return nt == 1 ? F::ROWS_OCCUPANCY : (nt == 2 && F::ROWS_AT_16 ? 2 : F::occupancy(nt)); }

Plan make_plan(const fhip_weight* w, size_t t) {
    Plan q;
    q.nt = t <= 8 ? 1 : (t <= 16 ? 2 : 4);
    q.nchunks = (int)((w->cols + CHUNK - 1) / CHUNK);
    const long long cus = fhip::device_cus() > 0 ? fhip::device_cus() : 256;
    // the eight-wave kernel (groups of 256 rows, one workgroup per CU): up to 8 rows on a K-quant weight of 48 MB and more whose
    // groups it cuts along K with every CU holding one share
    q.group = 128;
    if (q.nt == 1 && (w->type == FHIP_Q4_K || w->type == FHIP_Q5_K || w->type == FHIP_Q6_K) && w->nbytes >= ((size_t)48 << 20)) {
        const long long g8 = ((long long)w->rows + 255) / 256, u8 = g8 * q.nchunks, per8 = (u8 + cus - 1) / cus;
        if (u8 >= cus && per8 * 4 < (long long)q.nchunks * 3) q.group = 256;
    }
    const long long groups = ((long long)w->rows + q.group - 1) / q.group;
    q.units = groups * q.nchunks;
    const long long wgs = q.group == 256 ? cus : cus * (w->type == FHIP_Q6_K ? slots<Q6K>(q.nt) : w->type == FHIP_Q8_0 ? slots<Q80>(q.nt) :
                                 w->type == FHIP_Q5_K ? slots<Q5K>(q.nt) : slots<Q4K>(q.nt));
    // one workgroup per resident slot, each with the same share of the units (a grid of 2.66 workgroups per CU leaves
    // two thirds of the CUs with half as much again to do as the rest); shares of three quarters of a group's chunks or
    // more are rounded to whole groups, which store instead of adding
    const long long per = (q.units + wgs - 1) / wgs;
    if (per >= q.nchunks || per * 4 >= (long long)q.nchunks * 3) q.grid = (unsigned)groups;
    else q.grid = (unsigned)(q.units < wgs ? q.units : wgs);
    q.split = q.grid != (unsigned)groups;
    q.groups = groups;
    q.kmax = 1;
    for (long long g = 0; g < groups && q.split; g++) {
        const int nk = holder_of((g + 1) * q.nchunks - 1, q.grid, q.units) - holder_of(g * q.nchunks, q.grid, q.units) + 1;
        if (nk > q.kmax) q.kmax = nk;
    }
    return q;
}

template <class F>
int launch_xsplit_fmt(const float* d_x, size_t t, size_t k, bool swiglu, const Plan& q, uint16_t* d_xp, hipStream_t s, float* zero,
                      size_t zero_n, const fhip::F16Parts& src) {
    const dim3 grid((unsigned)q.nchunks, (unsigned)(8 * q.nt)), wg(256);
    if (swiglu) hipLaunchKernelGGL((xsplit_f16_kernel<F, true>), grid, wg, 0, s, d_x, (int)t, (int)k, q.nt, d_xp, zero, zero_n, src);
    else hipLaunchKernelGGL((xsplit_f16_kernel<F, false>), grid, wg, 0, s, d_x, (int)t, (int)k, q.nt, d_xp, zero, zero_n, src);
    return fhip::check_hip(hipGetLastError(), "xsplit_f16 launch");
}

template <class F>
int launch_fmt(const fhip_weight* w, const uint16_t* d_xp, size_t t, float* d_y, hipStream_t s, bool y_cleared, float* d_part, fhip::F16Parts* deferred) {
    const Plan q = make_plan(w, t);
    F16Params p;
    p.W = w->d_raw; p.Xp = d_xp; p.Y = d_y;
    p.part = q.split ? d_part : nullptr; p.kmax = q.kmax;
    p.T = (int)t; p.N = (int)w->rows; p.nchunks = q.nchunks; p.row_bytes = w->row_bytes;
    p.nblk = (int)(w->cols / 32);
    p.units = q.units; p.group = q.group;
    if (q.split && !y_cleared && !d_part) {
        const size_t n = t * w->rows;
        hipLaunchKernelGGL(zero_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, d_y, n);
    }
    if (q.nt == 1 && q.group == 256) {
        if constexpr (F::ROW_PER_LANE) hipLaunchKernelGGL((gemm_q_f16x2_rows_kernel<F, 1, 8>), dim3(q.grid), dim3(512), 0, s, p);
    } else if (q.nt == 1) hipLaunchKernelGGL((gemm_q_f16x2_rows_kernel<F, 1, 4>), dim3(q.grid), dim3(256), 0, s, p);
    else if (q.nt == 2 && F::ROWS_AT_16) hipLaunchKernelGGL((gemm_q_f16x2_rows_kernel<F, 2, 4>), dim3(q.grid), dim3(256), 0, s, p);
    else if constexpr (F::ROW_PER_LANE) {
        if (q.nt == 2) hipLaunchKernelGGL((gemm_q_f16x2_kernel<F, 2>), dim3(q.grid), dim3(256), 0, s, p);
        else hipLaunchKernelGGL((gemm_q_f16x2_kernel<F, 4>), dim3(q.grid), dim3(256), 0, s, p);
    } else {
        return fhip::set_error(FHIP_ERR_SHAPE, "f16x2 matmul: this format takes at most 16 activation rows, got %zu", t);
    }
    if (deferred) *deferred = fhip::F16Parts{p.part, p.kmax, p.nchunks, (int)q.grid, p.units, q.group};
    if (p.part && !deferred)
        hipLaunchKernelGGL(sum_split_kernel, dim3((unsigned)q.groups, (unsigned)((t * q.group + 255) / 256)), dim3(256), 0, s, d_y, (const float*)d_part, p.T, p.N,
                           p.nchunks, p.units, (int)q.grid, p.kmax, q.group);
    return fhip::check_hip(hipGetLastError(), "gemm_q_f16x2 launch");
}

}  // namespace

namespace fhip {

bool gemm_f16x2_supports(const fhip_weight* w, size_t t) {
    if (!w || t < 1 || w->cols == 0 || w->cols > (size_t)MAXW * 1024) return false;
    if (w->type == FHIP_Q8_0) return t <= 16 && w->cols % 32 == 0;   // rows of any whole number of blocks
    return (w->type == FHIP_Q4_K || w->type == FHIP_Q5_K || w->type == FHIP_Q6_K) && t <= 32 && w->cols % CHUNK == 0;
}

size_t gemm_f16x2_xp_bytes(const fhip_weight* w, size_t t) {
    const Plan q = make_plan(w, t);
    return (size_t)q.nchunks * 16 * q.nt * XR * sizeof(uint16_t);
}

bool gemm_f16x2_adds_into_y(const fhip_weight* w, size_t t) { return make_plan(w, t).split; }

size_t gemm_f16x2_part_bytes(const fhip_weight* w, size_t t) {
    const Plan q = make_plan(w, t);
    return q.split ? (size_t)q.groups * q.kmax * 32 * q.group * sizeof(float) : 0;
}
// the most any batch of up to t rows needs (fewer rows can mean more resident workgroups, and so more contributors)
size_t gemm_f16x2_part_bytes_upto(const fhip_weight* w, size_t t) {
    size_t m = gemm_f16x2_part_bytes(w, t);
    for (size_t u : {(size_t)8, (size_t)16})
        if (u < t) m = std::max(m, gemm_f16x2_part_bytes(w, u));
    return m;
}

int launch_xsplit_f16(const fhip_weight* w, const float* d_x, size_t t, bool swiglu, uint16_t* d_xp, hipStream_t s, float* zero, size_t zero_n,
                      const F16Parts* src_in) {
    const Plan q = make_plan(w, t);
    const F16Parts src = src_in ? *src_in : F16Parts{nullptr, 0, 0, 0, 0, 128};
    switch (w->type) {
        case FHIP_Q4_K: return launch_xsplit_fmt<Q4K>(d_x, t, w->cols, swiglu, q, d_xp, s, zero, zero_n, src);
        case FHIP_Q5_K: return launch_xsplit_fmt<Q5K>(d_x, t, w->cols, swiglu, q, d_xp, s, zero, zero_n, src);
        case FHIP_Q6_K: return launch_xsplit_fmt<Q6K>(d_x, t, w->cols, swiglu, q, d_xp, s, zero, zero_n, src);
        case FHIP_Q8_0: return launch_xsplit_fmt<Q80>(d_x, t, w->cols, swiglu, q, d_xp, s, zero, zero_n, src);
        default: return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "f16x2 matmul: no kernel for ggml type %u", w->type);
    }
}

int launch_gemm_f16x2(const fhip_weight* w, const uint16_t* d_xp, size_t t, float* d_y, hipStream_t s, bool y_cleared, float* d_part,
                      F16Parts* deferred) {
    switch (w->type) {
        case FHIP_Q4_K: return launch_fmt<Q4K>(w, d_xp, t, d_y, s, y_cleared, d_part, deferred);
        case FHIP_Q5_K: return launch_fmt<Q5K>(w, d_xp, t, d_y, s, y_cleared, d_part, deferred);
        case FHIP_Q6_K: return launch_fmt<Q6K>(w, d_xp, t, d_y, s, y_cleared, d_part, deferred);
        case FHIP_Q8_0: return launch_fmt<Q80>(w, d_xp, t, d_y, s, y_cleared, d_part, deferred);
        default: return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "f16x2 matmul: no kernel for ggml type %u", w->type);
    }
}

}  // namespace fhip
