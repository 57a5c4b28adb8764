// Prefill dequant-GEMM on the matrix cores, gfx950:  Y[t, n] = sum_k X[t, k] * dequant(W[n, k])
// X bf16 [T, K], W raw GGUF blocks [N, K], Y f32 [T, N], f32 accumulate.
//
// Stands for the reference's cooperative-matrix prefill kernels (crates/ferric-tensor/src/dtype.rs:2059-2096
// Q4_K, :1217-1257 Q6_K, :1333-1370 Q8_0, :1074-1131 Q5_K), which dequantize an 8x8 weight tile into shared memory and
// feed an 8x8 f32 matrix unit. Here the unit is v_mfma_f32_32x32x16_bf16.
//
// Shape of the kernel. The reference found this path bound by the unpack arithmetic, not the matrix
// unit (crates/ferric-core/src/lib.rs:90-101), and the same holds here: a weight costs ~3 VALU
// operations to turn into bf16, an MFMA retires 16K multiply-adds in 32 cycles. So
//   * each lane dequantizes 8 consecutive quants of one weight row, which is exactly the B fragment a lane
//     holds in a 32x32x16 MFMA: no transposition for the weights;
//   * a dequantized fragment is published once in LDS and used by both waves of a T-pair for every 32-row
//     slab they own, so unpack cost is amortised over the workgroup's 64*MI activation rows;
//   * the fragments of step s+1 are produced while the MFMAs of step s run, one MFMA alternating with its
//     share of the unpack arithmetic, with two waves per SIMD to fill each other's issue gaps;
//   * the activation tile, which all 8 waves of a workgroup share, is staged through LDS (padded rows,
//     16-byte reads);
//   * the 16 k of one MFMA are chosen inside ONE scale sub-block (the k order inside an MFMA is free as
//     long as both operands agree), so a fragment needs a single (scale, min) pair;
//   * weight bytes are fetched a whole 256-column chunk ahead into the registers the previous chunk has
//     just vacated (consume, then refill), so no weight load is waited for in the steady state.
// One k-step is 64 columns = 4 MFMA slices; a chunk is 4 steps = one K-quant super-block or 8 Q8_0 blocks.
// Dequantized values are exactly the f32 the CPU dequantizer produces, rounded to bf16 (RNE) by
// v_cvt_pk_bf16_f32.
// Three kernels: the tiled one (64, 128 or 256 activation rows x 256 or 128 outputs per workgroup), its 160-column variant
// (256 or 128 rows) for output widths that 160 deals to the chip's workgroups exactly, and one for up to 32 rows; the
// launcher picks by a cost estimate. A launch that cuts output tiles along K sums the partial tiles in a fixed order: the same inputs give the
// same bits on every run.
#include "common.hpp"
#include "loads.hpp"

#include <hip/hip_fp16.h>

#include <cstdlib>
#include <type_traits>

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float f16_bits(uint32_t b) { return __half2float(__ushort_as_half((unsigned short)b)); }
__device__ __forceinline__ float ub(uint32_t v, int k) { return (float)((v >> (8 * k)) & 0xFFu); }
__device__ __forceinline__ uint32_t pk_bf16(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){a, b}, bf16x2));
}
// 8 weights w_i = fma(s, q_i, o) from the bytes of two dwords -> one MFMA operand (8 bf16)
__device__ __forceinline__ bf16x8 frag8(uint32_t q0, uint32_t q1, float s, float o) {
    // Hide from the optimiser which bits of the bytes are known zero: with that knowledge it narrows every
    // byte extraction to a bit-field extract and adds one instruction per weight in front of the byte-lane
    // conversions v_cvt_f32_ubyte0..3, which take the byte lane as it is.
    asm("" : "+v"(q0));
    asm("" : "+v"(q1));
    u32x4 r;
    r[0] = pk_bf16(fmaf(s, ub(q0, 0), o), fmaf(s, ub(q0, 1), o));
    r[1] = pk_bf16(fmaf(s, ub(q0, 2), o), fmaf(s, ub(q0, 3), o));
    r[2] = pk_bf16(fmaf(s, ub(q1, 0), o), fmaf(s, ub(q1, 1), o));
    r[3] = pk_bf16(fmaf(s, ub(q1, 2), o), fmaf(s, ub(q1, 3), o));
    return __builtin_bit_cast(bf16x8, r);
}

constexpr int KSTEP = 64;            // columns per k-step: 4 MFMA slices of 16
constexpr int CHUNK = 256;           // columns per chunk: 4 steps
constexpr int LDS_ROW = KSTEP + 8;   // bf16 per staged activation row (+16 B pad: conflict-free 16-byte reads)

// Column of the 8 consecutive k that lane half h (= lane / 32) holds in slice t of a step, for both
// operands and every format: sub-block (t >> 1) of the step, elements 16h + 8(t & 1) + [0, 8).
__device__ __forceinline__ constexpr int kcol(int t, int h) { return 32 * (t >> 1) + 16 * h + 8 * (t & 1); }

// ------------------------------------------------------------------------------------------------
// Per-format weight streams. `Raw` is the per-lane register image of one chunk of one weight row (the
// half h of it this lane unpacks). prime() loads chunk c whole. For step G of a chunk, begin<G>() derives
// the step's scales into a `Ctx`, frag<G, T>() builds the B fragment of slice T, and refill<G>() reloads
// the registers step G has just read with the same bytes of chunk `nc` (the following chunk, clamped by
// the caller to one that exists).
// ------------------------------------------------------------------------------------------------

struct Q4K {
    static constexpr int BLOCK = 144;
    static constexpr float UNPACK_US = 1.4f;   // unpack of a 256 x 256 chunk by one workgroup
    // one chunk of a workgroup tile of 64 x 256, 128 x 256, 256 x 256, 256 x 160, 128 x 128, 64 x 128, 128 x 160, in us (fitted, see plan_cost_us)
    static constexpr float CHUNK_US[7] = {3.43f, 4.76f, 8.15f, 5.19f, 2.84f, 2.00f, 3.29f};
    static constexpr bool PARTIAL = false;
    static __host__ __device__ int chunks(int K) { return K / 256; }
    struct Raw { u32x4 hd, hdn, q[4]; };
    struct Ctx { float d0, o0, d1, o1; };
    static __device__ __forceinline__ void prime(Raw& r, const uint8_t* row, int c, int h, int) {
        const uint8_t* blk = row + (size_t)c * BLOCK;
        r.hd = *(const u32x4*)blk;
        r.hdn = r.hd;
#pragma unroll
        for (int g = 0; g < 4; g++) r.q[g] = *(const u32x4*)(blk + 16 + 32 * g + 16 * h);
    }
    // get_sc_min (crates/ferric-gguf/src/lib.rs:795-804) for sub-block j (a compile-time constant after inlining)
    static __device__ __forceinline__ void sc_min(const u32x4& hd, int j, float& sc, float& mn) {
        const uint32_t a = hd[1], b = hd[2], c = hd[3];
        if (j < 4) {
            sc = (float)((a >> (8 * j)) & 63u);
            mn = (float)((b >> (8 * j)) & 63u);
        } else {
            const int i = j - 4;
            sc = (float)(((c >> (8 * i)) & 0xFu) | (((a >> (8 * i + 6)) & 3u) << 4));
            mn = (float)(((c >> (8 * i + 4)) & 0xFu) | (((b >> (8 * i + 6)) & 3u) << 4));
        }
    }
    template <int G>
    static __device__ __forceinline__ void begin(Raw& r, int, int, int, Ctx& x) {
        if (G == 0) r.hd = r.hdn;
        const float d = f16_bits(r.hd[0] & 0xFFFFu), dmin = f16_bits(r.hd[0] >> 16);
        float s0, m0, s1, m1;
        sc_min(r.hd, 2 * G, s0, m0);
        sc_min(r.hd, 2 * G + 1, s1, m1);
        // y = (d*sc)*q - (dmin*m): the product is exact in f32, so the fused form rounds identically.
        // The high nibbles stay in place (q * 16) and their scale carries the 1/16, an exact power of two.
        x.d0 = d * s0; x.o0 = -(dmin * m0); x.d1 = (d * s1) * 0.0625f; x.o1 = -(dmin * m1);
    }
    // slice T: sub-block 2G + (T >> 1) = low (T < 2) or high nibbles of bytes 32G + 16h + 8(T & 1) + [0, 8)
    template <int G, int T>
    static __device__ __forceinline__ bf16x8 frag(const Raw& r, const Ctx& x) {
        constexpr uint32_t M = T < 2 ? 0x0F0F0F0Fu : 0xF0F0F0F0u;
        return frag8(r.q[G][2 * (T & 1)] & M, r.q[G][2 * (T & 1) + 1] & M, T < 2 ? x.d0 : x.d1, T < 2 ? x.o0 : x.o1);
    }
    template <int G>
    static __device__ __forceinline__ void refill(Raw& r, const uint8_t* row, int nc, int h, int) {
        const uint8_t* nb = row + (size_t)nc * BLOCK;
        r.q[G] = *(const u32x4*)(nb + 16 + 32 * G + 16 * h);
        if (G == 1) r.hdn = *(const u32x4*)nb;
    }
};

// Q5_K is Q4_K with a fifth bit per quant (the reference's matmul_q5_k_coop, crates/ferric-tensor/src/dtype.rs:1074-1131):
// 176 B = [f16 d][f16 dmin][scales 12 B][qh 32 B][qs 128 B]; bit s of qh[l] is the fifth bit of element l of sub-block s
// (crates/ferric-gguf/src/lib.rs:692-716), q = nibble + 16 * bit in 0..31, y = (d*sc)*q - dmin*m. A lane half h works on
// elements 16h + [0, 16) of every sub-block, so it holds the same 16 bytes qh[16h, 16h + 16) for the whole chunk; slice T of
// step G takes bit 2G + (T >> 1) of them. The high nibbles are shifted down (with the fifth bit on top they do not fit a
// byte in place), so both sub-block scales are plain d * sc.
struct Q5K {
    static constexpr int BLOCK = 176;
    static constexpr float UNPACK_US = 1.8f;
    static constexpr float CHUNK_US[7] = {3.83f, 5.16f, 9.41f, 6.12f, 3.17f, 2.26f, 3.78f};
    static constexpr bool PARTIAL = false;
    static __host__ __device__ int chunks(int K) { return K / 256; }
    struct Raw { u32x4 hd, hdn, qh, qhn, q[4]; };
    struct Ctx { float d0, o0, d1, o1; };
    static __device__ __forceinline__ void prime(Raw& r, const uint8_t* row, int c, int h, int) {
        const uint8_t* blk = row + (size_t)c * BLOCK;
        r.hd = *(const u32x4*)blk;
        r.hdn = r.hd;
        r.qh = *(const u32x4*)(blk + 16 + 16 * h);
        r.qhn = r.qh;
#pragma unroll
        for (int g = 0; g < 4; g++) r.q[g] = *(const u32x4*)(blk + 48 + 32 * g + 16 * h);
    }
    template <int G>
    static __device__ __forceinline__ void begin(Raw& r, int, int, int, Ctx& x) {
        if (G == 0) { r.hd = r.hdn; r.qh = r.qhn; }
        const float d = f16_bits(r.hd[0] & 0xFFFFu), dmin = f16_bits(r.hd[0] >> 16);
        float s0, m0, s1, m1;
        Q4K::sc_min(r.hd, 2 * G, s0, m0);
        Q4K::sc_min(r.hd, 2 * G + 1, s1, m1);
        // every product is exact in f32 (11-bit d, 6-bit scale, 5-bit quant), so the fused form rounds as the reference's
        x.d0 = d * s0; x.o0 = -(dmin * m0); x.d1 = d * s1; x.o1 = -(dmin * m1);
    }
    template <int G, int T>
    static __device__ __forceinline__ bf16x8 frag(const Raw& r, const Ctx& x) {
        constexpr int w = 2 * (T & 1), s = 2 * G + (T >> 1);
        uint32_t v[2];
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const uint32_t nib = T < 2 ? r.q[G][w + i] & 0x0F0F0F0Fu : (r.q[G][w + i] >> 4) & 0x0F0F0F0Fu;
            const uint32_t bit = (s >= 4 ? r.qh[w + i] >> (s - 4) : r.qh[w + i] << (4 - s)) & 0x10101010u;
            v[i] = nib | bit;
        }
        return frag8(v[0], v[1], T < 2 ? x.d0 : x.d1, T < 2 ? x.o0 : x.o1);
    }
    template <int G>
    static __device__ __forceinline__ void refill(Raw& r, const uint8_t* row, int nc, int h, int) {
        const uint8_t* nb = row + (size_t)nc * BLOCK;
        r.q[G] = *(const u32x4*)(nb + 48 + 32 * G + 16 * h);
        if (G == 1) { r.hdn = *(const u32x4*)nb; r.qhn = *(const u32x4*)(nb + 16 + 16 * h); }
    }
};

struct Q6K {
    // Step G covers half hf = G >> 1 of the super-block and its groups g0 = 2(G & 1), g0 + 1 (low nibbles of
    // ql for G even, high nibbles for G odd); slice T is group g = g0 + (T >> 1), l = 16h + 8(T & 1) + [0, 8),
    // whose scale is sc[8hf + 2g + h]  (crates/ferric-gguf/src/lib.rs:833-851).
    static constexpr int BLOCK = 210;
    static constexpr float UNPACK_US = 2.3f;
    static constexpr float CHUNK_US[7] = {5.93f, 6.83f, 9.84f, 6.27f, 4.68f, 3.95f, 4.35f};
    static constexpr bool PARTIAL = false;
    static __host__ __device__ int chunks(int K) { return K / 256; }
    struct Raw { u32x4 ql[2][2], qh[2], sc, scn; uint32_t d, dn; };
    struct Ctx { float d; };
    static __device__ __forceinline__ u32x4 ld16(const uint8_t* p) { return fhip::load16_a2(p); }   // 210-byte blocks: see loads.hpp
    static __device__ __forceinline__ void prime(Raw& r, const uint8_t* row, int c, int h, int) {
        const uint8_t* blk = row + (size_t)c * BLOCK;
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
            r.ql[hf][0] = ld16(blk + 64 * hf + 16 * h);
            r.ql[hf][1] = ld16(blk + 64 * hf + 32 + 16 * h);
            r.qh[hf] = ld16(blk + 128 + 32 * hf + 16 * h);
        }
        r.scn = ld16(blk + 192);
        r.dn = *(const uint16_t*)(blk + 208);
        r.sc = r.scn;
        r.d = r.dn;
    }
    template <int G>
    static __device__ __forceinline__ void begin(Raw& r, int, int h, int, Ctx& x) {
        if (G == 0) {
            // byte h of every 16-bit pair is this lane half's scale: shift it down once per chunk
#pragma unroll
            for (int w = 0; w < 4; w++) r.sc[w] = r.scn[w] >> (8 * h);
            r.d = r.dn;
        }
        x.d = f16_bits(r.d);
    }
    template <int G, int T>
    static __device__ __forceinline__ bf16x8 frag(const Raw& r, const Ctx& x) {
        constexpr int hf = G >> 1, g = 2 * (G & 1) + (T >> 1), par = T >> 1, w = 2 * (T & 1);
        const uint32_t l0 = r.ql[hf][par][w], l1 = r.ql[hf][par][w + 1];
        const uint32_t h0 = r.qh[hf][w], h1 = r.qh[hf][w + 1];
        uint32_t n0, n1, u0, u1;
        if (G & 1) { n0 = (l0 >> 4) & 0x0F0F0F0Fu; n1 = (l1 >> 4) & 0x0F0F0F0Fu; }
        else       { n0 = l0 & 0x0F0F0F0Fu;        n1 = l1 & 0x0F0F0F0Fu; }
        if (g < 2) { u0 = (h0 << (g < 2 ? 4 - 2 * g : 0)) & 0x30303030u; u1 = (h1 << (g < 2 ? 4 - 2 * g : 0)) & 0x30303030u; }
        else       { u0 = (h0 >> (g < 2 ? 0 : 2 * g - 4)) & 0x30303030u; u1 = (h1 >> (g < 2 ? 0 : 2 * g - 4)) & 0x30303030u; }
        const uint32_t scw = r.sc[2 * hf + (g >> 1)];
        const float ds = x.d * (float)(int8_t)((scw >> (16 * (g & 1))) & 0xFFu);
        // (d*sc)*(q-32) = ds*q - 32*ds, every term exact in f32
        return frag8(n0 | u0, n1 | u1, ds, -32.0f * ds);
    }
    template <int G>
    static __device__ __forceinline__ void refill(Raw& r, const uint8_t* row, int nc, int h, int) {
        constexpr int hf = G >> 1;
        const uint8_t* nb = row + (size_t)nc * BLOCK;
        if (G & 1) {   // both nibble planes of this half are spent
            r.ql[hf][0] = ld16(nb + 64 * hf + 16 * h);
            r.ql[hf][1] = ld16(nb + 64 * hf + 32 + 16 * h);
            r.qh[hf] = ld16(nb + 128 + 32 * hf + 16 * h);
        }
        if (G == 1) {
            r.scn = ld16(nb + 192);
            r.dn = *(const uint16_t*)(nb + 208);
        }
    }
};

struct Q80 {
    // A chunk is 8 blocks of 34 bytes; step G covers blocks 2G, 2G+1; slice T is block 2G + (T >> 1),
    // elements 16h + 8(T & 1) + [0, 8). A trailing partial chunk is allowed: blocks past the row's end are
    // read from the last valid block's address and given scale 0 (their activations are staged as 0 too).
    static constexpr int BLOCK = 34;
    static constexpr float UNPACK_US = 5.1f;
    static constexpr float CHUNK_US[7] = {9.51f, 9.88f, 11.93f, 6.86f, 7.16f, 6.65f, 5.76f};
    static constexpr bool PARTIAL = true;   // a row may end inside a chunk
    static __host__ __device__ int chunks(int K) { return (K + 255) / 256; }
    struct Raw { u32x4 q[4][2]; uint32_t d[4][2]; };
    struct Ctx { float d[2]; };
    static __device__ __forceinline__ const uint8_t* blk(const uint8_t* row, int c, int i, int nblk) {
        int bi = 8 * c + i;
        bi = bi < nblk ? bi : nblk - 1;
        return row + (size_t)bi * BLOCK;
    }
    static __device__ __forceinline__ void prime(Raw& r, const uint8_t* row, int c, int h, int nblk) {
#pragma unroll
        for (int g = 0; g < 4; g++)
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const uint8_t* p = blk(row, c, 2 * g + u, nblk);
                r.d[g][u] = *(const uint16_t*)p;
                r.q[g][u] = fhip::load16_a2(p + 2 + 16 * h);
            }
    }
    template <int G>
    static __device__ __forceinline__ void begin(Raw& r, int c, int, int nblk, Ctx& x) {
#pragma unroll
        for (int u = 0; u < 2; u++) x.d[u] = (8 * c + 2 * G + u) < nblk ? f16_bits(r.d[G][u]) : 0.0f;
    }
    template <int G, int T>
    static __device__ __forceinline__ bf16x8 frag(const Raw& r, const Ctx& x) {
        // q = (q ^ 0x80) - 128 with the biased byte unsigned: d*q = d*u - 128*d, every term exact in f32
        const float d = x.d[T >> 1];
        return frag8(r.q[G][T >> 1][2 * (T & 1)] ^ 0x80808080u, r.q[G][T >> 1][2 * (T & 1) + 1] ^ 0x80808080u, d, -128.0f * d);
    }
    template <int G>
    static __device__ __forceinline__ void refill(Raw& r, const uint8_t* row, int nc, int h, int nblk) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const uint8_t* p = blk(row, nc, 2 * G + u, nblk);
            r.d[G][u] = *(const uint16_t*)p;
            r.q[G][u] = fhip::load16_a2(p + 2 + 16 * h);
        }
    }
};

struct GemmParams {
    const uint8_t* W;
    const uint16_t* X;   // bf16 bits [T, K]
    float* Y;            // [T, N]
    int T, N, K;
    int nblk;            // blocks per weight row
    size_t row_bytes;
    int tiles_n;         // workgroup tiles along N
    int nchunks;         // chunks per weight row
    int whole_rounds;    // rounds of whole tiles every workgroup computes first: tile = round * gridDim.x + blockIdx.x
    long long units;     // the remaining tiles' (tile, chunk) work units, chunk fastest
    int per;             // of those, units per workgroup
    float* ws;           // partial tiles of the left-over tiles that several runs share: [left-over tile][contributor][BM x 256]
    int kmax;            // contributor slots per left-over tile
};

template <int I, int N, class Fn>
__device__ __forceinline__ void static_for(Fn&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// Workgroup = 8 waves, 2 along T x 4 along N; wave tile = (32*MI) x 64; workgroup tile = (64*MI) x 256.
// Two waves per SIMD: a wave issues one VALU instruction per ~6 cycles and one 16-byte LDS read per ~16, so
// a single wave cannot feed its own MFMAs and unpack at the same time; two can.
// The two waves of a T-pair need the same 64 weight rows. Each unpacks 32 of them (all four slices of a
// step) and publishes the fragments in LDS in MFMA operand order (lane L's 16 bytes at L*16), where both
// read them back: unpack work per MFMA halves, and a wave carries the raw bytes of one row only.
//
// Work distribution. One workgroup per CU. Every workgroup first computes `whole_rounds` whole tiles (tile =
// round * gridDim.x + blockIdx.x, so the workgroups running side by side share activation rows in L2). The
// tiles left over, fewer than one per workgroup, are cut along K: their (tile, chunk) units are dealt out in
// equal contiguous runs of `per`, so every CU does the same amount of MFMA work whatever the tile count (no
// partial last round). A run may start and end inside a tile: a segment that covers its tile's whole K stores
// the tile, any other stores its partial sums into the workspace slot (tile, contributor), contributor = the run's rank among
// the runs that touch the tile, and sum_split_tiles_kernel adds a tile's slots in that order afterwards: the result does not
// depend on which workgroup finishes first (f32 atomics into Y, which this replaced, gave run-to-run differences in the
// last bits wherever a tile had three contributors or more).
//
// NI = 1 is the same layout at half the width, a workgroup tile of (64*MI) x 128 for short prompts: a T-pair then needs one
// block of 32 weight rows, both waves carry its raw bytes and each unpacks two of a step's four slices, so that at 128
// activation rows (MI = 2) every weight is unpacked once (the 64 x 256 tile unpacks it twice, once per tile row) with the
// same partial-tile bytes per workgroup.
template <class F, int MI, int NI>
__global__ void __launch_bounds__(512) gemm_q_bf16_kernel(GemmParams p) {
    constexpr int BM = 64 * MI, BN = 128 * NI;
    constexpr int FRAG = 512;                                   // bf16 per published fragment (64 lanes x 8)
    __shared__ __attribute__((aligned(16))) uint16_t As[2][BM * LDS_ROW];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[2][16 * NI * FRAG];   // [n-block 0..4 NI - 1][slice 0..3]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave & 3, wm = wave >> 2;
    const int h = lane >> 5, c = lane & 31;
    const int nchunks = p.nchunks;
    long long u = (long long)blockIdx.x * p.per;
    const long long u_end = u + p.per < p.units ? u + p.per : p.units;
  for (int round = 0;; round++) {
    int tile, c_begin, c_end;
    if (round < p.whole_rounds) {
        tile = round * gridDim.x + blockIdx.x;
        c_begin = 0;
        c_end = nchunks;
    } else {
        if (u >= u_end) break;
        const int rt = (int)(u / nchunks);
        tile = p.whole_rounds * gridDim.x + rt;
        c_begin = (int)(u - (long long)rt * nchunks);
        c_end = (long long)(nchunks - c_begin) < u_end - u ? nchunks : c_begin + (int)(u_end - u);
        u += c_end - c_begin;
    }
    const bool whole = c_begin == 0 && c_end == nchunks;
    const int tile_y = tile / p.tiles_n, tile_x = tile - tile_y * p.tiles_n;
    const int t0 = tile_y * BM + wm * (32 * MI);
    const int n0 = tile_x * BN + wn * (32 * NI);
    const int c_last = c_end - 1;

    // the weight row this lane unpacks: n-block 2*wn + wm of the workgroup tile (NI = 1: n-block wn, of which this wave
    // unpacks slices 2*wm and 2*wm + 1); clamped: rows past N are computed but not stored
    const uint8_t* wrow;
    {
        int n = n0 + (NI == 2 ? 32 * wm : 0) + c;
        wrow = p.W + (size_t)(n < p.N ? n : p.N - 1) * p.row_bytes;
    }
    const int b_wr = ((NI == 2 ? 2 * wn + wm : wn) * 4) * FRAG + lane * 8;    // + t * FRAG
    const int b_rd = ((NI * wn) * 4) * FRAG + lane * 8;                        // + (4 * j + t) * FRAG
    auto mine = [&](int t) { return NI == 2 || (t >> 1) == wm; };             // does this wave unpack slice t (wave-uniform)

    f32x16 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // Activation staging: BM rows x 64 bf16 per step; thread `tid` moves the 16-byte piece (tid & 7) of rows
    // (tid >> 3) + 64q, q < MI. Rows past T are read from row T-1 (their outputs are never stored); columns
    // past K (a partial last chunk) are staged as zeros.
    const int a_col = (tid & 7) * 8;
    uint32_t a_src[MI];   // element offsets into X (the launcher checks T*K fits 31 bits)
#pragma unroll
    for (int q = 0; q < MI; q++) {
        int t = tile_y * BM + (tid >> 3) + 64 * q;
        a_src[q] = (uint32_t)(t < p.T ? t : p.T - 1) * (uint32_t)p.K + a_col;
    }
    const int a_dst = (tid >> 3) * LDS_ROW + a_col;
    u32x4 stage[MI];
    auto load_a = [&](int s) {   // s = absolute step index (64 columns each)
        if constexpr (F::PARTIAL) {
            const bool ok = s * KSTEP + a_col < p.K;
            const int off = ok ? s * KSTEP : 0;
            const uint32_t keep = ok ? 0xFFFFFFFFu : 0u;
#pragma unroll
            for (int q = 0; q < MI; q++) {
                u32x4 v = *(const u32x4*)(p.X + (a_src[q] + off));
                stage[q] = (u32x4){v[0] & keep, v[1] & keep, v[2] & keep, v[3] & keep};
            }
        } else {
            const int off = s * KSTEP < p.K ? s * KSTEP : 0;   // past the end: any valid address, the tile is never read
#pragma unroll
            for (int q = 0; q < MI; q++) stage[q] = *(const u32x4*)(p.X + (a_src[q] + off));
        }
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int q = 0; q < MI; q++) *(u32x4*)(&As[buf][a_dst + 64 * q * LDS_ROW]) = stage[q];
    };
    const int a_rd = (wm * 32 * MI + c) * LDS_ROW + 16 * h;   // + 32*i rows, + kcol(t, 0)
    typename F::Raw raw;
    F::prime(raw, wrow, c_begin, h, p.nblk);
    load_a(4 * c_begin);
    {
        const int nc = c_begin + 1 < c_last ? c_begin + 1 : c_last;
        typename F::Ctx x;
        F::template begin<0>(raw, c_begin, h, p.nblk, x);
        static_for<0, 4>([&](auto T) {
            if (mine(T.value)) *(bf16x8*)(&Bs[0][b_wr + T.value * FRAG]) = F::template frag<0, T.value>(raw, x);
        });
        F::template refill<0>(raw, wrow, nc, h, p.nblk);
    }
    store_a(0);
    __syncthreads();

    // One k-step: the MFMAs of step (chunk ck, G) from LDS buffers G & 1, while this wave's fragments of the
    // following step are unpacked and published into the other B buffer and the following activations
    // travel global -> registers -> LDS. The step is cut into its four slices; each slice first reads the
    // next slice's operands from LDS, then alternates one MFMA with its share of the unpack arithmetic.
    // Nothing moves between slices.
    constexpr int VPM = (26 + MI * NI - 1) / (MI * NI);   // VALU instructions issued behind each MFMA
    auto step = [&](auto Gc, int ck) {
        constexpr int G = decltype(Gc)::value;
        constexpr int GN = (G + 1) & 3;
        constexpr int buf = G & 1;
        // fragments of step G+1 of this chunk, or of step 0 of the next one
        const int pc = G == 3 ? (ck + 1 < c_last ? ck + 1 : c_last) : ck;
        const int nc = pc + 1 < c_last ? pc + 1 : c_last;
        typename F::Ctx ctx;
        bf16x8 a[2][MI], b[2][NI];
        auto read_ops = [&](int t, bf16x8 (&da)[MI], bf16x8 (&db)[NI]) {
#pragma unroll
            for (int i = 0; i < MI; i++) da[i] = *(const bf16x8*)(&As[buf][a_rd + 32 * i * LDS_ROW + kcol(t, 0)]);
#pragma unroll
            for (int j = 0; j < NI; j++) db[j] = *(const bf16x8*)(&Bs[buf][b_rd + (4 * j + t) * FRAG]);
        };
        read_ops(0, a[0], b[0]);
        load_a(4 * ck + G + 1);
        F::template begin<GN>(raw, pc, h, p.nblk, ctx);
        __builtin_amdgcn_sched_barrier(0);
        static_for<0, 4>([&](auto S) {
            constexpr int t = decltype(S)::value;
            if constexpr (t < 3) read_ops(t + 1, a[(t + 1) & 1], b[(t + 1) & 1]);
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int j = 0; j < NI; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[t & 1][i], b[t & 1][j], acc[i][j], 0, 0, 0);
            if (mine(t)) *(bf16x8*)(&Bs[buf ^ 1][b_wr + t * FRAG]) = F::template frag<GN, t>(raw, ctx);
            if constexpr (t < 3) __builtin_amdgcn_sched_group_barrier(0x100, MI + NI, 0);
#pragma unroll
            for (int u = 0; u < MI * NI; u++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, VPM, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
            __builtin_amdgcn_sched_barrier(0);
        });
        F::template refill<GN>(raw, wrow, nc, h, p.nblk);
        store_a(buf ^ 1);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
    };

    for (int ck = c_begin; ck < c_end; ck++) {
        step(std::integral_constant<int, 0>{}, ck);
        step(std::integral_constant<int, 1>{}, ck);
        step(std::integral_constant<int, 2>{}, ck);
        step(std::integral_constant<int, 3>{}, ck);
    }

    // a partial tile goes to the slot of this run in the tile's contributor list: runs are numbered by blockIdx.x, and the
    // first run that touches left-over tile rt is the one that holds unit rt * nchunks
    float* part = nullptr;
    if (!whole) {
        const int rt = tile - p.whole_rounds * (int)gridDim.x;
        const int k = (int)blockIdx.x - (int)(((long long)rt * nchunks) / p.per);
        part = p.ws + ((size_t)rt * p.kmax + k) * (size_t)(BM * BN);
    }
    // D layout of the 32x32 MFMA: register r of lane (h, c) is row 8*(r/4) + 4*h + (r%4), column c
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++) {
            const int n = n0 + 32 * j + c;
            if (n >= p.N) continue;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int t = t0 + 32 * i + 8 * (r >> 2) + 4 * h + (r & 3);
                if (t < p.T) {
                    if (whole) p.Y[(size_t)t * p.N + n] = acc[i][j][r];
                    else part[(size_t)(t - tile_y * BM) * BN + (n - tile_x * BN)] = acc[i][j][r];
                }
            }
        }
  }
}

// ------------------------------------------------------------------------------------------------
// The same kernel with a 256 x 160 workgroup tile. An output width of 5120 is 20 tiles of 256 columns but 32 of 160, and
// 32 x (T / 256) tile rows deal 2048, 1024 or 512 activation rows to the chip's 256 workgroups exactly: one whole tile
// each, or every tile cut along K in exactly two or four (no run that starts in one tile and ends in the next, so one
// partial tile per workgroup). Wave layout: 8 waves along T, 32 rows each, every wave holding all five 32-column blocks
// (MI = 1, NI = 5: 1.2 LDS operand reads per MFMA instead of 0.75). Waves 0..4 each unpack one 32-row weight block and
// publish its fragments; waves 5..7 only multiply (and, for the formats dear to unpack, move the activations: below). (The fifth block shared by waves
// 4..7, one slice each, so that every SIMD carries the same unpack arithmetic, was slower: 130 -> 141 us at T = 2048 --
// four more waves fetch raw bytes and derive scales every step.) Work distribution and K-split slots are the tall
// kernel's at MI = 4.
// MI = 2 is the tile at 128 rows, for prompts of 96 ... 256 rows, where the 256-row tile multiplies rows that do not exist
// or is cut along K more finely: four waves along T, and the five column blocks dealt to two wave groups, three to waves
// 0..3 and two to waves 4..7 -- wave w and wave w + 4 share a SIMD, so every SIMD still carries five blocks of MFMAs per
// slice. Measured against the best other tile, us: Q4_K 5120 x 5120 at 256 rows 36.1 -> 32.9, 34816 x 5120 at 128 rows
// 75.7 -> 68.9, Q6_K 5120 x 17408 at 128 rows 64.6 -> 59.0, Q8_0 12288 x 4096 at 128 rows 57.8 -> 52.3; at 512 rows of
// 5120 x 5120 (128 tiles cut in two instead of 64 cut in four) it is level, 49.2 against 48.0.
// ------------------------------------------------------------------------------------------------
template <class F, int MI>
__global__ void __launch_bounds__(512) gemm_q_bf16_n160_kernel(GemmParams p) {
    constexpr int NB = 5;
    constexpr int BM = 64 * MI, BN = 32 * NB;
    constexpr int TW = BM / 32, NBW = TW == 8 ? NB : 3;         // waves along T; column blocks a wave holds at most
    constexpr int FRAG = 512;
    __shared__ __attribute__((aligned(16))) uint16_t As[2][BM * LDS_ROW];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[2][NB * 4 * FRAG];   // [n-block 0..4][slice 0..3]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, c = lane & 31;
    const bool unpacker = wave < NB;                            // wave-uniform
    const int tw = TW == 8 ? wave : (wave & 3);                 // the wave's 32 activation rows of the tile
    const int j0 = TW == 8 ? 0 : (wave < 4 ? 0 : 3);            // its first column block ...
    const int nj = TW == 8 ? NB : (wave < 4 ? 3 : 2);           // ... and how many it holds (wave-uniform)
    const int nchunks = p.nchunks;
    long long u = (long long)blockIdx.x * p.per;
    const long long u_end = u + p.per < p.units ? u + p.per : p.units;
  for (int round = 0;; round++) {
    int tile, c_begin, c_end;
    if (round < p.whole_rounds) {
        tile = round * gridDim.x + blockIdx.x;
        c_begin = 0;
        c_end = nchunks;
    } else {
        if (u >= u_end) break;
        const int rt = (int)(u / nchunks);
        tile = p.whole_rounds * gridDim.x + rt;
        c_begin = (int)(u - (long long)rt * nchunks);
        c_end = (long long)(nchunks - c_begin) < u_end - u ? nchunks : c_begin + (int)(u_end - u);
        u += c_end - c_begin;
    }
    const bool whole = c_begin == 0 && c_end == nchunks;
    const int tile_y = tile / p.tiles_n, tile_x = tile - tile_y * p.tiles_n;
    const int t0 = tile_y * BM + 32 * tw;
    const int n0 = tile_x * BN;
    const int c_last = c_end - 1;

    // the weight row an unpacking lane works on: row c of n-block `wave` of the tile (clamped: rows past N are computed but
    // not stored); the other waves point at a valid row and never read it
    const uint8_t* wrow;
    {
        int n = n0 + 32 * (unpacker ? wave : 0) + c;
        wrow = p.W + (size_t)(n < p.N ? n : p.N - 1) * p.row_bytes;
    }
    const int b_wr = (wave * 4) * FRAG + lane * 8;              // + t * FRAG (unpackers)
    const int b_rd = (4 * j0) * FRAG + lane * 8;                // + (4 * j + t) * FRAG

    f32x16 acc[NBW];
#pragma unroll
    for (int j = 0; j < NBW; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[j][r] = 0.f;

    // Activation staging, BM rows x 64 bf16 per step, global -> registers one step ahead -> padded LDS. Rows past T are read
    // from row T-1 (their outputs are never stored); columns past K (a partial last chunk) are staged as zeros. Who moves
    // them depends on what a weight costs to unpack. Q4_K: every thread, the 16-byte piece (tid & 7) of rows (tid >> 3) +
    // 64 q, as in the tall kernel. Q6_K and Q8_0: the three waves that unpack nothing -- lane sl of those 192 moves piece
    // (sl & 7) of rows (sl >> 3) + 24 q, q < 11 (the eleventh round holds 16 rows, for the first two of the three waves) --
    // which takes 20 of some 190 instructions a step off the waves that set the pace (Q8_0 5120 x 4096 at T = 2048 150 ->
    // 133 us, Q6_K 5120 x 17408 444 -> 432 us; Q4_K 5120 x 5120 131 -> 135 us, so it keeps the even split).
    // (at 128 rows: six rounds, the sixth holds 8 rows, for the first of the three waves)
    constexpr bool SPLIT = F::UNPACK_US > 2.f;
    constexpr int NQ = SPLIT ? (MI == 4 ? 11 : 6) : MI, RSTEP = SPLIT ? 24 : 64;
    const bool stager = SPLIT ? !unpacker : true;               // wave-uniform
    const bool qlast = SPLIT ? wave < NB + (MI == 4 ? 2 : 1) : true;   // wave-uniform: the wave has a piece in the last round
    const int sl = SPLIT ? (wave - NB) * 64 + lane : tid;
    const int a_col = (sl & 7) * 8;
    uint32_t a_src[NQ];
    u32x4 stage[NQ];
    if (stager) {
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const int t = tile_y * BM + (sl >> 3) + RSTEP * q;
            a_src[q] = (uint32_t)(t < p.T ? t : p.T - 1) * (uint32_t)p.K + a_col;
        }
    }
    const int a_dst = (sl >> 3) * LDS_ROW + a_col;              // + RSTEP q LDS_ROW
    auto load_a = [&](int s) {
        if constexpr (F::PARTIAL) {
            const bool ok = s * KSTEP + a_col < p.K;
            const int off = ok ? s * KSTEP : 0;
            const uint32_t keep = ok ? 0xFFFFFFFFu : 0u;
#pragma unroll
            for (int q = 0; q < NQ; q++)
                if (q < NQ - 1 || qlast) {
                    u32x4 v = *(const u32x4*)(p.X + (a_src[q] + off));
                    stage[q] = (u32x4){v[0] & keep, v[1] & keep, v[2] & keep, v[3] & keep};
                }
        } else {
            const int off = s * KSTEP < p.K ? s * KSTEP : 0;   // past the end: any valid address, the tile is never read
#pragma unroll
            for (int q = 0; q < NQ; q++)
                if (q < NQ - 1 || qlast) stage[q] = *(const u32x4*)(p.X + (a_src[q] + off));
        }
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int q = 0; q < NQ; q++)
            if (q < NQ - 1 || qlast) *(u32x4*)(&As[buf][a_dst + RSTEP * q * LDS_ROW]) = stage[q];
    };
    const int a_rd = (32 * tw + c) * LDS_ROW + 16 * h;          // + kcol(t, 0)
    typename F::Raw raw;
    if (stager) load_a(4 * c_begin);
    if (unpacker) {
        F::prime(raw, wrow, c_begin, h, p.nblk);
        const int nc = c_begin + 1 < c_last ? c_begin + 1 : c_last;
        typename F::Ctx x;
        F::template begin<0>(raw, c_begin, h, p.nblk, x);
        static_for<0, 4>([&](auto T) {
            *(bf16x8*)(&Bs[0][b_wr + T.value * FRAG]) = F::template frag<0, T.value>(raw, x);
        });
        F::template refill<0>(raw, wrow, nc, h, p.nblk);
    }
    if (stager) store_a(0);
    __syncthreads();

    // one k-step, as in the tall kernel; UNPACK: the wave produces its block's fragments, one behind each slice's MFMAs
    // (NJ: the column blocks the wave holds, a constant of the loop it runs)
    auto step = [&](auto Gc, auto Uc, auto Jc, int ck) {
        constexpr int G = decltype(Gc)::value;
        constexpr bool UNPACK = decltype(Uc)::value;
        constexpr int NJ = decltype(Jc)::value;
        constexpr int GN = (G + 1) & 3;
        constexpr int buf = G & 1;
        constexpr int VPM = (26 + NJ - 1) / NJ;
        const int pc = G == 3 ? (ck + 1 < c_last ? ck + 1 : c_last) : ck;
        const int nc = pc + 1 < c_last ? pc + 1 : c_last;
        typename F::Ctx ctx;
        bf16x8 a[2], b[2][NJ];
        auto read_ops = [&](int t, bf16x8& da, bf16x8 (&db)[NJ]) {
            da = *(const bf16x8*)(&As[buf][a_rd + kcol(t, 0)]);
#pragma unroll
            for (int j = 0; j < NJ; j++) db[j] = *(const bf16x8*)(&Bs[buf][b_rd + (4 * j + t) * FRAG]);
        };
        read_ops(0, a[0], b[0]);
        if constexpr (!(UNPACK && SPLIT)) load_a(4 * ck + G + 1);
        if constexpr (UNPACK) F::template begin<GN>(raw, pc, h, p.nblk, ctx);
        __builtin_amdgcn_sched_barrier(0);
        static_for<0, 4>([&](auto S) {
            constexpr int t = decltype(S)::value;
            if constexpr (t < 3) read_ops(t + 1, a[(t + 1) & 1], b[(t + 1) & 1]);
#pragma unroll
            for (int j = 0; j < NJ; j++) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[t & 1], b[t & 1][j], acc[j], 0, 0, 0);
            if constexpr (UNPACK) *(bf16x8*)(&Bs[buf ^ 1][b_wr + t * FRAG]) = F::template frag<GN, t>(raw, ctx);
            if constexpr (t < 3) __builtin_amdgcn_sched_group_barrier(0x100, 1 + NJ, 0);
#pragma unroll
            for (int m = 0; m < NJ; m++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if constexpr (UNPACK) __builtin_amdgcn_sched_group_barrier(0x002, VPM, 0);
            }
            if constexpr (UNPACK) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
            __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (UNPACK) F::template refill<GN>(raw, wrow, nc, h, p.nblk);
        if constexpr (!(UNPACK && SPLIT)) store_a(buf ^ 1);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
    };

    auto run = [&](auto Uc, auto Jc) {
        for (int ck = c_begin; ck < c_end; ck++) {
            step(std::integral_constant<int, 0>{}, Uc, Jc, ck);
            step(std::integral_constant<int, 1>{}, Uc, Jc, ck);
            step(std::integral_constant<int, 2>{}, Uc, Jc, ck);
            step(std::integral_constant<int, 3>{}, Uc, Jc, ck);
        }
    };
    if constexpr (TW == 8) {
        if (unpacker) run(std::true_type{}, std::integral_constant<int, NB>{});
        else run(std::false_type{}, std::integral_constant<int, NB>{});
    } else {
        if (wave < 4) run(std::true_type{}, std::integral_constant<int, 3>{});
        else if (unpacker) run(std::true_type{}, std::integral_constant<int, 2>{});
        else run(std::false_type{}, std::integral_constant<int, 2>{});
    }

    float* part = nullptr;
    if (!whole) {
        const int rt = tile - p.whole_rounds * (int)gridDim.x;
        const int k = (int)blockIdx.x - (int)(((long long)rt * nchunks) / p.per);
        part = p.ws + ((size_t)rt * p.kmax + k) * (size_t)(BM * BN);
    }
    // D layout of the 32x32 MFMA: register r of lane (h, c) is row 8*(r/4) + 4*h + (r%4), column c
#pragma unroll
    for (int j = 0; j < NBW; j++) {
        const int n = n0 + 32 * (j0 + j) + c;
        if (j >= nj || n >= p.N) continue;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int t = t0 + 8 * (r >> 2) + 4 * h + (r & 3);
            if (t < p.T) {
                if (whole) p.Y[(size_t)t * p.N + n] = acc[j][r];
                else part[(size_t)(t - tile_y * BM) * BN + (n - tile_x * BN)] = acc[j][r];
            }
        }
    }
  }
}

// Left-over tile `blockIdx.x` (BM x BN outputs, BN a multiple of 4), if more than one run contributed to it: Y = slot 0 +
// slot 1 + ... in that order. A thread owns four adjacent columns of one row (item blockIdx.y * 256 + threadIdx.x of the
// tile's BM * BN / 4) and asks for up to eight slots at once: the launch is a few dependent trips to memory long, so it
// is cut as finely as that allows (a thread per 16 rows took 7.6 us for the 40 tiles of 5120 x 5120 at T = 128).
__global__ void __launch_bounds__(256) sum_split_tiles_kernel(float* __restrict__ Y, const float* __restrict__ ws, int T, int N, int BM, int BN,
                                                            int tiles_n, int nchunks, int per, int kmax, int first_tile) {
    const int rt = blockIdx.x, tile = first_tile + rt;
    const long long u0 = (long long)rt * nchunks;
    const int nk = (int)((u0 + nchunks - 1) / per) - (int)(u0 / per) + 1;
    if (nk == 1) return;                          // one run covered the whole K of this tile and stored it
    const int tile_y = tile / tiles_n, tile_x = tile - tile_y * tiles_n;
    const int item = blockIdx.y * 256 + threadIdx.x, bn4 = BN >> 2;
    const int lt = item / bn4, c4 = (item - lt * bn4) * 4;
    const int t = tile_y * BM + lt, col = tile_x * BN + c4;
    if (lt >= BM || t >= T || col >= N) return;
    const size_t slot = (size_t)BM * BN;
    const float* q = ws + (size_t)rt * kmax * slot + (size_t)lt * BN + c4;
    float4 a = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < nk; k0 += 8) {
        float4 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = *(const float4*)(q + (size_t)(k0 + j < nk ? k0 + j : 0) * slot);
        if (k0 == 0) a = v[0];
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (k0 + j > 0 && k0 + j < nk) { a.x += v[j].x; a.y += v[j].y; a.z += v[j].z; a.w += v[j].w; }
    }
    float* y = Y + (size_t)t * N + col;
    if ((N & 3) == 0) *(float4*)y = a;
    else {
        y[0] = a.x;
        if (col + 1 < N) y[1] = a.y;
        if (col + 2 < N) y[2] = a.z;
        if (col + 3 < N) y[3] = a.w;
    }
}

// ------------------------------------------------------------------------------------------------
// T <= 32 (batched decode, short prompts): one 32-row MFMA slab of activations, so the kernel is bound by
// the weight stream and its unpack arithmetic, not by the matrix pipe. A workgroup is 4 waves on 4 adjacent
// 32-row weight blocks; each wave unpacks its own block straight into its B operand (no LDS for weights)
// with the weight bytes one chunk ahead, the same register image and refill order as the tiled kernel. The
// activations of a chunk (TP rows x 256 columns, TP = 8 or 32) are staged once per workgroup in LDS, double
// buffered, one barrier per chunk. The (128-row group, chunk) units, chunk fastest, are dealt to the
// workgroups in equal contiguous runs, two to four workgroups per CU; a segment that covers its group's whole K
// stores its tile, any other stores partial sums into the workspace slot (group, contributor) and sum_split_groups_kernel
// adds a group's slots in contributor order afterwards, as for the tiled kernel.
// ------------------------------------------------------------------------------------------------
struct SkinnyParams {
    const uint8_t* W;
    const uint16_t* X;
    float* Y;
    int T, N, K;
    int nblk;
    size_t row_bytes;
    int nchunks;
    long long units;   // 128-row groups * nchunks
    int per;           // units per workgroup
    float* ws;         // partial sums of groups that several runs share: [group][contributor][TP x 128]
    int kmax;          // contributor slots per group
};

constexpr int XROW = CHUNK + 8;   // bf16 per staged activation row of a chunk (+16 B pad)

template <class F, int TP>
__global__ void __launch_bounds__(256, TP == 8 ? 4 : 2) gemm_q_bf16_skinny_kernel(SkinnyParams p) {
    __shared__ __attribute__((aligned(16))) uint16_t Xs[2][TP * XROW];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, c = lane & 31;
    const int nchunks = p.nchunks;
    long long u = (long long)blockIdx.x * p.per;
    const long long u_end = u + p.per < p.units ? u + p.per : p.units;
    // staging: thread `tid` moves the 16-byte piece (tid & 31) of rows (tid >> 5) + 8q, q < TP / 8; rows past T
    // repeat row T-1 (their outputs are never stored)
    constexpr int NQ = TP / 8;
    const int s_col = (tid & 31) * 8;
    uint32_t s_src[NQ];
#pragma unroll
    for (int q = 0; q < NQ; q++) {
        int t = (tid >> 5) + 8 * q;
        s_src[q] = (uint32_t)(t < p.T ? t : p.T - 1) * (uint32_t)p.K;
    }
    const int s_dst = (tid >> 5) * XROW + s_col;
    const int k_last = p.K - 8;   // a partial last chunk reads earlier columns of the same row (their weights are 0)
    u32x4 stage[NQ];
    auto load_x = [&](int ck) {
        int col = ck * CHUNK + s_col;
        col = col < k_last ? col : k_last;
#pragma unroll
        for (int q = 0; q < NQ; q++) stage[q] = *(const u32x4*)(p.X + (s_src[q] + col));
    };
    auto store_x = [&](int buf) {
#pragma unroll
        for (int q = 0; q < NQ; q++) *(u32x4*)(&Xs[buf][s_dst + 8 * q * XROW]) = stage[q];
    };
    const int a_rd = (c & (TP - 1)) * XROW + 16 * h;   // + 64 * step + kcol(t, 0)

    for (int seg = 0; u < u_end; seg++) {
        const int grp = (int)(u / nchunks);
        const int c_begin = (int)(u - (long long)grp * nchunks);
        const int c_end = (long long)(nchunks - c_begin) < u_end - u ? nchunks : c_begin + (int)(u_end - u);
        u += c_end - c_begin;
        const bool whole = c_begin == 0 && c_end == nchunks;
        const int c_last = c_end - 1;
        const int n = grp * 128 + wave * 32 + c;
        const uint8_t* wrow = p.W + (size_t)(n < p.N ? n : p.N - 1) * p.row_bytes;

        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0.f;
        // Weight bytes: the whole next chunk is requested at the top of a chunk, all its loads back to back, so
        // the two or three cache lines a row's block spans are fetched from L2 once (loads of one block spread
        // over the chunk's steps would find the line evicted from L1 each time and refetch it).
        typename F::Raw raw, nxt;
        bf16x8 a[4], b[4];   // both operands of the step in flight; each slice is replaced as soon as its MFMA has issued
        F::prime(raw, wrow, c_begin, h, p.nblk);
        load_x(c_begin);
        if (seg > 0) __syncthreads();   // the previous segment's last reads of buffer 0 are done
        store_x(0);
        {
            typename F::Ctx x;
            F::template begin<0>(raw, c_begin, h, p.nblk, x);
            static_for<0, 4>([&](auto T) { b[T.value] = F::template frag<0, T.value>(raw, x); });
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < 4; t++) a[t] = *(const bf16x8*)(&Xs[0][a_rd + kcol(t, 0)]);

        for (int ck = c_begin; ck < c_end; ck++) {
            const int buf = (ck - c_begin) & 1;
            const int cn = ck + 1 < c_end ? ck + 1 : ck;
            F::prime(nxt, wrow, cn, h, p.nblk);
            load_x(cn);
            static_for<0, 4>([&](auto Gc) {
                constexpr int G = decltype(Gc)::value;
                constexpr int GN = (G + 1) & 3;
                typename F::Ctx x;
                if constexpr (G == 3) {
                    F::template begin<0>(nxt, cn, h, p.nblk, x);
                    static_for<0, 4>([&](auto T) {
                        constexpr int t = decltype(T)::value;
                        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[t], b[t], acc, 0, 0, 0);
                        b[t] = F::template frag<0, t>(nxt, x);
                    });
                    store_x(buf ^ 1);
                    __syncthreads();
#pragma unroll
                    for (int t = 0; t < 4; t++) a[t] = *(const bf16x8*)(&Xs[buf ^ 1][a_rd + kcol(t, 0)]);
                } else {
                    F::template begin<GN>(raw, ck, h, p.nblk, x);
                    static_for<0, 4>([&](auto T) {
                        constexpr int t = decltype(T)::value;
                        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[t], b[t], acc, 0, 0, 0);
                        a[t] = *(const bf16x8*)(&Xs[buf][a_rd + KSTEP * (G + 1) + kcol(t, 0)]);
                        b[t] = F::template frag<GN, t>(raw, x);
                    });
                }
            });
            raw = nxt;
        }
        // runs are numbered by blockIdx.x; the first run that touches group grp is the one that holds unit grp * nchunks
        float* part = whole ? nullptr
                            : p.ws + ((size_t)grp * p.kmax + ((int)blockIdx.x - (int)(((long long)grp * nchunks) / p.per))) * (size_t)(TP * 128) + wave * 32 + c;
        if (n < p.N) {
#pragma unroll
            for (int r = 0; r < (TP == 8 ? 4 : 16); r++) {
                const int t = 8 * (r >> 2) + 4 * h + (r & 3);
                if (t < p.T) {
                    if (whole) p.Y[(size_t)t * p.N + n] = acc[r];
                    else part[t * 128] = acc[r];
                }
            }
        }
    }
}

// Group `blockIdx.x` of 128 outputs, if more than one run contributed to it: Y = slot 0 + slot 1 + ... in that order.
// Thread = output column (threadIdx.x & 127) of row 2 * blockIdx.y + (threadIdx.x >> 7); eight slots are requested at a time.
__global__ void __launch_bounds__(256) sum_split_groups_kernel(float* __restrict__ Y, const float* __restrict__ ws, int T, int N, int TP,
                                                             int nchunks, int per, int kmax) {
    const int grp = blockIdx.x;
    const long long u0 = (long long)grp * nchunks;
    const int nk = (int)((u0 + nchunks - 1) / per) - (int)(u0 / per) + 1;
    if (nk == 1) return;
    const int col = threadIdx.x & 127, n = grp * 128 + col, t = 2 * blockIdx.y + (threadIdx.x >> 7);
    if (n >= N || t >= T) return;
    const size_t slot = (size_t)TP * 128;
    const float* q = ws + (size_t)grp * kmax * slot + t * 128 + col;
    float a = q[0];
    for (int k0 = 1; k0 < nk; k0 += 8) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = q[(size_t)(k0 + j < nk ? k0 + j : 0) * slot];
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (k0 + j < nk) a += v[j];
    }
    Y[(size_t)t * N + n] = a;
}

struct SkinnyPlan { long long groups, units, per; unsigned grid; int kmax; int tp; bool split; };

static SkinnyPlan plan_skinny(size_t rows, int nchunks, size_t t, long long cus) {
    SkinnyPlan q;
    q.groups = ((long long)rows + 127) / 128;
    q.units = q.groups * nchunks;
    q.tp = t <= 8 ? 8 : 32;
    // workgroups per CU as the register budget allows: four with 8 activation rows staged, two with 32
    const long long wgs = cus * (t <= 8 ? 4 : 2);
    long long per = (q.units + wgs - 1) / wgs;
    if (per * 4 >= (long long)nchunks * 3 && per < nchunks) per = nchunks;   // nearly whole groups: make them whole
    if (per < 1) per = 1;
    q.per = per;
    q.grid = (unsigned)((q.units + per - 1) / per);
    q.split = per % nchunks != 0;
    // a group's nchunks units lie in at most this many runs of `per`
    q.kmax = q.split ? (int)((nchunks + per - 2) / per) + 1 : 1;
    return q;
}

static size_t skinny_ws_bytes(const SkinnyPlan& q) { return q.split ? (size_t)q.groups * q.kmax * q.tp * 128 * sizeof(float) : 0; }

template <class F>
int launch_skinny(const fhip_weight* w, const uint16_t* d_x, size_t t, float* d_y, hipStream_t s, float* d_ws, size_t ws_bytes) {
    SkinnyParams p;
    p.W = w->d_raw; p.X = d_x; p.Y = d_y;
    p.T = (int)t; p.N = (int)w->rows; p.K = (int)w->cols; p.row_bytes = w->row_bytes;
    p.nblk = (int)(w->row_bytes / F::BLOCK);
    p.nchunks = F::chunks(p.K);
    const long long cus = fhip::device_cus() > 0 ? fhip::device_cus() : 256;
    const SkinnyPlan q = plan_skinny(w->rows, p.nchunks, t, cus);
    p.units = q.units;
    p.per = (int)q.per;
    p.ws = d_ws; p.kmax = q.kmax;
    if (q.split && (!d_ws || ws_bytes < skinny_ws_bytes(q)))
        return fhip::set_error(FHIP_ERR_ARG, "gemm_q_bf16: the launch cuts row groups along K and needs %zu bytes of workspace", skinny_ws_bytes(q));
    if (t <= 8) hipLaunchKernelGGL((gemm_q_bf16_skinny_kernel<F, 8>), dim3(q.grid), dim3(256), 0, s, p);
    else hipLaunchKernelGGL((gemm_q_bf16_skinny_kernel<F, 32>), dim3(q.grid), dim3(256), 0, s, p);
    if (q.split)
        hipLaunchKernelGGL(sum_split_groups_kernel, dim3((unsigned)q.groups, (unsigned)((t + 1) / 2)), dim3(256), 0, s, d_y, (const float*)d_ws, p.T, p.N, q.tp, p.nchunks,
                           p.per, p.kmax);
    return fhip::check_hip(hipGetLastError(), "gemm_q_bf16 launch");
}

// How a launch of the tiled kernel with tile height 64 * mi is dealt to the chip: `whole_rounds` whole tiles per workgroup,
// then the left-over tiles cut along K into runs of `per` chunks.
struct TilePlan {
    int mi, bn;                         // tile of 64 * mi activation rows x bn outputs (256, 128, or 160 with mi = 4 or 2)
    int whole_rounds, per;
    long long left, units, split_wgs;   // left-over tiles, their chunks, workgroups whose run ends in partial tiles
    int kmax;                           // most runs that touch one left-over tile
    long long slots;                    // partial tiles the launch writes: over the left-over tiles cut along K, the runs that touch each
    float extra_starts;                 // tiles a run touches beyond its first, on average (a run that ends in the next tile starts twice)
    unsigned grid;
};

static TilePlan plan_tiles(long long tiles_n, int nchunks, size_t t, int mi, long long cus, int bn = 256) {
    TilePlan q;
    q.mi = mi; q.bn = bn;
    const long long tiles = tiles_n * (long long)((t + 64 * mi - 1) / (64 * mi));
    q.whole_rounds = (int)(tiles / cus);
    q.left = tiles - q.whole_rounds * cus;
    q.units = q.left * nchunks;
    long long per = (q.units + cus - 1) / cus;
    // a run shorter than a tile's K that is close to it is rounded up to whole tiles: no partial tiles, no summing launch
    if (per * 4 >= (long long)nchunks * 3) per = nchunks;
    if (per < 1) per = 1;
    q.per = (int)per;
    const long long runs = (q.units + per - 1) / per;
    q.grid = q.whole_rounds > 0 ? (unsigned)cus : (unsigned)runs;
    q.split_wgs = (q.left > 0 && per % nchunks != 0) ? runs : 0;
    q.kmax = 1;
    q.slots = 0;
    long long segs = 0;
    for (long long rt = 0; rt < q.left && q.split_wgs > 0; rt++) {
        const long long u0 = rt * nchunks;
        const int k = (int)((u0 + nchunks - 1) / per - u0 / per) + 1;
        if (k > q.kmax) q.kmax = k;
        if (k > 1) q.slots += k;
        segs += k;
    }
    q.extra_starts = q.split_wgs > 0 ? (float)segs / (float)runs - 1.f : 0.f;
    return q;
}

// Estimated duration of a plan in us: 4.3 for the launch, 1.5 per tile or run a workgroup starts (4.0 more per further tile a
// run reaches into), chunks per workgroup x the cost of a chunk of that tile and format (F::CHUNK_US), and, when tiles are cut
// along K, the partial tiles and the launch that sums them: 7.8 per 256 partial tiles of 64 x 256 written and read back, plus a
// constant per tile shape. A linear model fitted (relative least squares, 7 % rms) to 620 forced-tile launches: ten weights of
// the four formats (5120 x 5120, 34816 x 5120, 7168 x 5120, 10240 x 5120, 4096 x 4096 Q4_K; 5120 x 17408, 5120 x 5120 Q6_K;
// 4096 x 4096, 12288 x 4096 Q8_0; 5120 x 5120 Q5_K) at 48 ... 2048 rows, every tile. On those the tile it picks is 1.0 % slower
// than the measured best on average (worst: 17 %, Q6_K 5120 x 5120 at 256 rows).
constexpr float FIXUP_US[7] = {0.9f, -2.3f, -13.2f, -5.2f, -1.0f, 1.5f, 0.4f};
static int tile_index(const TilePlan& q) { return q.bn == 256 ? (q.mi == 1 ? 0 : q.mi == 2 ? 1 : 2) : q.bn == 160 ? (q.mi == 4 ? 3 : 6) : (q.mi == 2 ? 4 : 5); }
template <class F>
static float plan_cost_us(const TilePlan& q, int nchunks, long long cus) {
    const int ti = tile_index(q);
    const float chunks = (float)q.whole_rounds * (float)nchunks + (q.left > 0 ? (float)q.per : 0.f);
    const float starts = (float)q.whole_rounds + (q.left > 0 ? 1.f : 0.f);
    float fix = 0.f;
    if (q.split_wgs > 0) {
        fix = FIXUP_US[ti] + 7.77f * (float)q.mi * ((float)q.bn / 256.f) * (float)q.slots / (float)cus;
        fix = fix > 0.f ? fix : 0.f;
    }
    return 4.29f + 1.5f * starts + 3.96f * q.extra_starts + chunks * F::CHUNK_US[ti] + fix;
}

static size_t plan_ws_bytes(const TilePlan& q) {
    return q.split_wgs > 0 ? (size_t)q.left * q.kmax * (size_t)(64 * q.mi * q.bn) * sizeof(float) : 0;
}

template <class F, int MI, int BN>
int launch_cfg(const fhip_weight* w, const uint16_t* d_x, size_t t, float* d_y, hipStream_t s, const TilePlan& q, long long cus, float* d_ws,
               size_t ws_bytes) {
    GemmParams p;
    p.W = w->d_raw; p.X = d_x; p.Y = d_y;
    p.T = (int)t; p.N = (int)w->rows; p.K = (int)w->cols; p.row_bytes = w->row_bytes;
    p.nblk = (int)(w->row_bytes / F::BLOCK);
    p.nchunks = F::chunks(p.K);
    p.tiles_n = (int)((w->rows + BN - 1) / BN);
    // one workgroup per CU (its LDS tiles take most of a CU's 160 KB)
    p.whole_rounds = q.whole_rounds;
    p.units = q.units;
    p.per = q.per;
    p.ws = d_ws; p.kmax = q.kmax;
    if (q.split_wgs > 0 && (!d_ws || ws_bytes < plan_ws_bytes(q)))
        return fhip::set_error(FHIP_ERR_ARG, "gemm_q_bf16: the launch cuts tiles along K and needs %zu bytes of workspace", plan_ws_bytes(q));
    if constexpr (BN == 256) hipLaunchKernelGGL((gemm_q_bf16_kernel<F, MI, 2>), dim3(q.grid), dim3(512), 0, s, p);
    else if constexpr (BN == 128) hipLaunchKernelGGL((gemm_q_bf16_kernel<F, MI, 1>), dim3(q.grid), dim3(512), 0, s, p);
    else hipLaunchKernelGGL((gemm_q_bf16_n160_kernel<F, MI>), dim3(q.grid), dim3(512), 0, s, p);
    if (q.split_wgs > 0)
        hipLaunchKernelGGL(sum_split_tiles_kernel, dim3((unsigned)q.left, (unsigned)((64 * MI * BN / 4 + 255) / 256)), dim3(256), 0, s, d_y, (const float*)d_ws, p.T, p.N, 64 * MI,
                           BN, p.tiles_n, p.nchunks, p.per, p.kmax, (int)(p.whole_rounds * cus));
    return fhip::check_hip(hipGetLastError(), "gemm_q_bf16 launch");
}

int g_force_tile = -1;   // tests: 0..3 = 64, 128, 256 rows x 256 columns, 256 x 160; 4, 5 = 128, 64 rows x 128 columns; 6 = 128 x 160; anything else: the estimate decides

// the tile the estimate picks for this launch (one of the seven the loop lists) with its plan
template <class F>
static void choose_plan(const fhip_weight* w, size_t t, TilePlan& out) {
    const long long cus = fhip::device_cus() > 0 ? fhip::device_cus() : 256;
    const int nchunks = F::chunks((int)w->cols);
    float best_cost = 0.f;
    for (int i = 0; i < 7; i++) {                 // 64, 128, 256 rows x 256 columns, 256 x 160, 128 and 64 rows x 128 columns, 128 x 160
        constexpr int MI_OF[7] = {1, 2, 4, 4, 2, 1, 2}, BN_OF[7] = {256, 256, 256, 160, 128, 128, 160};
        const int mi = MI_OF[i], bn = BN_OF[i];
        if (g_force_tile >= 0 && g_force_tile <= 6 && i != g_force_tile) continue;
        const TilePlan q = plan_tiles((long long)((w->rows + bn - 1) / bn), nchunks, t, mi, cus, bn);
        const float c = plan_cost_us<F>(q, nchunks, cus);
        if (best_cost == 0.f || c < 0.98f * best_cost) { best_cost = c; out = q; }
    }
}

template <class F>
static size_t ws_bytes_fmt(const fhip_weight* w, size_t t) {
    if (t <= 32) return skinny_ws_bytes(plan_skinny(w->rows, F::chunks((int)w->cols), t, fhip::device_cus() > 0 ? fhip::device_cus() : 256));
    TilePlan q;
    choose_plan<F>(w, t, q);
    return plan_ws_bytes(q);
}

template <class F>
int launch_fmt(const fhip_weight* w, const uint16_t* d_x, size_t t, float* d_y, hipStream_t s, float* d_ws, size_t ws_bytes) {
    if (t <= 32) return launch_skinny<F>(w, d_x, t, d_y, s, d_ws, ws_bytes);
    // Which tile. The 256 x 256 tile unpacks each weight once per 256 activation rows, but when there is no whole round of
    // such tiles for the chip every tile is cut along K, each workgroup writes a whole partial tile for a few chunks of
    // work, and a lower tile (twice the tiles, half the fix-up, longer runs), the 256 x 160 tile (whose count divides the
    // chip for output widths like 5120 and 4096) or, for short prompts, a 128-column tile (half the partial-tile bytes a
    // workgroup writes, every weight unpacked once at 128 rows) can win: the estimate decides. Measured, us at 64 / 128 / 256
    // rows x 256, 256 x 160, 128 / 64 rows x 128: Q4_K 5120 x 5120 T = 64 21 / 25 / 32 / 34 / 21 / 18, T = 128 25 / 27 / 35 / 36 /
    // 22 / 27, T = 512 67 / 56 / 53 / 47 / 54 / 62; Q4_K 34816 x 5120 T = 64 57 / 68 / 102 / 96 / 68 / 55, T = 256 157 / 113 / 119 /
    // 100 / 132 / 187; Q6_K 5120 x 17408 T = 128 80 / 62 / 77 / 73 / 67 / 103, T = 512 254 / 157 / 133 / 116 / 209 / 327; Q8_0
    // 4096 x 4096 T = 128 35 / 33 / 37 / 32 / 31 / 40.
    const long long cus = fhip::device_cus() > 0 ? fhip::device_cus() : 256;
    TilePlan q;
    choose_plan<F>(w, t, q);
    if (q.bn == 160) return q.mi == 4 ? launch_cfg<F, 4, 160>(w, d_x, t, d_y, s, q, cus, d_ws, ws_bytes)
                                      : launch_cfg<F, 2, 160>(w, d_x, t, d_y, s, q, cus, d_ws, ws_bytes);
    if (q.bn == 128) return q.mi == 2 ? launch_cfg<F, 2, 128>(w, d_x, t, d_y, s, q, cus, d_ws, ws_bytes)
                                      : launch_cfg<F, 1, 128>(w, d_x, t, d_y, s, q, cus, d_ws, ws_bytes);
    if (q.mi == 4) return launch_cfg<F, 4, 256>(w, d_x, t, d_y, s, q, cus, d_ws, ws_bytes);
    if (q.mi == 2) return launch_cfg<F, 2, 256>(w, d_x, t, d_y, s, q, cus, d_ws, ws_bytes);
    return launch_cfg<F, 1, 256>(w, d_x, t, d_y, s, q, cus, d_ws, ws_bytes);
}

// f32 -> bf16 (round to nearest even), 8 values per thread, the tail one by one
__global__ void __launch_bounds__(256) cvt_f32_bf16_kernel(const float* __restrict__ x, uint16_t* __restrict__ out, size_t n) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i >= n) return;
    if (i + 8 <= n) {
        const float4 a = *(const float4*)(x + i), b = *(const float4*)(x + i + 4);
        u32x4 r = {pk_bf16(a.x, a.y), pk_bf16(a.z, a.w), pk_bf16(b.x, b.y), pk_bf16(b.z, b.w)};
        *(u32x4*)(out + i) = r;
    } else {
        for (size_t k = i; k < n; k++) out[k] = (uint16_t)(pk_bf16(x[k], 0.f) & 0xFFFFu);
    }
}

// SwiGLU of a [t, 2d] = [gate | up] f32 matrix, written as bf16 [t, d] for the down projection's A operand.
// Same arithmetic as the un-fused f32 op (crates/ferric-tensor/src/lib.rs:2603-2618), then one RNE rounding.
__global__ void __launch_bounds__(256) swiglu_bf16_kernel(const float* __restrict__ gu, size_t n, size_t d, uint16_t* __restrict__ out) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t row = i / d, col = i % d;
    const float g = gu[row * 2 * d + col], u = gu[row * 2 * d + d + col];
    out[i] = (uint16_t)(pk_bf16((g / (1.0f + expf(-g))) * u, 0.f) & 0xFFFFu);
}

}  // namespace

namespace fhip {

int launch_swiglu_bf16(const float* d_gu, size_t t, size_t d, uint16_t* d_out, hipStream_t s) {
    const size_t n = t * d;
    if (n == 0) return FHIP_OK;
    hipLaunchKernelGGL(swiglu_bf16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, d_gu, n, d, d_out);
    return check_hip(hipGetLastError(), "swiglu_bf16 launch");
}

int launch_cvt_bf16(const float* d_x, size_t n, uint16_t* d_out, hipStream_t s) {
    if (n == 0) return FHIP_OK;
    if ((((uintptr_t)d_x | (uintptr_t)d_out) & 15) != 0) return set_error(FHIP_ERR_ARG, "cvt_f32_bf16: pointers must be 16-byte aligned");
    hipLaunchKernelGGL(cvt_f32_bf16_kernel, dim3((unsigned)((n + 2047) / 2048)), dim3(256), 0, s, d_x, d_out, n);
    return check_hip(hipGetLastError(), "cvt_f32_bf16 launch");
}

int gemm_bf16_force_tile(int tile) {
    const int before = g_force_tile;
    g_force_tile = tile;
    return before;
}

size_t gemm_bf16_ws_bytes(const fhip_weight* w, size_t t) {
    if (!w || t == 0 || w->rows == 0) return 0;
    switch (w->type) {
        case FHIP_Q4_K: return ws_bytes_fmt<Q4K>(w, t);
        case FHIP_Q6_K: return ws_bytes_fmt<Q6K>(w, t);
        case FHIP_Q8_0: return ws_bytes_fmt<Q80>(w, t);
        case FHIP_Q5_K: return ws_bytes_fmt<Q5K>(w, t);
        default: return 0;
    }
}

int launch_gemm_bf16(const fhip_weight* w, const uint16_t* d_x, size_t t, float* d_y, hipStream_t s, float* d_ws, size_t ws_bytes) {
    if (t == 0 || w->rows == 0) return FHIP_OK;
    if (((uintptr_t)d_x & 15) != 0) return set_error(FHIP_ERR_ARG, "gemm_q_bf16: x must be 16-byte aligned");
    if ((unsigned long long)t * w->cols >= (1ull << 31))
        return set_error(FHIP_ERR_SHAPE, "gemm_q_bf16: t * cols must be below 2^31 (got %zu x %zu)", t, w->cols);
    switch (w->type) {
        case FHIP_Q4_K: return launch_fmt<Q4K>(w, d_x, t, d_y, s, d_ws, ws_bytes);
        case FHIP_Q6_K: return launch_fmt<Q6K>(w, d_x, t, d_y, s, d_ws, ws_bytes);
        case FHIP_Q8_0: return launch_fmt<Q80>(w, d_x, t, d_y, s, d_ws, ws_bytes);
        case FHIP_Q5_K: return launch_fmt<Q5K>(w, d_x, t, d_y, s, d_ws, ws_bytes);
        default: return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "QMatrix: no native matmul for ggml type %u", w->type);
    }
}

}  // namespace fhip
