// Prefill dequant-GEMM on the matrix cores, gfx950:  Y[t, n] = sum_k X[t, k] * dequant(W[n, k])
// X bf16 [T, K], W raw GGUF blocks [N, K], Y f32 [T, N], f32 accumulate.
//
// Stands for the reference's cooperative-matrix prefill kernels (crates/ferric-tensor/src/dtype.rs:2059-2096
// Q4_K, :1217-1257 Q6_K, :1333-1370 Q8_0), which dequantize an 8x8 weight tile into shared memory and
// feed an 8x8 f32 matrix unit. Here the unit is v_mfma_f32_32x32x16_bf16.
//
// Shape of the kernel. The reference found this path bound by the unpack arithmetic, not the matrix
// unit (crates/ferric-core/src/lib.rs:90-101), and the same holds here: a Q4_K weight costs ~3 VALU
// operations to turn into bf16, an MFMA retires 16K multiply-adds in 32 cycles. So
//   * each lane dequantizes straight into the B-operand registers of the MFMA it feeds (the B fragment of
//     a 32x32x16 MFMA is 8 consecutive k of one weight row per lane, which is 8 consecutive quants of the
//     GGUF stream: no LDS round trip, no transposition for the weights);
//   * a dequantized fragment is reused for every 32-row slab of the activation tile the wave owns
//     (MI slabs), so unpack cost is amortised over BM = 32*MI activation rows;
//   * the activation tile, which all 4 waves of a workgroup share, is staged through LDS (padded rows,
//     16-byte reads) and each fragment read feeds NI MFMAs;
//   * the 16 k of one MFMA are chosen inside ONE scale sub-block (the k order inside an MFMA is free as
//     long as both operands agree), so a fragment needs a single (scale, min) pair.
// One k-step is 64 columns = 4 MFMA slices. Dequantized values are exactly the f32 the CPU dequantizer
// produces, rounded to bf16 (RNE) by v_cvt_pk_bf16_f32.
#include "common.hpp"

#include <hip/hip_fp16.h>

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
struct __attribute__((packed, aligned(2))) U4A2 { u32x4 v; };
struct __attribute__((packed, aligned(2))) U2A2 { u32x2 v; };

__device__ __forceinline__ float f16_bits(uint32_t b) { return __half2float(__ushort_as_half((unsigned short)b)); }
__device__ __forceinline__ float ub(uint32_t v, int k) { return (float)((v >> (8 * k)) & 0xFFu); }
__device__ __forceinline__ float sb(uint32_t v, int k) { return (float)(int8_t)((v >> (8 * k)) & 0xFFu); }
__device__ __forceinline__ uint32_t pk_bf16(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){a, b}, bf16x2));
}
// 8 weights w_i = fma(s, q_i, o) from the bytes of two dwords -> one MFMA operand (8 bf16)
__device__ __forceinline__ bf16x8 frag8(uint32_t q0, uint32_t q1, float s, float o) {
    u32x4 r;
    r[0] = pk_bf16(fmaf(s, ub(q0, 0), o), fmaf(s, ub(q0, 1), o));
    r[1] = pk_bf16(fmaf(s, ub(q0, 2), o), fmaf(s, ub(q0, 3), o));
    r[2] = pk_bf16(fmaf(s, ub(q1, 0), o), fmaf(s, ub(q1, 1), o));
    r[3] = pk_bf16(fmaf(s, ub(q1, 2), o), fmaf(s, ub(q1, 3), o));
    return __builtin_bit_cast(bf16x8, r);
}

constexpr int KSTEP = 64;            // columns per k-step: 4 MFMA slices of 16
constexpr int LDS_ROW = KSTEP + 8;   // bf16 per staged activation row (+16 B pad: conflict-free 16-byte reads)

// ------------------------------------------------------------------------------------------------
// Per-format fragment builders. For k-step s of row `row` and lane half h (= lane / 32), produce the four
// B fragments; slice t of the step covers, for lane half h, the 8 columns
//     k0 + koff(t) + 8h' ... with the per-format column map given by `kcol`, which the activation side uses
// to fetch the matching 8 columns.
// ------------------------------------------------------------------------------------------------

struct Q4K {
    // step = group g of block b: slice t -> sub-block 2g + (t>>1), elements 16h + 8(t&1) + [0,8)
    static __device__ __forceinline__ int kcol(int t, int h) { return 32 * (t >> 1) + 16 * h + 8 * (t & 1); }
    struct Raw { u32x4 hd, q; };
    static __device__ __forceinline__ Raw load(const uint8_t* row, int step, int h) {
        const uint8_t* blk = row + (size_t)(step >> 2) * 144;
        Raw r;
        r.hd = *(const u32x4*)blk;
        r.q = *(const u32x4*)(blk + 16 + 32 * (step & 3) + 16 * h);
        return r;
    }
    static __device__ __forceinline__ void frags(const Raw& r, int step, int, bf16x8 (&b)[4]) {
        const int g = step & 3;
        // get_sc_min for sub-blocks 2g, 2g+1 (crates/ferric-gguf/src/lib.rs:795-804), two packed bytes each
        const int sh = 16 * (g & 1);
        uint32_t a = r.hd[1] >> sh, bb = r.hd[2] >> sh, c = r.hd[3] >> sh;
        uint32_t scp = g >= 2 ? ((c & 0x0F0Fu) | ((a >> 2) & 0x3030u)) : (a & 0x3F3Fu);
        uint32_t mp = g >= 2 ? (((c >> 4) & 0x0F0Fu) | ((bb >> 2) & 0x3030u)) : (bb & 0x3F3Fu);
        float d = f16_bits(r.hd[0] & 0xFFFFu), dmin = f16_bits(r.hd[0] >> 16);
        // y = (d*sc)*q - (dmin*m): the product is exact in f32, so the fused form rounds identically
        float d0 = d * ub(scp, 0), d1 = d * ub(scp, 1), m0 = -(dmin * ub(mp, 0)), m1 = -(dmin * ub(mp, 1));
        const uint32_t M = 0x0F0F0F0Fu;
        b[0] = frag8(r.q[0] & M, r.q[1] & M, d0, m0);
        b[1] = frag8(r.q[2] & M, r.q[3] & M, d0, m0);
        b[2] = frag8((r.q[0] >> 4) & M, (r.q[1] >> 4) & M, d1, m1);
        b[3] = frag8((r.q[2] >> 4) & M, (r.q[3] >> 4) & M, d1, m1);
    }
};

struct Q6K {
    // step = 64 columns of half hf: groups g0 = 2*(step&1), g0+1; slice t -> group g0 + (t>>1),
    // l = 16(t&1) + 8h + [0,8)  (one scale per slice: sc[8hf + 2g + l/16])
    static __device__ __forceinline__ int kcol(int t, int h) { return 32 * (t >> 1) + 16 * (t & 1) + 8 * h; }
    struct Raw { u32x2 ql[4], qh[2], sc8; uint32_t d; };
    static __device__ __forceinline__ Raw load(const uint8_t* row, int step, int h) {
        const uint8_t* blk = row + (size_t)(step >> 2) * 210;
        const int hf = (step >> 1) & 1;
        Raw r;
        r.d = *(const uint16_t*)(blk + 208);
        r.sc8 = ((const U2A2*)(blk + 192 + 8 * hf))->v;               // sc[8hf .. 8hf+8)
#pragma unroll
        for (int t = 0; t < 4; t++)                                   // group parity (t>>1), l = 16(t&1) + 8h
            r.ql[t] = ((const U2A2*)(blk + 64 * hf + 32 * (t >> 1) + 16 * (t & 1) + 8 * h))->v;
#pragma unroll
        for (int u = 0; u < 2; u++) r.qh[u] = ((const U2A2*)(blk + 128 + 32 * hf + 16 * u + 8 * h))->v;
        return r;
    }
    static __device__ __forceinline__ void frags(const Raw& r, int step, int, bf16x8 (&b)[4]) {
        const int g0 = 2 * (step & 1);                                // groups g0 (t = 0,1) and g0+1 (t = 2,3)
        float d = f16_bits(r.d);
        uint32_t scw = g0 ? r.sc8[1] : r.sc8[0];                      // sc[8hf + 2g0 + t], t = 0..3
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int g = g0 + (t >> 1);                              // ql byte parity g&1 = t>>1, nibble = g>=2 = (g0 != 0)
            uint32_t n0 = (g0 ? r.ql[t][0] >> 4 : r.ql[t][0]) & 0x0F0F0F0Fu, n1 = (g0 ? r.ql[t][1] >> 4 : r.ql[t][1]) & 0x0F0F0F0Fu;
            uint32_t h0 = ((r.qh[t & 1][0] >> (2 * g)) & 0x03030303u) << 4, h1 = ((r.qh[t & 1][1] >> (2 * g)) & 0x03030303u) << 4;
            float ds = d * sb(scw, t);
            // (d*sc)*(q-32) = ds*q - 32*ds, every term exact in f32
            b[t] = frag8(n0 | h0, n1 | h1, ds, -32.0f * ds);
        }
    }
};

struct Q80 {
    // step = blocks 2s, 2s+1: slice t -> block 2s + (t>>1), elements 16(t&1) + 8h + [0,8)
    static __device__ __forceinline__ int kcol(int t, int h) { return 32 * (t >> 1) + 16 * (t & 1) + 8 * h; }
    struct Raw { u32x2 q[4]; uint32_t d[2]; };
    static __device__ __forceinline__ Raw load(const uint8_t* row, int step, int h) {
        Raw r;
#pragma unroll
        for (int u = 0; u < 2; u++) r.d[u] = *(const uint16_t*)(row + (size_t)(2 * step + u) * 34);
#pragma unroll
        for (int t = 0; t < 4; t++) r.q[t] = ((const U2A2*)(row + (size_t)(2 * step + (t >> 1)) * 34 + 2 + 16 * (t & 1) + 8 * h))->v;
        return r;
    }
    static __device__ __forceinline__ void frags(const Raw& r, int, int, bf16x8 (&b)[4]) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            float d = f16_bits(r.d[t >> 1]);
            u32x4 o;
            o[0] = pk_bf16(sb(r.q[t][0], 0) * d, sb(r.q[t][0], 1) * d);
            o[1] = pk_bf16(sb(r.q[t][0], 2) * d, sb(r.q[t][0], 3) * d);
            o[2] = pk_bf16(sb(r.q[t][1], 0) * d, sb(r.q[t][1], 1) * d);
            o[3] = pk_bf16(sb(r.q[t][1], 2) * d, sb(r.q[t][1], 3) * d);
            b[t] = __builtin_bit_cast(bf16x8, o);
        }
    }
};

struct GemmParams {
    const uint8_t* W;
    const uint16_t* X;   // bf16 bits [T, K]
    float* Y;            // [T, N]
    int T, N, K;
    size_t row_bytes;
    int steps_per_split; // k-steps each grid.z slice walks
    int atomic;          // 1: several k-splits add into a zeroed Y
};

// Workgroup = 4 waves side by side along N; wave tile = (32*MI) x (32*NI); workgroup tile = (32*MI) x (128*NI).
template <class F, int MI, int NI>
__global__ void __launch_bounds__(256) gemm_q_bf16_kernel(GemmParams p) {
    constexpr int BM = 32 * MI;
    __shared__ __attribute__((aligned(16))) uint16_t As[2][BM * LDS_ROW];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int h = lane >> 5, c = lane & 31;
    const int t0 = blockIdx.y * BM;
    const int n0 = blockIdx.x * (128 * NI) + wave * (32 * NI);
    const int nsteps = p.K / KSTEP;
    const int s_begin = blockIdx.z * p.steps_per_split;
    const int s_end = s_begin + p.steps_per_split < nsteps ? s_begin + p.steps_per_split : nsteps;

    // weight row of each of this lane's NI fragments (clamped: rows past N are computed but not stored)
    const uint8_t* wrow[NI];
#pragma unroll
    for (int j = 0; j < NI; j++) {
        int n = n0 + 32 * j + c;
        wrow[j] = p.W + (size_t)(n < p.N ? n : p.N - 1) * p.row_bytes;
    }

    f32x16 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // activation staging: BM rows x 64 bf16 = BM * 128 B per step; each thread moves 16 B pieces
    constexpr int PIECES = BM * 8 / 256;  // 16-byte pieces per thread per step
    u32x4 stage[PIECES];
    auto load_a = [&](int s) {
#pragma unroll
        for (int q = 0; q < PIECES; q++) {
            int piece = tid + 256 * q, r = piece >> 3, col = (piece & 7) * 8;
            int t = t0 + r;
            if (t < p.T) stage[q] = *(const u32x4*)(p.X + (size_t)t * p.K + (size_t)s * KSTEP + col);
            else stage[q] = (u32x4){0, 0, 0, 0};
        }
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int q = 0; q < PIECES; q++) {
            int piece = tid + 256 * q, r = piece >> 3, col = (piece & 7) * 8;
            *(u32x4*)(&As[buf][r * LDS_ROW + col]) = stage[q];
        }
    };

    typename F::Raw raw[NI];
    if (s_begin < s_end) {
        load_a(s_begin);
#pragma unroll
        for (int j = 0; j < NI; j++) raw[j] = F::load(wrow[j], s_begin, h);
        store_a(0);
    }
    __syncthreads();
    for (int s = s_begin; s < s_end; s++) {
        const int buf = (s - s_begin) & 1;
        bf16x8 b[NI][4];
#pragma unroll
        for (int j = 0; j < NI; j++) F::frags(raw[j], s, h, b[j]);
        if (s + 1 < s_end) {                         // next step's activations and weight bytes in flight during the MFMAs
            load_a(s + 1);
#pragma unroll
            for (int j = 0; j < NI; j++) raw[j] = F::load(wrow[j], s + 1, h);
        }
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int kc = F::kcol(t, h);
#pragma unroll
            for (int i = 0; i < MI; i++) {
                bf16x8 a = *(const bf16x8*)(&As[buf][(32 * i + c) * LDS_ROW + kc]);
#pragma unroll
                for (int j = 0; j < NI; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b[j][t], acc[i][j], 0, 0, 0);
            }
        }
        if (s + 1 < s_end) store_a(buf ^ 1);
        __syncthreads();
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
                    float* y = p.Y + (size_t)t * p.N + n;
                    if (p.atomic) unsafeAtomicAdd(y, acc[i][j][r]);
                    else *y = acc[i][j][r];
                }
            }
        }
}

__global__ void zero_f32_kernel(float* __restrict__ out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = 0.f;
}

template <class F, int MI, int NI>
int launch_cfg(const fhip_weight* w, const uint16_t* d_x, size_t t, float* d_y, hipStream_t s) {
    GemmParams p;
    p.W = w->d_raw; p.X = d_x; p.Y = d_y;
    p.T = (int)t; p.N = (int)w->rows; p.K = (int)w->cols; p.row_bytes = w->row_bytes;
    const int nsteps = p.K / KSTEP;
    dim3 grid((unsigned)((w->rows + 128 * NI - 1) / (128 * NI)), (unsigned)((t + 32 * MI - 1) / (32 * MI)), 1);
    // Too few output tiles to occupy the CUs: split K over grid.z and add the slices into a zeroed Y.
    const int cus = fhip::device_cus() > 0 ? fhip::device_cus() : 256;
    int split = 1;
    const size_t tiles = (size_t)grid.x * grid.y;
    if (tiles < (size_t)cus) {
        split = (int)((cus + tiles - 1) / tiles);
        if (split > nsteps) split = nsteps;
        if (split > 16) split = 16;
    }
    p.steps_per_split = (nsteps + split - 1) / split;
    grid.z = (unsigned)((nsteps + p.steps_per_split - 1) / p.steps_per_split);
    p.atomic = grid.z > 1;
    if (p.atomic) {
        size_t n = t * w->rows;
        hipLaunchKernelGGL(zero_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, d_y, n);
    }
    hipLaunchKernelGGL((gemm_q_bf16_kernel<F, MI, NI>), grid, dim3(256), 0, s, p);
    return fhip::check_hip(hipGetLastError(), "gemm_q_bf16 launch");
}

template <class F>
int launch_fmt(const fhip_weight* w, const uint16_t* d_x, size_t t, float* d_y, hipStream_t s) {
    if (t > 64) return launch_cfg<F, 4, 2>(w, d_x, t, d_y, s);   // 128 x 256 workgroup tile
    if (t > 32) return launch_cfg<F, 2, 2>(w, d_x, t, d_y, s);
    return launch_cfg<F, 1, 2>(w, d_x, t, d_y, s);
}

}  // namespace

namespace fhip {

int launch_gemm_bf16(const fhip_weight* w, const uint16_t* d_x, size_t t, float* d_y, hipStream_t s) {
    if (w->cols % KSTEP != 0)
        return set_error(FHIP_ERR_SHAPE, "gemm_q_bf16: cols must be a multiple of %d (got %zu)", KSTEP, w->cols);
    if (((uintptr_t)d_x & 15) != 0) return set_error(FHIP_ERR_ARG, "gemm_q_bf16: x must be 16-byte aligned");
    switch (w->type) {
        case FHIP_Q4_K: return launch_fmt<Q4K>(w, d_x, t, d_y, s);
        case FHIP_Q6_K: return launch_fmt<Q6K>(w, d_x, t, d_y, s);
        case FHIP_Q8_0: return launch_fmt<Q80>(w, d_x, t, d_y, s);
        default: return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "QMatrix: no native matmul for ggml type %u", w->type);
    }
}

}  // namespace fhip
