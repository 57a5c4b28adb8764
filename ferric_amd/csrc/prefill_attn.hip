// Causal attention for a block of query rows against the cache (prefill, chunked prefill, prefix-cached suffixes), gfx950.
//
//   out[i, h] = softmax_j(q[i, h] . K[j, kv(h)] / sqrt(dh)) @ V[:, kv(h)],   j <= off + i,   off = S - T
//
// One op for the reference's causal_attention (crates/ferric-tensor/src/nn.rs:40-57), causal_attention_win (:66-88, keys older
// than `window` masked), chunked_attention (:239-265, T query rows against S >= T cached rows, query i at position off + i)
// and flash_attention_prefill (crates/ferric-llama/src/qwen3.rs:925: "all three are the same math"), with the Gemma-2 score
// softcap (:59-61). The reference composes it from permutes, two batched matmuls and a masked softmax over a [nh, T, S] score
// tensor (or a WGSL flash kernel up to its shared-memory limit); here it is one flash-style launch on the matrix cores in f32.
//
// Why f32 matrix instructions. v_mfma_f32_16x16x4_f32 multiplies f32 operands exactly and accumulates in f32: results have the
// grade of the reference's f32 arithmetic (the tests hold them to 1e-5 of the largest output against an f64 evaluation), where
// bf16 operands would leave three digits. It runs at the chip's f32 matrix rate (157 TFLOP/s), a sixteenth of bf16's.
//
// Tiling. A wave owns 16 query rows of one head; lane (c, ks) = (lane % 16, lane / 16). It keeps its query fragment in
// registers for the whole launch (query c, quarter ks of the dims: dh / 4 registers) and walks the key tiles of 32 rows that
// its queries may see. Per tile, with the two 16-key halves u = 0, 1:
//   S^T_u [16 keys x 16 queries] = K_u [16 x dh] . Q^T         (dh / 4 instructions each; an instruction's four k are one
//                                                               dim of every quarter)
//   online softmax down each column: a lane holds keys 16 u + 4 ks + i (i < 4) of ITS query, the other three lane groups the
//                                    rest, so a query's statistics are 8 register operations and two exchanges
//   O^T [dh x 16 queries] += V_tile^T [dh x 32 keys] . P^T     (dh / 16 output tiles x 8 instructions)
// Computing the transposes is what makes the second product free of data movement: register i of S^T_u in lane group ks is the
// probability of key 16 u + 4 ks + i for the lane's query, which is exactly the B operand of an instruction whose four k are
// the keys 16 u + 4 ks' + i (ks' = 0..3); the A operand reads those keys' value rows from LDS. The probabilities never leave
// their registers. Which dim an output row stands for is free as well: row m of output tile d is dim (dh / 16) m + d, so a
// lane's A operands of the dh / 16 instructions of a step are consecutive floats of one value row.
// Sixteen-row tiles rather than 32 x 32 ones keep a wave at 32 + 32 + 8 registers of fragments instead of 64 + 64 + 16, which
// is what leaves room to request the next K and V tile a tile ahead: with the larger tile the compiler had to move every
// prefetched piece out of the way as it arrived, one memory round trip after the other.
// The K and V tiles of a KV head go through LDS (K rows padded by 4 floats so that the 16-byte reads of a lane group start 4
// banks apart), shared by the 8 waves (128 queries) of a workgroup; workgroups of the same KV head read the same rows out of
// L2. Query blocks are issued longest first across all heads.
#include "common.hpp"

#include <math.h>

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// NW: waves (16 query rows each) per workgroup.
template <int HD, int NW>
__global__ __launch_bounds__(64 * NW, NW == 8 ? 4 : 2) void causal_attn_kernel(const float* __restrict__ q, const float* __restrict__ K, const float* __restrict__ V, int T,
                                                              int S, int n_head, int n_kv, float scale, int window, float softcap,
                                                              float* __restrict__ out) {
    constexpr int KS = HD + 4;              // floats per K row in LDS
    constexpr int QD = HD / 4;              // dims per quarter
    constexpr int NDT = HD / 16;            // output tiles of 16 rows
    constexpr int QROWS = 16 * NW;          // query rows per workgroup
    constexpr int NF = 32 * (HD / 4) / (64 * NW);   // 16-byte pieces of a K (and of a V) tile per thread
    static_assert(NF >= 1 && NF * 64 * NW == 32 * (HD / 4), "the tile divides over the threads");
    __shared__ __attribute__((aligned(16))) float Ks[32 * KS];
    __shared__ __attribute__((aligned(16))) float Vs[32 * HD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, ks = lane >> 4;
    // Workgroups are handed out x first: all heads' last query blocks (which see the most keys), then all heads' second to
    // last, ... -- longest first over the whole launch, so the long ones do not start late and finish alone.
    const int head = blockIdx.x, kvh = head / (n_head / n_kv);
    const int qb = (int)gridDim.y - 1 - (int)blockIdx.y;
    const int off = S - T;
    const int wg_first = qb * QROWS, wg_last = min(T - 1, wg_first + QROWS - 1);
    const int i0 = wg_first + wave * 16;
    const bool wave_live = i0 < T;                              // a wave past the last query row only helps to load tiles
    const int i_last = min(i0 + 15, T - 1);
    const int i = min(i0 + c, T - 1), qpos = off + i;           // this lane's query row and its absolute position
    // key tiles the workgroup walks, and the ones this wave's queries can see
    const int kt_hi = (off + wg_last) / 32;
    const int kt_lo = window > 0 ? max(0, off + wg_first - window + 1) / 32 : 0;
    const int my_hi = wave_live ? (off + i_last) / 32 : -1;
    const int my_lo = window > 0 ? max(0, off + i0 - window + 1) / 32 : 0;

    float qf[QD];
    {
        const float* qp = q + ((size_t)i * n_head + head) * HD + ks * QD;
#pragma unroll
        for (int t = 0; t < QD; t += 4) {
            const float4 v = *(const float4*)(qp + t);
            qf[t] = v.x; qf[t + 1] = v.y; qf[t + 2] = v.z; qf[t + 3] = v.w;
        }
    }
    f32x4 oacc[NDT];
#pragma unroll
    for (int d = 0; d < NDT; d++) oacc[d] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m = -3.0e38f, l = 0.f;
    const size_t kv_stride = (size_t)n_kv * HD;
    const float* Kh = K + (size_t)kvh * HD;
    const float* Vh = V + (size_t)kvh * HD;

    // The next tile's pieces wait in registers while the current tile is worked on (native vectors, indexed by unrolled
    // loops only: anything the compiler cannot keep in registers here lands in scratch memory, and every piece is then waited
    // for and stored as it arrives, one memory round trip after the other).
    f32x4 kreg[NF], vreg[NF];
    int prow[NF], pcol[NF];
#pragma unroll
    for (int n = 0; n < NF; n++) {
        const int f = tid + n * 64 * NW;
        prow[n] = f / (HD / 4);
        pcol[n] = (f % (HD / 4)) * 4;
    }
#pragma unroll
    for (int n = 0; n < NF; n++) {
        const size_t src = (size_t)min(kt_lo * 32 + prow[n], S - 1) * kv_stride + (size_t)pcol[n];
        kreg[n] = *(const f32x4*)(Kh + src);
        vreg[n] = *(const f32x4*)(Vh + src);
    }
    for (int kt = kt_lo; kt <= kt_hi; kt++) {
        __syncthreads();                                        // every wave is done with the previous tile
#pragma unroll
        for (int n = 0; n < NF; n++) {
            *(f32x4*)(Ks + prow[n] * KS + pcol[n]) = kreg[n];
            *(f32x4*)(Vs + prow[n] * HD + pcol[n]) = vreg[n];
        }
        __syncthreads();
        const int nxt = min(kt + 1, kt_hi);                     // in flight under this tile's arithmetic
#pragma unroll
        for (int n = 0; n < NF; n++) {
            // rows past the cache repeat its last row; they are masked below
            const size_t src = (size_t)min(nxt * 32 + prow[n], S - 1) * kv_stride + (size_t)pcol[n];
            kreg[n] = *(const f32x4*)(Kh + src);
            vreg[n] = *(const f32x4*)(Vh + src);
        }
        if (kt < my_lo || kt > my_hi) continue;                 // wave-uniform; the barriers above are reached by every wave

        // the two halves' chains alternate, so an instruction does not wait for the result of the one before it
        f32x4 sacc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
        const float* krow = Ks + c * KS + ks * QD;
#pragma unroll
        for (int t = 0; t < QD; t += 4) {
            const float4 k0 = *(const float4*)(krow + t), k1 = *(const float4*)(krow + 16 * KS + t);
            sacc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(k0.x, qf[t], sacc[0], 0, 0, 0);
            sacc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(k1.x, qf[t], sacc[1], 0, 0, 0);
            sacc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(k0.y, qf[t + 1], sacc[0], 0, 0, 0);
            sacc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(k1.y, qf[t + 1], sacc[1], 0, 0, 0);
            sacc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(k0.z, qf[t + 2], sacc[0], 0, 0, 0);
            sacc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(k1.z, qf[t + 2], sacc[1], 0, 0, 0);
            sacc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(k0.w, qf[t + 3], sacc[0], 0, 0, 0);
            sacc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(k1.w, qf[t + 3], sacc[1], 0, 0, 0);
        }
        // scores of this lane's query against its 8 keys of the tile; a tile every query of the wave sees whole needs no mask
        const bool whole = kt * 32 + 31 <= off + i0 && (window == 0 || off + i_last - kt * 32 < window);
        float mt = -3.0e38f;
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float s = sacc[u][r] * scale;
                if (softcap > 0.f) s = softcap * tanhf(s / softcap);        // cap * tanh(x / cap), crates/ferric-tensor/src/lib.rs:308
                if (!whole) {
                    const int j = kt * 32 + 16 * u + 4 * ks + r;
                    const bool ok = j <= qpos && (window == 0 || qpos - j < window);   // nn.rs:128-133
                    s = ok ? s : -3.0e38f;
                }
                sacc[u][r] = s;
                mt = fmaxf(mt, s);
            }
        mt = fmaxf(mt, __shfl_xor(mt, 16));
        mt = fmaxf(mt, __shfl_xor(mt, 32));
        const float m_new = fmaxf(m, mt);
        const float corr = __expf(m - m_new);
        float ps = 0.f;
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float p = sacc[u][r] > -2.9e38f ? __expf(sacc[u][r] - m_new) : 0.f;
                sacc[u][r] = p;
                ps += p;
            }
        l = fmaf(l, corr, ps);
        m = m_new;
#pragma unroll
        for (int d = 0; d < NDT; d++) oacc[d] *= corr;
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float* vrow = Vs + (16 * u + 4 * ks + r) * HD + NDT * c;
                float va[NDT];
#pragma unroll
                for (int d = 0; d < NDT; d += 4) {
                    const float4 t4 = *(const float4*)(vrow + d);
                    va[d] = t4.x; va[d + 1] = t4.y; va[d + 2] = t4.z; va[d + 3] = t4.w;
                }
#pragma unroll
                for (int d = 0; d < NDT; d++) oacc[d] = __builtin_amdgcn_mfma_f32_16x16x4f32(va[d], sacc[u][r], oacc[d], 0, 0, 0);
            }
    }
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    if (!wave_live || i0 + c >= T) return;
    const float inv = 1.0f / l;
    // register r of output tile d is row m = 4 ks + r, i.e. dim NDT m + d
    float* op = out + ((size_t)i * n_head + head) * HD;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        float* dst = op + NDT * (4 * ks + r);
#pragma unroll
        for (int d = 0; d < NDT; d += 4)
            *(float4*)(dst + d) = float4{oacc[d][r] * inv, oacc[d + 1][r] * inv, oacc[d + 2][r] * inv, oacc[d + 3][r] * inv};
    }
}

}  // namespace

namespace fhip {

int launch_causal_attention(const float* q, const float* K, const float* V, size_t t, size_t s, int n_head, int n_kv, int hd, size_t window,
                            float softcap, float* out, hipStream_t st) {
    if (t == 0 || n_head == 0 || hd == 0) return FHIP_OK;
    if (s < t) return set_error(FHIP_ERR_SHAPE, "cache (%zu) cannot be shorter than the query block (%zu)", s, t);   // nn.rs:73, :249
    if (n_kv <= 0 || n_head % n_kv != 0) return set_error(FHIP_ERR_SHAPE, "causal_attention: n_heads must be a multiple of n_kv_heads");
    if (hd != 64 && hd != 128) return set_error(FHIP_ERR_SHAPE, "causal_attention: head_dim must be 64 or 128");
    if (s > 0x3FFFFFFFull || n_head > 65535) return set_error(FHIP_ERR_SHAPE, "causal_attention: too large for one launch");
    // waves (16 query rows each) per workgroup: 8, or 4 while that leaves the chip fewer than two workgroups per CU
    const int cus = device_cus() > 0 ? device_cus() : 256;
    int nw = 8;
    if (((t + 127) / 128) * (size_t)n_head < 2 * (size_t)cus) nw = 4;
    const size_t qblocks = (t + (size_t)nw * 16 - 1) / ((size_t)nw * 16);
    if (qblocks > 65535) return set_error(FHIP_ERR_SHAPE, "causal_attention: too many query rows for one launch");
    const dim3 grid((unsigned)n_head, (unsigned)qblocks), wg(64 * nw);
    const float scale = 1.0f / sqrtf((float)hd);
    const int win = window == 0 || window >= s ? 0 : (int)window;     // a window that covers the cache is no window
    if (hd == 128 && nw == 8) hipLaunchKernelGGL((causal_attn_kernel<128, 8>), grid, wg, 0, st, q, K, V, (int)t, (int)s, n_head, n_kv, scale, win, softcap, out);
    else if (hd == 128) hipLaunchKernelGGL((causal_attn_kernel<128, 4>), grid, wg, 0, st, q, K, V, (int)t, (int)s, n_head, n_kv, scale, win, softcap, out);
    else if (nw == 8) hipLaunchKernelGGL((causal_attn_kernel<64, 8>), grid, wg, 0, st, q, K, V, (int)t, (int)s, n_head, n_kv, scale, win, softcap, out);
    else hipLaunchKernelGGL((causal_attn_kernel<64, 4>), grid, wg, 0, st, q, K, V, (int)t, (int)s, n_head, n_kv, scale, win, softcap, out);
    return check_hip(hipGetLastError(), "causal_attention launch");
}

}  // namespace fhip
