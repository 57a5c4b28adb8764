// Shared host-side declarations of libferric_hip: the weight handle, error plumbing and the
// kernel launchers each .hip translation unit provides.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/ferric_hip.h"
#include "../../include/ferric_hip_debug.h"

struct fhip_weight {
    uint32_t type;      // ggml id: 2 / 3 / 6 / 7 / 8 / 12 / 13 / 14 / 20 / 23 / 39
    size_t rows, cols;  // [out, in]
    size_t row_bytes;   // cols / block_values * block_bytes
    size_t nbytes;      // rows * row_bytes
    const uint8_t* d_raw;  // raw GGUF block stream in HBM
    bool owns;          // allocated by fhip_weight_create (freed on destroy)
    // How launches on this weight compute, fixed when the handle is made (from the process defaults of that moment) and
    // changed only through the handle's own setters: launches on other handles never see it.
    int planes;         // activation planes of its streaming mat-vec: 3 = 24-bit (the f32 significand), 2 = 16-bit
    int batch_policy;   // FHIP_BATCH_*: which kernels its batches of three rows and more take
};

namespace fhip {

// Expert selection for the mixture-of-experts "_id" matmuls (crates/ferric-tensor/src/dtype.rs:2463-2700).
// The weight is a slab of n_expert experts of `expert_rows` rows each. The launch is replicated over `npairs`
// (token, slot) pairs, slot s along grid.y and token ti along grid.z (sel_grid); pair p = ti * k + s uses expert e = selw[ti*2k + k + s] (the index half of a
// moe_topk row, stored as f32), activation row (x_per_pair ? p : ti) and writes at y + p * y_stride.
// selw == nullptr: a plain launch.
struct SelParams {
    const float* selw;
    int k, n_expert;
    size_t expert_rows;
    int x_per_pair;
    size_t y_stride;
    int npairs;
    int relu2;   // the pair's outputs leave as max(v, 0)^2 (the squared-ReLU expert MLP, dtype.rs:1703-1729)
};
// grid of a launch of `wgs` workgroups per pair
inline dim3 sel_grid(unsigned wgs, const SelParams& sel) {
    const unsigned k = sel.selw && sel.k > 0 ? (unsigned)sel.k : 1u;
    return dim3(wgs, k, sel.selw ? (unsigned)sel.npairs / k : 1u);
}
// applied at the top of a kernel: moves the three base pointers to this y-slice's expert / row / output
template <class P>
__device__ __forceinline__ void apply_selection(P& p) {
    if (p.sel.selw) {
        const int s = blockIdx.y, ti = blockIdx.z, pair = ti * p.sel.k + s;   // grid (workgroups, k, tokens): no division
        int e = (int)p.sel.selw[(size_t)ti * 2 * p.sel.k + p.sel.k + s];
        e = e < 0 ? 0 : (e >= p.sel.n_expert ? p.sel.n_expert - 1 : e);   // a corrupt index must not leave the slab
        e = __builtin_amdgcn_readfirstlane(e);
        p.W += (size_t)e * p.sel.expert_rows * p.row_bytes;
        p.x += (size_t)(p.sel.x_per_pair ? pair : ti) * p.cols;
        p.y += (size_t)pair * p.sel.y_stride;
    }
}

// Input norm fused into a batch-1 mat-vec: the activation row is rmsnorm(x [+ resid]) * norm_w; x + resid goes to x_out
// (optional, must not be x).
struct NormParams {
    const float* norm_w;
    const float* resid;
    float* x_out;
    float eps;
};
constexpr int NORM_NOT_FUSED = -100;   // internal: launch_gemv_norm launched nothing, run the two steps apart

int set_error(int code, const char* fmt, ...);
int check_hip(hipError_t e, const char* what);
int device_cus();
size_t device_lds_bytes();  // LDS one workgroup may use

// dequant.hip
int launch_f16_to_f32(const uint16_t* d_bits, size_t n, float* d_out, hipStream_t s);
int launch_bf16_to_f32(const uint16_t* d_bits, size_t n, float* d_out, hipStream_t s);
int launch_dequant(uint32_t type, const uint8_t* d_raw, size_t nblocks, float* d_out, hipStream_t s);

// gemv.hip
// y[rows_x, out_rows] = x * W^T; when n_ff > 0 the weight stacks gate|up (2*n_ff rows) and
// y[rows_x, n_ff] = silu(gate.x) * (up.x).
int launch_gemv(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, size_t n_ff, hipStream_t s);
// gemv.hip is built once per activation precision (two or three byte planes per run: a 16- or 24-bit significand at the run
// maximum); launch_gemv, launch_gemv_norm, launch_gemv_sel and gemv_force_generic (api.hip) forward to the copy the weight's
// `planes` names.
#define FHIP_GEMV_COPY(sfx)                                                                                                         \
    int launch_gemv##sfx(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, size_t n_ff, hipStream_t s);            \
    int launch_gemv_norm##sfx(const fhip_weight* w, const float* d_x, float* d_y, size_t n_ff, const struct NormParams& norm,        \
                              hipStream_t s);                                                                                       \
    int launch_gemv_sel##sfx(const fhip_weight* w, const float* d_x, float* d_y, size_t out_rows, bool swiglu,                      \
                             const struct SelParams& sel, hipStream_t s);                                                           \
    void gemv_force_generic##sfx(bool on);                                                                                         \
    bool gemv_streams##sfx(const fhip_weight* w, size_t n_ff);                                                                      \
    bool gemv_quad_supports##sfx(const fhip_weight* w, size_t rows_x, size_t n_ff);                                                 \
    int launch_gemv_quad##sfx(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, size_t n_ff, hipStream_t s);
FHIP_GEMV_COPY(_p2)
FHIP_GEMV_COPY(_p3)
#undef FHIP_GEMV_COPY
// gemv_generic.hip: same contract, any cols the format allows (up to 32768)
int launch_gemv_generic(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, size_t n_ff, hipStream_t s);
int launch_swiglu(const float* d_gu, size_t t, size_t d, float* d_out, hipStream_t s);
void gemv_force_generic(bool on);   // debugging / tests: every mat-vec through gemv_generic.hip
bool gemv_quad_matvec(bool on);     // debugging / tests: off keeps batches of three and more off gemv_quad.hip; returns the setting before
// One batch-1 GEMV per (token, slot) pair on the selected expert's `out_rows` rows (fused SwiGLU over its
// gate|up halves when swiglu: then expert_rows = 2 * out_rows). Both files provide it, same contract as above.
int launch_gemv_norm(const fhip_weight* w, const float* d_x, float* d_y, size_t n_ff, const NormParams& norm, hipStream_t s);
int launch_gemv_sel(const fhip_weight* w, const float* d_x, float* d_y, size_t out_rows, bool swiglu, const SelParams& sel,
                    hipStream_t s);
int launch_gemv_generic_sel(const fhip_weight* w, const float* d_x, float* d_y, size_t out_rows, bool swiglu,
                            const SelParams& sel, hipStream_t s);

// probe.hip: reads nbytes (a multiple of 16 is read) and stores nothing to speak of
int launch_read_probe(const void* d_src, size_t nbytes, uint32_t* d_sink, hipStream_t s);
int launch_mfma_probe(int iters, float* d_sink, hipStream_t s, double* flops);

// moe.hip
int launch_moe_topk(const float* d_logits, const float* d_bias, size_t t, size_t ne, int k, int sigmoid, float scale, int norm,
                    float* d_out, hipStream_t s);
int launch_moe_wsum(const float* d_parts, const float* d_selw, size_t t, int k, size_t out_pe, float* d_y, hipStream_t s);

// gemm_mfma.hip
// d_ws / ws_bytes: gemm_bf16_ws_bytes(w, t) bytes of scratch for launches that cut output tiles along K (0: none needed)
int launch_gemm_bf16(const fhip_weight* w, const uint16_t* d_x, size_t t, float* d_y, hipStream_t s, float* d_ws = nullptr, size_t ws_bytes = 0);
size_t gemm_bf16_ws_bytes(const fhip_weight* w, size_t t);
int gemm_bf16_force_tile(int tile);   // debugging / tests: 0..3 pins the tile of launches of more than 32 rows, -1 frees it; returns the old value
// conversions in front of the GEMM
int launch_cvt_bf16(const float* d_x, size_t n, uint16_t* d_out, hipStream_t s);
int launch_swiglu_bf16(const float* d_gu, size_t t, size_t d, uint16_t* d_out, hipStream_t s);

// gemm_f16x2.hip: 2..32 activation rows in one pass over the weights, f16 matrix cores, f32-grade results
bool gemm_f16x2_supports(const fhip_weight* w, size_t t);
size_t gemm_f16x2_xp_bytes(const fhip_weight* w, size_t t);       // prepared-activation buffer for t rows
bool gemm_f16x2_adds_into_y(const fhip_weight* w, size_t t);      // true: the launch adds into y, a cleared y saves it a launch
// splits the rows of x [t, cols] (swiglu: of silu(gate) * up of x [t, 2 cols]) chunk by chunk into scaled f16 hi / lo
// operand rows, each carrying the factor that takes its scale out again
// Where the K-split groups of a matmul's output still lie as partial sums, one slot per (128-output group, contributor):
// output n of activation row t is slot 0 + slot 1 + ... of its group in that order (one contributor: the value in y itself).
struct F16Parts {
    const float* part;    // null: every output is in y
    int kmax, nchunks, grid;
    long long units;
    int group;            // outputs of a group: 128, or 256 where the eight-wave row-streaming kernel made the sums
};
// src: x is the output of a matmul whose ordered sum was left to this launch (launch_gemm_f16x2 with `deferred`)
int launch_xsplit_f16(const fhip_weight* w, const float* d_x, size_t t, bool swiglu, uint16_t* d_xp, hipStream_t s, float* zero = nullptr,
                      size_t zero_n = 0, const F16Parts* src = nullptr);
// d_part: null, or gemm_f16x2_part_bytes(w, t) bytes: partial sums of K-split groups go there and are added in a fixed
// order by a launch behind the matmul (y then needs no clearing) instead of being added into y atomically
// deferred: with d_part, the launch that adds the partial sums is left out and *deferred says where they lie; the reader of y
// (launch_xsplit_f16 with `src`) adds them in the same order
int launch_gemm_f16x2(const fhip_weight* w, const uint16_t* d_xp, size_t t, float* d_y, hipStream_t s, bool y_cleared = false,
                      float* d_part = nullptr, F16Parts* deferred = nullptr);
size_t gemm_f16x2_part_bytes(const fhip_weight* w, size_t t);
size_t gemm_f16x2_part_bytes_upto(const fhip_weight* w, size_t t);   // the largest over batches of 1..t rows

// decode_ops.hip: the steps either side of the matmuls in a decode layer
int launch_rmsnorm(const float* a, const float* b, const float* weight, size_t rows, size_t d, float eps, float* sum_out, float* norm_out,
                   hipStream_t s);
int launch_add(const float* a, const float* b, size_t n, float* out, hipStream_t s);
int launch_u32_add(uint32_t* w, size_t n, uint32_t delta, hipStream_t s);
// block-quantized K / V cache (kvquant.hip); scales addressed as uint16 [block] (Q4_1: [block][2])
int launch_kvq_append(int fmt, const float* src, size_t src_row_stride, size_t t, size_t width, const uint32_t* d_pos, uint32_t pos_off,
                      bool src_at_pos, size_t cap, uint32_t* codes, uint16_t* scales, hipStream_t s, const float* src2 = nullptr,
                      uint32_t* codes2 = nullptr, uint16_t* scales2 = nullptr);
int launch_decode_attention_kvq(int fmt, const float* q, const uint32_t* k_codes, const uint16_t* k_scales, const uint32_t* v_codes,
                                const uint16_t* v_scales, int n_head, int n_kv, int hd, size_t len, const uint32_t* d_len, size_t window,
                                float softcap, float* ws, float* out, hipStream_t s);
int launch_kvq_dequantize(int fmt, const uint32_t* codes, const uint16_t* scales, size_t row0, size_t rows, size_t width, const uint32_t* d_last_pos,
                          float* out, hipStream_t s);
int launch_causal_attention(const float* q, const float* K, const float* V, size_t t, size_t s, int n_head, int n_kv, int hd, size_t window,
                            float softcap, float* out, hipStream_t st);
int launch_mul_sigmoid(const float* a, const float* g, size_t n, float* out, hipStream_t s);   // out = a * sigmoid(g); out may be a
int launch_geglu(const float* gu, size_t t, size_t d, float* out, hipStream_t s);              // rows [gate | up] -> gelu_tanh(gate) * up
int launch_rope(const float* x, size_t src_row_stride, size_t t, int heads, int hd, int n_rot, float base, const uint32_t* d_pos, uint32_t pos_off,
                const float* freq_scale, int interleaved, float* out, hipStream_t s);
int launch_qkv_post(const float* qkv, const float* bias, const float* q_norm, const float* k_norm, const uint32_t* d_pos, const float* freq_scale,
                    size_t t, int n_head, int n_kv, int hd, int n_rot, int interleaved, float eps, float base, float* q_out, float* k_cache,
                    float* v_cache, size_t cap, hipStream_t s, bool kv_packed = false);   // kv_packed: K / V rows to packed [t, n_kv * hd] outputs
int launch_kv_append(const float* k, const float* v, size_t t, size_t width, const uint32_t* d_pos, uint32_t pos_off, size_t cap, float* kc,
                     float* vc, hipStream_t s);
int attn_splits(size_t len, int n_kv);
int attn_ws_splits(size_t len, int n_head, int n_kv);
int launch_qkv_post_attention(const float* qkv, const float* bias, const float* q_norm, const float* k_norm, const uint32_t* d_pos,
                              const float* freq_scale, int n_head, int n_kv, int hd, int n_rot, bool interleaved, float eps, float base,
                              float* k_cache, float* v_cache, size_t cap, size_t len, size_t window, float softcap, float* ws, float* out,
                              hipStream_t s);
int launch_decode_attention(const float* q, const float* K, const float* V, int n_head, int n_kv, int hd, size_t len, const uint32_t* d_len,
                            size_t window, float softcap, float* ws, float* out, hipStream_t s);

}  // namespace fhip
