/*
 * ferric_hip.h -- C ABI of the MI355X (gfx950) quantized-GGUF matmul path.
 *
 * One shared library, libferric_hip.so, exports exactly these symbols. They are the functions a
 * `ferric-hip` backend crate binds (extern "C") to stand in for the reference's quantized-linear
 * entry points; each declaration cites the reference interface it replaces (paths are relative to
 * the reference checkout).
 *
 * Conventions
 *   - Weights are [rows = out, cols = in], row-major, as the RAW GGUF block byte stream
 *     (Q8_0 34 B / 32 values, Q4_K 144 B / 256, Q6_K 210 B / 256). No repack is needed or done.
 *   - Activations x are f32 [rows_x, cols] contiguous, outputs y are f32 [rows_x, rows] contiguous,
 *     both in device memory owned by the caller.
 *   - Every compute call only enqueues work on `stream` (a hipStream_t passed as void*, NULL = the
 *     default stream) and returns; there is no hidden synchronisation or allocation in them.
 *   - Return value: FHIP_OK (0) or a negative FHIP_ERR_* code; the text is available from
 *     fhip_last_error() (thread-local). Nothing in this library aborts the process: shape
 *     violations that the reference turns into `assert!` panics come back as FHIP_ERR_SHAPE so the
 *     binding can re-raise them on its own side.
 *   - Handles are immutable after creation and may be shared read-only between threads; one host
 *     thread drives one stream.
 */
#ifndef FERRIC_HIP_H
#define FERRIC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids of the supported formats (crates/ferric-gguf/src/lib.rs:471-494). */
#define FHIP_Q8_0 8u
#define FHIP_Q4_K 12u
#define FHIP_Q6_K 14u
/* further block formats of the same reader (crates/ferric-gguf/src/lib.rs:618-716, 748-791, 843-908): unpackers, mat-vec / small batch and
 * the "_id" variants; the matrix-core entry points take the three formats above only */
#define FHIP_Q4_0 2u
#define FHIP_Q4_1 3u
#define FHIP_Q5_0 6u
#define FHIP_Q5_1 7u
#define FHIP_Q5_K 13u
#define FHIP_IQ4_NL 20u
#define FHIP_IQ4_XS 23u
#define FHIP_MXFP4 39u
/* unquantized tensor types (crates/ferric-gguf/src/lib.rs:473-475, 499-501): sizes and deq_raw only; a weight handle
 * takes block formats only (crates/ferric-tensor/src/dtype.rs:853-855 sends these to the dense matmul) */
#define FHIP_F32 0u
#define FHIP_F16 1u
#define FHIP_BF16 30u

#define FHIP_OK 0
#define FHIP_ERR_UNSUPPORTED_TYPE (-1) /* reference: Err("unsupported ggml type N") / Err("QMatrix: no native matmul ...") */
#define FHIP_ERR_SHAPE (-2)            /* reference: assert!/assert_eq! panic on cols % block, byte length, inner dim */
#define FHIP_ERR_HIP (-3)              /* a HIP runtime call failed */
#define FHIP_ERR_ARG (-4)              /* NULL pointer or otherwise unusable argument */
#define FHIP_ERR_FORMAT (-5)           /* reference: Err(String) from the GGUF reader (not GGUF, truncated, stride refusal, no such tensor) */

typedef struct fhip_weight fhip_weight; /* opaque: one packed weight resident in HBM */

/* ---- library / device ---------------------------------------------------------------------- */

/* Select the device and probe it. Stands where the reference creates its device context
 * (crates/ferric-core/src/lib.rs:109 Context::new). Must be called once before anything else. */
int fhip_init(int device);

/* Thread-local text of the last error returned on this thread ("" if none). */
const char* fhip_last_error(void);

/* Number of compute units of the initialised device (0 before fhip_init). */
int fhip_device_cus(void);

/* ---- sizes --------------------------------------------------------------------------------- */

/* crates/ferric-gguf/src/lib.rs:471 type_size(ty, n): bytes of n elements; 0 = unsupported type
 * (the reference returns Err). Integer division truncates as in the reference (n/32*34 ...). */
size_t fhip_type_size(uint32_t ggml_type, size_t n);

/* crates/ferric-tensor/src/dtype.rs:873 QMatrix::block_bytes: (values, bytes) of one block.
 * Returns FHIP_OK or FHIP_ERR_UNSUPPORTED_TYPE (reference: None). */
int fhip_block_bytes(uint32_t ggml_type, size_t* values, size_t* bytes);

/* ---- device memory, streams, events (plumbing the binding needs to own tensors) ------------- */
/* These stand where the reference's Tensor creates/reads wgpu buffers
 * (crates/ferric-tensor/src/lib.rs:1481 empty(), :141 to_vec(), :1816 readback). */
int fhip_malloc(void** d_ptr, size_t nbytes);
int fhip_free(void* d_ptr);
int fhip_memcpy_h2d(void* d_dst, const void* h_src, size_t nbytes, void* stream); /* async on stream */
int fhip_memcpy_d2h(void* h_dst, const void* d_src, size_t nbytes, void* stream); /* synchronises stream before returning */
int fhip_memcpy_d2d(void* d_dst, const void* d_src, size_t nbytes, void* stream);
/* `height` rows of `width` bytes between two pitched device arrays, async on stream (what Tensor::cat along the last
 * dim of a matrix comes to, crates/ferric-tensor/src/lib.rs:201-221: each side is copied into its columns of the result) */
int fhip_memcpy_2d_d2d(void* d_dst, size_t dpitch, const void* d_src, size_t spitch, size_t width, size_t height, void* stream);
int fhip_memset(void* d_dst, int byte, size_t nbytes, void* stream);
int fhip_stream_create(void** stream);
int fhip_stream_destroy(void* stream);
int fhip_stream_sync(void* stream);
int fhip_event_create(void** event);
int fhip_event_destroy(void* event);
int fhip_event_record(void* event, void* stream);
int fhip_event_sync(void* event);
int fhip_event_elapsed_ms(void* start, void* stop, float* ms);

/* Record-then-replay of a sequence of calls on one stream, standing for the reference's
 * batch(ctx, ..) recorder that encodes every dispatch of a decode step into one submission
 * (crates/ferric-tensor/src/lib.rs:1802). Between begin and end, compute calls on `stream` (which
 * must come from fhip_stream_create) are captured into a HIP graph instead of executed; the
 * returned executable graph replays them with one launch. Buffers used by the captured calls must
 * stay alive and in place while the graph exists. */
int fhip_graph_capture_begin(void* stream);
int fhip_graph_capture_end(void* stream, void** graph_exec);
int fhip_graph_launch(void* graph_exec, void* stream);
int fhip_graph_destroy(void* graph_exec);

/* ---- packed weights ------------------------------------------------------------------------ */

/* crates/ferric-tensor/src/dtype.rs:893 QMatrix::from_bytes(ctx, bytes, ggml_type, rows, cols) and the
 * per-format constructors Q8_0Weights/Q4_KWeights/Q6_KWeights::from_bytes (dtype.rs:1270/1388/1147).
 * Copies `nbytes` host bytes into HBM (the caller keeps nothing alive). The device layout IS the
 * GGUF byte stream; one allocation holds any size, so there is no row-sharding.
 * Errors: unsupported type -> FHIP_ERR_UNSUPPORTED_TYPE; cols % block_values != 0 or
 * nbytes != rows*(cols/block_values)*block_bytes -> FHIP_ERR_SHAPE. */
int fhip_weight_create(uint32_t ggml_type, const uint8_t* h_raw, size_t nbytes, size_t rows, size_t cols,
                       fhip_weight** out);

/* The same from several host buffers laid end to end (the byte stacking of crates/ferric-llama/src/qwen35.rs:393-395
 * and of Proj::load, crates/ferric-llama/src/qwen3.rs:197-213, without the host-side Vec): part i is uploaded behind
 * part i - 1; the parts' sizes must add up to rows * row_bytes. */
int fhip_weight_create_parts(uint32_t ggml_type, const uint8_t* const* h_parts, const size_t* part_bytes, size_t n_parts,
                             size_t rows, size_t cols, fhip_weight** out);

/* Same, but adopts block bytes that are already in device memory (no copy; the caller keeps the
 * buffer alive until fhip_weight_destroy). Used when a loader streams a file straight into HBM. d_raw: 16-byte aligned, and
 * the allocation it lies in must extend 256 bytes past the weight's last block (readable, content irrelevant), as the library's
 * own weights do: buffers from fhip_malloc always qualify; anything else is checked and refused with FHIP_ERR_ARG. */
int fhip_weight_wrap_device(uint32_t ggml_type, const uint8_t* d_raw, size_t nbytes, size_t rows, size_t cols,
                            fhip_weight** out);

void fhip_weight_destroy(fhip_weight* w);

/* dtype.rs:927-930 QMatrix::{rows, cols, nbytes}; ggml type of the handle. */
size_t fhip_weight_rows(const fhip_weight* w);
size_t fhip_weight_cols(const fhip_weight* w);
size_t fhip_weight_nbytes(const fhip_weight* w);
uint32_t fhip_weight_type(const fhip_weight* w);

/* ---- unpackers (bit-exact with the reference CPU dequantizers) ------------------------------- */

/* crates/ferric-gguf/src/lib.rs:605 rd_f16 / crates/ferric-tensor/src/cpu_simd.rs:29 f16:
 * n IEEE binary16 patterns (device) -> f32 (device), exact incl. subnormal / inf / nan. */
int fhip_f16_to_f32(const uint16_t* d_bits, size_t n, float* d_out, void* stream);

/* crates/ferric-gguf/src/lib.rs:608 deq_q8_0, :793 deq_q4_k, :721 deq_q6_k applied to rows
 * [row0, row0+nrows) of a resident weight: d_out receives nrows*cols f32, row-major.
 * (The callers dequantize embedding rows this way: crates/ferric-llama/src/qwen3.rs:749.) */
int fhip_dequant_rows(const fhip_weight* w, size_t row0, size_t nrows, float* d_out, void* stream);

/* crates/ferric-gguf/src/lib.rs:497 deq_raw(raw, n, ty) with host buffers on both sides: uploads,
 * dequantizes on the GPU, downloads, synchronises. h_out must hold n f32. *n_written receives what
 * the reference's Vec would hold: n for the K-quants (a ragged tail stays 0.0), whole blocks only
 * for Q8_0. Only min(n / block_values, nbytes / block_bytes) whole blocks are read. The unquantized types
 * (FHIP_F32 / FHIP_F16 / FHIP_BF16, lib.rs:499-501) give exactly n values and need n elements' bytes: fewer is
 * FHIP_ERR_SHAPE (the reference's slice panics). F32 is a byte copy on the host; the other two convert on the GPU. */
int fhip_deq_raw(const uint8_t* h_raw, size_t nbytes, size_t n, uint32_t ggml_type, float* h_out, size_t* n_written);

/* ---- matmuls ------------------------------------------------------------------------------- */

/* crates/ferric-tensor/src/dtype.rs:935 Tensor::matmul_q (and :1292 matmul_q8_0, :1426 matmul_q4_k,
 * :1172 matmul_q6_k): y[rows_x, rows] = x[rows_x, cols] * W^T, f32 in, f32 accumulate, f32 out.
 * rows_x = 1 is the decode GEMV; any rows_x >= 1 is accepted.
 * Which kernel a batch takes (fhip_batch_policy): one or two rows go through the streaming mat-vec; three and four rows of a
 * Q4_K / Q5_K / Q6_K weight with rows of up to 10240 columns (Q8_0: 5120) through its four-row form (the same arithmetic on the int8 matrix
 * instruction: every row has the bits it has in a batch of one; one launch, no workspace); otherwise, from three rows on (five
 * for Q8_0) Q4_K / Q5_K / Q6_K / Q8_0 weights are read once per group of up to 32 (Q8_0: 16) rows by the f16 hi/lo matrix-core
 * kernels (see fhip_matmul_q_f16x2: f32-grade, 22-bit activations), longer batches group by group. That path keeps its
 * prepared activations in a workspace the library owns per stream (fhip_workspace_reserve); inside a graph capture the
 * workspace cannot grow, and the call then fails with FHIP_ERR_ARG and says how many bytes to reserve beforehand.
 * Non-finite activations: on the mat-vec kernel a NaN or infinite x gives what the f32 dot gives (NaN, +-inf by the weight's
 * sign); on the matrix-core kernels the whole output row of such an activation row is non-finite and no other row is touched. */
int fhip_matmul_q(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, void* stream);

/* crates/ferric-tensor/src/dtype.rs:949 try_matmul_swiglu / :1551 matmul_q4_k_swiglu / :1802
 * matmul_q6_k_swiglu: `gate_up` stacks gate rows [0, n_ff) then up rows [n_ff, 2 n_ff);
 * y[rows_x, n_ff] = silu(x*gate^T) * (x*up^T), silu(g) = g / (1 + exp(-g)).
 * Errors: odd row count -> FHIP_ERR_SHAPE; Q8_0 -> FHIP_ERR_UNSUPPORTED_TYPE (reference: None,
 * the caller then runs matmul_q + swiglu). Batches of three and four rows (Q4_K, Q5_K, Q6_K, rows of up to 10240 columns): one pass
 * of the mat-vec's arithmetic for four rows at a time (the int8 matrix instruction; every row has the bits it has in a batch of one, no
 * workspace). Other batches of three rows and more: as fhip_matmul_q, then the un-fused SwiGLU of
 * crates/ferric-tensor/src/lib.rs:2603-2618 over the [rows, 2 n_ff] intermediate in the library's workspace. */
int fhip_matmul_q_swiglu(const fhip_weight* gate_up, const float* d_x, size_t rows_x, float* d_y, void* stream);

/* crates/ferric-tensor/src/lib.rs:728 Tensor::swiglu(d): gu is [t, 2d] = [gate | up] per row,
 * out[t, d] = silu(gate) * up. */
int fhip_swiglu(const float* d_gu, size_t t, size_t d, float* d_out, void* stream);

/* The FFN block of crates/ferric-llama/src/qwen3.rs:944-964: y = down( swiglu( gate_up(x) ) ).
 * d_ws is caller-provided scratch of at least rows_x * n_ff f32 (n_ff = gate_up rows / 2). Batches of three rows and more
 * run as fhip_ffn_f16x2 does (one pass over each weight per group of up to 32 rows) out of the library's workspace; in a
 * group of three or four rows gate|up + SwiGLU is the call fhip_matmul_q_swiglu makes for such a batch, and the block gives
 * the bits of that call followed by fhip_matmul_q on the down projection. */
int fhip_ffn(const fhip_weight* gate_up, const fhip_weight* down, const float* d_x, size_t rows_x, float* d_y,
             float* d_ws, void* stream);

/* Prefill dequant-GEMM, stands for crates/ferric-tensor/src/dtype.rs:1818 matmul_q4_k_coop (:1199
 * Q6_K, :1316 Q8_0): x is bf16 [t, cols] (raw 16-bit patterns), y f32 [t, rows]; weights are
 * dequantized tile by tile into LDS as bf16 and contracted on the matrix cores, f32 accumulate. A launch that cuts
 * output tiles along K keeps their partial tiles in the library's workspace of the stream (fhip_workspace_bytes_coop)
 * and adds them in a fixed order: the same inputs give the same bits on every run. */
int fhip_gemm_q_bf16(const fhip_weight* w, const uint16_t* d_x_bf16, size_t t, float* d_y, void* stream);

/* ---- mixture-of-experts decode: the "_id" variants that sit behind the same matmul entry points ---------- */

/* crates/ferric-tensor/src/dtype.rs:1582 Tensor::moe_topk / :1596 moe_topk_ex (kernel :2415-2461). logits
 * [t, n_expert] f32, bias n_expert f32 or NULL; out [t, 2k] = [w_0..w_{k-1} | idx_0..idx_{k-1}], indices as f32.
 * Scores: softmax over all experts, or sigmoid; selection by score + bias, ties to the lowest index; weights =
 * selected scores (without bias), / their sum when norm, * scale. k not in 1..=8 or n_expert > 1024 ->
 * FHIP_ERR_SHAPE (the reference's asserts, dtype.rs:1599-1600). */
int fhip_moe_topk(const float* d_logits, const float* d_bias, size_t t, size_t n_expert, size_t k, int sigmoid, float scale, int norm,
                  float* d_out, void* stream);

/* dtype.rs:1620 matmul_q4_k_swiglu_id / :1731 matmul_q8_0_swiglu_id (kernels :2463, :2618): x [t, cols], w packs all
 * experts' fused gate|up rows expert-major (rows = n_expert * 2 * eff: gate rows, then up rows, per expert), selw the
 * [t, 2k] moe_topk output; y [t, k, eff] = silu(gate_e . x_t) * (up_e . x_t) for every (token, selected expert).
 * Any of the three formats. An index outside the slab is clamped into it. */
int fhip_matmul_q_swiglu_id(const fhip_weight* w, const float* d_x, size_t t, const float* d_selw, size_t k, size_t eff, float* d_y,
                            void* stream);

/* dtype.rs:1703-1729 matmul_q5_0_relu2_id (kernel :3714-3758): the selected-expert UP projection of a squared-ReLU expert
 * MLP (no gate slab). x [t, cols], w packs all experts' up rows expert-major (rows = n_expert * eff), selw the [t, 2k]
 * moe_topk output; y [t, k, eff] = max(up_e . x_t, 0)^2 for every (token, selected expert), the activation applied as the
 * dot product leaves the kernel. The reference has it for Q5_0; any format with a native mat-vec is taken. */
int fhip_matmul_q_relu2_id(const fhip_weight* w, const float* d_x, size_t t, const float* d_selw, size_t k, size_t eff, float* d_y,
                           void* stream);

/* dtype.rs:1640 matmul_q6_k_id (kernel :2509): x [k, cols] (row s = slot s's SwiGLU output), w packs all experts' down
 * rows expert-major (rows = n_expert * out_pe), selw one moe_topk row [2k]; y [k, out_pe]. Any of the three formats. */
int fhip_matmul_q_id(const fhip_weight* w, const float* d_x, const float* d_selw, size_t k, size_t out_pe, float* d_y, void* stream);

/* dtype.rs:1662 matmul_q6_k_id_wsum / :1765 matmul_q4_k_id_wsum / :1748 matmul_q8_0_id_wsum (kernels :2538, :2571,
 * :2654): x [t, k, cols]; y [t, out_pe], row t = sum_s w_{t,s} * down_{e_{t,s}}(x_{t,s}), slots added in order.
 * d_ws: caller-provided scratch of t * k * out_pe f32 (the per-slot projections before the weighted sum). */
int fhip_matmul_q_id_wsum(const fhip_weight* w, const float* d_x, size_t t, const float* d_selw, size_t k, size_t out_pe, float* d_y,
                          float* d_ws, void* stream);

/* ---- the steps either side of the matmuls in one decode layer (crates/ferric-llama/src/qwen3.rs:861-942 `attn`,
 * :979-1052 `apply_layer`). f32 throughout; every pointer is device memory; all enqueue on `stream` and return. ---- */

/* crates/ferric-tensor/src/lib.rs:346 Tensor::rmsnorm (kernel :2018): out[r, j] = x[r, j] / sqrt(mean_j x[r, :]^2 + eps)
 * * weight[j], rows x d. The sum of squares is a fixed-shape tree over the row instead of the reference's one-thread
 * serial loop: same value to rounding, not the same bits. */
int fhip_rmsnorm(const float* d_x, const float* d_weight, size_t rows, size_t d, float eps, float* d_out, void* stream);

/* lib.rs:372 Tensor::add_rmsnorm (kernel :2057): sum = a + b (bit-exact), norm = rmsnorm(sum, weight). d_sum may be d_a
 * (the residual updated in place). */
int fhip_add_rmsnorm(const float* d_a, const float* d_b, const float* d_weight, size_t rows, size_t d, float eps, float* d_sum,
                     float* d_norm, void* stream);

/* lib.rs:279 Tensor::add, same shapes: out = a + b, n elements. */
int fhip_add(const float* d_a, const float* d_b, size_t n, float* d_out, void* stream);
/* out = a * sigmoid(g), n values; d_out may be d_a. The gate of a gated-attention layer on the attention output,
 * crates/ferric-llama/src/qwen3.rs:936-938 (`o.mul(&h.matmul_q(wg).sigmoid())`), sigmoid as lib.rs:299 / :1915. */
int fhip_mul_sigmoid(const float* d_a, const float* d_g, size_t n, float* d_out, void* stream);
/* out [t, d] = gelu_tanh(gate) * up for rows gu [t, 2 d] = [gate | up]: Gemma's GEGLU, qwen3.rs:953-958, with the
 * tanh-approximated GELU of lib.rs:304 / :1926. The unfused counterpart of fhip_swiglu for that activation. */
int fhip_geglu(const float* d_gu, size_t t, size_t d, float* d_out, void* stream);

/* lib.rs:417 Tensor::rope / :409 rope_interleaved / :429 rope_partial / :465 rope_at / :489 rope_at_ex (kernels :2118,
 * :2094). x: t rows of n_heads * head_dim, row i at d_x + i * src_row_stride (a strided window such as a slice of the
 * fused qkv row is read in place; 0 = packed rows); out packed [t, n_heads * head_dim]. Row i sits at position
 * d_positions[i] (device u32) or, when that is NULL, pos_off + i. Pair c rotates by position * base^(-2c / n_rot)
 * [* d_freq_scale[c]]; partners are (c, c + n_rot/2), or (2c, 2c + 1) when interleaved; dims >= n_rot are copied.
 * n_rot odd or > head_dim -> FHIP_ERR_SHAPE (the reference's assert, lib.rs:437). */
int fhip_rope(const float* d_x, size_t src_row_stride, size_t t, size_t n_heads, size_t head_dim, size_t n_rot, float base,
              const uint32_t* d_positions, uint32_t pos_off, const float* d_freq_scale, int interleaved, float* d_out, void* stream);

/* lib.rs:1379 append2: rows of k and v [t, width] into the two caches [cap, width] at rows d_positions[i] (or pos_off +
 * i), one launch. The caches are caller-owned, fixed-capacity buffers (the reference's KvBuf grows by reallocating, which
 * a captured step cannot do); a row at or past cap is dropped. */
int fhip_kv_append2(const float* d_k, const float* d_v, size_t t, size_t width, const uint32_t* d_positions, uint32_t pos_off,
                    float* d_k_cache, float* d_v_cache, size_t cap, void* stream);

/* qwen3.rs:861-905 in one launch, for t tokens' fused qkv rows [t, (n_head + 2 n_kv) * head_dim]: + d_bias (optional,
 * :848), per-head RMSNorm of the query and key heads with d_q_norm / d_k_norm [head_dim] (optional, :851-855), rotary
 * embedding of both at d_positions[i] (as fhip_rope), query heads to d_q_out [t, n_head * head_dim], key and value heads
 * to row d_positions[i] of the caches [cap, n_kv * head_dim]. No single counterpart in the reference: it issues these as
 * 4-5 dispatches. */
int fhip_qkv_post(const float* d_qkv, const float* d_bias, const float* d_q_norm, const float* d_k_norm, const uint32_t* d_positions,
                  const float* d_freq_scale, size_t t, size_t n_head, size_t n_kv, size_t head_dim, size_t n_rot, int interleaved,
                  float eps, float base, float* d_q_out, float* d_k_cache, float* d_v_cache, size_t cap, void* stream);

/* Block-quantized K / V cache, crates/ferric-tensor/src/kvquant.rs (KvqFmt :57-64): rows of `width` values (a multiple of
 * 32, else FHIP_ERR_SHAPE with the reference's message, :470) stored as llama.cpp-layout blocks of 32 along the row, block
 * b = row * (width / 32) + col / 32. d_codes: 8 (Q8_0) or 4 (Q4_0, Q4_1) u32 words per block; d_scales: f16 bit patterns,
 * two blocks per u32 word for Q8_0 / Q4_0 (block b in half b % 2 of word b / 2), one word d | min << 16 per block for Q4_1:
 * the reference's `codes` / `scales` buffers byte for byte, and its arithmetic operation for operation (`mod reference`,
 * :943-1186: d = amax / 127 with roundf; d = extreme / -8 with floor(x + 8.5); d = (max - min) / 15 with floor(x + 0.5)), so
 * codes, scales and dequantized values are bit-identical to the reference's. */
#define FHIP_KVQ_Q8_0 0
#define FHIP_KVQ_Q4_0 1
#define FHIP_KVQ_Q4_1 2
/* KvqFmt::code_words / scale_words (:66-81) for rows x width: u32 words of each array. */
int fhip_kvq_sizes(int fmt, size_t rows, size_t width, size_t* code_words, size_t* scale_words);
/* QKvCache::append (:464-517) without the growth (the caller owns arrays of `cap` rows): quantizes exactly the t rows handed
 * over and writes their blocks at their flat offsets; nothing already stored is touched or read. Source row i is at
 * d_src + i * src_row_stride (0 = packed; a window of a fused qkv row is read in place) and goes to cache row
 * d_positions[i] (device u32) or pos_off + i. src_at_pos != 0: the source row index is the cache row too (the newest row of
 * an f32 staging cache of full length), for a captured decode step whose position lives in a device word. */
int fhip_kvq_append(int fmt, const float* d_src, size_t src_row_stride, size_t t, size_t width, const uint32_t* d_positions, uint32_t pos_off,
                    int src_at_pos, size_t cap, uint32_t* d_codes, uint32_t* d_scales, void* stream);
/* QKvCache::dequantize_rows (:621-650; dequantize :617 is row0 = 0, rows = len): cache rows row0 .. row0 + rows to f32
 * d_out [rows, width]. d_last_pos (optional, device u32): rows past *d_last_pos are not written, so a captured step can pass
 * the capacity as `rows` and the position word of the token being decoded. The arrays carry no length: row0 + rows (and, with
 * d_last_pos, *d_last_pos + 1) must not exceed the `rows` the caller sized them for with fhip_kvq_sizes -- an unchecked
 * precondition, as for every other device pointer of this header. */
int fhip_kvq_dequantize_rows(int fmt, const uint32_t* d_codes, const uint32_t* d_scales, size_t row0, size_t rows, size_t width,
                             const uint32_t* d_last_pos, float* d_out, void* stream);

/* K and V rows of the same tokens into their two caches in one launch (the quantized twin of fhip_kv_append2; the
 * reference appends them apart, crates/ferric-llama/src/qwen3.rs:909-910). Both sources share the row stride. */
int fhip_kvq_append2(int fmt, const float* d_k, const float* d_v, size_t src_row_stride, size_t t, size_t width, const uint32_t* d_positions,
                     uint32_t pos_off, size_t cap, uint32_t* d_k_codes, uint32_t* d_k_scales, uint32_t* d_v_codes, uint32_t* d_v_scales,
                     void* stream);
/* fhip_decode_attention_ex over a block-quantized cache read in place: each key / value row is dequantized in registers as it
 * is loaded (the use the reference chose the block layout for and left unbuilt, kvquant.rs:30-37, qwen3.rs:897-905: it
 * materialises `dequantize()` of the whole history per layer and step and attends over that). The values that enter the
 * softmax are exactly fhip_kvq_dequantize_rows', so the result has the bits of fhip_decode_attention_ex over the dequantized
 * rows, at 8.5 / 4.5 / 5 bits per value of traffic instead of 32 + 32 written and read back. */
int fhip_decode_attention_kvq(int fmt, const float* d_q, const uint32_t* d_k_codes, const uint32_t* d_k_scales, const uint32_t* d_v_codes,
                              const uint32_t* d_v_scales, size_t n_head, size_t n_kv, size_t head_dim, size_t len, const uint32_t* d_last_pos,
                              size_t window, float softcap, float* d_ws, float* d_out, void* stream);

/* Causal attention of t query rows q [t, n_head * head_dim] against the first s >= t rows of K and V [., n_kv * head_dim]:
 * query i sits at absolute position (s - t) + i and attends to keys 0 ..= (s - t) + i, or only to the newest `window` of them
 * when window > 0; softcap > 0 replaces each scaled score x by softcap * tanh(x / softcap). One entry point for
 * crates/ferric-tensor/src/nn.rs:40 causal_attention (s == t), :66 causal_attention_win, :239 chunked_attention (prefix-cached
 * and chunked prefill) and the flash prefill kernel crates/ferric-llama/src/qwen3.rs:925 picks when it can -- "all three are
 * the same math". s < t -> FHIP_ERR_SHAPE with the reference's message (nn.rs:73). head_dim 64 or 128; f32 throughout (f32
 * matrix instructions), out [t, n_head * head_dim]; pointers 16-byte aligned. */
int fhip_causal_attention(const float* d_q, const float* d_k, const float* d_v, size_t t, size_t s, size_t n_head, size_t n_kv, size_t head_dim,
                          size_t window, float softcap, float* d_out, void* stream);

/* fhip_qkv_post with the key and value heads written to packed outputs [t, n_kv * head_dim] (row i for token i) instead of
 * cache rows: for callers that store them themselves, as the quantized arm of qwen3.rs:906-912 does. */
int fhip_qkv_post_packed(const float* d_qkv, const float* d_bias, const float* d_q_norm, const float* d_k_norm, const uint32_t* d_positions,
                         const float* d_freq_scale, size_t t, size_t n_head, size_t n_kv, size_t head_dim, size_t n_rot, int interleaved,
                         float eps, float base, float* d_q_out, float* d_k_out, float* d_v_out, void* stream);

/* crates/ferric-tensor/src/nn.rs:140 decode_attention -> lib.rs:762 fused_decode_attention (kernels :2675, :2740 ff.):
 * one query row q [n_head * head_dim] against the cache rows [0, len) of K and V [., n_kv * head_dim];
 * out[h] = softmax_j(q_h . K[j, h / g] / sqrt(head_dim)) @ V[:, h / g], g = n_head / n_kv (1..=8), head_dim 64 or 128.
 * When d_last_pos is given the length is *d_last_pos + 1 read on the device (clamped to len), so one captured launch
 * serves a growing cache; len still sizes the launch. d_ws: fhip_decode_attention_ws_bytes(...) bytes of scratch (the
 * per-split partial sums; may be NULL when that is 0). */
size_t fhip_decode_attention_ws_bytes(size_t n_head, size_t n_kv, size_t head_dim, size_t len);
int fhip_decode_attention(const float* d_q, const float* d_k_cache, const float* d_v_cache, size_t n_head, size_t n_kv, size_t head_dim,
                          size_t len, const uint32_t* d_last_pos, float* d_ws, float* d_out, void* stream);
/* nn.rs:92 decode_attention_win and the softcapped scores of nn.rs:61 / lib.rs:308 (Gemma-2), which the reference's fused
 * kernel does not take (it falls back to ~12 composed dispatches): window > 0 attends to the last `window` keys only
 * (0, or >= the length: all keys); softcap > 0 replaces each scaled score x by softcap * tanh(x / softcap). With
 * (0, 0.0f) this is fhip_decode_attention. */
int fhip_decode_attention_ex(const float* d_q, const float* d_k_cache, const float* d_v_cache, size_t n_head, size_t n_kv, size_t head_dim,
                             size_t len, const uint32_t* d_last_pos, size_t window, float softcap, float* d_ws, float* d_out, void* stream);

/* fhip_qkv_post and fhip_decode_attention_ex for ONE new token in one launch (crates/ferric-llama/src/qwen3.rs:861-905 followed
 * by crates/ferric-tensor/src/nn.rs:140-166): every attention workgroup forms its own query heads from the raw QKV row
 * [(n_head + 2 n_kv) * head_dim] (bias, per-head RMSNorm, rotation at *d_pos), and the workgroups whose keys include position
 * *d_pos (one, or one per query head of the KV head) form and append that token's K and V rows, the same bits from each,
 * before they read them back. Attention is over rows [0, min(*d_pos + 1,
 * len)) of the caches; `len` (at most cap) is the host-side upper bound that sizes the launch, as in fhip_decode_attention.
 * d_ws: fhip_decode_attention_ws_bytes(n_head, n_kv, head_dim, len) bytes. Same results as the two calls. */
int fhip_qkv_post_attention(const float* d_qkv, const float* d_bias, const float* d_q_norm, const float* d_k_norm, const uint32_t* d_pos,
                            const float* d_freq_scale, size_t n_head, size_t n_kv, size_t head_dim, size_t n_rot, int interleaved, float eps,
                            float base, float* d_k_cache, float* d_v_cache, size_t cap, size_t len, size_t window, float softcap, float* d_ws,
                            float* d_out, void* stream);

/* rmsnorm / add_rmsnorm (lib.rs:346, :372) fused into the mat-vec that consumes it, for ONE activation row:
 *   h = rmsnorm(x [+ resid], norm_w, eps);   y = h W^T   (swiglu != 0: y = silu(gate . h) * (up . h), as fhip_matmul_q_swiglu)
 * and, when d_x_out is given, x_out = x + resid (the next residual). Neither x_out nor y may overlap x, resid, norm_w or each
 * other (FHIP_ERR_ARG): every workgroup reads the whole inputs while the outputs are being stored. The norm is formed while the
 * activation row is staged, so the layer saves a launch; weights whose shape the streaming kernel does not take run the two
 * steps apart through d_h_scratch [cols] (required). d_resid may be NULL (plain rmsnorm). Same value as the unfused pair to
 * rounding (the sum of squares is added in a different order), not the same bits. No single counterpart in the reference. */
int fhip_norm_matmul_q(const fhip_weight* w, const float* d_x, const float* d_resid, const float* d_norm_w, float eps, float* d_x_out,
                       float* d_h_scratch, int swiglu, float* d_y, void* stream);

/* fhip_ffn for callers that cannot allocate or bring a workspace (code under graph capture, tight serving loops, harnesses
 * that forbid hipMalloc): the [rows_x, n_ff] intermediate lives in a 512 KiB array built into the library's code object (one
 * copy per device, held until the process ends), so the call takes inputs and outputs only and calls no allocating routine.
 * Always the mat-vec kernels (two rows per pass over the weights), so its result has the bits of fhip_ffn under
 * FHIP_BATCH_F32_MATVEC. rows_x * n_ff > 131072 floats: FHIP_ERR_SHAPE. Every call on a device shares that device's array:
 * calls that overlap in time on one GPU (two streams, two threads) race on it. It has no counterpart in the reference. */
int fhip_ffn_noalloc(const fhip_weight* gate_up, const fhip_weight* down, const float* d_x, size_t rows_x, float* d_y, void* stream);

/* Which kernels a weight's batches of three rows or more take in fhip_matmul_q, fhip_matmul_q_swiglu and fhip_ffn. It is a
 * property of the weight handle (the reference's QMatrix is immutable after from_bytes, crates/ferric-tensor/src/dtype.rs:865-931;
 * so is this handle as far as launches go: nothing process-wide is read when a launch is enqueued).
 * FHIP_BATCH_ORDERED (what a new handle starts with): the one-pass matrix-core kernels described at fhip_matmul_q; where a
 * launch cuts a weight row's columns between workgroups the pieces go to the library workspace (fhip_workspace_bytes counts
 * them) and one more launch adds them in a fixed order, so the same call on the same inputs returns the same bits on every run.
 * FHIP_BATCH_AUTO: the same kernels with the pieces added by f32 atomics instead: a few microseconds per matmul faster, the
 * last bits vary from run to run (within 2e-6 of the largest output).
 * FHIP_BATCH_F32_MATVEC: the streaming mat-vec's arithmetic for every row; an output row then has the same bits whatever
 * batch it was part of (the guarantee the reference's CPU path gives, crates/ferric-tensor/src/cpu_simd.rs:175-200), at the
 * price of one pass over the weights per four rows (Q4_K, Q5_K, Q6_K and short-row Q8_0: the products of four rows at a time go through the
 * 4 x 4 x 4 int8 matrix instruction, three quarters of the time of two dot-product passes; other formats: two to four rows
 * a pass on the dot-product kernel).
 * fhip_weight_batch_policy sets one handle's policy and returns the one before; any value that is no policy only queries. Set it
 * before sizing or reserving the workspace and not while another thread launches on the handle.
 * fhip_batch_policy sets what handles made AFTERWARDS start with (existing handles keep theirs) and returns the previous
 * default. */
#define FHIP_BATCH_AUTO 0
#define FHIP_BATCH_F32_MATVEC 1
#define FHIP_BATCH_ORDERED 2
int fhip_weight_batch_policy(fhip_weight* w, int policy);
int fhip_batch_policy(int policy);

/* The library's workspace of a stream (NULL: the default stream): device memory the batched paths of fhip_matmul_q,
 * fhip_matmul_q_swiglu and fhip_ffn use for prepared activations and intermediates. It is allocated on first need, only
 * grows (to a power of two), is shared by the calls enqueued on that stream, and is freed by fhip_workspace_release or
 * fhip_stream_destroy (both wait for the stream first). fhip_workspace_bytes: what a call with these weights (down may be
 * NULL) and rows_x rows needs at most, 0 when it takes the mat-vec kernel. fhip_workspace_reserve: grow it to nbytes now,
 * e.g. before a graph capture, during which it cannot grow. A buffer that was outgrown stays allocated until the release,
 * because a graph captured earlier may still name it. No counterpart in the reference (wgpu allocates per dispatch).
 * fhip_workspace_bytes_coop: the same for the matrix-core entry points fhip_gemm_q_bf16, fhip_matmul_q_coop (down NULL) and
 * fhip_ffn_coop, which keep there the partial tiles of a launch that cuts output tiles along K (0 when no tile is cut). */
size_t fhip_workspace_bytes(const fhip_weight* w, const fhip_weight* down, size_t rows_x);
size_t fhip_workspace_bytes_coop(const fhip_weight* w, const fhip_weight* down, size_t rows_x);
int fhip_workspace_reserve(void* stream, size_t nbytes);
void fhip_workspace_release(void* stream);

/* Precision of the activations inside the streaming mat-vec kernels (fhip_matmul_q, _swiglu, fhip_ffn, the "_id" entry points,
 * fhip_norm_matmul_q): per run of 32 (16 for Q6_K) columns the activations are held as block fixed point with a `bits`-bit
 * significand at the run's largest magnitude, the weights exactly, the sums exactly, and everything above the sub-block in
 * f32. A property of the weight handle, like the batch policy.
 * bits = 24 (what a new handle starts with): the significand of f32 itself, results within 1e-5 of the largest output -- the
 * bar the reference's own examples hold its scalar kernels to (crates/ferric-tensor/examples/q4_k.rs:54, q6_k.rs:33,
 * q8_0.rs:21), so a handle left alone passes them.
 * bits = 16 (opt-in): dot products within about 1e-4 of the largest output, still three orders of magnitude inside
 * 1e-3 * ||w_row|| * ||x||, but NOT inside the 1e-5 of those examples; 1-6 % faster.
 * fhip_weight_matvec_precision sets one handle (bits = 0 only queries) and returns its setting before the call (16 or 24), or
 * FHIP_ERR_ARG; not while another thread launches on the handle. fhip_matvec_precision sets what handles made AFTERWARDS start
 * with and returns the previous default. The reference has no such switch: its kernels multiply f32 by f32. */
int fhip_weight_matvec_precision(fhip_weight* w, int bits);
int fhip_matvec_precision(int bits);

/* words[i] += delta for n device u32 words: advances the position word(s) at the end of a captured decode step. */
int fhip_u32_add(uint32_t* d_words, size_t n, uint32_t delta, void* stream);

/* f32 -> bf16 bit patterns, round to nearest even, n values (both pointers 16-byte aligned). The reference's
 * matrix-unit kernels read f32 activations (crates/ferric-tensor/src/dtype.rs:1824-1830, `xp.buf`); the
 * matrix cores here take bf16, so this is the conversion in front of fhip_gemm_q_bf16. */
int fhip_cvt_f32_bf16(const float* d_x, size_t n, uint16_t* d_out_bf16, void* stream);

/* crates/ferric-tensor/src/dtype.rs:1818 Tensor::matmul_q4_k_coop(w) (:1199 matmul_q6_k_coop, :1316
 * matmul_q8_0_coop) with the reference's own operand types: x f32 [rows_x, cols] -> y f32 [rows_x, rows].
 * Converts x into the caller's scratch d_ws_bf16 (rows_x * cols 16-bit values, 16-byte aligned) and runs
 * fhip_gemm_q_bf16 on it. Any rows_x (no padding to 8 as at dtype.rs:1823: the kernel masks). */
int fhip_matmul_q_coop(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, uint16_t* d_ws_bf16,
                       void* stream);

/* The FFN block of crates/ferric-llama/src/qwen3.rs:944-964 built from the matrix-unit matmuls
 * (crates/ferric-tensor/src/dtype.rs:1818, :1199, :1316) for a batch of rows: x f32 -> bf16, gate_up GEMM,
 * SwiGLU rounded to bf16, down GEMM, y f32 [rows_x, down rows]. d_ws: caller-provided scratch of
 * fhip_ffn_coop_ws_bytes(...) bytes, 256-byte aligned. Any of the three formats for either weight. */
size_t fhip_ffn_coop_ws_bytes(const fhip_weight* gate_up, const fhip_weight* down, size_t rows_x);
int fhip_ffn_coop(const fhip_weight* gate_up, const fhip_weight* down, const float* d_x, size_t rows_x, float* d_y,
                  void* d_ws, void* stream);

/* crates/ferric-tensor/src/dtype.rs:935-944 Tensor::matmul_q for 1..32 activation rows in ONE pass over the weights
 * with f32-grade results (the reference's kernels, :2995-3051 and :3423-3469, walk the weight row once per activation
 * row): x f32 [rows_x, cols] -> y f32 [rows_x, rows]. Q4_K, Q5_K and Q6_K (cols a multiple of 256, as the formats
 * require), and Q8_0 (:2948-2990; cols a multiple of 32) for up to 16 rows.
 * Each 256-column chunk of an activation row is scaled by a power of two and split into two f16 operand rows (22
 * significant bits at the chunk's largest magnitude), the
 * weights enter the f16 matrix cores as exact integers (sub-block scale x quant; the int8 quant for Q8_0) and the f32
 * block scale is applied to the f32 accumulator. d_ws: caller-provided scratch of fhip_matmul_q_f16x2_ws_bytes(...)
 * bytes, 256-byte aligned. rows_x > 32 (> 16 for Q8_0): FHIP_ERR_SHAPE; other formats: FHIP_ERR_UNSUPPORTED_TYPE
 * (ws_bytes returns 0 for both). */
size_t fhip_matmul_q_f16x2_ws_bytes(const fhip_weight* w, size_t rows_x);
int fhip_matmul_q_f16x2(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, void* d_ws, void* stream);

/* The FFN block of crates/ferric-llama/src/qwen3.rs:944-964 for a batch of 1..32 rows on the same path: gate_up
 * matmul, SwiGLU (crates/ferric-tensor/src/lib.rs:2603-2618, f32) fused into the split of the down projection's
 * activations, down matmul; y f32 [rows_x, down rows]. Same checks and messages as fhip_ffn. */
size_t fhip_ffn_f16x2_ws_bytes(const fhip_weight* gate_up, const fhip_weight* down, size_t rows_x);
int fhip_ffn_f16x2(const fhip_weight* gate_up, const fhip_weight* down, const float* d_x, size_t rows_x, float* d_y,
                   void* d_ws, void* stream);

/* ---- GGUF ingest: file -> HBM without a host copy or repack (host code; no device needed to parse) ------- */

typedef struct fhip_gguf fhip_gguf;

/* crates/ferric-gguf/src/lib.rs:105 parse(bytes): header, metadata, tensor table, then check_declared_strides
 * (:387) against the data section. `bytes` must outlive the handle. Errors (FHIP_ERR_FORMAT, text as the
 * reference's): "not a GGUF file", "GGUF header truncated or malformed", the two stride refusals.
 * fhip_gguf_open maps the file read-only and parses the mapping (the native GgufFile, :520-573, without its
 * read-per-tensor: the mapping IS the raw view). */
int fhip_gguf_parse(const uint8_t* bytes, size_t n, fhip_gguf** out);
int fhip_gguf_open(const char* path, fhip_gguf** out);
void fhip_gguf_close(fhip_gguf* g);
uint32_t fhip_gguf_version(const fhip_gguf* g);
uint64_t fhip_gguf_data_start(const fhip_gguf* g);

/* TensorInfo (lib.rs:41-47), in file order; pointers stay valid until close. fhip_gguf_find: index or -1
 * (Gguf::tensor, lib.rs:441). */
size_t fhip_gguf_n_tensors(const fhip_gguf* g);
int fhip_gguf_tensor(const fhip_gguf* g, size_t i, const char** name, uint32_t* n_dims, const uint64_t** dims, uint32_t* ggml_type,
                     uint64_t* offset);
long fhip_gguf_find(const fhip_gguf* g, const char* name);

/* Gguf::raw / GgufFile::raw (lib.rs:443-449, :566-573): the tensor's packed bytes exactly as stored, as a view into
 * the parsed buffer / mapping (no copy). Unknown name -> FHIP_ERR_FORMAT "no tensor 'name'". */
int fhip_gguf_raw(const fhip_gguf* g, const char* name, const uint8_t** bytes, size_t* nbytes);

/* Metadata (lib.rs:38 enum Meta): kind 0 U, 1 I, 2 F, 3 Bool, 4 Str, 5 Arr, or -1 when absent; arr_len is set for
 * arrays. The typed getters read the value itself (j = (size_t)-1) or element j of an array. */
size_t fhip_gguf_n_meta(const fhip_gguf* g);
const char* fhip_gguf_meta_key(const fhip_gguf* g, size_t i);
int fhip_gguf_meta_kind(const fhip_gguf* g, const char* key, size_t* arr_len);
int fhip_gguf_meta_u64(const fhip_gguf* g, const char* key, size_t j, uint64_t* out);
int fhip_gguf_meta_i64(const fhip_gguf* g, const char* key, size_t j, int64_t* out);
int fhip_gguf_meta_f64(const fhip_gguf* g, const char* key, size_t j, double* out);
int fhip_gguf_meta_str(const fhip_gguf* g, const char* key, size_t j, const char** s, size_t* len);

/* QShard::build from a GGUF tensor (crates/ferric-tensor/src/dtype.rs:839-857 over GgufSource::raw): uploads the
 * tensor's bytes straight from the mapping. dims are [in, out] or, for an expert slab, [in, rows per expert,
 * n_expert] (rows = product of the trailing dims). Types 2 / 3 / 6 / 7 / 8 / 12 / 13 / 14 / 20 / 23 / 39 only. */
int fhip_weight_from_gguf(const fhip_gguf* g, const char* name, fhip_weight** out);

/* crates/ferric-llama/src/qwen35.rs:379-402 qm_cat(ctx, g, names) (fused QKV, fused gate|up): several tensors of one
 * format and one input width stacked along the output dim into ONE weight. Each tensor's bytes go from the mapping to
 * their place in the device allocation; nothing is concatenated on the host. Errors with the reference's messages:
 * "no tensor 'X'", "X: mixed quant formats in one fused matmul", "X: input dim differs" (FHIP_ERR_FORMAT, the
 * reference's Err(String)). */
int fhip_weight_from_gguf_cat(const fhip_gguf* g, const char* const* names, size_t n_names, fhip_weight** out);

/* crates/ferric-tensor/src/cpu_simd.rs:79 matvec_q8_0(x, w, rows, cols) with HOST buffers on both
 * sides (upload, GEMV, download, synchronise) -- the drop-in for the CPU mat-vec call.
 * Errors as the reference's asserts: cols % 32, w_len != rows * cols/32*34 -> FHIP_ERR_SHAPE. */
int fhip_matvec_q8_0_host(const float* h_x, const uint8_t* h_w, size_t w_len, size_t rows, size_t cols, float* h_y);

/* crates/ferric-tensor/src/cpu_simd.rs:238-300 Pool and :303-331 matvec_q8_0_pooled(pool, x, w, cols, lo, hi): rows
 * [lo, hi) of y = x . W^T with host buffers on both sides, on a pool that is set up once. The reference's pool saves
 * the thread creation of every call; what a host-buffer call pays here is the upload of the weight, so the pool keeps
 * the bytes of the last `h_w` it was given resident in HBM (with its staging buffers and a stream of its own) and a
 * call with the same (h_w, w_len, cols) uploads the activations only. `w` is an immutable Arc<Vec<u8>> in the
 * reference; a caller that rewrites the bytes in place, or frees them (another buffer may then appear at the same address),
 * calls fhip_pool_forget first -- a binding keeps a clone of the Arc beside the pool for as long as it is the key. As a
 * second line of defence the key also holds a fingerprint of the bytes (first and last 4 KiB and 64 spread samples, hashed on
 * every call): a buffer rewritten or reused at the same address and length is uploaded again unless the change misses all of
 * those, so the fingerprint replaces no fhip_pool_forget.
 * h_y receives hi - lo values.
 * `threads` is kept for Pool::threads() (at least 1) and partitions nothing here. lo > hi, a span past the rows in
 * h_w or fewer than cols activations: FHIP_ERR_SHAPE (the reference's assert and slice panics). One call at a time
 * per pool (the reference serialises Pool::run behind a mutex). */
typedef struct fhip_pool fhip_pool;
int fhip_pool_create(size_t threads, fhip_pool** out);
size_t fhip_pool_threads(const fhip_pool* p);
size_t fhip_pool_uploads(const fhip_pool* p);   /* weight uploads so far: 1 after any number of calls on one weight */
void fhip_pool_forget(fhip_pool* p);
void fhip_pool_destroy(fhip_pool* p);
int fhip_matvec_q8_0_pooled(fhip_pool* p, const float* h_x, size_t x_len, const uint8_t* h_w, size_t w_len, size_t cols,
                            size_t lo, size_t hi, float* h_y);

#ifdef __cplusplus
}
#endif
#endif /* FERRIC_HIP_H */
