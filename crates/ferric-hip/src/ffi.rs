//! Raw bindings of libferric_hip.so, one declaration per entry point of include/ferric_hip.h (same order; the header's
//! comments give each function's contract and the reference interface it replaces). Device pointers are plain raw pointers;
//! `stream` arguments take a handle from `fhip_stream_create` or null for the default stream.
use std::os::raw::{c_char, c_void};

#[repr(C)] pub struct FhipWeight { _private: [u8; 0] }
#[repr(C)] pub struct FhipPool { _private: [u8; 0] }
#[repr(C)] pub struct FhipGguf { _private: [u8; 0] }

pub const FHIP_OK: i32 = 0;
pub const FHIP_ERR_UNSUPPORTED_TYPE: i32 = -1;
pub const FHIP_ERR_SHAPE: i32 = -2;
pub const FHIP_ERR_HIP: i32 = -3;
pub const FHIP_ERR_ARG: i32 = -4;
pub const FHIP_ERR_FORMAT: i32 = -5;
pub const FHIP_BATCH_AUTO: i32 = 0;
pub const FHIP_BATCH_F32_MATVEC: i32 = 1;

#[link(name = "ferric_hip")]
extern "C" {
    pub fn fhip_init(device: i32) -> i32;
    pub fn fhip_last_error() -> *const c_char;
    pub fn fhip_device_cus() -> i32;
    pub fn fhip_type_size(ggml_type: u32, n: usize) -> usize;
    pub fn fhip_block_bytes(ggml_type: u32, values: *mut usize, bytes: *mut usize) -> i32;
    pub fn fhip_malloc(d_ptr: *mut *mut c_void, nbytes: usize) -> i32;
    pub fn fhip_free(d_ptr: *mut c_void) -> i32;
    pub fn fhip_memcpy_h2d(d_dst: *mut c_void, h_src: *const c_void, nbytes: usize, stream: *mut c_void) -> i32;
    pub fn fhip_memcpy_d2h(h_dst: *mut c_void, d_src: *const c_void, nbytes: usize, stream: *mut c_void) -> i32;
    pub fn fhip_memcpy_d2d(d_dst: *mut c_void, d_src: *const c_void, nbytes: usize, stream: *mut c_void) -> i32;
    pub fn fhip_memcpy_2d_d2d(d_dst: *mut c_void, dpitch: usize, d_src: *const c_void, spitch: usize, width: usize, height: usize, stream: *mut c_void) -> i32;
    pub fn fhip_memset(d_dst: *mut c_void, byte: i32, nbytes: usize, stream: *mut c_void) -> i32;
    pub fn fhip_stream_create(stream: *mut *mut c_void) -> i32;
    pub fn fhip_stream_destroy(stream: *mut c_void) -> i32;
    pub fn fhip_stream_sync(stream: *mut c_void) -> i32;
    pub fn fhip_event_create(event: *mut *mut c_void) -> i32;
    pub fn fhip_event_destroy(event: *mut c_void) -> i32;
    pub fn fhip_event_record(event: *mut c_void, stream: *mut c_void) -> i32;
    pub fn fhip_event_sync(event: *mut c_void) -> i32;
    pub fn fhip_event_elapsed_ms(start: *mut c_void, stop: *mut c_void, ms: *mut f32) -> i32;
    pub fn fhip_graph_capture_begin(stream: *mut c_void) -> i32;
    pub fn fhip_graph_capture_end(stream: *mut c_void, graph_exec: *mut *mut c_void) -> i32;
    pub fn fhip_graph_launch(graph_exec: *mut c_void, stream: *mut c_void) -> i32;
    pub fn fhip_graph_destroy(graph_exec: *mut c_void) -> i32;
    pub fn fhip_weight_create(ggml_type: u32, h_raw: *const u8, nbytes: usize, rows: usize, cols: usize, out_: *mut *mut FhipWeight) -> i32;
    pub fn fhip_weight_create_parts(ggml_type: u32, h_parts: *const *const u8, part_bytes: *const usize, n_parts: usize, rows: usize, cols: usize, out_: *mut *mut FhipWeight) -> i32;
    pub fn fhip_weight_wrap_device(ggml_type: u32, d_raw: *const u8, nbytes: usize, rows: usize, cols: usize, out_: *mut *mut FhipWeight) -> i32;
    pub fn fhip_weight_destroy(w: *mut FhipWeight);
    pub fn fhip_weight_rows(w: *const FhipWeight) -> usize;
    pub fn fhip_weight_cols(w: *const FhipWeight) -> usize;
    pub fn fhip_weight_nbytes(w: *const FhipWeight) -> usize;
    pub fn fhip_weight_type(w: *const FhipWeight) -> u32;
    pub fn fhip_f16_to_f32(d_bits: *const u16, n: usize, d_out: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_dequant_rows(w: *const FhipWeight, row0: usize, nrows: usize, d_out: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_deq_raw(h_raw: *const u8, nbytes: usize, n: usize, ggml_type: u32, h_out: *mut f32, n_written: *mut usize) -> i32;
    pub fn fhip_matmul_q(w: *const FhipWeight, d_x: *const f32, rows_x: usize, d_y: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_matmul_q_swiglu(gate_up: *const FhipWeight, d_x: *const f32, rows_x: usize, d_y: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_swiglu(d_gu: *const f32, t: usize, d: usize, d_out: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_ffn(gate_up: *const FhipWeight, down: *const FhipWeight, d_x: *const f32, rows_x: usize, d_y: *mut f32, d_ws: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_gemm_q_bf16(w: *const FhipWeight, d_x_bf16: *const u16, t: usize, d_y: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_moe_topk(d_logits: *const f32, d_bias: *const f32, t: usize, n_expert: usize, k: usize, sigmoid: i32, scale: f32, norm: i32, d_out: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_matmul_q_swiglu_id(w: *const FhipWeight, d_x: *const f32, t: usize, d_selw: *const f32, k: usize, eff: usize, d_y: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_matmul_q_id(w: *const FhipWeight, d_x: *const f32, d_selw: *const f32, k: usize, out_pe: usize, d_y: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_matmul_q_id_wsum(w: *const FhipWeight, d_x: *const f32, t: usize, d_selw: *const f32, k: usize, out_pe: usize, d_y: *mut f32, d_ws: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_rmsnorm(d_x: *const f32, d_weight: *const f32, rows: usize, d: usize, eps: f32, d_out: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_add_rmsnorm(d_a: *const f32, d_b: *const f32, d_weight: *const f32, rows: usize, d: usize, eps: f32, d_sum: *mut f32, d_norm: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_add(d_a: *const f32, d_b: *const f32, n: usize, d_out: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_rope(d_x: *const f32, src_row_stride: usize, t: usize, n_heads: usize, head_dim: usize, n_rot: usize, base: f32, d_positions: *const u32, pos_off: u32, d_freq_scale: *const f32, interleaved: i32, d_out: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_kv_append2(d_k: *const f32, d_v: *const f32, t: usize, width: usize, d_positions: *const u32, pos_off: u32, d_k_cache: *mut f32, d_v_cache: *mut f32, cap: usize, stream: *mut c_void) -> i32;
    pub fn fhip_qkv_post(d_qkv: *const f32, d_bias: *const f32, d_q_norm: *const f32, d_k_norm: *const f32, d_positions: *const u32, d_freq_scale: *const f32, t: usize, n_head: usize, n_kv: usize, head_dim: usize, n_rot: usize, interleaved: i32, eps: f32, base: f32, d_q_out: *mut f32, d_k_cache: *mut f32, d_v_cache: *mut f32, cap: usize, stream: *mut c_void) -> i32;
    pub fn fhip_decode_attention_ws_bytes(n_head: usize, n_kv: usize, head_dim: usize, len: usize) -> usize;
    pub fn fhip_decode_attention(d_q: *const f32, d_k_cache: *const f32, d_v_cache: *const f32, n_head: usize, n_kv: usize, head_dim: usize, len: usize, d_last_pos: *const u32, d_ws: *mut f32, d_out: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_decode_attention_ex(d_q: *const f32, d_k_cache: *const f32, d_v_cache: *const f32, n_head: usize, n_kv: usize, head_dim: usize, len: usize, d_last_pos: *const u32, window: usize, softcap: f32, d_ws: *mut f32, d_out: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_qkv_post_attention(d_qkv: *const f32, d_bias: *const f32, d_q_norm: *const f32, d_k_norm: *const f32, d_pos: *const u32, d_freq_scale: *const f32, n_head: usize, n_kv: usize, head_dim: usize, n_rot: usize, interleaved: i32, eps: f32, base: f32, d_k_cache: *mut f32, d_v_cache: *mut f32, cap: usize, len: usize, window: usize, softcap: f32, d_ws: *mut f32, d_out: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_norm_matmul_q(w: *const FhipWeight, d_x: *const f32, d_resid: *const f32, d_norm_w: *const f32, eps: f32, d_x_out: *mut f32, d_h_scratch: *mut f32, swiglu: i32, d_y: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_ffn_noalloc(gate_up: *const FhipWeight, down: *const FhipWeight, d_x: *const f32, rows_x: usize, d_y: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_batch_policy(policy: i32) -> i32;
    pub fn fhip_workspace_bytes(w: *const FhipWeight, down: *const FhipWeight, rows_x: usize) -> usize;
    pub fn fhip_workspace_reserve(stream: *mut c_void, nbytes: usize) -> i32;
    pub fn fhip_workspace_release(stream: *mut c_void);
    pub fn fhip_debug_generic_matvec(on: i32) -> i32;
    pub fn fhip_debug_read_probe(d_src: *const c_void, nbytes: usize, d_sink: *mut u32, stream: *mut c_void) -> i32;
    pub fn fhip_debug_matmul_q_loop(ws: *const *const FhipWeight, n_weights: usize, launches: usize, d_x: *const f32, swiglu: i32, d_y: *mut f32, stream: *mut c_void) -> i32;
    pub fn fhip_matvec_precision(bits: i32) -> i32;
    pub fn fhip_u32_add(d_words: *mut u32, n: usize, delta: u32, stream: *mut c_void) -> i32;
    pub fn fhip_cvt_f32_bf16(d_x: *const f32, n: usize, d_out_bf16: *mut u16, stream: *mut c_void) -> i32;
    pub fn fhip_matmul_q_coop(w: *const FhipWeight, d_x: *const f32, rows_x: usize, d_y: *mut f32, d_ws_bf16: *mut u16, stream: *mut c_void) -> i32;
    pub fn fhip_ffn_coop_ws_bytes(gate_up: *const FhipWeight, down: *const FhipWeight, rows_x: usize) -> usize;
    pub fn fhip_ffn_coop(gate_up: *const FhipWeight, down: *const FhipWeight, d_x: *const f32, rows_x: usize, d_y: *mut f32, d_ws: *mut c_void, stream: *mut c_void) -> i32;
    pub fn fhip_matmul_q_f16x2_ws_bytes(w: *const FhipWeight, rows_x: usize) -> usize;
    pub fn fhip_matmul_q_f16x2(w: *const FhipWeight, d_x: *const f32, rows_x: usize, d_y: *mut f32, d_ws: *mut c_void, stream: *mut c_void) -> i32;
    pub fn fhip_ffn_f16x2_ws_bytes(gate_up: *const FhipWeight, down: *const FhipWeight, rows_x: usize) -> usize;
    pub fn fhip_ffn_f16x2(gate_up: *const FhipWeight, down: *const FhipWeight, d_x: *const f32, rows_x: usize, d_y: *mut f32, d_ws: *mut c_void, stream: *mut c_void) -> i32;
    pub fn fhip_gguf_parse(bytes: *const u8, n: usize, out_: *mut *mut FhipGguf) -> i32;
    pub fn fhip_gguf_open(path: *const c_char, out_: *mut *mut FhipGguf) -> i32;
    pub fn fhip_gguf_close(g: *mut FhipGguf);
    pub fn fhip_gguf_version(g: *const FhipGguf) -> u32;
    pub fn fhip_gguf_data_start(g: *const FhipGguf) -> u64;
    pub fn fhip_gguf_n_tensors(g: *const FhipGguf) -> usize;
    pub fn fhip_gguf_tensor(g: *const FhipGguf, i: usize, name: *mut *const c_char, n_dims: *mut u32, dims: *mut *const u64, ggml_type: *mut u32, offset: *mut u64) -> i32;
    pub fn fhip_gguf_find(g: *const FhipGguf, name: *const c_char) -> std::os::raw::c_long;
    pub fn fhip_gguf_raw(g: *const FhipGguf, name: *const c_char, bytes: *mut *const u8, nbytes: *mut usize) -> i32;
    pub fn fhip_gguf_n_meta(g: *const FhipGguf) -> usize;
    pub fn fhip_gguf_meta_key(g: *const FhipGguf, i: usize) -> *const c_char;
    pub fn fhip_gguf_meta_kind(g: *const FhipGguf, key: *const c_char, arr_len: *mut usize) -> i32;
    pub fn fhip_gguf_meta_u64(g: *const FhipGguf, key: *const c_char, j: usize, out_: *mut u64) -> i32;
    pub fn fhip_gguf_meta_i64(g: *const FhipGguf, key: *const c_char, j: usize, out_: *mut i64) -> i32;
    pub fn fhip_gguf_meta_f64(g: *const FhipGguf, key: *const c_char, j: usize, out_: *mut f64) -> i32;
    pub fn fhip_gguf_meta_str(g: *const FhipGguf, key: *const c_char, j: usize, s: *mut *const c_char, len: *mut usize) -> i32;
    pub fn fhip_weight_from_gguf(g: *const FhipGguf, name: *const c_char, out_: *mut *mut FhipWeight) -> i32;
    pub fn fhip_weight_from_gguf_cat(g: *const FhipGguf, names: *const *const c_char, n_names: usize, out_: *mut *mut FhipWeight) -> i32;
    pub fn fhip_matvec_q8_0_host(h_x: *const f32, h_w: *const u8, w_len: usize, rows: usize, cols: usize, h_y: *mut f32) -> i32;
    pub fn fhip_pool_create(threads: usize, out_: *mut *mut FhipPool) -> i32;
    pub fn fhip_pool_threads(p: *const FhipPool) -> usize;
    pub fn fhip_pool_uploads(p: *const FhipPool) -> usize;
    pub fn fhip_pool_forget(p: *mut FhipPool);
    pub fn fhip_pool_destroy(p: *mut FhipPool);
    pub fn fhip_matvec_q8_0_pooled(p: *mut FhipPool, h_x: *const f32, x_len: usize, h_w: *const u8, w_len: usize, cols: usize, lo: usize, hi: usize, h_y: *mut f32) -> i32;
}
