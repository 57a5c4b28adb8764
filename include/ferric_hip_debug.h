/* Measurement and test aids of libferric_hip.so. They are exported by the same library but are no part of the interface a
 * caller of the quantized-linear path binds (include/ferric_hip.h): none of them has a counterpart in the reference. */
#ifndef FERRIC_HIP_DEBUG_H
#define FERRIC_HIP_DEBUG_H

#include "ferric_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Debugging and tests: on != 0 sends every mat-vec to the shape-complete f32 kernel instead of the streaming one (process-wide,
 * not thread-safe against concurrent launches). No counterpart in the reference. */
int fhip_debug_generic_matvec(int on);

/* Debugging and tests: pins the workgroup tile of the matrix-core GEMM (fhip_gemm_q_bf16, fhip_matmul_q_coop, fhip_ffn_coop)
 * for launches of more than 32 rows: 0, 1, 2 = 64, 128, 256 activation rows x 256 outputs, 3 = 256 x 160, 4, 5 = 128, 64 rows x
 * 128 outputs, 6 = 128 x 160; -1 (the default) lets the cost estimate choose. Returns the value before the call. Process-wide, not thread-safe against concurrent
 * launches; fhip_workspace_bytes_coop follows it. No counterpart in the reference. */
int fhip_debug_gemm_tile(int tile);

/* Debugging and tests: on == 0 keeps Q4_K / Q5_K / Q6_K / Q8_0 batches of three and more rows off the kernel that multiplies on the
 * 4 x 4 x 4 int8 matrix instruction, so that the mat-vec entry points run them on the dot-product kernel two rows at a time
 * (the two give the same bits; the tests compare them this way). Returns the setting before the call (1 = on, the default).
 * Process-wide, not thread-safe against concurrent launches. No counterpart in the reference. */
int fhip_debug_quad_matvec(int on);

/* Measurement aid: one launch that reads nbytes at d_src (16-byte loads over the whole chip) and does nothing else; d_sink is
 * one device word that is practically never written. Timed beside a mat-vec of the same size it gives the time a perfect reader
 * needs for those bytes on this device. No counterpart in the reference (its matvec_roofline example prints bytes / time of the
 * kernel itself, crates/ferric-tensor/examples/matvec_roofline.rs:85-100). */
int fhip_debug_read_probe(const void* d_src, size_t nbytes, uint32_t* d_sink, void* stream);

/* Measurement aid: one launch of matrix instructions only (v_mfma_f32_32x32x16_bf16 on register-resident operands with random
 * mantissas; one workgroup of eight waves per CU, `iters` rounds of four instructions per wave). *flops (may be NULL) receives
 * the floating-point operations of the launch: 2 * 32 * 32 * 16 per instruction. Timed, it is what the matrix pipe gives on this
 * device at the clock its power limit allows, the ceiling the dequant-GEMM is priced against. d_sink is one device float that
 * is practically never written. No counterpart in the reference. */
int fhip_debug_mfma_probe(int iters, float* d_sink, double* flops, void* stream);

/* Measurement aid: `launches` one-row calls of fhip_matmul_q (swiglu != 0: fhip_matmul_q_swiglu) enqueued back to back from
 * native code, launch i on weight ws[i % n_weights], all with the same x and y. A profiler run that cannot replay graphs gets
 * the same steady stream of launches from it that a captured graph gives. No counterpart in the reference. */
int fhip_debug_matmul_q_loop(const fhip_weight* const* ws, size_t n_weights, size_t launches, const float* d_x, int swiglu, float* d_y,
                             void* stream);

#ifdef __cplusplus
}
#endif

#endif /* FERRIC_HIP_DEBUG_H */
