// Shared host-side declarations of libferric_hip: the weight handle, error plumbing and the
// kernel launchers each .hip translation unit provides.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/ferric_hip.h"

struct fhip_weight {
    uint32_t type;      // ggml id: 8 / 12 / 14
    size_t rows, cols;  // [out, in]
    size_t row_bytes;   // cols / block_values * block_bytes
    size_t nbytes;      // rows * row_bytes
    const uint8_t* d_raw;  // raw GGUF block stream in HBM
    bool owns;          // allocated by fhip_weight_create (freed on destroy)
};

namespace fhip {

int set_error(int code, const char* fmt, ...);
int check_hip(hipError_t e, const char* what);
int device_cus();
size_t device_lds_bytes();  // LDS one workgroup may use

// dequant.hip
int launch_f16_to_f32(const uint16_t* d_bits, size_t n, float* d_out, hipStream_t s);
int launch_dequant(uint32_t type, const uint8_t* d_raw, size_t nblocks, float* d_out, hipStream_t s);

// gemv.hip
// y[rows_x, out_rows] = x * W^T; when n_ff > 0 the weight stacks gate|up (2*n_ff rows) and
// y[rows_x, n_ff] = silu(gate.x) * (up.x).
int launch_gemv(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, size_t n_ff, hipStream_t s);
// gemv_generic.hip: same contract, any cols the format allows (up to 32768)
int launch_gemv_generic(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, size_t n_ff, hipStream_t s);
int launch_swiglu(const float* d_gu, size_t t, size_t d, float* d_out, hipStream_t s);

// gemm_mfma.hip
// y_cleared: the caller has zeroed y on this stream already (see gemm_bf16_adds_into_y)
int launch_gemm_bf16(const fhip_weight* w, const uint16_t* d_x, size_t t, float* d_y, hipStream_t s, bool y_cleared = false);
bool gemm_bf16_adds_into_y(size_t t);   // true: a launch for t rows may add into y, so a cleared y saves it a launch
// conversions in front of the GEMM; each can also clear `zero_n` floats at `zero`
int launch_cvt_bf16(const float* d_x, size_t n, uint16_t* d_out, hipStream_t s, float* zero = nullptr, size_t zero_n = 0);
int launch_swiglu_bf16(const float* d_gu, size_t t, size_t d, uint16_t* d_out, hipStream_t s, float* zero = nullptr,
                       size_t zero_n = 0);

}  // namespace fhip
