// Prefill dequant-GEMM (placeholder until the matrix-core kernel lands).
#include "common.hpp"

namespace fhip {
int launch_gemm_bf16(const fhip_weight*, const uint16_t*, size_t, float*, hipStream_t) {
    return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "fhip_gemm_q_bf16: not built yet");
}
}  // namespace fhip
