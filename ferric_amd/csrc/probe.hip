// Measurement aid: a kernel that only reads. What it reaches on a buffer is the ceiling this device offers a mat-vec of the
// same size in the same launch conditions (one launch, cold data): no arithmetic, no reduction, 16-byte loads, 8 in flight
// per lane. bench.py times it beside the mat-vec kernels ("reader_floor_us").
#include "common.hpp"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(256) read_probe_kernel(const u32x4* __restrict__ src, size_t n16, uint32_t* __restrict__ sink) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    u32x4 acc = {0, 0, 0, 0};
    for (; i + 7 * stride < n16; i += 8 * stride) {
        u32x4 v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) v[k] = src[i + k * stride];
#pragma unroll
        for (int k = 0; k < 8; k++) acc |= v[k];
    }
    for (; i < n16; i += stride) acc |= src[i];
    const uint32_t r = acc[0] | acc[1] | acc[2] | acc[3];
    if (r == 0x9E3779B9u) sink[0] = r;   // practically never: the loads must stay, the store must not cost
}

}  // namespace

namespace fhip {

int launch_read_probe(const void* d_src, size_t nbytes, uint32_t* d_sink, hipStream_t s) {
    const size_t n16 = nbytes / 16;
    if (n16 == 0) return FHIP_OK;
    size_t wgs = (n16 + 256 * 8 - 1) / (256 * 8);
    const size_t cap = (size_t)(device_cus() > 0 ? device_cus() : 256) * 8;
    if (wgs > cap) wgs = cap;
    hipLaunchKernelGGL(read_probe_kernel, dim3((unsigned)wgs), dim3(256), 0, s, (const u32x4*)d_src, n16, d_sink);
    return check_hip(hipGetLastError(), "read probe launch");
}

}  // namespace fhip
