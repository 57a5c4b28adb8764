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

// Measurement aid: matrix instructions on operands that stay in registers. Eight waves a workgroup (two per SIMD), one
// workgroup per CU, four independent 32 x 32 accumulators per wave, `iters` rounds of four v_mfma_f32_32x32x16_bf16 each:
// what the matrix pipe gives in wall-clock terms when nothing else has to happen (operands with random mantissas, so the
// multipliers switch as they do on real data and the clock settles where the power limit puts it).
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__global__ void __launch_bounds__(512) mfma_probe_kernel(int iters, float* __restrict__ sink) {
    uint32_t h = (uint32_t)(blockIdx.x * 512 + threadIdx.x) * 0x9E3779B9u + 0x7F4A7C15u;
    auto next = [&]() {   // a bf16 pair in [1, 2) with random mantissas and signs
        h = h * 1664525u + 1013904223u;
        return (h & 0x807F807Fu) | 0x3F803F80u;
    };
    u32x4 ar[2], br[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        ar[j] = (u32x4){next(), next(), next(), next()};
        br[j] = (u32x4){next(), next(), next(), next()};
    }
    f32x16 acc[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[j][r] = 0.f;
#pragma unroll 1
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int j = 0; j < 4; j++)
            acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ar[j & 1]), __builtin_bit_cast(bf16x8, br[j >> 1]),
                                                             acc[j], 0, 0, 0);
    }
    float t = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) t += acc[j][r];
    if (t == 12345.678f) sink[0] = t;   // practically never: the arithmetic must stay, the store must not cost
}

}  // namespace

namespace fhip {

int launch_mfma_probe(int iters, float* d_sink, hipStream_t s, double* flops) {
    const int cus = device_cus() > 0 ? device_cus() : 256;
    if (flops) *flops = (double)cus * 8.0 * (double)iters * 4.0 * 2.0 * 32.0 * 32.0 * 16.0;
    hipLaunchKernelGGL(mfma_probe_kernel, dim3((unsigned)cus), dim3(512), 0, s, iters, d_sink);
    return check_hip(hipGetLastError(), "mfma probe launch");
}

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
