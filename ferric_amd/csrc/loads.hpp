// Wide loads from addresses that are only 2-byte aligned (Q6_K blocks are 210 bytes, Q8_0 blocks 34, the legacy 4/5-bit
// blocks 18..24). The memory pipeline splits a dwordx2 / dwordx4 load whose address is not a multiple of 4 and runs it
// at about 60 % of the aligned rate (measured on the Q6_K down projection: 47 us with such loads, 31 us aligned). So
// the load is made from the dword boundary at or below the address and the bytes are shifted into place: one
// v_alignbyte_b32 per dword. The last two bytes come from their own 2-byte load, so nothing outside [p, p + n) is read
// beyond the two bytes below p that lie in the same dword.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace fhip {

typedef uint32_t ld_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t ld_u32x2 __attribute__((ext_vector_type(2)));
struct __attribute__((packed, aligned(4))) LdU4A4 { ld_u32x4 v; };
struct __attribute__((packed, aligned(4))) LdU2A4 { ld_u32x2 v; };

__device__ __forceinline__ ld_u32x4 load16_a2(const uint8_t* p) {
    const uint32_t m = (uint32_t)(uintptr_t)p & 2u;
    const ld_u32x4 w = ((const LdU4A4*)(p - m))->v;
    const uint32_t e = *(const uint16_t*)(p + 14);
    return (ld_u32x4){__builtin_amdgcn_alignbyte(w[1], w[0], m), __builtin_amdgcn_alignbyte(w[2], w[1], m),
                      __builtin_amdgcn_alignbyte(w[3], w[2], m), __builtin_amdgcn_alignbyte(e, w[3], m)};
}

__device__ __forceinline__ ld_u32x2 load8_a2(const uint8_t* p) {
    const uint32_t m = (uint32_t)(uintptr_t)p & 2u;
    const ld_u32x2 w = ((const LdU2A4*)(p - m))->v;
    const uint32_t e = *(const uint16_t*)(p + 6);
    return (ld_u32x2){__builtin_amdgcn_alignbyte(w[1], w[0], m), __builtin_amdgcn_alignbyte(e, w[1], m)};
}

}  // namespace fhip
