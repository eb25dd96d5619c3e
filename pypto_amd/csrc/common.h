// Shared device/host helpers for the gfx950 kernels of libpypto_amd.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pto {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Two fp32 -> one dword holding two bf16 (round to nearest even), low half = a.
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b)
{
    bf16x2 v;
    v[0] = (__bf16)a;
    v[1] = (__bf16)b;
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __builtin_bit_cast(float, bits16 << 16); }

// Order-preserving map fp32 -> u32 (larger float <=> larger key).
__device__ __forceinline__ uint32_t f32_to_ordered(float f)
{
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

} // namespace pto
