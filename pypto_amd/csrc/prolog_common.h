// Device helpers shared by the prolog kernels (lightning-indexer prolog, MLA prolog).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "common.h"

namespace pto {
namespace {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
__device__ __forceinline__ s16x4 lds_read_tr(const uint8_t* p)
{
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)const_cast<uint8_t*>(p));
}
typedef int v2i __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) v2i lds_v2i;
__device__ __forceinline__ v2i lds_read_tr8(const uint8_t* p)
{
    return __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i*)const_cast<uint8_t*>(p));
}
__device__ __forceinline__ float bf16_to_f32(uint16_t v) { return __builtin_bit_cast(float, (uint32_t)v << 16); }
// The golden's "127 / max": torch evaluates scalar / tensor as reciprocal(tensor) * scalar, two roundings
__device__ __forceinline__ float quant_scale(float mx) { return (1.0f / mx) * 127.0f; }
__device__ __forceinline__ uint16_t f32_to_bf16(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
__device__ __forceinline__ float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }


} // namespace
} // namespace pto
