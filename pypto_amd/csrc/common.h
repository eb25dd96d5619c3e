// Shared device/host helpers for the gfx950 kernels of libpypto_amd.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace pto {

// Host side: set-up that has to happen once on every device the library launches on (a kernel's attributes belong to
// the device its code object is loaded on).  f must be idempotent: two threads that arrive together both run it.
class DeviceOnce {
    std::atomic<uint64_t> done_{0}; // one bit per device ordinal
public:
    template <class F>
    hipError_t run(F&& f)
    {
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        const uint64_t bit = 1ull << (dev & 63);
        if (done_.load(std::memory_order_acquire) & bit) return hipSuccess;
        if ((e = f()) != hipSuccess) return e;
        done_.fetch_or(bit, std::memory_order_release);
        return hipSuccess;
    }
};

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Wavefront-wide maximum of non-negative or arbitrary floats, the same value in every lane, in the vector unit's own lane
// network (DPP row_shr steps inside the rows of 16 lanes, row_bcast15 / row_bcast31 across them) instead of six
// dependent permutes through LDS.  The maximum does not depend on the order, so the result is the butterfly's.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_from_f32(float v, float ident)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, ident), __builtin_bit_cast(int, v),
                                                                 CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float wave_max_f32(float v)
{
    const float lo = -__builtin_inff();
    v = fmaxf(v, dpp_from_f32<0x111, 0xf>(v, lo));
    v = fmaxf(v, dpp_from_f32<0x112, 0xf>(v, lo));
    v = fmaxf(v, dpp_from_f32<0x114, 0xf>(v, lo));
    v = fmaxf(v, dpp_from_f32<0x118, 0xf>(v, lo));
    v = fmaxf(v, dpp_from_f32<0x142, 0xa>(v, lo));
    v = fmaxf(v, dpp_from_f32<0x143, 0xc>(v, lo));
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Wavefront-wide sum, the same value in every lane, with the additions of the xor butterfly (partners 1, 2, 4, 8, 16, 32
// lanes away, in that order) but without its six dependent permutes through LDS.  After the first two steps (quad
// permutes) a quad's lanes hold the same value, so mirroring a half row pairs every lane with a lane that holds what
// its xor-4 partner holds; likewise the row mirror for xor 8; the two swaps exchange whole rows and half-waves.  a + b
// is b + a, so every lane adds the same two numbers as in the butterfly: the result is the butterfly's, bit for bit.
template <int CTRL>
__device__ __forceinline__ float dpp_perm_f32(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float wave_sum_butterfly(float v)
{
    v += dpp_perm_f32<0xB1>(v);  // quad_perm [1, 0, 3, 2]
    v += dpp_perm_f32<0x4E>(v);  // quad_perm [2, 3, 0, 1]
    v += dpp_perm_f32<0x141>(v); // row_half_mirror
    v += dpp_perm_f32<0x140>(v); // row_mirror
    {
        const auto sw = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned, v), __builtin_bit_cast(unsigned, v), false, false);
        v = __builtin_bit_cast(float, (unsigned)sw[0]) + __builtin_bit_cast(float, (unsigned)sw[1]);
    }
    {
        const auto sw = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, v), __builtin_bit_cast(unsigned, v), false, false);
        v = __builtin_bit_cast(float, (unsigned)sw[0]) + __builtin_bit_cast(float, (unsigned)sw[1]);
    }
    return v;
}

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
