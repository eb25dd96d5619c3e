// Grouped expert selection (GLM-4.5 router): sigmoid, + bias, group maximum, top groups, top-k experts, renormalised
// weights.  Reference: models/glm_v4_5/glm_select_experts.py:60-228 (kernel) and :274-313 (golden);
// python/tests/ut/interpreter/_ops/moe_gating_topk.py:223-287 (groups, -inf fill, scaling factor).
//
// The whole problem is a few MB (8192 x 160 logits), so the kernel is bound by launch and memory latency, not by a
// roofline: one wavefront per token; groups are ranked by counting (rank of g = number of groups that come before g in
// the order "value descending, index ascending"), experts by top_k rounds of a wave-wide arg-max on 64-bit keys.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "common.h"
#include "kernels.h"
#include "timing.h"

namespace pto {
namespace {

constexpr int SE_MAX_NE = 256;
constexpr int SE_MAX_GROUPS = 64;
constexpr int SE_MAX_K = 32;

__device__ __forceinline__ float load_as_f32(const float* p, int64_t i) { return p[i]; }
__device__ __forceinline__ float load_as_f32(const uint16_t* p, int64_t i) { return __uint_as_float((uint32_t)p[i] << 16); }

// true when (v2, e2) comes before (v, e)
__device__ __forceinline__ int before(float v2, int e2, float v, int e) { return (v2 > v) || (v2 == v && e2 < e); }

template <typename LT, typename BT>
__global__ __launch_bounds__(64) void select_experts_kernel(SelectExpertsArgs a)
{
    __shared__ __align__(16) float s_sig[SE_MAX_NE];
    __shared__ __align__(16) float s_x[SE_MAX_NE];
    __shared__ float s_g[SE_MAX_GROUPS];
    __shared__ int s_keep[SE_MAX_GROUPS];
    __shared__ float s_w[SE_MAX_K];

    const int lane = threadIdx.x;
    const int ne = a.ne, ng = a.n_group, gs = ne / ng;
    const LT* logits = static_cast<const LT*>(a.logits);
    const BT* bias = static_cast<const BT*>(a.bias);
    const float fill = a.fill_neg_inf ? -__builtin_inff() : 0.0f;

    for (int64_t tok = blockIdx.x; tok < a.t; tok += gridDim.x) {
        float own_x[4], own_s[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = lane + 64 * j;
            own_x[j] = 0.f;
            own_s[j] = 0.f;
            if (e < ne) {
                const float x = load_as_f32(logits, tok * ne + e);
                // sigmoid in double, rounded once: the correctly rounded fp32 value whatever the libm
                const float sg = (float)(1.0 / (1.0 + exp(-(double)x)));
                own_s[j] = sg;
                own_x[j] = sg + load_as_f32(bias, e);
                s_sig[e] = sg;
                s_x[e] = own_x[j];
            }
        }
        __syncthreads();
        if (lane < ng) {
            float m = s_x[lane * gs];
            for (int i = 1; i < gs; ++i) m = fmaxf(m, s_x[lane * gs + i]);
            s_g[lane] = m;
        }
        __syncthreads();
        if (lane < ng) {
            const float m = s_g[lane];
            int rank = 0;
            for (int g2 = 0; g2 < ng; ++g2) rank += before(s_g[g2], g2, m, lane);
            s_keep[lane] = rank < a.topk_group;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = lane + 64 * j;
            if (e < ne && !s_keep[e / gs]) {
                own_x[j] = fill;
                s_x[e] = fill;
            }
        }
        __syncthreads();
        // top_k rounds of a wave-wide arg-max over 64-bit keys (ordered score << 32 | ~expert): the largest key is the
        // largest score and, among equal scores, the smallest expert id
        unsigned long long key[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = lane + 64 * j;
            key[j] = e < ne ? ((unsigned long long)f32_to_ordered(own_x[j] + 0.0f) << 32) | (uint32_t)(~e) : 0ull;
        }
        for (int r = 0; r < a.top_k; ++r) {
            unsigned long long best = key[0] > key[1] ? key[0] : key[1];
            const unsigned long long b2 = key[2] > key[3] ? key[2] : key[3];
            best = best > b2 ? best : b2;
#pragma unroll
            for (int sh = 1; sh < 64; sh <<= 1) {
                const unsigned long long o = __shfl_xor(best, sh);
                best = best > o ? best : o;
            }
            const int e = (int)~(uint32_t)best;
            if (lane == 0) {
                a.topk_ids[tok * a.top_k + r] = e;
                s_w[r] = s_sig[e];
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) key[j] = key[j] == best ? 0ull : key[j];
        }
        __syncthreads();
        if (lane < a.top_k) {
            float w = s_w[lane];
            if (a.renormalize) {
                float sum = 0.f;
                for (int i = 0; i < a.top_k; ++i) sum += s_w[i];
                w = w / sum;
            }
            a.topk_weights[tok * a.top_k + lane] = w * a.routed_scaling_factor;
        }
        __syncthreads();
    }
}

} // namespace

bool select_experts_supported(int ne, int n_group, int top_k)
{
    return ne > 0 && ne <= SE_MAX_NE && n_group > 0 && n_group <= SE_MAX_GROUPS && ne % n_group == 0 && top_k > 0 &&
           top_k <= SE_MAX_K && top_k <= ne;
}

hipError_t select_experts_launch(const SelectExpertsArgs& a, hipStream_t stream)
{
    if (a.t == 0) return hipSuccess;
    const int grid = (int)(a.t < 16384 ? a.t : 16384);
    ScopedKernelTimer timer(KID_SELECT_EXPERTS, stream);
    if (a.logits_bf16) {
        if (a.bias_bf16) hipLaunchKernelGGL((select_experts_kernel<uint16_t, uint16_t>), dim3(grid), dim3(64), 0, stream, a);
        else hipLaunchKernelGGL((select_experts_kernel<uint16_t, float>), dim3(grid), dim3(64), 0, stream, a);
    } else {
        if (a.bias_bf16) hipLaunchKernelGGL((select_experts_kernel<float, uint16_t>), dim3(grid), dim3(64), 0, stream, a);
        else hipLaunchKernelGGL((select_experts_kernel<float, float>), dim3(grid), dim3(64), 0, stream, a);
    }
    return hipGetLastError();
}

} // namespace pto
