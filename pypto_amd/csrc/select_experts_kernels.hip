// Grouped expert selection (GLM-4.5 router): sigmoid, + bias, group maximum, top groups, top-k experts, renormalised
// weights.  Reference: models/glm_v4_5/glm_select_experts.py:60-228 (kernel) and :274-313 (golden);
// python/tests/ut/interpreter/_ops/moe_gating_topk.py:223-287 (groups, -inf fill, scaling factor).
//
// The whole problem is a few MB (8192 x 160 logits), so the kernel is bound by launch and memory latency, not by a
// roofline: one wavefront per token, the token's scores in LDS, ranks by counting (rank of e = number of experts that
// come before e in the order "value descending, index ascending"), which needs no sort network and is exact on ties.
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

    // pad the tail of the score array so that the 4-wide ranking loop never counts it
    for (int e = ne + lane; e < SE_MAX_NE; e += 64) s_x[e] = -__builtin_inff();

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
        int rank[4] = {0, 0, 0, 0};
        const int ne4 = (ne + 3) & ~3;
        for (int e2 = 0; e2 < ne4; e2 += 4) {
            const float4 v = *reinterpret_cast<const float4*>(&s_x[e2]);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int e = lane + 64 * j;
                rank[j] += before(v.x, e2, own_x[j], e) + before(v.y, e2 + 1, own_x[j], e) +
                           before(v.z, e2 + 2, own_x[j], e) + before(v.w, e2 + 3, own_x[j], e);
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = lane + 64 * j;
            if (e < ne && rank[j] < a.top_k) {
                a.topk_ids[tok * a.top_k + rank[j]] = e;
                s_w[rank[j]] = own_s[j];
            }
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
