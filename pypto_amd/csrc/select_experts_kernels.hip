// Grouped expert selection (GLM-4.5 router): sigmoid, + bias, group maximum, top groups, top-k experts, renormalised
// weights.  Reference: models/glm_v4_5/glm_select_experts.py:60-228 (kernel) and :274-313 (golden);
// python/tests/ut/interpreter/_ops/moe_gating_topk.py:223-287 (groups, -inf fill, scaling factor).
//
// The whole problem is a few MB (8192 x 160 logits): what bounds the kernels is vector instruction issue, more than half
// of it the double-precision sigmoid.  Groups are ranked by counting (rank of g = number of groups that come before g
// in the order "value descending, index ascending"), experts by top_k rounds of an arg-max on (ordered score, ~id).
// select_experts_rows_kernel puts four tokens in a wavefront (the router's shapes); select_experts_kernel, one token per
// wavefront, takes the shapes with more than 16 groups or 16 selected experts.
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

// Wavefront-wide maximum of a u32, the same value in every lane, in the vector unit's own lane network (DPP row_shr
// steps inside the rows of 16 lanes, row_bcast15 / row_bcast31 across them).
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t se_dpp_from(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, false);
}
__device__ __forceinline__ uint32_t se_wave_max(uint32_t v)
{
    v = max(v, se_dpp_from<0x111, 0xf>(v));
    v = max(v, se_dpp_from<0x112, 0xf>(v));
    v = max(v, se_dpp_from<0x114, 0xf>(v));
    v = max(v, se_dpp_from<0x118, 0xf>(v));
    v = max(v, se_dpp_from<0x142, 0xa>(v));
    v = max(v, se_dpp_from<0x143, 0xc>(v));
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}
__device__ __forceinline__ float ordered_to_f32(uint32_t k)
{
    return __builtin_bit_cast(float, (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// One wavefront per token, everything but the group maxima in registers: lane l holds experts l, l + 64, l + 128,
// l + 192.  Group maxima by LDS atomic maxima on order-preserving keys; group ranks by counting against the other groups'
// maxima read lane by lane (v_readlane); experts by top_k rounds of a wave-wide arg-max in two steps - the largest
// ordered score, then the smallest expert id among the lanes that hold it - both in the lane network (DPP), no trip
// through LDS.  The selected experts' sigmoid values are picked out of their owners' registers with v_readlane.
template <typename LT, typename BT>
__global__ __launch_bounds__(64) void select_experts_kernel(SelectExpertsArgs a)
{
    __shared__ uint32_t s_gkey[SE_MAX_GROUPS];

    const int lane = threadIdx.x;
    const int ne = a.ne, ng = a.n_group, gs = ne / ng;
    const LT* logits = static_cast<const LT*>(a.logits);
    const BT* bias = static_cast<const BT*>(a.bias);
    const float fill = a.fill_neg_inf ? -__builtin_inff() : 0.0f;
    // what does not depend on the token: this lane's experts' groups and bias
    int grp[4];
    float bs[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = lane + 64 * j;
        grp[j] = e < ne ? e / gs : 0;
        bs[j] = e < ne ? load_as_f32(bias, e) : 0.f;
    }

    for (int64_t tok = blockIdx.x; tok < a.t; tok += gridDim.x) {
        float own_x[4], own_s[4];
        if (lane < ng) s_gkey[lane] = 0u;
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
                own_x[j] = sg + bs[j];
            }
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (lane + 64 * j < ne) atomicMax(&s_gkey[grp[j]], f32_to_ordered(own_x[j]));
        __syncthreads();
        // lane g < ng: the maximum of group g, its rank among the groups (value descending, index ascending)
        const float m = ordered_to_f32(s_gkey[lane < ng ? lane : 0]);
        int rank = 0;
        for (int g2 = 0; g2 < ng; ++g2) {
            const float m2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, m), g2));
            rank += before(m2, g2, m, lane);
        }
        const uint64_t keep = __ballot(lane < ng && rank < a.topk_group);
        // ordered score and inverted id of this lane's experts (0 / 0 for the slots past the last expert and for the
        // experts already taken): the largest (score, ~id) is the largest score and, among equal scores, the smallest id
        uint32_t hi[4], lo[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = lane + 64 * j;
            if (!((keep >> grp[j]) & 1ull)) own_x[j] = fill;
            hi[j] = e < ne ? f32_to_ordered(own_x[j] + 0.0f) : 0u;
            lo[j] = e < ne ? (uint32_t)(~e) : 0u;
        }
        int my_id = 0;
        float my_w = 0.f, sum = 0.f;
        for (int r = 0; r < a.top_k; ++r) {
            const uint32_t hmax = se_wave_max(max(max(hi[0], hi[1]), max(hi[2], hi[3])));
            uint32_t cand = 0u;
#pragma unroll
            for (int j = 0; j < 4; ++j) cand = max(cand, hi[j] == hmax ? lo[j] : 0u);
            const uint32_t lmax = se_wave_max(cand);
            const int e = (int)~lmax;
            // the expert's sigmoid value sits in register e / 64 of lane e % 64
            const int ej = e >> 6;
            const float src = ej == 0 ? own_s[0] : ej == 1 ? own_s[1] : ej == 2 ? own_s[2] : own_s[3];
            const float w = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, src), e & 63));
            sum += w;
            if (lane == r) {
                my_id = e;
                my_w = w;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) hi[j] = (hi[j] == hmax && lo[j] == lmax) ? 0u : hi[j];
        }
        if (lane < a.top_k) {
            a.topk_ids[tok * a.top_k + lane] = my_id;
            const float w = a.renormalize ? my_w / sum : my_w;
            a.topk_weights[tok * a.top_k + lane] = w * a.routed_scaling_factor;
        }
        __syncthreads(); // the group maxima are cleared for the next token only after every lane has read them
    }
}

// The same selection with four tokens per wavefront, one per row of 16 lanes: lane c of a row holds experts c, c + 16,
// ... (NS of them), so no lane idles at 160 experts and every cross-lane step serves four tokens at once.  Reductions run
// inside the rows - a maximum by four rotations (row_ror 8, 4, 2, 1: every lane of the row ends up with it) - group ranks by
// rotating the row's group maxima past every lane.  For up to 16 groups and 16 selected experts (the router's shapes).
template <int N>
__device__ __forceinline__ uint32_t row_ror(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x120 + N, 0xf, 0xf, false);
}
__device__ __forceinline__ uint32_t row_max_u32(uint32_t v)
{
    v = max(v, row_ror<8>(v));
    v = max(v, row_ror<4>(v));
    v = max(v, row_ror<2>(v));
    v = max(v, row_ror<1>(v));
    return v;
}
template <int K>
__device__ __forceinline__ void rank_step(int& rank, float m, int c, int delta, int ng)
{
    if constexpr (K < 16) {
        const float m2 = __builtin_bit_cast(float, row_ror<K>(__builtin_bit_cast(uint32_t, m)));
        const int g2 = (c + K * delta) & 15; // the lane of the row the rotation brought here
        rank += (g2 < ng) & before(m2, g2, m, c);
        rank_step<K + 1>(rank, m, c, delta, ng);
    }
}

template <typename LT, typename BT, int NS>
__global__ __launch_bounds__(64) void select_experts_rows_kernel(SelectExpertsArgs a)
{
    __shared__ uint32_t s_gkey[4][16];

    const int lane = threadIdx.x, row = lane >> 4, c = lane & 15;
    const int ne = a.ne, ng = a.n_group, gs = ne / ng;
    const LT* logits = static_cast<const LT*>(a.logits);
    const BT* bias = static_cast<const BT*>(a.bias);
    const float fill = a.fill_neg_inf ? -__builtin_inff() : 0.0f;
    // which way row_ror turns, found out once: lane c receives lane (c + delta) & 15
    const int delta = ((int)row_ror<1>((uint32_t)c) - c) & 15;
    int grp[NS];
    float bs[NS];
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int e = c + 16 * j;
        grp[j] = e < ne ? e / gs : 0;
        bs[j] = e < ne ? load_as_f32(bias, e) : 0.f;
    }

    for (int64_t tok0 = (int64_t)blockIdx.x * 4; tok0 < a.t; tok0 += (int64_t)gridDim.x * 4) {
        const int64_t tok = tok0 + row;
        const bool live = tok < a.t;
        const int64_t tl = live ? tok : a.t - 1; // (rows past the last token work on the last one and store nothing)
        float own_x[NS], own_s[NS];
        if (c < ng) s_gkey[row][c] = 0u;
#pragma unroll
        for (int j = 0; j < NS; ++j) {
            const int e = c + 16 * j;
            own_x[j] = 0.f;
            own_s[j] = 0.f;
            if (e < ne) {
                const float x = load_as_f32(logits, tl * ne + e);
                // sigmoid in double, rounded once: the correctly rounded fp32 value whatever the libm
                const float sg = (float)(1.0 / (1.0 + exp(-(double)x)));
                own_s[j] = sg;
                own_x[j] = sg + bs[j];
            }
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < NS; ++j)
            if (c + 16 * j < ne) atomicMax(&s_gkey[row][grp[j]], f32_to_ordered(own_x[j]));
        __syncthreads();
        // lane g < ng of a row: the maximum of the token's group g and its rank (value descending, index ascending)
        const float m = ordered_to_f32(s_gkey[row][c < ng ? c : 0]);
        int rank = 0;
        rank_step<1>(rank, m, c, delta, ng);
        const uint64_t keep = __ballot(c < ng && rank < a.topk_group); // bit 16 row + g
        uint32_t hi[NS], lo[NS];
#pragma unroll
        for (int j = 0; j < NS; ++j) {
            const int e = c + 16 * j;
            if (!((keep >> (16 * row + grp[j])) & 1ull)) own_x[j] = fill;
            hi[j] = e < ne ? f32_to_ordered(own_x[j] + 0.0f) : 0u;
            lo[j] = e < ne ? (uint32_t)(~e) : 0u;
        }
        int my_id = 0;
        float my_w = 0.f, sum = 0.f;
        for (int r = 0; r < a.top_k; ++r) {
            uint32_t h = hi[0];
#pragma unroll
            for (int j = 1; j < NS; ++j) h = max(h, hi[j]);
            const uint32_t hmax = row_max_u32(h);
            uint32_t cand = 0u;
#pragma unroll
            for (int j = 0; j < NS; ++j) cand = max(cand, hi[j] == hmax ? lo[j] : 0u);
            const uint32_t lmax = row_max_u32(cand);
            // the winner's sigmoid value (positive, so its bits order like the value): only its owner offers it
            uint32_t wb = 0u;
#pragma unroll
            for (int j = 0; j < NS; ++j) {
                const bool win = hi[j] == hmax && lo[j] == lmax;
                wb = max(wb, win ? __builtin_bit_cast(uint32_t, own_s[j]) : 0u);
                hi[j] = win ? 0u : hi[j];
            }
            const float w = __builtin_bit_cast(float, row_max_u32(wb));
            sum += w;
            if (c == r) {
                my_id = (int)~lmax;
                my_w = w;
            }
        }
        if (live && c < a.top_k) {
            a.topk_ids[tok * a.top_k + c] = my_id;
            const float w = a.renormalize ? my_w / sum : my_w;
            a.topk_weights[tok * a.top_k + c] = w * a.routed_scaling_factor;
        }
        __syncthreads(); // the group maxima are cleared for the next tokens only after every lane has read them
    }
}

} // namespace

bool select_experts_supported(int ne, int n_group, int top_k)
{
    return ne > 0 && ne <= SE_MAX_NE && n_group > 0 && n_group <= SE_MAX_GROUPS && ne % n_group == 0 && top_k > 0 &&
           top_k <= SE_MAX_K && top_k <= ne;
}

template <typename LT, typename BT>
static void launch_typed(const SelectExpertsArgs& a, hipStream_t stream)
{
    if (a.n_group <= 16 && a.top_k <= 16) {
        const int64_t wgs = (a.t + 3) / 4;
        const int grid = (int)(wgs < 16384 ? wgs : 16384);
        if (a.ne <= 160)
            hipLaunchKernelGGL((select_experts_rows_kernel<LT, BT, 10>), dim3(grid), dim3(64), 0, stream, a);
        else
            hipLaunchKernelGGL((select_experts_rows_kernel<LT, BT, 16>), dim3(grid), dim3(64), 0, stream, a);
    } else {
        const int grid = (int)(a.t < 16384 ? a.t : 16384);
        hipLaunchKernelGGL((select_experts_kernel<LT, BT>), dim3(grid), dim3(64), 0, stream, a);
    }
}

hipError_t select_experts_launch(const SelectExpertsArgs& a, hipStream_t stream)
{
    if (a.t == 0) return hipSuccess;
    ScopedKernelTimer timer(KID_SELECT_EXPERTS, stream);
    if (a.logits_bf16) {
        if (a.bias_bf16) launch_typed<uint16_t, uint16_t>(a, stream);
        else launch_typed<uint16_t, float>(a, stream);
    } else {
        if (a.bias_bf16) launch_typed<float, uint16_t>(a, stream);
        else launch_typed<float, float>(a, stream);
    }
    return hipGetLastError();
}

} // namespace pto
