// Lightning indexer (int8 index scores + top-k) - gfx950 kernels.
//
// Replaces the device side of lightning_indexer_decode_compute
// (models/deepseek_v32_exp/lightning_indexer_quant_impl.py:38-216); arithmetic follows the golden
// (models/deepseek_v32_exp/deepseekv32_lightning_indexer_quant.py:178-263):
//   w_scale[h] = fp16(q_scale[h] * weight[h])
//   y[h, n]    = fp16(relu(int32 dot(q[h], k[n])) * 2^-11)
//   score[n]   = (sum_h fp32(w_scale[h]) * fp32(y[h, n])) * fp32(k_scale[n])
//   top-k over score[0 : eff_seq), eff_seq = act_seq - (s1 - 1 - i); best first, equal scores by ascending
//   index (framework/src/interface/interpreter/calculator/calc_torch.cpp:2481-2494); unused slots = -1.
//
// indexer_score_kernel: v_mfma_i32_16x16x64_i8 with the query heads as rows (A, resident in registers)
// and 16 cached keys as columns (B, loaded from the paged cache straight in operand layout: lane l reads
// 16 bytes of key l%16).  The result has one key per lane, so the relu / fp16 rounding / weighted head sum
// is an in-lane chain over 16 accumulators and two cross-lane adds.  Scores go to a dense fp32 row per
// query token.
//
// indexer_topk_kernel: one workgroup per query token.  Three radix-select passes (11+11+10 bits of an
// order-preserving key) find the k-th largest key, a compaction pass collects the winners, a bitonic sort
// of (key, ~index) words orders them.
#include "common.h"
#include "kernels.h"
#include "timing.h"

namespace pto {
namespace {

constexpr int D = 128;          // index head dim
constexpr int CHUNK = 512;      // keys per workgroup of the score kernel
constexpr int MAX_K = 2048;     // top-k capacity

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }

// S1 query tokens of one sequence share every key fragment.
template <int S1, int NHB>
__global__ __launch_bounds__(256) void indexer_score_kernel(IndexerArgs a, int s1_base_stride)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int bi = blockIdx.y;
    const int sgrp = blockIdx.z; // group of S1 consecutive query tokens of the sequence
    const int L = a.act_seq[bi];
    const int tok_begin = blockIdx.x * CHUNK;
    if (tok_begin >= L) return;
    const int tok_end = min(L, tok_begin + CHUNK);
    const int row0 = bi * a.s1 + sgrp * S1;

    // A fragments: head hb*16 + l16, bytes 64*ks + 16*g .. +15
    i32x4 qf[S1][NHB][2];
    float wsc[S1][NHB][4]; // fp32(w_scale) of heads hb*16 + 4*g + r
#pragma unroll
    for (int s = 0; s < S1; ++s)
#pragma unroll
        for (int hb = 0; hb < NHB; ++hb) {
            const int8_t* qp = a.q + ((int64_t)(row0 + s) * a.nh + hb * 16 + l16) * D + 16 * g;
            qf[s][hb][0] = *reinterpret_cast<const i32x4*>(qp);
            qf[s][hb][1] = *reinterpret_cast<const i32x4*>(qp + 64);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t h = (int64_t)(row0 + s) * a.nh + hb * 16 + 4 * g + r;
                const _Float16 qs = __builtin_bit_cast(_Float16, a.q_scale[h]);
                const _Float16 w = __builtin_bit_cast(_Float16, a.weights[h]);
                wsc[s][hb][r] = (float)(_Float16)(qs * w); // one fp16 rounding
            }
        }

    for (int t0 = tok_begin + wave * 16; t0 < tok_end; t0 += 64) {
        const int tok = t0 + l16;
        const bool ok = tok < tok_end;
        int64_t krow = 0;
        if (ok) {
            const int page = a.block_table[(int64_t)bi * a.bt_stride + tok / a.block_size];
            krow = (int64_t)page * a.block_size + tok % a.block_size;
            if (page < 0 || page >= a.n_blocks) krow = -1;
        }
        i32x4 kf0 = {0, 0, 0, 0}, kf1 = {0, 0, 0, 0};
        float ksc = 0.f;
        if (ok && krow >= 0) {
            const int8_t* kp = a.k_cache + krow * D + 16 * g;
            kf0 = *reinterpret_cast<const i32x4*>(kp);
            kf1 = *reinterpret_cast<const i32x4*>(kp + 64);
            ksc = f16_bits_to_f32(a.k_scale[krow]);
        }
#pragma unroll
        for (int s = 0; s < S1; ++s) {
            float part = 0.f;
#pragma unroll
            for (int hb = 0; hb < NHB; ++hb) {
                i32x4 acc = {0, 0, 0, 0};
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(qf[s][hb][0], kf0, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(qf[s][hb][1], kf1, acc, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float x = (float)max(acc[r], 0) * (1.0f / 2048.0f);
                    const float y = (float)(_Float16)x;
                    part = __builtin_fmaf(wsc[s][hb][r], y, part);
                }
            }
            part += __shfl_xor(part, 16);
            part += __shfl_xor(part, 32);
            if (ok && g == 0) a.scores[(int64_t)(row0 + s) * a.score_stride + tok] = part * ksc;
        }
    }
}

__device__ __forceinline__ uint32_t score_key(float f) { return f32_to_ordered(f + 0.0f); } // -0 -> +0

__device__ __forceinline__ uint64_t make_cand(uint32_t key, int idx)
{
    return ((uint64_t)key << 32) | (uint32_t)(0xffffffffu - (uint32_t)idx);
}

// block-wide inclusive suffix sum over 1024 lanes (lane t gets sum of v[t..1023]); tmp holds 16 words
__device__ __forceinline__ uint32_t block_suffix_sum(uint32_t v, uint32_t* tmp)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t o = __shfl_down(v, d);
        if (lane + d < 64) v += o;
    }
    __syncthreads();
    if (lane == 0) tmp[wave] = v;
    __syncthreads();
    uint32_t add = 0;
    for (int w = wave + 1; w < 16; ++w) add += tmp[w];
    return v + add;
}

__global__ __launch_bounds__(1024) void indexer_topk_kernel(const float* __restrict__ scores, int score_stride,
                                                            const int32_t* __restrict__ act_seq, int s1, int k,
                                                            int32_t* __restrict__ out)
{
    __shared__ uint32_t hist[2048];
    __shared__ uint64_t cand[MAX_K];
    __shared__ uint32_t tmp[16];
    __shared__ uint32_t s_bin, s_krem, s_cnt_gt, s_cnt_eq, s_bin_count;

    const int tid = threadIdx.x;
    const int row = blockIdx.x;
    const int bi = row / s1, si = row - bi * s1;
    int n = act_seq[bi] - (s1 - 1 - si);
    n = min(max(n, 0), score_stride);
    const float* x = scores + (int64_t)row * score_stride;

    for (int i = tid; i < MAX_K; i += 1024) cand[i] = 0ull;
    __syncthreads();

    if (n <= k) {
        for (int i = tid; i < n; i += 1024) cand[i] = make_cand(score_key(x[i]), i);
    } else {
        uint32_t prefix = 0; // key bits already fixed (aligned to the top)
        uint32_t krem = (uint32_t)k;
        uint32_t eq_total = 0;
#pragma unroll 1
        for (int pass = 0; pass < 3; ++pass) {
            const int shift = pass == 0 ? 21 : (pass == 1 ? 10 : 0);
            const int bits = pass == 2 ? 10 : 11;
            const uint32_t mask = (1u << bits) - 1u;
            hist[tid] = 0;
            hist[tid + 1024] = 0;
            __syncthreads();
            for (int i = tid; i < n; i += 1024) {
                const uint32_t u = score_key(x[i]);
                const bool in = pass == 0 || (u >> (shift + bits)) == (prefix >> (shift + bits));
                if (in) atomicAdd(&hist[(u >> shift) & mask], 1u);
            }
            __syncthreads();
            // lane t owns bins 2t (low) and 2t+1 (high)
            const uint32_t h_lo = hist[2 * tid], h_hi = hist[2 * tid + 1];
            const uint32_t incl = block_suffix_sum(h_lo + h_hi, tmp);
            const uint32_t above_hi = incl - h_lo - h_hi; // elements in bins > 2t+1
            const uint32_t above_lo = above_hi + h_hi;     // elements in bins > 2t
            if (above_hi < krem && krem <= above_hi + h_hi) {
                s_bin = 2 * tid + 1;
                s_krem = krem - above_hi;
                s_bin_count = h_hi;
            } else if (above_lo < krem && krem <= above_lo + h_lo) {
                s_bin = 2 * tid;
                s_krem = krem - above_lo;
                s_bin_count = h_lo;
            }
            __syncthreads();
            prefix |= s_bin << shift;
            krem = s_krem;
            eq_total = s_bin_count;
            __syncthreads();
        }
        // prefix = k-th largest key; take every key above it and the krem smallest indices equal to it
        const uint32_t n_gt = (uint32_t)k - krem;
        if (tid == 0) {
            s_cnt_gt = 0;
            s_cnt_eq = 0;
        }
        __syncthreads();
        const bool take_all_eq = eq_total == krem;
        for (int i = tid; i < n; i += 1024) {
            const uint32_t u = score_key(x[i]);
            if (u > prefix) {
                cand[atomicAdd(&s_cnt_gt, 1u)] = make_cand(u, i);
            } else if (take_all_eq && u == prefix) {
                cand[n_gt + atomicAdd(&s_cnt_eq, 1u)] = make_cand(u, i);
            }
        }
        if (!take_all_eq) {
            // more ties than slots: walk the row in index order and keep the first krem of them
            uint32_t base = 0;
            for (int i0 = 0; i0 < n && base < krem; i0 += 1024) {
                const int i = i0 + tid;
                const bool eq = i < n && score_key(x[i]) == prefix;
                const uint64_t bal = __ballot(eq);
                const int lane = tid & 63, wave = tid >> 6;
                const uint32_t in_wave = __popcll(bal & ((1ull << lane) - 1ull));
                __syncthreads();
                if (lane == 0) tmp[wave] = __popcll(bal);
                __syncthreads();
                uint32_t before = 0, total = 0;
                for (int w = 0; w < 16; ++w) {
                    const uint32_t c = tmp[w];
                    before += w < wave ? c : 0;
                    total += c;
                }
                const uint32_t rank = base + before + in_wave;
                if (eq && rank < krem) cand[n_gt + rank] = make_cand(prefix, i);
                base += total;
            }
        }
    }
    __syncthreads();

    // bitonic sort, descending, 2048 words, two per lane
    for (int size = 2; size <= MAX_K; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            const int pos = 2 * tid - (tid & (stride - 1)); // lower index of the pair
            const bool desc = (pos & size) == 0;
            const uint64_t lo = cand[pos], hi = cand[pos + stride];
            if ((lo < hi) == desc) {
                cand[pos] = hi;
                cand[pos + stride] = lo;
            }
            __syncthreads();
        }
    }
    for (int j = tid; j < k; j += 1024)
        out[(int64_t)row * k + j] = (int32_t)(0xffffffffu - (uint32_t)(cand[j] & 0xffffffffull));
}

} // namespace

uint64_t indexer_workspace_bytes(int t, int max_ctx) { return (uint64_t)t * (uint64_t)max_ctx * sizeof(float); }

hipError_t indexer_launch(const IndexerArgs& a, hipStream_t stream)
{
    const int t = a.b * a.s1;
    if (t == 0) return hipSuccess;
    const int max_ctx = a.score_stride;
    const int chunks = (max_ctx + CHUNK - 1) / CHUNK;
    {
        ScopedKernelTimer tm(KID_INDEXER_SCORE, stream);
        if (a.s1 % 2 == 0) {
            hipLaunchKernelGGL((indexer_score_kernel<2, 4>), dim3(chunks, a.b, a.s1 / 2), dim3(256), 0, stream, a, 0);
        } else {
            hipLaunchKernelGGL((indexer_score_kernel<1, 4>), dim3(chunks, a.b, a.s1), dim3(256), 0, stream, a, 0);
        }
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    {
        ScopedKernelTimer tm(KID_INDEXER_TOPK, stream);
        hipLaunchKernelGGL(indexer_topk_kernel, dim3(t), dim3(1024), 0, stream, a.scores, a.score_stride, a.act_seq,
                           a.s1, a.k, a.topk_res);
    }
    return hipGetLastError();
}

} // namespace pto
