// Paged grouped-query decode attention for gfx950 (GLM-4.5 shape: 96 query heads, 8 KV heads, head dim 128, bf16).
// Reference: models/glm_v4_5/glm_attention.py:427-568 (ifa_func_kernel), golden ifa_flash_torch :1374-1483.
//
// The operator streams every cached K and V row of a sequence once (4096 bytes per token over all KV heads) and
// does 12 flop per byte, so it is bound by HBM bandwidth; the design goal is to keep enough 16-byte loads in flight
// and to touch every byte once.
//
// Grid: (KV chunk, KV head x 16-head sub-group, query token); 256 lanes = 4 wavefronts that free-run (no barrier in
// the main loop).  A wave owns every fourth 32-token sub-tile of the chunk (so the four waves together walk whole
// 128-token pages), prefetches the next sub-tile's K and V into registers while it works on the current one, and
// keeps its own online-softmax state (m, l, O); the four states are merged through LDS at the end and written either
// as the final bf16 rows (one chunk) or as fp32 partials that gqa_combine_kernel merges.
//
//   S^T[token, head] = K Q^T : v_mfma_f32_16x16x32_bf16, A = K rows loaded from global memory straight into the
//       operand layout (lane = token l%16, 8 dims at 8*(l/16) + 32*j), B = Q (resident, heads padded to 16).
//   O^T[dim, head] += V^T P~^T : A = V^T through a wave-private, XOR-swizzled LDS tile and ds_read_b64_tr_b16,
//       B = P~ rounded to bf16, which is exactly the register layout S^T comes out in (lane = head l%16, 4 tokens
//       per 16-token block), so P~ never leaves registers.  The contraction index is visited in the order
//       {4g..4g+3, 16+4g..16+4g+3} per lane group g on both operands.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "common.h"
#include "kernels.h"
#include "timing.h"

namespace pto {
namespace {

constexpr int GD = 128;      // head dim
constexpr int GSUB = 32;     // tokens per wave sub-tile
constexpr int GWAVES = 4;
constexpr int GROW = GD * 2; // bytes per staged V row
constexpr float LOG2E = 1.4426950408889634f;

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

__device__ __forceinline__ s16x4 lds_read_tr(uint8_t* p) { return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p); }

// byte offset inside a staged row of token t of 16-byte chunk c16: the 32-byte units of a row are XOR-ed with t % 8
__device__ __forceinline__ int vswz(int t, int c16) { return ((((c16 >> 1) ^ (t & 7)) << 5) | ((c16 & 1) << 4)); }

struct SubTile {
    u32x4 k[2][4]; // [16-token block][k-step]: 8 dims of this lane's token
    u32x4 v[8];    // row 4*i + l/16, 16-byte chunk l%16
};

__global__ __launch_bounds__(256, 2) void gqa_decode_kernel(GqaArgs a)
{
    __shared__ __align__(16) uint8_t lds[GWAVES * GSUB * GROW]; // V staging, later the merge buffer (4 x 16 x 128 fp32)
    __shared__ float s_ml[GWAVES][16][2];

    const int split = blockIdx.x;
    const int n2 = blockIdx.y / a.hsub, hs = blockIdx.y % a.hsub;
    const int tq = blockIdx.z;
    const int bi = tq / a.s1, si = tq - bi * a.s1;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;

    int cur = a.act_seq[bi] - (a.s1 - 1 - si);
    cur = cur < 0 ? 0 : cur;
    const int reach = a.bt_stride * a.block_size;
    cur = cur > reach ? reach : cur;
    const int start = split * a.chunk;
    const int end = (start + a.chunk < cur) ? start + a.chunk : cur;

    const int g = a.nq / a.nkv;
    uint16_t* out = static_cast<uint16_t*>(a.out);
    if (start >= end) {
        if (a.nsplit == 1) { // nothing to attend: the output rows are zero
            const int n = tid >> 4, hloc = hs * 16 + n;
            if (hloc < g) {
                const u32x4 z = {0u, 0u, 0u, 0u};
                *reinterpret_cast<u32x4*>(out + ((int64_t)tq * a.nq + n2 * g + hloc) * GD + (tid & 15) * 8) = z;
            }
        }
        return;
    }

    // Q fragment: B operand, lane = head r16 of this sub-group, dims 8*g4 + 32*j
    u32x4 qf[4];
    {
        const int hloc = hs * 16 + r16;
        const bool ok = hloc < g;
        const uint16_t* qp = static_cast<const uint16_t*>(a.q) + ((int64_t)tq * a.nq + n2 * g + (ok ? hloc : 0)) * GD;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            qf[j] = *reinterpret_cast<const u32x4*>(qp + 8 * (g4 + 4 * j));
            if (!ok) qf[j] = u32x4{0u, 0u, 0u, 0u};
        }
    }

    const uint8_t* kbase = static_cast<const uint8_t*>(a.k) + (int64_t)n2 * GROW;
    const uint8_t* vbase = static_cast<const uint8_t*>(a.v) + (int64_t)n2 * GROW;
    const int64_t row_pitch = (int64_t)a.nkv * GROW;
    const int32_t* bt = a.block_table + (int64_t)bi * a.bt_stride;
    uint8_t* myv = lds + w * (GSUB * GROW);

    const int nsub = (end - start + GSUB - 1) / GSUB;
    const float sc = a.softmax_scale * LOG2E;

    f32x4 o[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    // a sub-tile lies inside one page (block_size is a multiple of 32 and chunks start on multiples of 128)
    auto load = [&](int i, SubTile& t) {
        const int p0 = start + GSUB * i;
        const int page = p0 / a.block_size;
        int blk = __builtin_amdgcn_readfirstlane(bt[page]);
        blk = (blk < 0 || blk >= a.n_blocks) ? 0 : blk; // an unmapped page is masked in compute(); keep the loads in bounds
        const int64_t row0 = (int64_t)blk * a.block_size + (p0 - page * a.block_size);
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                t.k[tb][j] = *reinterpret_cast<const u32x4*>(kbase + (row0 + tb * 16 + r16) * row_pitch + (g4 + 4 * j) * 16);
#pragma unroll
        for (int i8 = 0; i8 < 8; ++i8)
            t.v[i8] = *reinterpret_cast<const u32x4*>(vbase + (row0 + 4 * i8 + g4) * row_pitch + r16 * 16);
    };

    auto compute = [&](int i, const SubTile& t) {
        const int p0 = start + GSUB * i;
        const int page = p0 / a.block_size;
        const int blk = __builtin_amdgcn_readfirstlane(bt[page]);
        const bool mapped = blk >= 0 && blk < a.n_blocks;
        f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, t.k[0][j]),
                                                         __builtin_bit_cast(bf16x8, qf[j]), s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, t.k[1][j]),
                                                         __builtin_bit_cast(bf16x8, qf[j]), s1, 0, 0, 0);
        }
        // stage V for the transposing reads while the scores are in flight
#pragma unroll
        for (int i8 = 0; i8 < 8; ++i8) {
            const int tv = 4 * i8 + g4;
            *reinterpret_cast<u32x4*>(myv + tv * GROW + vswz(tv, r16)) = t.v[i8];
        }
        float sv[8];
        float mt = -INFINITY;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const int tok = p0 + (r >> 2) * 16 + 4 * g4 + (r & 3);
            const float x = (r < 4 ? s0[r & 3] : s1[r & 3]) * sc;
            sv[r] = (tok < end && mapped) ? x : -INFINITY;
            mt = fmaxf(mt, sv[r]);
        }
        mt = fmaxf(mt, __shfl_xor(mt, 16));
        mt = fmaxf(mt, __shfl_xor(mt, 32));
        const float m_new = fmaxf(m_run, mt);
        const float mref = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = exp2f(m_run - mref);
        float p[8], psum = 0.f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            p[r] = exp2f(sv[r] - mref);
            psum += p[r];
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (__any(alpha != 1.f)) {
#pragma unroll
            for (int db = 0; db < 8; ++db) o[db] *= alpha;
        }
        const u32x4 pf = {pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]), pack_bf16x2(p[4], p[5]),
                          pack_bf16x2(p[6], p[7])};
        const int tok_lo = 4 * g4 + (r16 >> 2);
#pragma unroll
        for (int db = 0; db < 8; ++db) {
            const s16x4 lo = lds_read_tr(myv + tok_lo * GROW + ((db ^ (tok_lo & 7)) << 5) + (r16 & 3) * 8);
            const s16x4 hi = lds_read_tr(myv + (tok_lo + 16) * GROW + ((db ^ (tok_lo & 7)) << 5) + (r16 & 3) * 8);
            const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, both),
                                                            __builtin_bit_cast(bf16x8, pf), o[db], 0, 0, 0);
        }
    };

    if (w < nsub) {
        SubTile cur_t, nxt_t;
        int i = w;
        load(i, cur_t);
        for (; i + GWAVES < nsub; i += GWAVES) {
            load(i + GWAVES, nxt_t);
            compute(i, cur_t);
            cur_t = nxt_t;
        }
        compute(i, cur_t);
    }
    l_run += __shfl_xor(l_run, 16);
    l_run += __shfl_xor(l_run, 32);

    // merge the four waves
    __syncthreads();
    float* mo = reinterpret_cast<float*>(lds);
#pragma unroll
    for (int db = 0; db < 8; ++db)
        *reinterpret_cast<f32x4*>(mo + (w * 16 + r16) * GD + 16 * db + 4 * g4) = o[db];
    if (g4 == 0) {
        s_ml[w][r16][0] = m_run;
        s_ml[w][r16][1] = l_run;
    }
    __syncthreads();
    {
        const int n = tid >> 4, d0 = (tid & 15) * 8;
        const int hloc = hs * 16 + n;
        if (hloc >= g) return;
        float M = -INFINITY;
#pragma unroll
        for (int ww = 0; ww < GWAVES; ++ww) M = fmaxf(M, s_ml[ww][n][0]);
        float L = 0.f, acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (M > -INFINITY) {
#pragma unroll
            for (int ww = 0; ww < GWAVES; ++ww) {
                const float wgt = exp2f(s_ml[ww][n][0] - M);
                L += wgt * s_ml[ww][n][1];
                const f32x4 x0 = *reinterpret_cast<const f32x4*>(mo + (ww * 16 + n) * GD + d0);
                const f32x4 x1 = *reinterpret_cast<const f32x4*>(mo + (ww * 16 + n) * GD + d0 + 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc[e] += wgt * x0[e];
                    acc[4 + e] += wgt * x1[e];
                }
            }
        }
        const int64_t head_row = (int64_t)tq * a.nq + n2 * g + hloc;
        if (a.nsplit == 1) {
            const float inv = L > 0.f ? 1.f / L : 0.f;
            const u32x4 pk = {pack_bf16x2(acc[0] * inv, acc[1] * inv), pack_bf16x2(acc[2] * inv, acc[3] * inv),
                              pack_bf16x2(acc[4] * inv, acc[5] * inv), pack_bf16x2(acc[6] * inv, acc[7] * inv)};
            *reinterpret_cast<u32x4*>(out + head_row * GD + d0) = pk;
        } else {
            float* po = a.part_o + (head_row * a.nsplit + split) * GD + d0;
            *reinterpret_cast<f32x4*>(po) = f32x4{acc[0], acc[1], acc[2], acc[3]};
            *reinterpret_cast<f32x4*>(po + 4) = f32x4{acc[4], acc[5], acc[6], acc[7]};
            if ((tid & 15) == 0) {
                float* pm = a.part_ml + (head_row * a.nsplit + split) * 2;
                pm[0] = M;
                pm[1] = L;
            }
        }
    }
}

// One wave quarter (32 lanes x 4 dims) per head row: merges the chunks that hold tokens of this query token.
__global__ __launch_bounds__(128) void gqa_combine_kernel(GqaArgs a)
{
    const int64_t head_row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 5);
    if (head_row >= (int64_t)a.b * a.s1 * a.nq) return;
    const int d0 = (threadIdx.x & 31) * 4;
    const int tq = (int)(head_row / a.nq);
    const int bi = tq / a.s1, si = tq - bi * a.s1;
    int cur = a.act_seq[bi] - (a.s1 - 1 - si);
    cur = cur < 0 ? 0 : cur;
    const int reach = a.bt_stride * a.block_size;
    cur = cur > reach ? reach : cur;
    const int nvalid = (cur + a.chunk - 1) / a.chunk;
    const float* pm = a.part_ml + head_row * a.nsplit * 2;
    const float* po = a.part_o + head_row * a.nsplit * GD + d0;
    // eight chunks' loads in flight at a time (a chunk past the last valid one re-reads the last and is dropped): the
    // additions keep the order of the chunks
    constexpr int G = 8;
    float M = -INFINITY;
    for (int s0 = 0; s0 < nvalid; s0 += G) {
        float m[G];
#pragma unroll
        for (int j = 0; j < G; ++j) m[j] = pm[2 * min(s0 + j, nvalid - 1)];
#pragma unroll
        for (int j = 0; j < G; ++j) M = fmaxf(M, m[j]);
    }
    float L = 0.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    if (M > -INFINITY) {
        for (int s0 = 0; s0 < nvalid; s0 += G) {
            f32x4 v[G];
            float m[G], l[G];
#pragma unroll
            for (int j = 0; j < G; ++j) {
                const int s = min(s0 + j, nvalid - 1);
                m[j] = pm[2 * s];
                l[j] = pm[2 * s + 1];
                v[j] = *reinterpret_cast<const f32x4*>(po + (int64_t)s * GD);
            }
#pragma unroll
            for (int j = 0; j < G; ++j) {
                if (s0 + j < nvalid) {
                    const float wgt = exp2f(m[j] - M);
                    L += wgt * l[j];
                    acc += v[j] * wgt;
                }
            }
        }
    }
    const float inv = L > 0.f ? 1.f / L : 0.f;
    const u32x2 pk = {pack_bf16x2(acc[0] * inv, acc[1] * inv), pack_bf16x2(acc[2] * inv, acc[3] * inv)};
    *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(a.out) + head_row * GD + d0) = pk;
}

// attn_res <- 0 (cache without pages)
__global__ void gqa_zero_kernel(uint32_t* out, int64_t n_words)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_words) out[i] = 0u;
}

} // namespace

void gqa_pick_chunk(int max_ctx, int forced_chunk, int* chunk, int* nsplit)
{
    int c = forced_chunk > 0 ? (forced_chunk + 127) / 128 * 128 : 1024;
    int n = max_ctx > 0 ? (max_ctx + c - 1) / c : 1;
    if (forced_chunk <= 0 && n > 64) {
        c = ((max_ctx + 63) / 64 + 127) / 128 * 128;
        n = (max_ctx + c - 1) / c;
    }
    *chunk = c;
    *nsplit = n < 1 ? 1 : n;
}

uint64_t gqa_workspace_bytes(int64_t t, int nq, int nsplit)
{
    return nsplit > 1 ? (uint64_t)t * nq * nsplit * (GD + 2) * sizeof(float) : 0;
}

hipError_t gqa_launch(const GqaArgs& a, hipStream_t stream)
{
    const int64_t t = (int64_t)a.b * a.s1;
    if (t == 0 || a.nq == 0) return hipSuccess;
    if (a.n_blocks == 0) { // a cache without pages holds no token: every output row is zero (and no kernel reads the cache)
        const int64_t words = t * a.nq * 128 / 2;
        hipLaunchKernelGGL(gqa_zero_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream,
                           static_cast<uint32_t*>(a.out), words);
        return hipGetLastError();
    }
    {
        ScopedKernelTimer timer(KID_GQA_DECODE, stream);
        hipLaunchKernelGGL(gqa_decode_kernel, dim3(a.nsplit, a.nkv * a.hsub, (unsigned)t), dim3(256), 0, stream, a);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || a.nsplit == 1) return e;
    {
        ScopedKernelTimer timer(KID_GQA_COMBINE, stream);
        const int64_t rows = t * a.nq;
        hipLaunchKernelGGL(gqa_combine_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(128), 0, stream, a);
    }
    return hipGetLastError();
}

} // namespace pto
