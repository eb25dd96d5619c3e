// GLM-4.5 attention_pre_quant (the producer of the query / key / value rows of the paged GQA attention) - gfx950 kernels.
//
// Replaces the device side of attention_pre_quant (models/glm_v4_5/glm_attention_pre_quant.py:633-747; kernel
// quant_attention_pre_kernel :235-505), whose arithmetic is kept step by step:
//   s        = fp32(residual) + fp32(hidden_states);  residual_res = bf16(s)
//   x_norm   = bf16((s / sqrt(sum(s * s * (1 / h)) + eps)) * gamma + bias)                      (:361-386)
//   x_int8   = int8(saturate(rint(fp32(x_norm) * in_scale + in_offset)))                          (:389-396)
//   mm       = bf16(fp32(int32(x_int8 @ weight) + quant_bias) * deq_scale)                        (:398-403)
//   q | k | v = the first q_size, next kv_size, last kv_size outputs                              (:410-425)
//   q, k     = per head of 128: bf16((y / sqrt(sum(y * y / 128) + eps)) * norm_w + norm_b)       (:428-433, :188-218)
//              then on the head's first 2 * half dims (x1, x2): bf16(x1 cos - x2 sin), bf16(x2 cos + x1 sin)  (:446-490)
// Every product and sum above is a separately rounded fp32 operation (no contraction into fma).
//
// At decode sizes (8 - 64 tokens) the operator reads 9 MB of int8 weights once (hidden 5120 x 1792 outputs) and is bound by
// launch latency and that read; three launches:
//   apq_norm_kernel   one workgroup per token: the row is read once and stays in registers across the sum
//   apq_gemm_kernel   one workgroup per (128 outputs, 256 to 1024 contraction rows, 32 tokens): the weight tile (output
//                     dimension contiguous in memory) is loaded in one go, parked in LDS and read back with 8-bit
//                     transposing reads as the A operand of the int8 MFMA; int32 partial sums to the workspace (exact,
//                     so the split over the contraction changes nothing)
//   apq_head_kernel   one workgroup per (head, token): sum of the partials, bias, dequantisation, head norm, rotary
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>

#include "common.h"
#include "kernels.h"
#include "prolog_common.h"
#include "timing.h"

namespace pto {
namespace {

constexpr int AD = 128;      // head dim
constexpr int AK = 256;      // contraction rows per workgroup of apq_gemm_kernel
constexpr int AROW = 136;    // bytes per LDS row of the [256][128] int8 weight tile (padded, 8-byte aligned)
constexpr int ATOK = 32;     // tokens per workgroup of apq_gemm_kernel
constexpr int AMAX_H = 16384;

// sum over the 256 lanes of a workgroup in a fixed order; red is 4 floats of LDS
__device__ __forceinline__ float block_sum_256(float v, float* red, int tid)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    if ((tid & 63) == 0) red[tid >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

// ------------------------------------------------------------------------------------------------ residual + norm + quant
// grid (tokens), 256 lanes; lane l owns the 8-element pieces l, l + 256, ... of the row (NP of them at most)
template <int NP>
__global__ __launch_bounds__(256) void apq_norm_kernel(AttnPreArgs a)
{
#pragma clang fp contract(off)
    __shared__ float red[4];
    const int tok = blockIdx.x, tid = threadIdx.x;
    const int npieces = a.h / 8;
    const uint16_t* xrow = a.x + (int64_t)tok * a.h;
    const uint16_t* rrow = a.residual + (int64_t)tok * a.h;
    // every load of the kernel goes out before the first use (pieces past the row's end read its last piece again)
    u32x4 xr[NP], rr[NP], gr[NP], br[NP], sr[NP], fr[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int pc = min(tid + 256 * i, npieces - 1);
        xr[i] = reinterpret_cast<const u32x4*>(xrow)[pc];
        rr[i] = reinterpret_cast<const u32x4*>(rrow)[pc];
    }
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int pc = min(tid + 256 * i, npieces - 1);
        gr[i] = reinterpret_cast<const u32x4*>(a.gamma)[pc];
        br[i] = reinterpret_cast<const u32x4*>(a.bias)[pc];
        sr[i] = reinterpret_cast<const u32x4*>(a.in_scale)[pc];
        fr[i] = reinterpret_cast<const u32x4*>(a.in_offset)[pc];
    }
    float s[NP][8];
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const bool live = tid + 256 * i < npieces;
        u32x4 ro;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float lo = bf16_bits_to_f32(rr[i][e] & 0xffffu) + bf16_bits_to_f32(xr[i][e] & 0xffffu);
            const float hi = bf16_bits_to_f32(rr[i][e] >> 16) + bf16_bits_to_f32(xr[i][e] >> 16);
            s[i][2 * e] = lo;
            s[i][2 * e + 1] = hi;
            ro[e] = pack_bf16x2(lo, hi);
            if (live) {
                part += (lo * lo) * a.mean_coff;
                part += (hi * hi) * a.mean_coff;
            }
        }
        if (live) reinterpret_cast<u32x4*>(a.residual_out + (int64_t)tok * a.h)[tid + 256 * i] = ro;
    }
    const float denom = sqrtf(block_sum_256(part, red, tid) + a.eps);
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        if (tid + 256 * i >= npieces) continue;
        int8_t q[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int w = e >> 1, sh = (e & 1) * 16;
            const float g = bf16_bits_to_f32((gr[i][w] >> sh) & 0xffffu), b = bf16_bits_to_f32((br[i][w] >> sh) & 0xffffu);
            const float sc = bf16_bits_to_f32((sr[i][w] >> sh) & 0xffffu), of = bf16_bits_to_f32((fr[i][w] >> sh) & 0xffffu);
            const float xn = round_bf16((s[i][e] / denom) * g + b);
            const float v = __builtin_rintf(xn * sc + of);
            q[e] = (int8_t)(int)fminf(fmaxf(v, -128.f), 127.f);
        }
        *reinterpret_cast<u32x2*>(a.x_q + (int64_t)tok * a.h + 8 * (tid + 256 * i)) = __builtin_bit_cast(u32x2, q);
    }
}

// ------------------------------------------------------------------------------------------------ int8 projection
// grid (n_out / 128, splits of the contraction, token tiles of 32), 256 lanes: wave w owns outputs [32 w, 32 w + 32) of
// the tile.  A workgroup takes PER consecutive stages of 256 contraction rows (one where the grid would otherwise not
// fill the chip, more where there are workgroups to spare: fewer partial sums to write and to add up); every load of all
// its stages goes out before the first is used.
template <int PER>
__global__ __launch_bounds__(256) void apq_gemm_kernel(AttnPreArgs a)
{
    __shared__ __align__(16) uint8_t wl[AK * AROW];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int col0 = blockIdx.x * AD, split = blockIdx.y, tok0 = blockIdx.z * ATOK;
    const int stages = a.h / AK;
    // B operand (tokens): 16 contraction bytes per lane and MFMA, straight from the quantised rows
    i32x4 qf[PER][AK / 64][2];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int64_t kbase = (int64_t)min(split * PER + j, stages - 1) * AK; // past the end: the last stage again, dropped below
#pragma unroll
        for (int ks = 0; ks < AK / 64; ++ks)
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
                qf[j][ks][tb] = *reinterpret_cast<const i32x4*>(a.x_q + (int64_t)min(tok0 + 16 * tb + l16, a.t - 1) * a.h +
                                                                kbase + ks * 64 + 16 * g);
    }
    // the weight tiles: 256 rows of 128 bytes per stage, 16 bytes per lane and load
    const int srow = tid >> 3, spc = tid & 7;
    u32x4 stg[PER][AK / 32];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int64_t kbase = (int64_t)min(split * PER + j, stages - 1) * AK;
#pragma unroll
        for (int i = 0; i < AK / 32; ++i)
            stg[j][i] = *reinterpret_cast<const u32x4*>(a.w + (kbase + srow + 32 * i) * a.n_out + col0 + 16 * spc);
    }
    i32x4 acc[2][2];
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) acc[db][tb] = i32x4{0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        if (j > 0) __syncthreads();
#pragma unroll
        for (int i = 0; i < AK / 32; ++i) {
            u32x2* d = reinterpret_cast<u32x2*>(wl + (srow + 32 * i) * AROW + 16 * spc);
            d[0] = u32x2{stg[j][i][0], stg[j][i][1]};
            d[1] = u32x2{stg[j][i][2], stg[j][i][3]};
        }
        __syncthreads();
        if (split * PER + j >= stages) continue; // uniform over the workgroup
#pragma unroll
        for (int ks = 0; ks < AK / 64; ++ks) {
            // A operand: output 32 w + 16 db + l16, contraction bytes 16 g .. 16 g + 15 of the step.  An 8-bit transposing
            // read hands lane i of a 16-lane group byte i % 8 of the chunks addressed by lanes i / 8, i / 8 + 2, ...: with
            // lane i pointing at row i / 2, column half i % 2, lane i gets column i over rows 0 .. 7
            i32x4 wf[2];
#pragma unroll
            for (int db = 0; db < 2; ++db) {
                const uint8_t* p = wl + (ks * 64 + 16 * g + (l16 >> 1)) * AROW + 32 * wave + 16 * db + 8 * (l16 & 1);
                const v2i lo = lds_read_tr8(p), hi = lds_read_tr8(p + 8 * AROW);
                wf[db] = i32x4{lo[0], lo[1], hi[0], hi[1]};
            }
#pragma unroll
            for (int db = 0; db < 2; ++db)
#pragma unroll
                for (int tb = 0; tb < 2; ++tb)
                    acc[db][tb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[db], qf[j][ks][tb], acc[db][tb], 0, 0, 0);
        }
    }
    // register e of acc[db][tb]: output 32 w + 16 db + 4 g + e, token 16 tb + l16
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
        const int tok = tok0 + 16 * tb + l16;
        if (tok >= a.t) continue;
        int32_t* dst = a.part + ((int64_t)split * a.t + tok) * a.n_out + col0 + 32 * wave + 4 * g;
#pragma unroll
        for (int db = 0; db < 2; ++db) *reinterpret_cast<i32x4*>(dst + 16 * db) = acc[db][tb];
    }
}

// The projection at prefill sizes (128 tokens and more): a workgroup owns 128 tokens x 128 outputs over one split of
// the contraction and walks it in stages of 128 rows, both operands staged through LDS with the next stage's global
// loads in flight while the current stage is multiplied.  Wave (wr, wc) owns tokens [64 wr, +64) x outputs [64 wc, +64):
// every operand fragment read from LDS feeds four MFMAs, and the weights are read once per 128 tokens instead of once
// per 32.  Same int32 partial sums as apq_gemm_kernel (exact, so neither the tiling nor the split shows).
// grid (n_out / 128, splits, token tiles of 128), 256 lanes.
constexpr int BTOK = 128, BK = 128;
constexpr int BQROW = BK + 16; // bytes per LDS row of the [token][k] int8 tile (padded against bank conflicts)
__global__ __launch_bounds__(256, 3) void apq_gemm_big_kernel(AttnPreArgs a, int per)
{
    __shared__ __align__(16) uint8_t wl[BK * AROW];
    __shared__ __align__(16) uint8_t ql[BTOK * BQROW];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4, wr = wave >> 1, wc = wave & 1;
    const int col0 = blockIdx.x * AD, split = blockIdx.y, tok0 = blockIdx.z * BTOK;
    const int st0 = split * per, stages = min(a.h / BK, st0 + per) - st0; // this split's stages of 128 rows
    // 128 rows x 128 bytes of either operand per stage = 4 pieces of 16 bytes per lane (rows tid / 8 + 32 i, piece tid % 8)
    const int srow = tid >> 3, spc = tid & 7;
    const int8_t* wp = a.w + ((int64_t)st0 * BK + srow) * a.n_out + col0 + 16 * spc;
    const int8_t* qp[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) qp[i] = a.x_q + (int64_t)min(tok0 + srow + 32 * i, a.t - 1) * a.h + (int64_t)st0 * BK + 16 * spc;
    u32x4 wst[4], qst[4];
    auto load = [&](int st) {
#pragma unroll
        for (int i = 0; i < 4; ++i) qst[i] = *reinterpret_cast<const u32x4*>(qp[i] + st * BK);
#pragma unroll
        for (int i = 0; i < 4; ++i) wst[i] = *reinterpret_cast<const u32x4*>(wp + ((int64_t)st * BK + 32 * i) * a.n_out);
    };
    i32x4 acc[4][4]; // [db][tb]
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int tb = 0; tb < 4; ++tb) acc[db][tb] = i32x4{0, 0, 0, 0};
    load(0);
    for (int st = 0; st < stages; ++st) {
        __syncthreads(); // everyone is done with the previous stage's tiles
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            u32x2* d = reinterpret_cast<u32x2*>(wl + (srow + 32 * i) * AROW + 16 * spc);
            d[0] = u32x2{wst[i][0], wst[i][1]};
            d[1] = u32x2{wst[i][2], wst[i][3]};
            *reinterpret_cast<u32x4*>(ql + (srow + 32 * i) * BQROW + 16 * spc) = qst[i];
        }
        __syncthreads();
        load(min(st + 1, stages - 1)); // (unconditional: past the end the last stage is fetched again and dropped)
#pragma unroll
        for (int ks = 0; ks < BK / 64; ++ks) {
            i32x4 qf[4], wf[4];
#pragma unroll
            for (int tb = 0; tb < 4; ++tb)
                qf[tb] = *reinterpret_cast<const i32x4*>(ql + (64 * wr + 16 * tb + l16) * BQROW + ks * 64 + 16 * g);
            // (the byte-transposing read: see apq_gemm_kernel)
#pragma unroll
            for (int db = 0; db < 4; ++db) {
                const uint8_t* p = wl + (ks * 64 + 16 * g + (l16 >> 1)) * AROW + 64 * wc + 16 * db + 8 * (l16 & 1);
                const v2i lo = lds_read_tr8(p), hi = lds_read_tr8(p + 8 * AROW);
                wf[db] = i32x4{lo[0], lo[1], hi[0], hi[1]};
            }
#pragma unroll
            for (int db = 0; db < 4; ++db)
#pragma unroll
                for (int tb = 0; tb < 4; ++tb)
                    acc[db][tb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[db], qf[tb], acc[db][tb], 0, 0, 0);
        }
    }
    // register e of acc[db][tb]: output 64 wc + 16 db + 4 g + e, token 64 wr + 16 tb + l16
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) {
        const int tok = tok0 + 64 * wr + 16 * tb + l16;
        if (tok >= a.t) continue;
        int32_t* dst = a.part + ((int64_t)split * a.t + tok) * a.n_out + col0 + 64 * wc + 4 * g;
#pragma unroll
        for (int db = 0; db < 4; ++db) *reinterpret_cast<i32x4*>(dst + 16 * db) = acc[db][tb];
    }
}

// ------------------------------------------------------------------------------------------------ heads
// grid (q_heads + 2 kv_heads, tokens), 128 lanes: lane = dim of the head
__global__ __launch_bounds__(128) void apq_head_kernel(AttnPreArgs a)
{
#pragma clang fp contract(off)
    __shared__ float red[2];
    __shared__ float ys[AD];
    const int head = blockIdx.x, tok = blockIdx.y, dim = threadIdx.x;
    const int col = head * AD + dim;
    const bool is_q = head < a.q_heads, is_v = head >= a.q_heads + a.kv_heads;
    // what the epilogue reads goes out first
    const float deq = a.deq[col];
    const int32_t qb = a.qbias[col];
    const uint16_t* gp = is_q ? a.q_gamma : a.k_gamma;
    const uint16_t* bp = is_q ? a.q_bias : a.k_bias;
    const float gam = bf16_to_f32(gp[dim]), bia = bf16_to_f32(bp[dim]);
    const int rot = 2 * a.half;
    const int ci = dim < a.half ? dim : (dim < rot ? dim - a.half : 0);
    const float cs = bf16_to_f32(a.cos[(int64_t)tok * a.half + ci]), sn = bf16_to_f32(a.sin[(int64_t)tok * a.half + ci]);
    int32_t sum = 0;
    const int32_t* pp = a.part + (int64_t)tok * a.n_out + col;
    const int64_t pstride = (int64_t)a.t * a.n_out;
#pragma unroll 8
    for (int sidx = 0; sidx < a.ksplits; ++sidx) sum += pp[sidx * pstride];
    const float y = round_bf16((float)(sum + qb) * deq);
    if (is_v) {
        a.v[(int64_t)tok * a.kv_heads * AD + (head - a.q_heads - a.kv_heads) * AD + dim] = f32_to_bf16(y);
        return;
    }
    float m = (y * y) * (1.0f / AD);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m += __shfl_xor(m, o, 64);
    if ((dim & 63) == 0) red[dim >> 6] = m;
    __syncthreads();
    const float denom = sqrtf((red[0] + red[1]) + a.eps);
    const float yn = round_bf16((y / denom) * gam + bia);
    ys[dim] = yn;
    __syncthreads();
    float o = yn;
    if (dim < a.half) {
        o = yn * cs - ys[dim + a.half] * sn;
    } else if (dim < rot) {
        o = yn * cs + ys[dim - a.half] * sn;
    }
    uint16_t* dst = is_q ? a.q + ((int64_t)tok * a.q_heads + head) * AD : a.k + ((int64_t)tok * a.kv_heads + head - a.q_heads) * AD;
    dst[dim] = f32_to_bf16(o);
}

} // namespace

bool attention_pre_supported(int64_t h, int64_t d, int64_t half)
{
    return d == AD && h > 0 && h % AK == 0 && h <= AMAX_H && half >= 1 && 2 * half <= AD;
}

static uint64_t align256(uint64_t v) { return (v + 255) & ~(uint64_t)255; }

// stages of 256 contraction rows per workgroup of the projection: as many (1, 2 or 4) as still leave 448 workgroups
static int stages_per_split(int64_t t, int64_t h, int64_t n_out)
{
    const int64_t wgs = (n_out / AD) * (h / AK) * ((t + ATOK - 1) / ATOK);
    return wgs >= 8 * 448 ? 4 : wgs >= 2 * 448 ? 2 : 1;
}

// prefill sizes: stages of 128 rows per workgroup of apq_gemm_big_kernel - all of them while that still leaves
// 256 workgroups, otherwise as many as do
constexpr int BIG_T = 128;
static int big_stages_per_split(int64_t t, int64_t h, int64_t n_out)
{
    const int64_t tiles = (n_out / AD) * ((t + BTOK - 1) / BTOK), stages = h / BK;
    const int64_t splits = std::min<int64_t>(stages, std::max<int64_t>(1, (256 + tiles - 1) / tiles));
    return (int)((stages + splits - 1) / splits);
}

int attention_pre_ksplits(int64_t t, int64_t h, int64_t n_out)
{
    if (t >= BIG_T) {
        const int per = big_stages_per_split(t, h, n_out);
        return (int)((h / BK + per - 1) / per);
    }
    const int per = stages_per_split(t, h, n_out);
    return (int)((h / AK + per - 1) / per);
}

uint64_t attention_pre_workspace_bytes(int64_t t, int64_t h, int64_t n_out)
{
    return align256((uint64_t)t * h) + (uint64_t)attention_pre_ksplits(t, h, n_out) * t * n_out * sizeof(int32_t);
}

void attention_pre_bind_workspace(AttnPreArgs& a, void* ws)
{
    a.x_q = static_cast<int8_t*>(ws);
    a.part = reinterpret_cast<int32_t*>(static_cast<uint8_t*>(ws) + align256((uint64_t)a.t * a.h));
}

hipError_t attention_pre_launch(const AttnPreArgs& a, hipStream_t stream)
{
    if (a.t == 0) return hipSuccess;
    hipError_t e;
    {
        ScopedKernelTimer tm(KID_APQ_NORM, stream);
        if (a.h <= 3 * 2048)
            hipLaunchKernelGGL(apq_norm_kernel<3>, dim3(a.t), dim3(256), 0, stream, a);
        else
            hipLaunchKernelGGL(apq_norm_kernel<AMAX_H / 2048>, dim3(a.t), dim3(256), 0, stream, a);
    }
    if ((e = hipGetLastError()) != hipSuccess) return e;
    {
        ScopedKernelTimer tm(KID_APQ_GEMM, stream);
        const dim3 grid(a.n_out / AD, a.ksplits, (a.t + ATOK - 1) / ATOK);
        const int per = stages_per_split(a.t, a.h, a.n_out);
        if (a.ksplits != attention_pre_ksplits(a.t, a.h, a.n_out)) return hipErrorInvalidValue;
        if (a.t >= BIG_T)
            hipLaunchKernelGGL(apq_gemm_big_kernel, dim3(a.n_out / AD, a.ksplits, (a.t + BTOK - 1) / BTOK), dim3(256), 0, stream, a,
                               big_stages_per_split(a.t, a.h, a.n_out));
        else if (per == 4)
            hipLaunchKernelGGL(apq_gemm_kernel<4>, grid, dim3(256), 0, stream, a);
        else if (per == 2)
            hipLaunchKernelGGL(apq_gemm_kernel<2>, grid, dim3(256), 0, stream, a);
        else
            hipLaunchKernelGGL(apq_gemm_kernel<1>, grid, dim3(256), 0, stream, a);
    }
    if ((e = hipGetLastError()) != hipSuccess) return e;
    {
        ScopedKernelTimer tm(KID_APQ_HEAD, stream);
        hipLaunchKernelGGL(apq_head_kernel, dim3(a.q_heads + 2 * a.kv_heads, a.t), dim3(128), 0, stream, a);
    }
    return hipGetLastError();
}

} // namespace pto
