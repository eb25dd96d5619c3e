// MLA prolog, int8 form (the producer of the query and of the paged int8 cache that sparse flash attention reads) -
// gfx950 kernels.
//
// Replaces the device side of mla_prolog_quant_d / mla_prolog_quant_p
// (models/deepseek_v32_exp/mla_prolog_quant_impl.py:364-727, entry points :745-951); arithmetic follows the operator
// (RmsNorm with its epsilon, :127-163) and otherwise the golden mla_prolog_quant_v32_compute
// (models/deepseek_v32_exp/deepseekv32_mla_prolog_quant.py:131-283):
//   q_a   = bf16(x @ w_dq);  q_rms = bf16(gamma_cq * (q_a / sqrt(mean(q_a^2) + eps)))
//   q_norm, q_norm_scale = int8 rint(q_rms * 127 / max|q_rms|), fp32 max|q_rms| / 127         (per token)
//   q_b   = bf16(int32(q_norm @ w_uq_qr) * q_norm_scale * w_qb_scale)                          [t, n, 192]
//   q_nope[t, head] = bf16(q_b[t, head, :128] @ w_uk[head])                                    [t, n, 512]
//   q_rope = rotary(q_b[t, head, 128:])  (interleaved pairs (2i, 2i+1) -> positions (i, 32+i))  [t, n, 64]
//   kv    = bf16(x @ w_dkv_kr) [t, 576];  k_rms = bf16 RmsNorm(kv[:, :512], gamma_ckv)
//   cache row cache_index[t]: four groups of 128 of k_rms quantised like q_norm (int8 + 4 fp32 scales), rotary(kv[:, 512:])
//
// At decode sizes the operator streams 85 MB of weights once (w_dq 22, w_uq_qr 38, w_uk 17, w_dkv_kr 8) and is bound
// by that read.  All four weight matrices are stored with the output dimension contiguous, the opposite of what the
// MFMA operands want (contraction contiguous per lane), so every weight tile goes through LDS and is read back
// transposed: bf16 tiles with ds_read_b64_tr_b16, the int8 tile with ds_read_b64_tr_b8.
//   mla_xa_kernel    x @ [w_dq | w_dkv_kr], 256 contraction rows x 128 outputs per workgroup, fp32 partials
//   mla_norm_kernel  one workgroup per token: fixed-order sum of the partials, both RmsNorms, the quantisations, the
//                    key's rotary embedding, the three cache writes, q_norm / q_norm_scale
//   mla_qb_kernel    int8 MFMA GEMM q_norm @ w_uq_qr, 128 outputs x 32 tokens per workgroup, weights double-buffered
//                    through LDS; dequantisation and the query's rotary embedding in registers
//   mla_wuk_kernel   per (head, 128 outputs): q_b[:, head, :128] @ w_uk[head]
#include <hip/hip_runtime.h>

#include <algorithm>
#include <stdint.h>

#include "common.h"
#include "kernels.h"
#include "prolog_common.h"
#include "prolog_device.h"
#include "timing.h"

namespace pto {
namespace {

constexpr int MTOK = 32;          // tokens per workgroup tile
constexpr int MNOPE = 128, MROPE = 64, MQH = MNOPE + MROPE, MC = 512, MKV = MC + MROPE;
constexpr int MAX_R = 2048;       // largest q_lora_rank (LDS of mla_norm_kernel, registers of mla_qb_kernel)
constexpr int XA_K = 256;         // contraction rows per stage of mla_xa_kernel
constexpr int XA_SPLIT = 1024;    // contraction rows per workgroup of mla_xa_kernel (one fp32 partial sum each)
constexpr int XROW2 = 64 * 2 + 16; // bytes per LDS row of a [k][64] bf16 weight tile (padded against bank conflicts)
constexpr int TROW = 128 * 2 + 32; // bytes per LDS row of a [k][128] bf16 weight tile (padded against bank conflicts)
constexpr int QB_K = 128;         // contraction rows per stage of mla_qb_kernel
constexpr int MQROW = 136;         // bytes per LDS row of a [k][128] int8 weight tile (padded, 8-byte aligned)
constexpr int QB_GROUPS = 4;      // wavefront quads of mla_qb_kernel, each with its own stages in flight
constexpr int QB_MAXS = MAX_R / QB_K / QB_GROUPS; // stages per group at the largest q_lora_rank
constexpr int QB_QP = MTOK * (MAX_R / 16) / 1024; // 16-byte pieces of the q_norm tile per lane at the largest q_lora_rank
constexpr int BIG_T = 128;        // token count from which the kernels that own an output tile take over
constexpr int BIG_T2 = 256;       // token count above which their tiles are 256 tokens tall
#ifndef XA_BIG2_DEPTH
#define XA_BIG2_DEPTH 2
#endif


// 32 outputs x 32 tokens += W[KSTEPS steps of 16 rows, outputs]^T . X[tokens, k]: A by transposing reads of the [k][n]
// tile in LDS, rows of ROWB bytes.  Lane jj of a 16-lane group points at row 8 hl + jj / 4 (+ 4 for the second read) of
// the step, columns 16 mh + 4 (jj & 3); a read hands lane i the column 16 mh + i over the four rows its group's lanes
// i / 4, i / 4 + 4, ... point at, so lane half hl ends up with the contraction rows 8 hl .. 8 hl + 7 of the step - and B
// takes the same rows of X with ONE 16-byte load per step (x[token][16 ks + 8 hl ..]: 32 bytes contiguous per token row
// and instruction; narrower pieces cost the texture addresser twice the cycles, and it is what bounds these loads:
// every lane pair reads a different row).  Register e of the result: output 8 (e / 4) + 4 hl + e % 4, token lane % 32.
// The B operand is loaded by its own call so that a caller can put these loads ahead of a prefetch in program order:
// memory operations complete in order, and a wait for loads issued after a prefetch would wait for the prefetch too.
template <int KSTEPS>
__device__ __forceinline__ void load_b_rows(u32x4 (&b)[KSTEPS], const uint16_t* xrow, int lane)
{
    const uint16_t* xp = xrow + (lane >> 5) * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) b[ks] = *reinterpret_cast<const u32x4*>(xp + ks * 16);
}
template <int KSTEPS, int ROWB>
__device__ __forceinline__ void gemm_tr_tile(f32x16& acc, const uint8_t* wtile, int ncol0, const u32x4 (&b)[KSTEPS], int lane)
{
    const int jj = lane & 15, mh = (lane >> 4) & 1, hl = lane >> 5;
    const uint8_t* hp = wtile + (8 * hl + (jj >> 2)) * ROWB + (ncol0 + 16 * mh + 4 * (jj & 3)) * 2;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        const s16x4 lo = lds_read_tr(hp + ks * 16 * ROWB);
        const s16x4 hi = lds_read_tr(hp + (ks * 16 + 4) * ROWB);
        const bf16x8 av = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, __builtin_bit_cast(bf16x8, b[ks]), acc, 0, 0, 0);
    }
}

// ------------------------------------------------------------------------------------------------ x @ [w_dq | w_dkv_kr]
// grid (ceil(h / 1024), output tiles of 64, token tiles of 32), 1024 lanes = 4 groups of 4 wavefronts.  Group g takes rows
// [256 g, 256 g + 256) of the workgroup's 1024 contraction rows: 256 rows x 64 outputs of weights, loaded in one go (every
// load of the workgroup is in flight at once - at decode sizes the kernel is a single pass over the weights and its
// duration is one memory latency plus the transfer), transposed through the group's LDS buffer.  Within a group wave w
// owns the 32 outputs of block w & 1 over rows [128 (w >> 1), + 128).  The eight partial sums of an output are added
// through LDS in a fixed order; fp32 partial sums per 1024-row split go to the workspace.
// x [t, ldx] (bf16) times the 64 output columns at src (row stride ld), contraction rows [split * 1024, ..) of kdim;
// the workgroup's fp32 partial sums go to part_out[(split * t + token) * ncols + col0 + ..]
__device__ __forceinline__ void xa_body(const uint16_t* x, int ldx, int kdim, const uint16_t* src, int ld, float* part_out,
                                        int ncols, int col0, int split, int tok0, int t, uint8_t* xa_lds)
{
    const int tid = threadIdx.x & 255, grp = threadIdx.x >> 8, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hl = lane >> 5;
    const int stages = min(XA_SPLIT, kdim - split * XA_SPLIT) / XA_K; // 256-row stages of this split (4 but for the last)
    const int sg = min(grp, stages - 1);                              // idle groups re-read the last stage and drop it
    const int64_t kbase = (int64_t)split * XA_SPLIT + sg * XA_K;
    uint8_t* wl = xa_lds + grp * (XA_K * XROW2);
    const int nb = wave & 1, kh = wave >> 1;
    // the B operand first, then the weights (memory operations complete in order)
    u32x4 bx[8];
    load_b_rows<8>(bx, x + (int64_t)min(tok0 + l32, t - 1) * ldx + kbase + 128 * kh, lane);
    // 256 rows x 128 bytes = 8 pieces of 16 bytes per lane (rows tid/8 + 32 i, piece tid%8)
    const int srow = tid >> 3, spc = tid & 7;
    const uint16_t* sp = src + (kbase + srow) * ld + 8 * spc;
    u32x4 stg[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) stg[i] = *reinterpret_cast<const u32x4*>(sp + (int64_t)(32 * i) * ld);
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4*>(wl + (srow + 32 * i) * XROW2 + 16 * spc) = stg[i];
    __syncthreads();
    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
    gemm_tr_tile<8, XROW2>(acc, wl + 128 * kh * XROW2, 32 * nb, bx, lane);
    __syncthreads();
    // partial sums of (group, row half) -> LDS; the two collecting waves add them in the order of the rows
    float* red = reinterpret_cast<float*>(xa_lds);
    const int part = 2 * grp + kh;
    if (part > 0 && grp < stages) {
#pragma unroll
        for (int e = 0; e < 16; ++e) red[((part * 2 + nb) * 16 + e) * 64 + lane] = acc[e];
    }
    __syncthreads();
    if (part > 0) return;
    for (int pp = 1; pp < 2 * stages; ++pp)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[e] += red[((pp * 2 + nb) * 16 + e) * 64 + lane];
    const int gt = tok0 + l32;
    if (gt < t) {
        float* out = part_out + ((int64_t)split * t + gt) * ncols + col0 + 32 * nb + 4 * hl;
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4)
            *reinterpret_cast<f32x4*>(out + 8 * e4) = f32x4{acc[4 * e4], acc[4 * e4 + 1], acc[4 * e4 + 2], acc[4 * e4 + 3]};
    }
}

// Output tile `tile` (64 columns) of x @ [w_dq | w_dkv_kr | w_k | w_proj]: its weight columns and their row stride.
__device__ __forceinline__ const uint16_t* xa_source(const MlaPrologArgs& a, int tile, int& ld)
{
    const int qtiles = a.r / 64;
    if (tile < qtiles) {
        ld = a.r;
        return a.w_dq + tile * 64;
    }
    if (tile < qtiles + MKV / 64) {
        ld = MKV;
        return a.w_dkv_kr + (tile - qtiles) * 64;
    }
    if (tile < qtiles + MKV / 64 + PD / 64) { // fused with the indexer prolog: its x @ [w_k | w_proj] rides along
        ld = PD;
        return a.w_k + (tile - qtiles - MKV / 64) * 64;
    }
    ld = a.n_idx;
    return a.w_proj + (tile - qtiles - MKV / 64 - PD / 64) * 64;
}

__global__ __launch_bounds__(1024) void mla_xa_kernel(MlaPrologArgs a)
{
    extern __shared__ __align__(16) uint8_t xa_lds[]; // [4 groups][256 k][64 n] bf16, rows of XROW2 bytes
    int ld;
    const uint16_t* src = xa_source(a, blockIdx.y, ld);
    xa_body(a.x, a.h, a.h, src, ld, a.xa_part, a.ncols, blockIdx.y * 64, blockIdx.x, blockIdx.z * MTOK, a.t, xa_lds);
}

// The same product at prefill sizes (128 tokens and more): a workgroup owns an output tile of 128 tokens x 64 columns
// over one 1024-row split of the contraction and walks it in stages of 64 rows, both operands staged through LDS, so
// that the weights are read once per 128 tokens instead of once per 32 and a token row's piece is fetched by 8
// neighbouring lanes as one 128-byte run.  The global loads of BG_DEPTH stages are in flight at any time (register
// sets used round-robin): a stage's multiplication takes a few hundred nanoseconds and a load comes back after one to
// two microseconds, so with one stage ahead the sixteen stages of a split were sixteen memory latencies in a row
// (29 us at 512 tokens with 256 x 64 tiles; a 256 x 128 tile that halves the operand traffic but leaves one
// workgroup per CU was slower still: 33 us).  Wave w owns tokens [32 w, +32) x the 64 columns.  x is the A operand here,
// so a result register holds one token's value for 32 consecutive columns across the lanes and the partial sums leave
// as 128-byte runs.  grid (splits, output tiles of 64, token tiles), 256 lanes.
constexpr int BG_KS = 64;               // contraction rows per stage
constexpr int BG_XROW = BG_KS * 2 + 16; // bytes per LDS row of the [token][k] tile (padded against bank conflicts)
// TB: blocks of 32 tokens per wave (the workgroup's tile is 128 TB tokens x 64 columns; with TB = 2 a weight fragment read
// from LDS feeds two MFMAs and the weights are read half as often, which is what counts once the token count is large
// enough for the kernel to be bound by what the CUs draw from the L2); DEPTH: stages whose loads are in flight.
template <int TB, int DEPTH>
__global__ __launch_bounds__(256, TB == 1 ? 3 : 2) void mla_xa_big_kernel(MlaPrologArgs a)
{
    constexpr int TOK = 128 * TB;
    static_assert((XA_SPLIT / BG_KS) % DEPTH == 0 && XA_K % (BG_KS * DEPTH) == 0, "whole rounds of stages in every split");
    __shared__ __align__(16) uint8_t wt[BG_KS * XROW2];
    __shared__ __align__(16) uint8_t xt[TOK * BG_XROW];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hl = lane >> 5, jj = lane & 15, mh = (lane >> 4) & 1;
    int ld;
    const uint16_t* src = xa_source(a, blockIdx.y, ld);
    const int split = blockIdx.x, tok0 = blockIdx.z * TOK, col0 = blockIdx.y * 64;
    const int kbeg = split * XA_SPLIT;
    const int stages = (min(a.h, kbeg + XA_SPLIT) - kbeg) / BG_KS; // a multiple of DEPTH (h is one of 256)
    const int srow = tid >> 3, spc = tid & 7;
    const uint16_t* xp[4 * TB];
#pragma unroll
    for (int i = 0; i < 4 * TB; ++i) xp[i] = a.x + (int64_t)min(tok0 + srow + 32 * i, a.t - 1) * a.h + kbeg + 8 * spc;
    const uint16_t* wp = src + (int64_t)(kbeg + srow) * ld + 8 * spc;
    u32x4 xs[DEPTH][4 * TB], ws[DEPTH][2];
    auto load = [&](int st, int u) {
#pragma unroll
        for (int i = 0; i < 4 * TB; ++i) xs[u][i] = *reinterpret_cast<const u32x4*>(xp[i] + st * BG_KS);
#pragma unroll
        for (int i = 0; i < 2; ++i) ws[u][i] = *reinterpret_cast<const u32x4*>(wp + (int64_t)(st * BG_KS + 32 * i) * ld);
    };
    f32x16 acc[TB][2];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[tb][nb][e] = 0.f;
    const uint8_t* xr = xt + (32 * TB * wave + l32) * BG_XROW + 16 * hl;
    const uint8_t* hp = wt + (8 * hl + (jj >> 2)) * XROW2 + (16 * mh + 4 * (jj & 3)) * 2;
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) load(u, u);
    for (int st0 = 0; st0 < stages; st0 += DEPTH) {
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            __syncthreads(); // everyone is done with the previous stage's tiles
#pragma unroll
            for (int i = 0; i < 4 * TB; ++i) *reinterpret_cast<u32x4*>(xt + (srow + 32 * i) * BG_XROW + 16 * spc) = xs[u][i];
#pragma unroll
            for (int i = 0; i < 2; ++i) *reinterpret_cast<u32x4*>(wt + (srow + 32 * i) * XROW2 + 16 * spc) = ws[u][i];
            __syncthreads();
            load(min(st0 + u + DEPTH, stages - 1), u); // (unconditional: past the end the last stage is fetched again and dropped)
#pragma unroll
            for (int ks = 0; ks < BG_KS / 16; ++ks) {
                bf16x8 xf[TB], wf[2];
#pragma unroll
                for (int tb = 0; tb < TB; ++tb) xf[tb] = *reinterpret_cast<const bf16x8*>(xr + 32 * tb * BG_XROW + ks * 32);
#pragma unroll
                for (int nb = 0; nb < 2; ++nb) {
                    const s16x4 lo = lds_read_tr(hp + 64 * nb + ks * 16 * XROW2);
                    const s16x4 hi = lds_read_tr(hp + 64 * nb + (ks * 16 + 4) * XROW2);
                    wf[nb] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                }
#pragma unroll
                for (int tb = 0; tb < TB; ++tb)
#pragma unroll
                    for (int nb = 0; nb < 2; ++nb)
                        acc[tb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xf[tb], wf[nb], acc[tb][nb], 0, 0, 0);
            }
        }
    }
    // register e of acc[tb][nb]: token 32 TB w + 32 tb + 8 (e / 4) + 4 hl + e % 4, column 32 nb + lane % 32
#pragma unroll
    for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int gt = tok0 + 32 * TB * wave + 32 * tb + 8 * (e >> 2) + 4 * hl + (e & 3);
            if (gt >= a.t) continue;
            float* out = a.xa_part + ((int64_t)split * a.t + gt) * a.ncols + col0 + l32;
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) out[32 * nb] = acc[tb][nb][e];
        }
}

// bf16 form of the operator: q_b = q_norm (bf16 [t, r]) @ w_uq_qr (bf16 [r, n * 192]) with the same kernel body;
// grid (ceil(r / 1024), n * 192 / 64, token tiles of 32); partial sums to qb_part
__global__ __launch_bounds__(1024) void mla_qb16_kernel(MlaPrologArgs a)
{
    extern __shared__ __align__(16) uint8_t xa_lds[];
    const int nq = a.n * MQH;
    xa_body(reinterpret_cast<const uint16_t*>(a.q_norm), a.r, a.r, reinterpret_cast<const uint16_t*>(a.w_uq_qr) + blockIdx.y * 64,
            nq, a.qb_part, nq, blockIdx.y * 64, blockIdx.x, blockIdx.z * MTOK, a.t, xa_lds);
}

// bf16 form: q_b = bf16(sum of the partial sums); its first 128 dims of a head to qb_nope, the last 64 through the rotary
// embedding to q_rope.  grid (tokens, n * 192 / 1024 rounded up), 256 lanes: four columns (two pairs) per lane
__global__ __launch_bounds__(256) void mla_qb16_epilogue_kernel(MlaPrologArgs a)
{
#pragma clang fp contract(off)
    const int tok = blockIdx.x, col = (blockIdx.y * 256 + threadIdx.x) * 4;
    const int nq = a.n * MQH, splits = (a.r + XA_SPLIT - 1) / XA_SPLIT;
    if (col >= nq) return;
    f32x4 acc = *reinterpret_cast<const f32x4*>(a.qb_part + (int64_t)tok * nq + col);
    for (int sp = 1; sp < splits; ++sp) acc += *reinterpret_cast<const f32x4*>(a.qb_part + ((int64_t)sp * a.t + tok) * nq + col);
    uint16_t vb[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) vb[e] = f32_to_bf16(acc[e]);
    const int head = col / MQH, d = col % MQH;
    if (d < MNOPE) {
        const u32x2 pk = {(uint32_t)vb[0] | ((uint32_t)vb[1] << 16), (uint32_t)vb[2] | ((uint32_t)vb[3] << 16)};
        *reinterpret_cast<u32x2*>(a.qb_nope + ((int64_t)tok * a.n + head) * MNOPE + d) = pk;
    } else {
        const uint16_t* cp = a.cos + (int64_t)tok * MROPE;
        const uint16_t* snp = a.sin + (int64_t)tok * MROPE;
        uint16_t* out = a.q_rope + ((int64_t)tok * a.n + head) * MROPE;
#pragma unroll
        for (int pr = 0; pr < 2; ++pr) {
            const int i = (d - MNOPE) / 2 + pr;
            const float xe = bf16_to_f32(vb[2 * pr]), xo = bf16_to_f32(vb[2 * pr + 1]);
            const float o1 = xe * bf16_to_f32(cp[i]) + (-xo) * bf16_to_f32(snp[i]);
            const float o2 = xo * bf16_to_f32(cp[i + 32]) + xe * bf16_to_f32(snp[i + 32]);
            out[i] = f32_to_bf16(o1);
            out[i + 32] = f32_to_bf16(o2);
        }
    }
}

// ------------------------------------------------------------------------------------------------ norms, quantisation, cache
__device__ __forceinline__ float wave_sum(float v) { return wave_sum_butterfly(v); }
__device__ __forceinline__ float wave_max(float v) { return wave_max_f32(v); }

// one workgroup of 256 lanes per token
__device__ __forceinline__ void mla_norm_body(const MlaPrologArgs& a, int tok)
{
#pragma clang fp contract(off)
    __shared__ float buf[MAX_R + MKV];
    __shared__ float red[8];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = a.r, ncols = r + MKV;
    // everything that does not depend on the sums is loaded first, so that its latency hides behind them
    const int64_t row = a.cache_index[tok];
    const bool row_ok = row >= 0 && row < a.cache_rows;
    constexpr int NQ = MAX_R / 256;
    uint16_t gq[NQ];
#pragma unroll
    for (int j = 0; j < NQ; ++j) gq[j] = 256 * j + tid < r ? a.gamma_cq[256 * j + tid] : (uint16_t)0;
    const uint16_t gk0 = a.gamma_ckv[tid], gk1 = a.gamma_ckv[256 + tid];
    const int ri = tid & 31;
    const float rc0 = bf16_to_f32(a.cos[(int64_t)tok * MROPE + ri]), rc1 = bf16_to_f32(a.cos[(int64_t)tok * MROPE + ri + 32]);
    const float rs0 = bf16_to_f32(a.sin[(int64_t)tok * MROPE + ri]), rs1 = bf16_to_f32(a.sin[(int64_t)tok * MROPE + ri + 32]);
    // q_a and kv: partial sums in a fixed order, rounded to bf16 (lane: columns tid + 256 j; all of a split's loads in
    // flight together)
    {
        constexpr int NJ = (MAX_R + MKV + 255) / 256;
        // every load is unconditional (columns past the end re-read the last one and are dropped below): a load under
        // a condition makes the compiler wait for it on the spot, one memory round trip per load
        int cj[NJ];
        float sum[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            cj[j] = min(256 * j + tid, ncols - 1);
            sum[j] = 0.f;
        }
        // four splits' loads in flight together (a split past the end re-reads the last one and adds zero)
        for (int s0 = 0; s0 < a.ksplits; s0 += 4) {
            float v[4][NJ];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float* p = a.xa_part + ((int64_t)min(s0 + i, a.ksplits - 1) * a.t + tok) * a.ncols;
#pragma unroll
                for (int j = 0; j < NJ; ++j) v[i][j] = p[cj[j]];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j) sum[j] += s0 + i < a.ksplits ? v[i][j] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j)
            if (256 * j + tid < ncols) buf[256 * j + tid] = round_bf16(sum[j]);
    }
    __syncthreads();
    // query: RmsNorm over r, then per-token quantisation
    {
        const float coff = 1.0f / (float)r;
        float ss = 0.f;
        for (int c = tid; c < r; c += 256) ss += (buf[c] * buf[c]) * coff;
        ss = wave_sum(ss);
        if (lane == 0) red[wave] = ss;
        __syncthreads();
        const float y = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) + a.eps_cq);
        float mx = 0.f;
#pragma unroll
        for (int j = 0; j < NQ; ++j) {
            const int c = 256 * j + tid;
            if (c < r) {
                const float v = round_bf16(bf16_to_f32(gq[j]) * (buf[c] * y));
                buf[c] = v;
                mx = fmaxf(mx, fabsf(v));
            }
        }
        mx = wave_max(mx);
        if (lane == 0) red[4 + wave] = mx;
        __syncthreads();
        mx = fmaxf(fmaxf(red[4], red[5]), fmaxf(red[6], red[7]));
        if (a.quant) {
            const float sq = quant_scale(mx);
            // four values per lane and store
            for (int c = 4 * tid; c < r; c += 1024) {
                uint32_t pk = 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) pk |= ((uint32_t)(int)__builtin_rintf(buf[c + e] * sq) & 0xffu) << (8 * e);
                *reinterpret_cast<uint32_t*>(a.q_norm + (int64_t)tok * r + c) = pk;
            }
            if (tid == 0) a.q_norm_scale[tok] = 1.0f / sq;
        } else { // bf16 form: q_norm is the normalised row itself
            uint16_t* qo = reinterpret_cast<uint16_t*>(a.q_norm) + (int64_t)tok * r;
            for (int c = 4 * tid; c < r; c += 1024)
                *reinterpret_cast<u32x2*>(qo + c) = u32x2{(uint32_t)f32_to_bf16(buf[c]) | ((uint32_t)f32_to_bf16(buf[c + 1]) << 16),
                                                          (uint32_t)f32_to_bf16(buf[c + 2]) | ((uint32_t)f32_to_bf16(buf[c + 3]) << 16)};
        }
    }
    __syncthreads();
    // key: RmsNorm over 512 (lane: elements tid and tid + 256), groups of 128 quantised on their own
    {
        const float x0 = buf[r + tid], x1 = buf[r + 256 + tid];
        float ss = wave_sum((x0 * x0) * (1.0f / MC) + (x1 * x1) * (1.0f / MC));
        if (lane == 0) red[wave] = ss;
        __syncthreads();
        const float y = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) + a.eps_ckv);
        const float v0 = round_bf16(bf16_to_f32(gk0) * (x0 * y));
        const float v1 = round_bf16(bf16_to_f32(gk1) * (x1 * y));
        // waves 0, 1 hold group 0 (v0) and group 2 (v1); waves 2, 3 groups 1 and 3
        const float m0 = wave_max(fabsf(v0)), m1 = wave_max(fabsf(v1));
        __syncthreads();
        if (lane == 0) {
            red[wave] = m0;
            red[4 + wave] = m1;
        }
        __syncthreads();
        const int pair = wave & 2;
        const float sq0 = quant_scale(fmaxf(red[pair], red[pair + 1]));
        const float sq1 = quant_scale(fmaxf(red[4 + pair], red[4 + pair + 1]));
        if (row_ok && a.quant) {
            a.kv_cache[row * MC + tid] = (int8_t)(int)__builtin_rintf(v0 * sq0);
            a.kv_cache[row * MC + 256 + tid] = (int8_t)(int)__builtin_rintf(v1 * sq1);
            if ((tid & 127) == 0) {
                a.k_scale_cache[row * 4 + (tid >> 7)] = 1.0f / sq0;
                a.k_scale_cache[row * 4 + 2 + (tid >> 7)] = 1.0f / sq1;
            }
        } else if (row_ok) { // bf16 form: the cache row is the normalised key itself, no scales
            uint16_t* kvo = reinterpret_cast<uint16_t*>(a.kv_cache) + row * MC;
            kvo[tid] = f32_to_bf16(v0);
            kvo[256 + tid] = f32_to_bf16(v1);
        }
    }
    // key rotary: pair i = elements (2i, 2i+1) -> positions (i, 32 + i)
    if (tid < MROPE / 2 && row_ok) {
        const float xe = buf[r + MC + 2 * tid], xo = buf[r + MC + 2 * tid + 1];
        const float o1 = xe * rc0 + (-xo) * rs0;
        const float o2 = xo * rc1 + xe * rs1;
        a.kr_cache[row * MROPE + tid] = f32_to_bf16(o1);
        a.kr_cache[row * MROPE + 32 + tid] = f32_to_bf16(o2);
    }
}

// ------------------------------------------------------------------------------------------------ q_norm @ w_uq_qr
// grid (n * 192 / 128, token tiles of 32), 1024 lanes = 4 groups of 4 wavefronts.  Group g takes the contraction stages
// g, g + 4, ... (128 rows x 128 outputs each) and issues the loads of all of them at once (registers), so that the
// whole tile of weights is in flight together; a stage then goes through the group's LDS buffer to be read back byte-
// transposed.  The token tile of q_norm sits in LDS (loaded ahead of the weights: memory operations complete in
// order).  Within a group wave w owns outputs [32 w, 32 w + 32) of the tile.  The groups' int32 sums are added through LDS
// at the end (exact, so the result does not depend on the split).
__host__ __device__ constexpr int mla_qb_lds_bytes(int r)
{
    return QB_GROUPS * QB_K * MQROW + MTOK * (r + 16) + 2 * MTOK * MROPE * 2;
}
// qb_lds: [QB_GROUPS][QB_K * MQROW] weights | [32][r + 16] q_norm | [2][32][64] cos, sin
__device__ __forceinline__ void mla_qb_body(const MlaPrologArgs& a, int col0, int tok0, uint8_t* qb_lds)
{
#pragma clang fp contract(off)
    const int tid = threadIdx.x & 255, grp = threadIdx.x >> 8, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int r = a.r, qrowb = r + 16; // padded against bank conflicts (r is a multiple of 128)
    const int64_t nq = (int64_t)a.n * MQH;
    uint8_t* wl = qb_lds + grp * (QB_K * MQROW);
    uint8_t* ql = qb_lds + QB_GROUPS * (QB_K * MQROW);
    uint16_t* csl = reinterpret_cast<uint16_t*>(ql + MTOK * qrowb); // [2][32][64]: the token tile's cos and sin rows

    // q_norm tile: 32 rows of r bytes, 16-byte pieces over the 1024 lanes (at most QB_QP per lane)
    const int qpieces = MTOK * (r / 16);
    u32x4 qst[QB_QP];
#pragma unroll
    for (int i = 0; i < QB_QP; ++i) {
        const int pc = min((int)threadIdx.x + 1024 * i, qpieces - 1);
        const int row = pc / (r / 16), c = pc % (r / 16);
        qst[i] = *reinterpret_cast<const u32x4*>(a.q_norm + (int64_t)min(tok0 + row, a.t - 1) * r + 16 * c);
    }
    // the token tile's cos / sin rows and scales for the epilogue: loaded now, so that the epilogue waits for nothing
    u32x4 cst = {0u, 0u, 0u, 0u};
    if (threadIdx.x < 512) {
        const int which = threadIdx.x >> 8, row = (threadIdx.x & 255) >> 3, c = threadIdx.x & 7;
        cst = *reinterpret_cast<const u32x4*>((which ? a.sin : a.cos) + (int64_t)min(tok0 + row, a.t - 1) * MROPE + 8 * c);
    }
    float qs_pre[2];
    f32x4 ws_pre[2];
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) qs_pre[tb] = a.q_norm_scale[min(tok0 + 16 * tb + l16, a.t - 1)];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) ws_pre[nb] = *reinterpret_cast<const f32x4*>(a.w_qb_scale + col0 + 32 * wave + 16 * nb + 4 * g);
    // weights: every stage of this group, 128 rows x 128 bytes = 4 pieces of 16 bytes per lane (rows tid/8 + 32 i, piece
    // tid%8); stages past the end re-read the last one and are dropped
    const int stages = r / QB_K;
    const int srow = tid >> 3, spc = tid & 7;
    const int8_t* sp = static_cast<const int8_t*>(a.w_uq_qr) + (int64_t)srow * nq + col0 + 16 * spc;
    u32x4 stg[QB_MAXS][4];
#pragma unroll
    for (int j = 0; j < QB_MAXS; ++j) {
        const int s = min(grp + QB_GROUPS * j, stages - 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) stg[j][i] = *reinterpret_cast<const u32x4*>(sp + ((int64_t)s * QB_K + 32 * i) * nq);
    }
#pragma unroll
    for (int i = 0; i < QB_QP; ++i) {
        const int pc = (int)threadIdx.x + 1024 * i;
        if (pc < qpieces) *reinterpret_cast<u32x4*>(ql + (pc / (r / 16)) * qrowb + 16 * (pc % (r / 16))) = qst[i];
    }
    if (threadIdx.x < 512) reinterpret_cast<u32x4*>(csl)[threadIdx.x] = cst;
    i32x4 acc[2][2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) acc[nb][tb] = i32x4{0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < QB_MAXS; ++j) {
        const int s = grp + QB_GROUPS * j;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            u32x2* d = reinterpret_cast<u32x2*>(wl + (srow + 32 * i) * MQROW + 16 * spc);
            d[0] = u32x2{stg[j][i][0], stg[j][i][1]};
            d[1] = u32x2{stg[j][i][2], stg[j][i][3]};
        }
        __syncthreads();
        if (s < stages) {
#pragma unroll
            for (int ks = 0; ks < QB_K / 64; ++ks) {
                i32x4 qf[2], wf[2];
#pragma unroll
                for (int tb = 0; tb < 2; ++tb)
                    qf[tb] = *reinterpret_cast<const i32x4*>(ql + (16 * tb + l16) * qrowb + s * QB_K + ks * 64 + 16 * g);
                // A operand: output 32 w + 16 nb + l16, contraction bytes 16 g .. 16 g + 15 of the step.  An 8-bit
                // transposing read hands lane i of a 16-lane group byte i % 8 of the chunks addressed by lanes
                // i / 8, i / 8 + 2, ..., i / 8 + 14: with lane i pointing at row i / 2, column half i % 2, lane i gets
                // output column i over rows 0 .. 7 - eight of its sixteen contraction bytes per read
#pragma unroll
                for (int nb = 0; nb < 2; ++nb) {
                    const uint8_t* p = wl + (ks * 64 + 16 * g + (l16 >> 1)) * MQROW + 32 * wave + 16 * nb + 8 * (l16 & 1);
                    const v2i lo = lds_read_tr8(p), hi = lds_read_tr8(p + 8 * MQROW);
                    wf[nb] = i32x4{lo[0], lo[1], hi[0], hi[1]};
                }
#pragma unroll
                for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                    for (int tb = 0; tb < 2; ++tb)
                        acc[nb][tb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[nb], qf[tb], acc[nb][tb], 0, 0, 0);
            }
        }
        __syncthreads();
    }
    // add the groups' sums: groups 1.. leave theirs in their own (now idle) first buffer, group 0 collects
    if (grp > 0) {
        i32x4* red = reinterpret_cast<i32x4*>(wl);
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int tb = 0; tb < 2; ++tb) red[(2 * nb + tb) * 256 + tid] = acc[nb][tb];
    }
    __syncthreads();
    if (grp > 0) return;
#pragma unroll
    for (int og = 1; og < QB_GROUPS; ++og) {
        const i32x4* red = reinterpret_cast<const i32x4*>(qb_lds + og * (QB_K * MQROW));
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int tb = 0; tb < 2; ++tb) acc[nb][tb] += red[(2 * nb + tb) * 256 + tid];
    }
    // register e of acc[nb][tb]: output col0 + 32 w + 16 nb + 4 g + e, token 16 tb + l16
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
        const int gt = tok0 + 16 * tb + l16;
        if (gt >= a.t) continue;
        const float qs = qs_pre[tb];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const int col = col0 + 32 * wave + 16 * nb + 4 * g;
            const int head = col / MQH, d = col % MQH;
            const f32x4 ws = ws_pre[nb];
            uint16_t vb[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) vb[e] = f32_to_bf16(((float)acc[nb][tb][e] * qs) * ws[e]);
            if (d < MNOPE) {
                const u32x2 pk = {(uint32_t)vb[0] | ((uint32_t)vb[1] << 16), (uint32_t)vb[2] | ((uint32_t)vb[3] << 16)};
                *reinterpret_cast<u32x2*>(a.qb_nope + ((int64_t)gt * a.n + head) * MNOPE + d) = pk;
            } else {
                const uint16_t* cp = csl + (16 * tb + l16) * MROPE;
                const uint16_t* snp = csl + (MTOK + 16 * tb + l16) * MROPE;
                uint16_t* out = a.q_rope + ((int64_t)gt * a.n + head) * MROPE;
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    const int i = (d - MNOPE) / 2 + pr;
                    const float xe = bf16_to_f32(vb[2 * pr]), xo = bf16_to_f32(vb[2 * pr + 1]);
                    const float o1 = xe * bf16_to_f32(cp[i]) + (-xo) * bf16_to_f32(snp[i]);
                    const float o2 = xo * bf16_to_f32(cp[i + 32]) + xe * bf16_to_f32(snp[i + 32]);
                    out[i] = f32_to_bf16(o1);
                    out[i + 32] = f32_to_bf16(o2);
                }
            }
        }
    }
}

// grid (tokens), 256 lanes
__global__ __launch_bounds__(256) void mla_norm_kernel(MlaPrologArgs a) { mla_norm_body(a, blockIdx.x); }

// grid (n * 192 / 128, token tiles of 32), 1024 lanes
__global__ __launch_bounds__(1024) void mla_qb_kernel(MlaPrologArgs a)
{
    extern __shared__ __align__(16) uint8_t qb_lds[];
    mla_qb_body(a, blockIdx.x * 128, blockIdx.y * MTOK, qb_lds);
}

// The same product at prefill sizes (128 tokens and more): a workgroup owns 128 tokens x 128 outputs and walks the
// contraction in stages of 128 rows, both operands staged through LDS with the next stage's global loads in flight.  Wave
// (wr, wc) owns tokens [64 wr, +64) x outputs [64 wc, +64): every operand fragment read from LDS feeds four MFMAs.  The
// int32 sums are exact, so the results are the bits of mla_qb_kernel's.  The outputs go through LDS (in place of the
// operand tiles, which are no longer needed) so that they leave as the 128-byte runs they are in memory - a 128-column
// tile holds two 64-column segments, each either half of a head's 128 first dims or a head's 64 rotary dims, rotated
// into place on the way.  grid (n * 192 / 128, token tiles of 128), 256 lanes.
constexpr int QG_TOK = 128, QG_K = 128;
constexpr int QG_QROW = QG_K + 16;       // bytes per LDS row of the [token][k] int8 tile (padded against bank conflicts)
constexpr int QG_OROW = 128 * 2 + 16;    // bytes per LDS row of the [token][128 outputs] bf16 tile
constexpr int QG_STAGE_BYTES = QG_K * MQROW + QG_TOK * QG_QROW;
static_assert(QG_TOK * QG_OROW <= QG_STAGE_BYTES, "the output tile takes the operand tiles' place");
// DEPTH: stages whose loads are in flight (register sets used round-robin).  One keeps the kernel at 158 registers, three
// workgroups to a CU - what the 768 workgroups of 512 tokens want; at 256 tokens and fewer the grid leaves at most two
// workgroups to a CU anyway, and the twelve stages of a tile are otherwise twelve memory latencies in a row.
template <int DEPTH>
__device__ __forceinline__ void mla_qb_big_body(const MlaPrologArgs& a, int col0, int tok0, uint8_t* stage_lds)
{
#pragma clang fp contract(off)
    // stage_lds: QG_STAGE_BYTES, [128 k][MQROW] weights | [128 tokens][QG_QROW] q_norm
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4, wr = wave >> 1, wc = wave & 1;
    const int r = a.r;
    const int64_t nq = (int64_t)a.n * MQH;
    uint8_t* wl = stage_lds;
    uint8_t* ql = stage_lds + QG_K * MQROW;
    const int stages = r / QG_K;
    // 128 rows x 128 bytes of either operand per stage = 4 pieces of 16 bytes per lane (rows tid / 8 + 32 i, piece tid % 8)
    const int srow = tid >> 3, spc = tid & 7;
    const int8_t* wp = static_cast<const int8_t*>(a.w_uq_qr) + (int64_t)srow * nq + col0 + 16 * spc;
    const int8_t* qp[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) qp[i] = a.q_norm + (int64_t)min(tok0 + srow + 32 * i, a.t - 1) * r + 16 * spc;
    u32x4 wst[DEPTH][4], qst[DEPTH][4];
    auto load = [&](int st, int u) {
#pragma unroll
        for (int i = 0; i < 4; ++i) qst[u][i] = *reinterpret_cast<const u32x4*>(qp[i] + st * QG_K);
#pragma unroll
        for (int i = 0; i < 4; ++i) wst[u][i] = *reinterpret_cast<const u32x4*>(wp + ((int64_t)st * QG_K + 32 * i) * nq);
    };
    // the epilogue's scales, requested first
    float qs_pre[4];
    f32x4 ws_pre[4];
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) qs_pre[tb] = a.q_norm_scale[min(tok0 + 64 * wr + 16 * tb + l16, a.t - 1)];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) ws_pre[nb] = *reinterpret_cast<const f32x4*>(a.w_qb_scale + col0 + 64 * wc + 16 * nb + 4 * g);
    i32x4 acc[4][4]; // [nb][tb]
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int tb = 0; tb < 4; ++tb) acc[nb][tb] = i32x4{0, 0, 0, 0};
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) load(min(u, stages - 1), u);
    for (int st0 = 0; st0 < stages; st0 += DEPTH) {
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            if (st0 + u < stages) { // (uniform over the workgroup)
                __syncthreads(); // everyone is done with the previous stage's tiles
    #pragma unroll
                for (int i = 0; i < 4; ++i) {
                    u32x2* d = reinterpret_cast<u32x2*>(wl + (srow + 32 * i) * MQROW + 16 * spc);
                    d[0] = u32x2{wst[u][i][0], wst[u][i][1]};
                    d[1] = u32x2{wst[u][i][2], wst[u][i][3]};
                    *reinterpret_cast<u32x4*>(ql + (srow + 32 * i) * QG_QROW + 16 * spc) = qst[u][i];
                }
                __syncthreads();
                load(min(st0 + u + DEPTH, stages - 1), u); // (unconditional: past the end the last stage is fetched again and dropped)
    #pragma unroll
                for (int ks = 0; ks < QG_K / 64; ++ks) {
                    i32x4 qf[4], wf[4];
    #pragma unroll
                    for (int tb = 0; tb < 4; ++tb)
                        qf[tb] = *reinterpret_cast<const i32x4*>(ql + (64 * wr + 16 * tb + l16) * QG_QROW + ks * 64 + 16 * g);
                    // (the byte-transposing read: see mla_qb_body)
    #pragma unroll
                    for (int nb = 0; nb < 4; ++nb) {
                        const uint8_t* p = wl + (ks * 64 + 16 * g + (l16 >> 1)) * MQROW + 64 * wc + 16 * nb + 8 * (l16 & 1);
                        const v2i lo = lds_read_tr8(p), hi = lds_read_tr8(p + 8 * MQROW);
                        wf[nb] = i32x4{lo[0], lo[1], hi[0], hi[1]};
                    }
    #pragma unroll
                    for (int nb = 0; nb < 4; ++nb)
    #pragma unroll
                        for (int tb = 0; tb < 4; ++tb)
                            acc[nb][tb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[nb], qf[tb], acc[nb][tb], 0, 0, 0);
                }
            }
        }
    }
    __syncthreads(); // the operand tiles are free: the output tile takes their place
    // register e of acc[nb][tb]: output col0 + 64 wc + 16 nb + 4 g + e, token 64 wr + 16 tb + l16
    uint8_t* ot = stage_lds;
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) {
        const int tl = 64 * wr + 16 * tb + l16;
        const float qs = qs_pre[tb];
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
            const int cl = 64 * wc + 16 * nb + 4 * g; // column inside the tile
            const int d = (col0 + cl) % MQH;
            const f32x4 ws = ws_pre[nb];
            uint16_t vb[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) vb[e] = f32_to_bf16(((float)acc[nb][tb][e] * qs) * ws[e]);
            if (d < MNOPE) {
                const u32x2 pk = {(uint32_t)vb[0] | ((uint32_t)vb[1] << 16), (uint32_t)vb[2] | ((uint32_t)vb[3] << 16)};
                *reinterpret_cast<u32x2*>(ot + tl * QG_OROW + cl * 2) = pk;
            } else {
                const int64_t gtc = (int64_t)min(tok0 + tl, a.t - 1) * MROPE;
                const uint16_t* cp = a.cos + gtc;
                const uint16_t* snp = a.sin + gtc;
                uint16_t* seg = reinterpret_cast<uint16_t*>(ot + tl * QG_OROW) + (cl - (d - MNOPE)); // the head's 64 rotary dims
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    const int i = (d - MNOPE) / 2 + pr;
                    const float xe = bf16_to_f32(vb[2 * pr]), xo = bf16_to_f32(vb[2 * pr + 1]);
                    const float o1 = xe * bf16_to_f32(cp[i]) + (-xo) * bf16_to_f32(snp[i]);
                    const float o2 = xo * bf16_to_f32(cp[i + 32]) + xe * bf16_to_f32(snp[i + 32]);
                    seg[i] = f32_to_bf16(o1);
                    seg[i + 32] = f32_to_bf16(o2);
                }
            }
        }
    }
    __syncthreads();
    // 128 tokens x 2 segments x 128 bytes = 8 pieces of 16 bytes per lane
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int pc = tid + 256 * i, tl = pc >> 4, sg = (pc >> 3) & 1, c = pc & 7;
        const int gt = tok0 + tl;
        if (gt >= a.t) continue;
        const int col = col0 + 64 * sg, head = col / MQH, d0 = col % MQH;
        uint16_t* dst = d0 < MNOPE ? a.qb_nope + ((int64_t)gt * a.n + head) * MNOPE + d0 : a.q_rope + ((int64_t)gt * a.n + head) * MROPE;
        *reinterpret_cast<u32x4*>(dst + 8 * c) = *reinterpret_cast<const u32x4*>(ot + tl * QG_OROW + (64 * sg + 8 * c) * 2);
    }
}

template <int DEPTH>
__global__ __launch_bounds__(256, DEPTH == 1 ? 3 : 2) void mla_qb_big_kernel(MlaPrologArgs a)
{
    __shared__ __align__(16) uint8_t stage_lds[QG_STAGE_BYTES];
    mla_qb_big_body<DEPTH>(a, blockIdx.x * 128, blockIdx.y * QG_TOK, stage_lds);
}

// ------------------------------------------------------------------------------------------------ fused with the indexer prolog
// The fused operator runs the two prologs' per-token kernels side by side in one launch, and likewise the two int8
// GEMMs on q_norm (192 + 64 workgroups at model sizes: one per compute unit); the indexer's x @ [w_k | w_proj] rides along
// in mla_xa_kernel as three more output tiles.
// grid (tokens, 2), 256 lanes: y = 0 the MLA norms and cache rows, y = 1 the indexer's key path and weights (128 lanes)
__global__ __launch_bounds__(256) void fused_norm_kernel(MlaPrologArgs m, PrologArgs p)
{
    if (blockIdx.y == 0) {
        mla_norm_body(m, blockIdx.x);
    } else {
        if (threadIdx.x >= 128) return; // the barriers inside are among the two remaining waves
        prolog_k_body(p, blockIdx.x);
    }
}

// grid (n * 192 / 128 + index heads, token tiles of 32), 1024 lanes
__global__ __launch_bounds__(1024) void fused_qb_kernel(MlaPrologArgs m, PrologArgs p)
{
    extern __shared__ __align__(16) uint8_t fq_lds[];
    const int nqb = m.n * MQH / 128;
    if ((int)blockIdx.x < nqb)
        mla_qb_body(m, blockIdx.x * 128, blockIdx.y * MTOK, fq_lds);
    else
        prolog_q_body(p, blockIdx.x - nqb, blockIdx.y * PTOK, fq_lds);
}

// The same pair at prefill sizes: both products per 128 tokens, side by side.  The indexer's epilogue sets the LDS (68 KB:
// two workgroups to a CU), so both run with three stages of loads in flight.
// grid (n * 192 / 128 + index heads, token tiles of 128), 256 lanes
__global__ __launch_bounds__(256, 2) void fused_qb_big_kernel(MlaPrologArgs m, PrologArgs p)
{
    static_assert(QB_LDS_BYTES >= QG_STAGE_BYTES && QB_TOK == QG_TOK, "one LDS block and one token tiling serve both bodies");
    __shared__ __align__(16) uint8_t lds[QB_LDS_BYTES];
    const int nqb = m.n * MQH / 128;
    if ((int)blockIdx.x < nqb)
        mla_qb_big_body<QB_DEPTH>(m, blockIdx.x * 128, blockIdx.y * QG_TOK, lds);
    else
        prolog_q_big_body<QB_DEPTH>(p, blockIdx.x - nqb, blockIdx.y * QB_TOK, lds);
}

// Above 256 tokens the two products are launches of their own again: the MLA product then fills the chip at three
// workgroups to a CU (one stage of loads in flight, 36 KB of LDS), which the shared launch's 68 KB would not allow.
// grid (index heads, token tiles of 128), 256 lanes
__global__ __launch_bounds__(256, 2) void fused_q_big_kernel(PrologArgs p)
{
    __shared__ __align__(16) uint8_t lds[QB_LDS_BYTES];
    prolog_q_big_body<QB_DEPTH>(p, blockIdx.x, blockIdx.y * QB_TOK, lds);
}

// ------------------------------------------------------------------------------------------------ q_b[:, head, :128] @ w_uk[head]
// grid (heads, 512 / 128, z), 256 lanes: wave w owns outputs [32 w, 32 w + 32) of the tile.  The head's 128 x 128 weight
// tile stays in LDS while the workgroup walks the token tiles z, z + gridDim.z, ... (one at decode sizes; at prefill
// sizes the weights are then read once per workgroup instead of once per token tile); the next tile's operand rows are
// requested before the current tile's products.  TB blocks of 32 tokens per tile: 1 at decode sizes; 2 at prefill
// sizes, where every weight fragment read from LDS then feeds two MFMAs.
template <int TB>
__global__ __launch_bounds__(256) void mla_wuk_kernel(MlaPrologArgs a)
{
    constexpr int WTOK = MTOK * TB;    // tokens per tile
    constexpr int OROW = 128 * 2 + 16; // bytes per LDS row of the WTOK x 128 bf16 output tile (padded)
    __shared__ __align__(16) uint8_t wl[MNOPE * TROW];
    __shared__ __align__(16) uint8_t bt[WTOK * OROW]; // the token tile's operand rows
    __shared__ __align__(16) uint8_t ot[WTOK * OROW]; // its outputs
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hl = lane >> 5;
    const int head = blockIdx.x, ct = blockIdx.y;
    const int ttiles = (a.t + WTOK - 1) / WTOK;
    const uint16_t* src = a.w_uk + (int64_t)head * MNOPE * MC + ct * 128;
    // a tile's operand rows: WTOK tokens x 256 bytes, fetched once by the workgroup in 16-byte pieces (16 lanes per row) and
    // handed to the waves through LDS - a wave loading its own operand would fetch a different row with every lane pair,
    // which costs the texture addresser a cycle per row and instruction, four times over for the four waves
    const int prow = tid >> 4, pcol = tid & 15;
    auto fetch = [&](u32x4 (&q)[2 * TB], int tt) {
#pragma unroll
        for (int i = 0; i < 2 * TB; ++i)
            q[i] = *reinterpret_cast<const u32x4*>(a.qb_nope + ((int64_t)min(tt * WTOK + prow + 16 * i, a.t - 1) * a.n + head) * MNOPE +
                                                   8 * pcol);
    };
    auto park = [&](const u32x4 (&q)[2 * TB]) {
#pragma unroll
        for (int i = 0; i < 2 * TB; ++i) *reinterpret_cast<u32x4*>(bt + (prow + 16 * i) * OROW + 16 * pcol) = q[i];
    };
    u32x4 q0[2 * TB];
    fetch(q0, blockIdx.z);
#pragma unroll
    for (int i = tid; i < MNOPE * 16; i += 256) {
        const int k = i >> 4, c = i & 15;
        *reinterpret_cast<u32x4*>(wl + k * TROW + c * 16) = *reinterpret_cast<const u32x4*>(src + (int64_t)k * MC + c * 8);
    }
    park(q0);
    __syncthreads();
    const int jj = lane & 15, mh = (lane >> 4) & 1;
    const uint8_t* hp = wl + (8 * hl + (jj >> 2)) * TROW + (32 * wave + 16 * mh + 4 * (jj & 3)) * 2;
    for (int tt = blockIdx.z; tt < ttiles; tt += gridDim.z) {
        // the rows of the tile after this one, if there is one (uniform over the workgroup)
        const bool more = tt + (int)gridDim.z < ttiles;
        u32x4 qn[2 * TB];
        if (more) fetch(qn, tt + gridDim.z);
        f32x16 acc[TB];
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[tb][e] = 0.f;
        // (the weight fragment by transposing reads: see gemm_tr_tile)
#pragma unroll
        for (int ks = 0; ks < MNOPE / 16; ++ks) {
            const s16x4 lo = lds_read_tr(hp + ks * 16 * TROW);
            const s16x4 hi = lds_read_tr(hp + (ks * 16 + 4) * TROW);
            const bf16x8 av = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
            for (int tb = 0; tb < TB; ++tb) {
                const bf16x8 bx = *reinterpret_cast<const bf16x8*>(bt + (32 * tb + l32) * OROW + (ks * 16 + 8 * hl) * 2);
                acc[tb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bx, acc[tb], 0, 0, 0);
            }
        }
        // through LDS, so that a token's 128 outputs leave as one 256-byte run (16 lanes x 16 bytes)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                const u32x2 pk = {(uint32_t)f32_to_bf16(acc[tb][4 * e4]) | ((uint32_t)f32_to_bf16(acc[tb][4 * e4 + 1]) << 16),
                                  (uint32_t)f32_to_bf16(acc[tb][4 * e4 + 2]) | ((uint32_t)f32_to_bf16(acc[tb][4 * e4 + 3]) << 16)};
                *reinterpret_cast<u32x2*>(ot + (32 * tb + l32) * OROW + (32 * wave + 8 * e4 + 4 * hl) * 2) = pk;
            }
        __syncthreads(); // outputs parked; every wave is done with the operand rows
#pragma unroll
        for (int i = 0; i < 2 * TB; ++i) {
            const int tok = prow + 16 * i;
            if (tt * WTOK + tok < a.t)
                *reinterpret_cast<u32x4*>(a.q_nope + ((int64_t)(tt * WTOK + tok) * a.n + head) * MC + ct * 128 + 8 * pcol) =
                    *reinterpret_cast<const u32x4*>(ot + tok * OROW + 16 * pcol);
        }
        if (more) park(qn);
        __syncthreads();
    }
}

} // namespace

bool mla_prolog_supported(int64_t h, int64_t r, int64_t n, int64_t d_nope, int64_t d_rope, int64_t c)
{
    return d_nope == MNOPE && d_rope == MROPE && c == MC && n > 0 && (n * MQH) % 128 == 0 && r > 0 && r % 128 == 0 &&
           r <= MAX_R && h > 0 && h % XA_K == 0;
}

static uint64_t up256(uint64_t x) { return (x + 255) & ~(uint64_t)255; }

static uint64_t xa_part_bytes(int64_t t, int64_t h, int64_t ncols)
{
    return up256((uint64_t)((h + XA_SPLIT - 1) / XA_SPLIT) * t * ncols * sizeof(float));
}

uint64_t mla_prolog_workspace_bytes(int64_t t, int64_t h, int64_t r, int64_t n, int64_t n_idx, bool quant)
{
    // bf16 form: also the partial sums of q_norm @ w_uq_qr
    return xa_part_bytes(t, h, r + MKV + (n_idx ? PD + n_idx : 0)) + up256((uint64_t)t * n * MNOPE * 2) +
           (quant ? 0 : xa_part_bytes(t, r, n * MQH));
}

void mla_prolog_bind_workspace(MlaPrologArgs& a, void* ws)
{
    uint8_t* p = static_cast<uint8_t*>(ws);
    a.xa_part = reinterpret_cast<float*>(p);
    p += xa_part_bytes(a.t, a.h, a.ncols);
    a.qb_nope = reinterpret_cast<uint16_t*>(p);
    p += up256((uint64_t)a.t * a.n * MNOPE * 2);
    a.qb_part = reinterpret_cast<float*>(p);
}

bool fused_prolog_supported(int64_t n_idx) { return n_idx % 64 == 0; }

void fused_prolog_bind(MlaPrologArgs& m, PrologArgs& p, void* ws)
{
    m.w_k = p.w_k;
    m.w_proj = p.w_proj;
    m.n_idx = p.n;
    m.ncols = m.r + MKV + PD + p.n;
    mla_prolog_bind_workspace(m, ws);
    p.xw_part = m.xa_part;
    p.xw_stride = m.ncols;
    p.xw_col0 = m.r + MKV;
    p.ksplits = m.ksplits;
}

static hipError_t set_lds_limits()
{
    static DeviceOnce once;
    return once.run([] {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(mla_xa_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           4 * XA_K * XROW2);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(mla_qb_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                mla_qb_lds_bytes(MAX_R));
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(mla_qb16_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                4 * XA_K * XROW2);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(fused_qb_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                mla_qb_lds_bytes(MAX_R) > prolog_q_lds_bytes(QMAX_R) ? mla_qb_lds_bytes(MAX_R) : prolog_q_lds_bytes(QMAX_R));
        return e;
    });
}

// p == nullptr: the MLA prolog on its own; otherwise the fused operator (m and p bound by fused_prolog_bind)
static hipError_t launch_prologs(const MlaPrologArgs& a, const PrologArgs* p, hipStream_t stream)
{
    if (a.t == 0) return hipSuccess;
    const int ttiles = (a.t + MTOK - 1) / MTOK;
    hipError_t e = set_lds_limits();
    if (e != hipSuccess) return e;
    const bool big = a.t >= BIG_T; // prefill sizes: the kernels that own an output tile
    {
        ScopedKernelTimer tm(KID_MLA_XA, stream);
        if (big)
            if (a.t <= BIG_T2)
                hipLaunchKernelGGL((mla_xa_big_kernel<1, 4>), dim3(a.ksplits, a.ncols / 64, (a.t + 127) / 128), dim3(256), 0, stream, a);
            else
                hipLaunchKernelGGL((mla_xa_big_kernel<2, XA_BIG2_DEPTH>), dim3(a.ksplits, a.ncols / 64, (a.t + 255) / 256), dim3(256), 0, stream, a);
        else
            hipLaunchKernelGGL(mla_xa_kernel, dim3(a.ksplits, a.ncols / 64, ttiles), dim3(1024), 4 * XA_K * XROW2, stream, a);
    }
    if ((e = hipGetLastError()) != hipSuccess) return e;
    {
        ScopedKernelTimer tm(KID_MLA_NORM, stream);
        if (p)
            hipLaunchKernelGGL(fused_norm_kernel, dim3(a.t, 2), dim3(256), 0, stream, a, *p);
        else
            hipLaunchKernelGGL(mla_norm_kernel, dim3(a.t), dim3(256), 0, stream, a);
    }
    if ((e = hipGetLastError()) != hipSuccess) return e;
    {
        ScopedKernelTimer tm(KID_MLA_QB, stream);
        if (!a.quant) {
            const int nq = a.n * MQH;
            hipLaunchKernelGGL(mla_qb16_kernel, dim3((a.r + XA_SPLIT - 1) / XA_SPLIT, nq / 64, ttiles), dim3(1024),
                               4 * XA_K * XROW2, stream, a);
            hipLaunchKernelGGL(mla_qb16_epilogue_kernel, dim3(a.t, (nq / 4 + 255) / 256), dim3(256), 0, stream, a);
        } else if (big) {
            const dim3 qgrid(a.n * MQH / 128, (a.t + QG_TOK - 1) / QG_TOK);
            if (p && a.t <= BIG_T2) {
                hipLaunchKernelGGL(fused_qb_big_kernel, dim3(qgrid.x + p->n, qgrid.y), dim3(256), 0, stream, a, *p);
            } else {
                if (a.t <= BIG_T2)
                    hipLaunchKernelGGL(mla_qb_big_kernel<3>, qgrid, dim3(256), 0, stream, a);
                else
                    hipLaunchKernelGGL(mla_qb_big_kernel<1>, qgrid, dim3(256), 0, stream, a);
                if (p) hipLaunchKernelGGL(fused_q_big_kernel, dim3(p->n, qgrid.y), dim3(256), 0, stream, *p);
            }
        } else if (p) {
            const int smem = mla_qb_lds_bytes(a.r) > prolog_q_lds_bytes(a.r) ? mla_qb_lds_bytes(a.r) : prolog_q_lds_bytes(a.r);
            hipLaunchKernelGGL(fused_qb_kernel, dim3(a.n * MQH / 128 + p->n, ttiles), dim3(1024), smem, stream, a, *p);
        } else {
            hipLaunchKernelGGL(mla_qb_kernel, dim3(a.n * MQH / 128, ttiles), dim3(1024), mla_qb_lds_bytes(a.r), stream, a);
        }
    }
    if ((e = hipGetLastError()) != hipSuccess) return e;
    {
        ScopedKernelTimer tm(KID_MLA_WUK, stream);
        // token tiles per workgroup: one while that leaves the grid at about a thousand workgroups or fewer, more beyond
        if (big) {
            const int wtiles = (a.t + 2 * MTOK - 1) / (2 * MTOK);
            const int zdim = std::min(wtiles, std::max(1, 1024 / (a.n * (MC / 128))));
            hipLaunchKernelGGL(mla_wuk_kernel<2>, dim3(a.n, MC / 128, zdim), dim3(256), 0, stream, a);
        } else {
            const int zdim = std::min(ttiles, std::max(1, 1024 / (a.n * (MC / 128))));
            hipLaunchKernelGGL(mla_wuk_kernel<1>, dim3(a.n, MC / 128, zdim), dim3(256), 0, stream, a);
        }
    }
    return hipGetLastError();
}

hipError_t mla_prolog_launch(const MlaPrologArgs& a, hipStream_t stream) { return launch_prologs(a, nullptr, stream); }

hipError_t fused_prolog_launch(const MlaPrologArgs& m, const PrologArgs& p, hipStream_t stream)
{
    return launch_prologs(m, &p, stream);
}

} // namespace pto
