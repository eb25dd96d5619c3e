// Lightning-indexer prolog: device bodies of the query and the key kernels, shared by the operator's own kernels
// (prolog_kernels.hip) and by the fused MLA + indexer prolog (mla_prolog_kernels.hip).
#pragma once
#include "kernels.h"
#include "prolog_common.h"

namespace pto {
namespace {


constexpr int PD = 128;      // index head dim
constexpr int PROPE = 64;    // rotary dims
constexpr int PTOK = 32;     // tokens per workgroup tile
constexpr int XW_K = 256;    // contraction rows per workgroup of the x @ [w_k | w_proj] product
constexpr int XROW = PD * 2 + 16; // bytes per LDS row of the 32 x 128 bf16 tile (padded)
constexpr int QK = 128;      // contraction rows per stage of prolog_q_kernel
constexpr int QROW = 136;    // bytes per LDS row of a [k][128] int8 weight stage (padded, 8-byte aligned)
constexpr int QGROUPS = 4;   // wave groups of prolog_q_kernel, each with its own stages
constexpr int QMAX_R = 2048; // largest q_lora_rank
constexpr int QMAXS = QMAX_R / QK / QGROUPS;   // stages per group at the largest q_lora_rank
constexpr int QQP = PTOK * (QMAX_R / 16) / 1024; // 16-byte pieces of the q_norm tile per lane at the largest q_lora_rank

constexpr int QAUX = 2 * PTOK * PROPE * 2 + PD * 4 + PTOK * 4; // cos and sin rows of the token tile, w_qb_scale, q_norm_scale

__host__ __device__ constexpr int prolog_q_lds_bytes(int r) { return QGROUPS * QK * QROW + PTOK * (r + 16) + QAUX; }
static_assert(QGROUPS * QK * QROW >= PD * PD * 2 + PTOK * XROW + 4 * PTOK * 4, "the epilogue fits in the stage buffers");

// Rotary embedding of the first 64 dims of the 32 x 128 bf16 tile in LDS, fp32 arithmetic with every product and sum
// rounded (the golden's x * cos + rotate_half(x) * sin), back to bf16.  256 lanes: 4 (token, pair) items each.  csl is the
// tile's [2][32][64] cos and sin rows in LDS.
__device__ __forceinline__ void rope_tile(uint8_t* xt, const uint16_t* csl, int tid)
{
#pragma clang fp contract(off)
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int item = tid + 256 * it;
        const int tok = item >> 5, i = item & 31;
        uint16_t* row = reinterpret_cast<uint16_t*>(xt + tok * XROW);
        const uint16_t* cosp = csl + tok * PROPE;
        const uint16_t* sinp = csl + (PTOK + tok) * PROPE;
        const float x1 = bf16_to_f32(row[i]), x2 = bf16_to_f32(row[i + 32]);
        const float c1 = bf16_to_f32(cosp[i]), c2 = bf16_to_f32(cosp[i + 32]);
        const float s1 = bf16_to_f32(sinp[i]), s2 = bf16_to_f32(sinp[i + 32]);
        const float o1 = x1 * c1 + (-x2) * s1;
        const float o2 = x2 * c2 + x1 * s2;
        row[i] = f32_to_bf16(o1);
        row[i + 32] = f32_to_bf16(o2);
    }
}

// ------------------------------------------------------------------------------------------------ query path
// One workgroup of 1024 lanes = 4 groups of 4 wavefronts per (head, token tile of 32); plds is its dynamic LDS
// (prolog_q_lds_bytes).
__device__ __forceinline__ void prolog_q_body(const PrologArgs& a, int head, int tok0, uint8_t* plds)
{
    // LDS: [4 groups][QK x QROW] weight stages | [32][r + 16] q_norm tile | cos, sin rows and scales for the epilogue.
    // Once the GEMM is done the first region is
    // reused for hadamard_q [128][128] bf16, the head's bf16 tile [32][XROW] and the per-wave maxima.
    uint8_t* had = plds;
    uint8_t* xt = plds + PD * PD * 2;
    float(*smax)[PTOK] = reinterpret_cast<float(*)[PTOK]>(plds + PD * PD * 2 + PTOK * XROW);

    const int tid = threadIdx.x & 255, grp = threadIdx.x >> 8, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4, l32 = lane & 31, hl = lane >> 5;
    const int r = a.r, qrowb = r + 16;
    const int64_t nd = (int64_t)a.n * PD;
    uint8_t* wl = plds + grp * (QK * QROW);
    uint8_t* ql = plds + QGROUPS * (QK * QROW);
    uint8_t* aux = ql + PTOK * qrowb; // [2][32][64] bf16 cos, sin | [128] w_qb_scale | [32] q_norm_scale
    const uint16_t* csl = reinterpret_cast<const uint16_t*>(aux);
    const float* wsl = reinterpret_cast<const float*>(aux + 2 * PTOK * PROPE * 2);
    const float* qsl = wsl + PD;

    // loads in the order they are needed: hadamard_q (parked in registers until the GEMM is over), the q_norm tile,
    // then every weight stage of this group - all in flight together
    u32x4 hst[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) hst[i] = reinterpret_cast<const u32x4*>(a.had_q)[threadIdx.x + 1024 * i];
    const int qpieces = PTOK * (r / 16);
    u32x4 qst[QQP];
#pragma unroll
    for (int i = 0; i < QQP; ++i) {
        const int pc = min((int)threadIdx.x + 1024 * i, qpieces - 1);
        const int row = pc / (r / 16), c = pc % (r / 16);
        qst[i] = *reinterpret_cast<const u32x4*>(a.q_norm + (int64_t)min(tok0 + row, a.t - 1) * r + 16 * c);
    }
    // what the epilogue reads (rotary rows, scales): fetched now, so that it waits for nothing later
    // (every lane loads - a load under a condition would be waited for on the spot; lanes past 544 fetch piece 0 again)
    const int ai = threadIdx.x < 544 ? (int)threadIdx.x : 0;
    const uint8_t* ap = ai < 512 ? reinterpret_cast<const uint8_t*>((ai >> 8 ? a.sin : a.cos) +
                                                                     (int64_t)min(tok0 + ((ai & 255) >> 3), a.t - 1) * PROPE + 8 * (ai & 7))
                                 : reinterpret_cast<const uint8_t*>(a.w_qb_scale + (int64_t)head * PD + 4 * (ai - 512));
    const u32x4 ast = *reinterpret_cast<const u32x4*>(ap);
    const float qst1 = a.q_norm_scale[min(tok0 + (int)(threadIdx.x & 31), a.t - 1)];
    const int stages = r / QK;
    const int srow = tid >> 3, spc = tid & 7;
    const int8_t* sp = a.w_qb + (int64_t)srow * nd + head * PD + 16 * spc;
    u32x4 stg[QMAXS][4];
#pragma unroll
    for (int j = 0; j < QMAXS; ++j) {
        const int s = min(grp + QGROUPS * j, stages - 1); // past the end: the last stage again, dropped below
#pragma unroll
        for (int i = 0; i < 4; ++i) stg[j][i] = *reinterpret_cast<const u32x4*>(sp + ((int64_t)s * QK + 32 * i) * nd);
    }
#pragma unroll
    for (int i = 0; i < QQP; ++i) {
        const int pc = (int)threadIdx.x + 1024 * i;
        if (pc < qpieces) *reinterpret_cast<u32x4*>(ql + (pc / (r / 16)) * qrowb + 16 * (pc % (r / 16))) = qst[i];
    }
    if (threadIdx.x < 544) reinterpret_cast<u32x4*>(aux)[threadIdx.x] = ast;
    if (threadIdx.x < 32) reinterpret_cast<float*>(aux)[4 * 544 + threadIdx.x] = qst1;
    // C^T[dim, token] = W^T[dim, :] . q_norm[token, :]: wave w owns dims [32 w, 32 w + 32) x 32 tokens
    i32x4 acc[2][2];
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) acc[db][tb] = i32x4{0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < QMAXS; ++j) {
        const int s = grp + QGROUPS * j;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            u32x2* d = reinterpret_cast<u32x2*>(wl + (srow + 32 * i) * QROW + 16 * spc);
            d[0] = u32x2{stg[j][i][0], stg[j][i][1]};
            d[1] = u32x2{stg[j][i][2], stg[j][i][3]};
        }
        __syncthreads();
        if (s < stages) {
#pragma unroll
            for (int ks = 0; ks < QK / 64; ++ks) {
                i32x4 qf[2], wf[2];
#pragma unroll
                for (int tb = 0; tb < 2; ++tb)
                    qf[tb] = *reinterpret_cast<const i32x4*>(ql + (16 * tb + l16) * qrowb + s * QK + ks * 64 + 16 * g);
                // A operand: dim 32 w + 16 db + l16, contraction bytes 16 g .. 16 g + 15 of the step.  An 8-bit
                // transposing read hands lane i of a 16-lane group byte i % 8 of the chunks addressed by lanes
                // i / 8, i / 8 + 2, ..., i / 8 + 14: with lane i pointing at row i / 2, column half i % 2, lane i gets
                // column i over rows 0 .. 7 - eight of its sixteen contraction bytes per read
#pragma unroll
                for (int db = 0; db < 2; ++db) {
                    const uint8_t* p = wl + (ks * 64 + 16 * g + (l16 >> 1)) * QROW + 32 * wave + 16 * db + 8 * (l16 & 1);
                    const v2i lo = lds_read_tr8(p), hi = lds_read_tr8(p + 8 * QROW);
                    wf[db] = i32x4{lo[0], lo[1], hi[0], hi[1]};
                }
#pragma unroll
                for (int db = 0; db < 2; ++db)
#pragma unroll
                    for (int tb = 0; tb < 2; ++tb)
                        acc[db][tb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[db], qf[tb], acc[db][tb], 0, 0, 0);
            }
        }
        __syncthreads();
    }
    // add the groups' int32 sums (exact): groups 1.. leave theirs in their own stage buffer, group 0 collects
    if (grp > 0) {
        i32x4* red = reinterpret_cast<i32x4*>(wl);
#pragma unroll
        for (int db = 0; db < 2; ++db)
#pragma unroll
            for (int tb = 0; tb < 2; ++tb) red[(2 * db + tb) * 256 + tid] = acc[db][tb];
    }
    __syncthreads();
    if (grp == 0) {
#pragma unroll
        for (int og = 1; og < QGROUPS; ++og) {
            const i32x4* red = reinterpret_cast<const i32x4*>(plds + og * (QK * QROW));
#pragma unroll
            for (int db = 0; db < 2; ++db)
#pragma unroll
                for (int tb = 0; tb < 2; ++tb) acc[db][tb] += red[(2 * db + tb) * 256 + tid];
        }
    }
    __syncthreads();
    // the stage buffers are free now: hadamard_q moves in
#pragma unroll
    for (int i = 0; i < 2; ++i) reinterpret_cast<u32x4*>(had)[threadIdx.x + 1024 * i] = hst[i];
    __syncthreads();
    if (grp > 0) return; // the barriers below are among the first group's waves (a finished wave does not count)
    // register e of acc[db][tb]: dim 32 w + 16 db + 4 g + e, token 16 tb + l16
    {
#pragma clang fp contract(off)
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) {
            const int tok = 16 * tb + l16;
            const float qs = qsl[tok];
#pragma unroll
            for (int db = 0; db < 2; ++db) {
                const int dim = 32 * wave + 16 * db + 4 * g;
                const f32x4 ws = *reinterpret_cast<const f32x4*>(wsl + dim);
                uint16_t* dst = reinterpret_cast<uint16_t*>(xt + tok * XROW) + dim;
#pragma unroll
                for (int e = 0; e < 4; ++e) dst[e] = f32_to_bf16(((float)acc[db][tb][e] * qs) * ws[e]);
            }
        }
    }
    __syncthreads();
    rope_tile(xt, csl, tid);
    __syncthreads();

    // Y^T[n, token] = H^T[n, k] . X^T[k, token]: wave w owns n in [32 w, 32 w + 32).  A (H^T) by transposing reads of
    // the row-major H: lane jj of 16-lane group G points at row k0 + 4*hl + jj/4 (+ 8), columns 32 w + 16 (G&1) + 4 (jj&3)
    f32x16 y;
#pragma unroll
    for (int e = 0; e < 16; ++e) y[e] = 0.f;
    {
        const int jj = lane & 15, mh = (lane >> 4) & 1;
        const uint8_t* hp = had + (4 * hl + (jj >> 2)) * (PD * 2) + (32 * wave + 16 * mh + 4 * (jj & 3)) * 2;
        // the transposing reads hand lane half hl the contraction rows {4 hl .. 4 hl + 3} and {8 + 4 hl .. 8 + 4 hl + 3} of
        // a 16-row step, so the B operand takes the same rows of X: two 8-byte pieces
        const uint8_t* xp = xt + l32 * XROW + hl * 8;
#pragma unroll
        for (int ks = 0; ks < PD / 16; ++ks) {
            const s16x4 lo = lds_read_tr(hp + ks * 16 * (PD * 2));
            const s16x4 hi = lds_read_tr(hp + (ks * 16 + 8) * (PD * 2));
            const bf16x8 av = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
            const u32x2 b0 = *reinterpret_cast<const u32x2*>(xp + ks * 32);
            const u32x2 b1 = *reinterpret_cast<const u32x2*>(xp + ks * 32 + 16);
            const bf16x8 bv = __builtin_bit_cast(bf16x8, u32x4{b0[0], b0[1], b1[0], b1[1]});
            y = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, y, 0, 0, 0);
        }
    }
    // register e: n = 32 w + 8 (e/4) + 4 hl + e%4, token l32.  Round to bf16, then per-token absmax over the 128 n
    float yb[16], mx = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        yb[e] = bf16_to_f32(f32_to_bf16(y[e]));
        mx = fmaxf(mx, fabsf(yb[e]));
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    if (hl == 0) smax[wave][l32] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(smax[0][l32], smax[1][l32]), fmaxf(smax[2][l32], smax[3][l32]));
    const float sq = quant_scale(mx);
    const int gt = tok0 + l32;
    if (gt < a.t) {
        int8_t* qo = a.q_int8 + ((int64_t)gt * a.n + head) * PD + 32 * wave + 4 * hl;
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) {
            uint32_t pk = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) pk |= ((uint32_t)(int)__builtin_rintf(yb[4 * e4 + e] * sq) & 0xffu) << (8 * e);
            *reinterpret_cast<uint32_t*>(qo + 8 * e4) = pk;
        }
        if (wave == 0 && hl == 0)
            a.q_scale[(int64_t)gt * a.n + head] = __builtin_bit_cast(uint16_t, (_Float16)(1.0f / sq));
    }
}

// ------------------------------------------------------------------------------------------------ query path, prefill sizes
// The same product for 128 tokens and more: a workgroup of 256 lanes owns (head, 128 tokens) and walks the contraction
// in stages of 128 rows, both operands staged through LDS with the loads of the next DEPTH stages in flight.  Wave
// (wr, wc) owns tokens [64 wr, +64) x dims [64 wc, +64): every operand fragment read from LDS feeds four MFMAs, and the
// head's weight slice is fetched once per 128 tokens instead of once per 32.  Then, in LDS, for all 128 tokens: scale
// and round to bf16, rotary, hadamard (wave w: outputs [32 w, +32) of all tokens, every hadamard fragment feeding four
// MFMAs), quantisation.  The int32 sums are exact and the rest is the same operations in the same order, so the
// results are the bits of prolog_q_body's.
constexpr int QB_TOK = 128;
constexpr int QB_QROW = QK + 16; // bytes per LDS row of the [token][k] int8 tile (padded against bank conflicts)
constexpr int QB_STAGE_BYTES = QK * QROW + QB_TOK * QB_QROW;
constexpr int QB_EPI_BYTES = PD * PD * 2 + QB_TOK * XROW + 4 * QB_TOK * 4; // hadamard_q | bf16 tile | per-wave maxima
constexpr int QB_LDS_BYTES = QB_EPI_BYTES > QB_STAGE_BYTES ? QB_EPI_BYTES : QB_STAGE_BYTES;
constexpr int QB_DEPTH = 3; // stages of loads in flight (the epilogue's 68 KB of LDS leave two workgroups to a CU whatever the
                            // register count, so the depth costs no occupancy)

template <int DEPTH>
__device__ __forceinline__ void prolog_q_big_body(const PrologArgs& a, int head, int tok0, uint8_t* lds)
{
#pragma clang fp contract(off)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4, l32 = lane & 31, hl = lane >> 5, wr = wave >> 1, wc = wave & 1;
    const int r = a.r;
    const int64_t nd = (int64_t)a.n * PD;
    uint8_t* wl = lds;
    uint8_t* ql = lds + QK * QROW;
    const int stages = r / QK;
    // 128 rows x 128 bytes of either operand per stage = 4 pieces of 16 bytes per lane (rows tid / 8 + 32 i, piece tid % 8)
    const int srow = tid >> 3, spc = tid & 7;
    const int8_t* wp = a.w_qb + (int64_t)srow * nd + head * PD + 16 * spc;
    const int8_t* qp[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) qp[i] = a.q_norm + (int64_t)min(tok0 + srow + 32 * i, a.t - 1) * r + 16 * spc;
    u32x4 wst[DEPTH][4], qst[DEPTH][4];
    auto load = [&](int st, int u) {
#pragma unroll
        for (int i = 0; i < 4; ++i) qst[u][i] = *reinterpret_cast<const u32x4*>(qp[i] + st * QK);
#pragma unroll
        for (int i = 0; i < 4; ++i) wst[u][i] = *reinterpret_cast<const u32x4*>(wp + ((int64_t)st * QK + 32 * i) * nd);
    };
    // the epilogue's scales, requested first
    float qs_pre[4];
    f32x4 ws_pre[4];
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) qs_pre[tb] = a.q_norm_scale[min(tok0 + 64 * wr + 16 * tb + l16, a.t - 1)];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) ws_pre[nb] = *reinterpret_cast<const f32x4*>(a.w_qb_scale + (int64_t)head * PD + 64 * wc + 16 * nb + 4 * g);
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
                __syncthreads();    // everyone is done with the previous stage's tiles
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    u32x2* d = reinterpret_cast<u32x2*>(wl + (srow + 32 * i) * QROW + 16 * spc);
                    d[0] = u32x2{wst[u][i][0], wst[u][i][1]};
                    d[1] = u32x2{wst[u][i][2], wst[u][i][3]};
                    *reinterpret_cast<u32x4*>(ql + (srow + 32 * i) * QB_QROW + 16 * spc) = qst[u][i];
                }
                __syncthreads();
                load(min(st0 + u + DEPTH, stages - 1), u); // (unconditional: past the end the last stage is fetched again and dropped)
#pragma unroll
                for (int ks = 0; ks < QK / 64; ++ks) {
                    i32x4 qf[4], wf[4];
#pragma unroll
                    for (int tb = 0; tb < 4; ++tb)
                        qf[tb] = *reinterpret_cast<const i32x4*>(ql + (64 * wr + 16 * tb + l16) * QB_QROW + ks * 64 + 16 * g);
                    // (the byte-transposing read: see prolog_q_body)
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb) {
                        const uint8_t* p = wl + (ks * 64 + 16 * g + (l16 >> 1)) * QROW + 64 * wc + 16 * nb + 8 * (l16 & 1);
                        const v2i lo = lds_read_tr8(p), hi = lds_read_tr8(p + 8 * QROW);
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
    __syncthreads(); // the operand tiles are free: hadamard_q and the bf16 tile take their place
    uint8_t* had = lds;
    uint8_t* xt = lds + PD * PD * 2;
    float(*smax)[QB_TOK] = reinterpret_cast<float(*)[QB_TOK]>(lds + PD * PD * 2 + QB_TOK * XROW);
#pragma unroll
    for (int i = 0; i < PD * PD * 2 / 16 / 256; ++i) reinterpret_cast<u32x4*>(had)[tid + 256 * i] = reinterpret_cast<const u32x4*>(a.had_q)[tid + 256 * i];
    // register e of acc[nb][tb]: dim 64 wc + 16 nb + 4 g + e, token 64 wr + 16 tb + l16
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) {
        const int tl = 64 * wr + 16 * tb + l16;
        const float qs = qs_pre[tb];
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
            const int dim = 64 * wc + 16 * nb + 4 * g;
            const f32x4 ws = ws_pre[nb];
            uint16_t vb[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) vb[e] = f32_to_bf16(((float)acc[nb][tb][e] * qs) * ws[e]);
            *reinterpret_cast<u32x2*>(xt + tl * XROW + dim * 2) = u32x2{(uint32_t)vb[0] | ((uint32_t)vb[1] << 16), (uint32_t)vb[2] | ((uint32_t)vb[3] << 16)};
        }
    }
    __syncthreads();
    // rotary on the first 64 dims: 128 tokens x 32 pairs, 16 items per lane (the arithmetic of rope_tile)
#pragma unroll 4
    for (int it = 0; it < QB_TOK * 32 / 256; ++it) {
        const int item = tid + 256 * it;
        const int tok = item >> 5, i = item & 31;
        uint16_t* row = reinterpret_cast<uint16_t*>(xt + tok * XROW);
        const int64_t gtc = (int64_t)min(tok0 + tok, a.t - 1) * PROPE;
        const uint16_t* cosp = a.cos + gtc;
        const uint16_t* sinp = a.sin + gtc;
        const float x1 = bf16_to_f32(row[i]), x2 = bf16_to_f32(row[i + 32]);
        const float c1 = bf16_to_f32(cosp[i]), c2 = bf16_to_f32(cosp[i + 32]);
        const float s1 = bf16_to_f32(sinp[i]), s2 = bf16_to_f32(sinp[i + 32]);
        const float o1 = x1 * c1 + (-x2) * s1;
        const float o2 = x2 * c2 + x1 * s2;
        row[i] = f32_to_bf16(o1);
        row[i + 32] = f32_to_bf16(o2);
    }
    __syncthreads();
    // Y^T[n, token] = H^T[n, k] . X^T[k, token]: wave w owns n in [32 w, 32 w + 32) for the four blocks of 32 tokens
    // (operand addressing as in prolog_q_body)
    f32x16 y[4];
#pragma unroll
    for (int tb = 0; tb < 4; ++tb)
#pragma unroll
        for (int e = 0; e < 16; ++e) y[tb][e] = 0.f;
    {
        const int jj = lane & 15, mh = (lane >> 4) & 1;
        const uint8_t* hp = had + (4 * hl + (jj >> 2)) * (PD * 2) + (32 * wave + 16 * mh + 4 * (jj & 3)) * 2;
        const uint8_t* xp = xt + l32 * XROW + hl * 8;
#pragma unroll
        for (int ks = 0; ks < PD / 16; ++ks) {
            const s16x4 lo = lds_read_tr(hp + ks * 16 * (PD * 2));
            const s16x4 hi = lds_read_tr(hp + (ks * 16 + 8) * (PD * 2));
            const bf16x8 av = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
            for (int tb = 0; tb < 4; ++tb) {
                const u32x2 b0 = *reinterpret_cast<const u32x2*>(xp + 32 * tb * XROW + ks * 32);
                const u32x2 b1 = *reinterpret_cast<const u32x2*>(xp + 32 * tb * XROW + ks * 32 + 16);
                const bf16x8 bv = __builtin_bit_cast(bf16x8, u32x4{b0[0], b0[1], b1[0], b1[1]});
                y[tb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, y[tb], 0, 0, 0);
            }
        }
    }
    // register e of y[tb]: n = 32 w + 8 (e/4) + 4 hl + e%4, token 32 tb + l32.  Round to bf16, per-token absmax over the 128 n
    float mx[4];
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) {
        mx[tb] = 0.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            y[tb][e] = bf16_to_f32(f32_to_bf16(y[tb][e]));
            mx[tb] = fmaxf(mx[tb], fabsf(y[tb][e]));
        }
        mx[tb] = fmaxf(mx[tb], __shfl_xor(mx[tb], 32));
        if (hl == 0) smax[wave][32 * tb + l32] = mx[tb];
    }
    __syncthreads();
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) {
        const int tl = 32 * tb + l32;
        const float m = fmaxf(fmaxf(smax[0][tl], smax[1][tl]), fmaxf(smax[2][tl], smax[3][tl]));
        const float sq = quant_scale(m);
        const int gt = tok0 + tl;
        if (gt < a.t) {
            int8_t* qo = a.q_int8 + ((int64_t)gt * a.n + head) * PD + 32 * wave + 4 * hl;
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                uint32_t pk = 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) pk |= ((uint32_t)(int)__builtin_rintf(y[tb][4 * e4 + e] * sq) & 0xffu) << (8 * e);
                *reinterpret_cast<uint32_t*>(qo + 8 * e4) = pk;
            }
            if (wave == 0 && hl == 0) a.q_scale[(int64_t)gt * a.n + head] = __builtin_bit_cast(uint16_t, (_Float16)(1.0f / sq));
        }
    }
}
constexpr int PROLOG_BIG_T = 128;   // token count from which the query product runs per 128 tokens

// ------------------------------------------------------------------------------------------------ key path, weights
__device__ __forceinline__ float block_sum128(float v, float* red)
{
    v = wave_sum_butterfly(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return red[0] + red[1];
}
__device__ __forceinline__ float block_max128(float v, float* red)
{
    v = wave_max_f32(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return fmaxf(red[0], red[1]);
}

// One workgroup of 128 lanes per token: lane = output dim
__device__ __forceinline__ void prolog_k_body(const PrologArgs& a, int tok)
{
#pragma clang fp contract(off)
    __shared__ float red[2];
    __shared__ float kb[PD];
    const int tid = threadIdx.x;
    // everything that does not depend on the sums is loaded first (its latency hides behind them), and no load sits
    // under a condition (the compiler would wait for it on the spot)
    const int64_t row = a.k_cache_index[tok];
    const float gam = bf16_to_f32(a.ln_gamma[tid]), bet = bf16_to_f32(a.ln_beta[tid]);
    const int ri = tid & (PROPE - 1);
    const float rc = bf16_to_f32(a.cos[(int64_t)tok * PROPE + ri]), rs = bf16_to_f32(a.sin[(int64_t)tok * PROPE + ri]);
    uint16_t hk[PD]; // this lane's column of hadamard_k
#pragma unroll
    for (int k = 0; k < PD; ++k) hk[k] = a.had_k[k * PD + tid];
    float kv = 0.f, wv = 0.f;
    const int wcol = PD + min(tid, a.n - 1);
    // sixteen splits' loads in flight together (a split past the end re-reads the last one and adds zero); the order
    // of the additions is the order of the splits
    for (int s0 = 0; s0 < a.ksplits; s0 += 16) {
        float v0[16], v1[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const float* p = a.xw_part + ((int64_t)min(s0 + j, a.ksplits - 1) * a.t + tok) * a.xw_stride + a.xw_col0;
            v0[j] = p[tid];
            v1[j] = p[wcol];
        }
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            kv += s0 + j < a.ksplits ? v0[j] : 0.f;
            wv += s0 + j < a.ksplits ? v1[j] : 0.f;
        }
    }
    // LayerNorm in fp32 (biased variance), -> bf16
    const float mean = block_sum128(kv, red) / (float)PD;
    const float dlt = kv - mean;
    const float var = block_sum128(dlt * dlt, red) / (float)PD;
    float xn = dlt / sqrtf(var + a.eps);
    xn = xn * gam + bet;
    kb[tid] = bf16_to_f32(f32_to_bf16(xn));
    __syncthreads();
    // rotary on the first 64 dims
    float kr = kb[tid];
    if (tid < PROPE) {
        const float other = tid < 32 ? -kb[tid + 32] : kb[tid - 32];
        kr = bf16_to_f32(f32_to_bf16(kb[tid] * rc + other * rs));
    }
    __syncthreads();
    kb[tid] = kr;
    __syncthreads();
    // hadamard: y[n] = sum_k kr[k] H[k][n], fp32, -> bf16
    float y = 0.f;
#pragma unroll
    for (int k = 0; k < PD; ++k) y = __builtin_fmaf(kb[k], bf16_to_f32(hk[k]), y);
    y = bf16_to_f32(f32_to_bf16(y));
    const float mx = block_max128(fabsf(y), red);
    const float sq = quant_scale(mx);
    if (row >= 0 && row < a.cache_rows) {
        a.k_cache[row * PD + tid] = (int8_t)(int)__builtin_rintf(y * sq);
        if (tid == 0) a.k_scale_cache[row] = __builtin_bit_cast(uint16_t, (_Float16)(1.0f / sq));
    }
    if (tid < a.n) {
        const float w = bf16_to_f32(f32_to_bf16(wv));
        a.weights[(int64_t)tok * a.n + tid] = __builtin_bit_cast(uint16_t, (_Float16)((w * a.wscale_n) * a.wscale_d));
    }
}

} // namespace
} // namespace pto
