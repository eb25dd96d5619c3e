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
// transposed: bf16 tiles with ds_read_b64_tr_b16, the int8 tile byte by byte.
//   mla_xa_kernel    x @ [w_dq | w_dkv_kr], 256 contraction rows x 128 outputs per workgroup, fp32 partials
//   mla_norm_kernel  one workgroup per token: fixed-order sum of the partials, both RmsNorms, the quantisations, the
//                    key's rotary embedding, the three cache writes, q_norm / q_norm_scale
//   mla_qb_kernel    int8 MFMA GEMM q_norm @ w_uq_qr, 128 outputs x 32 tokens per workgroup, weights double-buffered
//                    through LDS; dequantisation and the query's rotary embedding in registers
//   mla_wuk_kernel   per (head, 128 outputs): q_b[:, head, :128] @ w_uk[head]
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "common.h"
#include "kernels.h"
#include "timing.h"

namespace pto {
namespace {

constexpr int MTOK = 32;          // tokens per workgroup tile
constexpr int MNOPE = 128, MROPE = 64, MQH = MNOPE + MROPE, MC = 512, MKV = MC + MROPE;
constexpr int XA_K = 256;         // contraction rows per workgroup of mla_xa_kernel
constexpr int TROW = 128 * 2 + 32; // bytes per LDS row of a [k][128] bf16 weight tile (padded against bank conflicts)
constexpr int QB_K = 128;         // contraction rows per stage of mla_qb_kernel
constexpr int QROW = 132;         // bytes per LDS row of a [k][128] int8 weight tile (padded)
constexpr int MAX_R = 2048;       // largest q_lora_rank mla_norm_kernel holds in LDS

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
__device__ __forceinline__ s16x4 lds_read_tr(const uint8_t* p)
{
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)const_cast<uint8_t*>(p));
}
__device__ __forceinline__ float bf16_to_f32(uint16_t v) { return __builtin_bit_cast(float, (uint32_t)v << 16); }
// The golden's "127 / max": torch evaluates scalar / tensor as reciprocal(tensor) * scalar, two roundings
__device__ __forceinline__ float quant_scale(float mx) { return (1.0f / mx) * 127.0f; }
__device__ __forceinline__ uint16_t f32_to_bf16(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
__device__ __forceinline__ float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

// 32 outputs x 32 tokens += W[k0 .. k0 + 16 steps, outputs]^T . X[tokens, k]: A by transposing reads of the [k][n] tile
// in LDS (lane jj of a 16-lane group points at row 4 hl + jj / 4 (+ 8) of the step, columns 16 mh + 4 (jj & 3)), which
// hand lane half hl the contraction rows {4 hl .. 4 hl + 3} and {8 + 4 hl .. + 3}; B takes the same rows of X as two
// 8-byte pieces.  Register e of the result: output 8 (e / 4) + 4 hl + e % 4, token lane % 32.
template <int KSTEPS>
__device__ __forceinline__ void gemm_tr_tile(f32x16& acc, const uint8_t* wtile, int ncol0, const uint16_t* xrow, int lane)
{
    const int jj = lane & 15, mh = (lane >> 4) & 1, hl = lane >> 5;
    const uint8_t* hp = wtile + (4 * hl + (jj >> 2)) * TROW + (ncol0 + 16 * mh + 4 * (jj & 3)) * 2;
    const uint16_t* xp = xrow + hl * 4;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        const u32x2 b0 = *reinterpret_cast<const u32x2*>(xp + ks * 16);
        const u32x2 b1 = *reinterpret_cast<const u32x2*>(xp + ks * 16 + 8);
        const bf16x8 bv = __builtin_bit_cast(bf16x8, u32x4{b0[0], b0[1], b1[0], b1[1]});
        const s16x4 lo = lds_read_tr(hp + ks * 16 * TROW);
        const s16x4 hi = lds_read_tr(hp + (ks * 16 + 8) * TROW);
        const bf16x8 av = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc, 0, 0, 0);
    }
}

// ------------------------------------------------------------------------------------------------ x @ [w_dq | w_dkv_kr]
// grid (h / 256, output tiles of 128, token tiles of 32), 256 lanes
__global__ __launch_bounds__(256) void mla_xa_kernel(MlaPrologArgs a)
{
    extern __shared__ __align__(16) uint8_t wl[]; // [256 k][128 n] bf16, rows of TROW bytes
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hl = lane >> 5;
    const int split = blockIdx.x, tile = blockIdx.y, tok0 = blockIdx.z * MTOK;
    const int64_t kbase = (int64_t)split * XA_K;
    const int qtiles = a.r / 128;
    const uint16_t* src;
    int ld, width;
    if (tile < qtiles) {
        src = a.w_dq + tile * 128;
        ld = a.r;
        width = 128;
    } else {
        const int c0 = (tile - qtiles) * 128;
        src = a.w_dkv_kr + c0;
        ld = MKV;
        width = min(128, MKV - c0);
    }
    const int pieces = width / 8; // 16-byte pieces per row
#pragma unroll 8
    for (int i = tid; i < XA_K * pieces; i += 256) {
        const int k = i / pieces, c = i % pieces;
        *reinterpret_cast<u32x4*>(wl + k * TROW + c * 16) = *reinterpret_cast<const u32x4*>(src + (kbase + k) * ld + c * 8);
    }
    __syncthreads();
    if (32 * wave >= width) return;
    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
    gemm_tr_tile<XA_K / 16>(acc, wl, 32 * wave, a.x + (int64_t)min(tok0 + l32, a.t - 1) * a.h + kbase, lane);
    const int gt = tok0 + l32;
    if (gt < a.t) {
        float* out = a.xa_part + ((int64_t)split * a.t + gt) * (a.r + MKV) + tile * 128 + 32 * wave + 4 * hl;
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4)
            *reinterpret_cast<f32x4*>(out + 8 * e4) = f32x4{acc[4 * e4], acc[4 * e4 + 1], acc[4 * e4 + 2], acc[4 * e4 + 3]};
    }
}

// ------------------------------------------------------------------------------------------------ norms, quantisation, cache
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) v += __shfl_xor(v, d);
    return v;
}
__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) v = fmaxf(v, __shfl_xor(v, d));
    return v;
}

// grid (tokens), 256 lanes
__global__ __launch_bounds__(256) void mla_norm_kernel(MlaPrologArgs a)
{
#pragma clang fp contract(off)
    __shared__ float buf[MAX_R + MKV];
    __shared__ float red[8];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, tok = blockIdx.x;
    const int r = a.r, ncols = r + MKV;
    // q_a and kv: partial sums in a fixed order, rounded to bf16
    for (int c = tid; c < ncols; c += 256) {
        float s = 0.f;
#pragma unroll 7
        for (int sp = 0; sp < a.ksplits; ++sp) s += a.xa_part[((int64_t)sp * a.t + tok) * ncols + c];
        buf[c] = round_bf16(s);
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
        for (int c = tid; c < r; c += 256) {
            const float v = round_bf16(bf16_to_f32(a.gamma_cq[c]) * (buf[c] * y));
            buf[c] = v;
            mx = fmaxf(mx, fabsf(v));
        }
        mx = wave_max(mx);
        if (lane == 0) red[4 + wave] = mx;
        __syncthreads();
        mx = fmaxf(fmaxf(red[4], red[5]), fmaxf(red[6], red[7]));
        const float sq = quant_scale(mx);
        // four values per lane and store
        for (int c = 4 * tid; c < r; c += 1024) {
            uint32_t pk = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) pk |= ((uint32_t)(int)__builtin_rintf(buf[c + e] * sq) & 0xffu) << (8 * e);
            *reinterpret_cast<uint32_t*>(a.q_norm + (int64_t)tok * r + c) = pk;
        }
        if (tid == 0) a.q_norm_scale[tok] = 1.0f / sq;
    }
    __syncthreads();
    const int64_t row = a.cache_index[tok];
    const bool row_ok = row >= 0 && row < a.cache_rows;
    // key: RmsNorm over 512 (lane: elements tid and tid + 256), groups of 128 quantised on their own
    {
        const float x0 = buf[r + tid], x1 = buf[r + 256 + tid];
        float ss = wave_sum((x0 * x0) * (1.0f / MC) + (x1 * x1) * (1.0f / MC));
        if (lane == 0) red[wave] = ss;
        __syncthreads();
        const float y = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) + a.eps_ckv);
        const float v0 = round_bf16(bf16_to_f32(a.gamma_ckv[tid]) * (x0 * y));
        const float v1 = round_bf16(bf16_to_f32(a.gamma_ckv[256 + tid]) * (x1 * y));
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
        if (row_ok) {
            a.kv_cache[row * MC + tid] = (int8_t)(int)__builtin_rintf(v0 * sq0);
            a.kv_cache[row * MC + 256 + tid] = (int8_t)(int)__builtin_rintf(v1 * sq1);
            if ((tid & 127) == 0) {
                a.k_scale_cache[row * 4 + (tid >> 7)] = 1.0f / sq0;
                a.k_scale_cache[row * 4 + 2 + (tid >> 7)] = 1.0f / sq1;
            }
        }
    }
    // key rotary: pair i = elements (2i, 2i+1) -> positions (i, 32 + i)
    if (tid < MROPE / 2 && row_ok) {
        const float xe = buf[r + MC + 2 * tid], xo = buf[r + MC + 2 * tid + 1];
        const uint16_t* cp = a.cos + (int64_t)tok * MROPE;
        const uint16_t* sp = a.sin + (int64_t)tok * MROPE;
        const float o1 = xe * bf16_to_f32(cp[tid]) + (-xo) * bf16_to_f32(sp[tid]);
        const float o2 = xo * bf16_to_f32(cp[tid + 32]) + xe * bf16_to_f32(sp[tid + 32]);
        a.kr_cache[row * MROPE + tid] = f32_to_bf16(o1);
        a.kr_cache[row * MROPE + 32 + tid] = f32_to_bf16(o2);
    }
}

// ------------------------------------------------------------------------------------------------ q_norm @ w_uq_qr
// grid (n * 192 / 128, token tiles of 32), 256 lanes: wave w owns outputs [32 w, 32 w + 32) of the tile
__global__ __launch_bounds__(256) void mla_qb_kernel(MlaPrologArgs a)
{
#pragma clang fp contract(off)
    __shared__ __align__(16) uint8_t wl[2][QB_K * QROW];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int col0 = blockIdx.x * 128, tok0 = blockIdx.y * MTOK;
    const int r = a.r;
    const int64_t nq = (int64_t)a.n * MQH;

    // staging: 128 rows x 128 bytes per stage = 4 pieces of 16 bytes per lane (rows tid/8 + 32 i, piece tid%8)
    const int srow = tid >> 3, spc = tid & 7;
    const int8_t* sp = a.w_uq_qr + (int64_t)srow * nq + col0 + 16 * spc;
    u32x4 stg[4];
    auto stage_load = [&](int s) {
#pragma unroll
        for (int i = 0; i < 4; ++i) stg[i] = *reinterpret_cast<const u32x4*>(sp + ((int64_t)s * QB_K + 32 * i) * nq);
    };
    auto stage_store = [&](int bufi) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t* d = reinterpret_cast<uint32_t*>(&wl[bufi][(srow + 32 * i) * QROW + 16 * spc]);
            d[0] = stg[i][0];
            d[1] = stg[i][1];
            d[2] = stg[i][2];
            d[3] = stg[i][3];
        }
    };
    i32x4 acc[2][2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) acc[nb][tb] = i32x4{0, 0, 0, 0};
    const int8_t* qrow[2];
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) qrow[tb] = a.q_norm + (int64_t)min(tok0 + 16 * tb + l16, a.t - 1) * r + 16 * g;

    const int stages = r / QB_K;
    stage_load(0);
    stage_store(0);
    __syncthreads();
    for (int s = 0; s < stages; ++s) {
        if (s + 1 < stages) stage_load(s + 1);
        const uint8_t* wb = wl[s & 1];
#pragma unroll
        for (int ks = 0; ks < QB_K / 64; ++ks) {
            i32x4 qf[2], wf[2];
#pragma unroll
            for (int tb = 0; tb < 2; ++tb) qf[tb] = *reinterpret_cast<const i32x4*>(qrow[tb] + s * QB_K + ks * 64);
            // A operand: output 32 w + 16 nb + l16, contraction bytes 16 g .. 16 g + 15 of the step - one byte per row
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                const uint8_t* p = wb + (ks * 64 + 16 * g) * QROW + 32 * wave + 16 * nb + l16;
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4)
                    wf[nb][q4] = (int)((uint32_t)p[(4 * q4) * QROW] | ((uint32_t)p[(4 * q4 + 1) * QROW] << 8) |
                                       ((uint32_t)p[(4 * q4 + 2) * QROW] << 16) | ((uint32_t)p[(4 * q4 + 3) * QROW] << 24));
            }
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int tb = 0; tb < 2; ++tb)
                    acc[nb][tb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[nb], qf[tb], acc[nb][tb], 0, 0, 0);
        }
        if (s + 1 < stages) stage_store((s + 1) & 1);
        __syncthreads();
    }
    // register e of acc[nb][tb]: output col0 + 32 w + 16 nb + 4 g + e, token 16 tb + l16
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
        const int gt = tok0 + 16 * tb + l16;
        if (gt >= a.t) continue;
        const float qs = a.q_norm_scale[gt];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const int col = col0 + 32 * wave + 16 * nb + 4 * g;
            const int head = col / MQH, d = col % MQH;
            const f32x4 ws = *reinterpret_cast<const f32x4*>(a.w_qb_scale + col);
            uint16_t vb[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) vb[e] = f32_to_bf16(((float)acc[nb][tb][e] * qs) * ws[e]);
            if (d < MNOPE) {
                const u32x2 pk = {(uint32_t)vb[0] | ((uint32_t)vb[1] << 16), (uint32_t)vb[2] | ((uint32_t)vb[3] << 16)};
                *reinterpret_cast<u32x2*>(a.qb_nope + ((int64_t)gt * a.n + head) * MNOPE + d) = pk;
            } else {
                const uint16_t* cp = a.cos + (int64_t)gt * MROPE;
                const uint16_t* snp = a.sin + (int64_t)gt * MROPE;
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

// ------------------------------------------------------------------------------------------------ q_b[:, head, :128] @ w_uk[head]
// grid (heads, 512 / 128, token tiles of 32), 256 lanes: wave w owns outputs [32 w, 32 w + 32) of the tile
__global__ __launch_bounds__(256) void mla_wuk_kernel(MlaPrologArgs a)
{
    __shared__ __align__(16) uint8_t wl[MNOPE * TROW];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hl = lane >> 5;
    const int head = blockIdx.x, ct = blockIdx.y, tok0 = blockIdx.z * MTOK;
    const uint16_t* src = a.w_uk + (int64_t)head * MNOPE * MC + ct * 128;
#pragma unroll
    for (int i = tid; i < MNOPE * 16; i += 256) {
        const int k = i >> 4, c = i & 15;
        *reinterpret_cast<u32x4*>(wl + k * TROW + c * 16) = *reinterpret_cast<const u32x4*>(src + (int64_t)k * MC + c * 8);
    }
    __syncthreads();
    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
    const int gt = tok0 + l32;
    gemm_tr_tile<MNOPE / 16>(acc, wl, 32 * wave, a.qb_nope + ((int64_t)min(gt, a.t - 1) * a.n + head) * MNOPE, lane);
    if (gt < a.t) {
        uint16_t* out = a.q_nope + ((int64_t)gt * a.n + head) * MC + ct * 128 + 32 * wave + 4 * hl;
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) {
            const u32x2 pk = {(uint32_t)f32_to_bf16(acc[4 * e4]) | ((uint32_t)f32_to_bf16(acc[4 * e4 + 1]) << 16),
                              (uint32_t)f32_to_bf16(acc[4 * e4 + 2]) | ((uint32_t)f32_to_bf16(acc[4 * e4 + 3]) << 16)};
            *reinterpret_cast<u32x2*>(out + 8 * e4) = pk;
        }
    }
}

} // namespace

bool mla_prolog_supported(int64_t h, int64_t r, int64_t n, int64_t d_nope, int64_t d_rope, int64_t c)
{
    return d_nope == MNOPE && d_rope == MROPE && c == MC && n > 0 && (n * MQH) % 128 == 0 && r > 0 && r % 128 == 0 &&
           r <= MAX_R && h > 0 && h % XA_K == 0;
}

static uint64_t up256(uint64_t x) { return (x + 255) & ~(uint64_t)255; }

uint64_t mla_prolog_workspace_bytes(int64_t t, int64_t h, int64_t r, int64_t n)
{
    return up256((uint64_t)(h / XA_K) * t * (r + MKV) * sizeof(float)) + up256((uint64_t)t * n * MNOPE * 2);
}

void mla_prolog_bind_workspace(MlaPrologArgs& a, void* ws)
{
    uint8_t* p = static_cast<uint8_t*>(ws);
    a.xa_part = reinterpret_cast<float*>(p);
    p += up256((uint64_t)a.ksplits * a.t * (a.r + MKV) * sizeof(float));
    a.qb_nope = reinterpret_cast<uint16_t*>(p);
}

hipError_t mla_prolog_launch(const MlaPrologArgs& a, hipStream_t stream)
{
    if (a.t == 0) return hipSuccess;
    const int ttiles = (a.t + MTOK - 1) / MTOK;
    hipError_t e;
    {
        const int smem = XA_K * TROW;
        static bool attr_done = false;
        if (!attr_done) {
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(mla_xa_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
            if (e != hipSuccess) return e;
            attr_done = true;
        }
        const int tiles = a.r / 128 + (MKV + 127) / 128;
        ScopedKernelTimer tm(KID_MLA_XA, stream);
        hipLaunchKernelGGL(mla_xa_kernel, dim3(a.ksplits, tiles, ttiles), dim3(256), smem, stream, a);
    }
    if ((e = hipGetLastError()) != hipSuccess) return e;
    {
        ScopedKernelTimer tm(KID_MLA_NORM, stream);
        hipLaunchKernelGGL(mla_norm_kernel, dim3(a.t), dim3(256), 0, stream, a);
    }
    if ((e = hipGetLastError()) != hipSuccess) return e;
    {
        ScopedKernelTimer tm(KID_MLA_QB, stream);
        hipLaunchKernelGGL(mla_qb_kernel, dim3(a.n * MQH / 128, ttiles), dim3(256), 0, stream, a);
    }
    if ((e = hipGetLastError()) != hipSuccess) return e;
    {
        ScopedKernelTimer tm(KID_MLA_WUK, stream);
        hipLaunchKernelGGL(mla_wuk_kernel, dim3(a.n, MC / 128, ttiles), dim3(256), 0, stream, a);
    }
    return hipGetLastError();
}

} // namespace pto
