// Lightning-indexer prolog (the producer of everything the lightning indexer reads) - gfx950 kernels.
//
// Replaces the device side of lightning_indexer_prolog_quant
// (models/deepseek_v32_exp/lightning_indexer_prolog_quant_impl.py:203-543); arithmetic follows the golden
// indexer_prolog (models/deepseek_v32_exp/deepseekv32_lightning_indexer_prolog_quant.py:209-288):
//   query   q = bf16(int32(q_norm @ w_qb) * q_norm_scale * w_qb_scale); rotary embedding on the first 64 of each head's
//           128 dims; q = bf16(q @ hadamard_q) (fp32 accumulate); per (token, head): s = 127 / max|q|, int8 rint(q s),
//           dequant scale fp16(1 / s)
//   key     k = bf16(LayerNorm(x @ w_k)); rotary; bf16(k @ hadamard_k); same quantisation; written into the paged int8
//           index cache and its fp16 scale cache at row k_cache_index[token]
//   weights fp16(bf16(x @ w_proj) * n^-0.5 * d^-0.5)
//
// At decode sizes (tens of tokens) the operator streams 15 MB of weights once and is bound by that read and by launch
// latency, not by the matrix cores; the kernels are laid out for coalesced weight reads:
//   prolog_qx_kernel         one workgroup of 1024 lanes per (head, 32 tokens): int8 MFMA GEMM over r - w_qb has the
//                            output dimension contiguous, so its tile (r x 128 bytes, every load issued at once) goes
//                            through LDS and is read back with 8-bit transposing reads; four wave groups split the
//                            contraction and add their int32 sums through LDS - then, on the first group, scale and
//                            round to bf16 into LDS, rotary in LDS, hadamard as a bf16 MFMA (matrix read with 16-bit
//                            transposing LDS reads), quantisation
//   (same launch)            x @ [w_k | w_proj] split over the contraction (256 rows of the weights per workgroup, staged
//                            in LDS and read with transposing reads); fp32 partials to the workspace
//   prolog_k_kernel          one workgroup per token: sums the partials in a fixed order, LayerNorm, rotary, hadamard,
//                            quantisation, cache write, weights
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "common.h"
#include "kernels.h"
#include "prolog_device.h"
#include "timing.h"

namespace pto {
namespace {


// grid (tokens), 128 lanes
__global__ __launch_bounds__(128) void prolog_k_kernel(PrologArgs a) { prolog_k_body(a, blockIdx.x); }

// ------------------------------------------------------------------------------------------------ x @ [w_k | w_proj]
// 256 lanes per (256 rows of the weights, token tile of 32 TB): partial sums over those rows; wl is [256 k][nw] bf16,
// nw = 128 + n.  TB blocks of 32 tokens per workgroup: 1 at decode sizes; 4 at prefill sizes, where the weight rows are
// then staged once per 128 tokens and every weight fragment read from LDS feeds four MFMAs.
template <int TB, int PARTS = 1>
__device__ __forceinline__ void prolog_xw_body(const PrologArgs& a, int split, int tok0, uint8_t* wl)
{
    // PARTS: the workgroup's 256 weight rows are staged in that many pieces, one after the other in the same LDS space
    // (two at prefill sizes: 49 KB instead of 98, so that two workgroups share a CU next to the query product's)
    constexpr int ROWS = XW_K / PARTS;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hl = lane >> 5;
    const int nw = PD + a.n, rowb = nw * 2;
    const int64_t kbase = (int64_t)split * XW_K;
    const int nblocks = nw / 32; // 32-wide output blocks; wave w takes blocks w, w + 4
    const int jj = lane & 15, mh = (lane >> 4) & 1;
    // B operand: the transposing reads below hand lane half hl the contraction rows 8 hl .. 8 hl + 7 of every 16-row step,
    // so B is one 16-byte load per step (32 bytes contiguous per token row and instruction), requested one step ahead
    const uint16_t* xp[TB];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) xp[tb] = a.x + (int64_t)min(tok0 + 32 * tb + l32, a.t - 1) * a.h + kbase + hl * 8;
    f32x16 acc[TB][2];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[tb][j][e] = 0.f;
    u32x4 xv[TB];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) xv[tb] = *reinterpret_cast<const u32x4*>(xp[tb]);
#pragma unroll
    for (int part = 0; part < PARTS; ++part) {
        if (part > 0) __syncthreads(); // everyone is done with the previous piece
        // stage the weights: w_k rows then w_proj rows, 16-byte pieces
        const int64_t k0 = kbase + part * ROWS;
#pragma unroll 8
        for (int i = tid; i < ROWS * (PD / 8); i += 256) {
            const int k = i / (PD / 8), c = i % (PD / 8);
            *reinterpret_cast<u32x4*>(wl + k * rowb + c * 16) = *reinterpret_cast<const u32x4*>(a.w_k + (k0 + k) * PD + c * 8);
        }
#pragma unroll 8
        for (int i = tid; i < ROWS * (a.n / 8); i += 256) {
            const int k = i / (a.n / 8), c = i % (a.n / 8);
            *reinterpret_cast<u32x4*>(wl + k * rowb + PD * 2 + c * 16) = *reinterpret_cast<const u32x4*>(a.w_proj + (k0 + k) * a.n + c * 8);
        }
        __syncthreads();
        for (int ks = part * (ROWS / 16); ks < (part + 1) * (ROWS / 16); ++ks) {
            bf16x8 bv[TB];
#pragma unroll
            for (int tb = 0; tb < TB; ++tb) bv[tb] = __builtin_bit_cast(bf16x8, xv[tb]);
            // (TB = 1 runs beside the query product in a 1024-lane launch, at 128 registers: no room for the step ahead,
            // the load sits at the end of the step instead)
            const int kn = min(ks + 1, XW_K / 16 - 1); // (past the end: the last step again, dropped)
            if constexpr (TB > 1) {
#pragma unroll
                for (int tb = 0; tb < TB; ++tb) xv[tb] = *reinterpret_cast<const u32x4*>(xp[tb] + kn * 16);
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int nb = wave + 4 * j;
                if (nb < nblocks) {
                    const uint8_t* hp = wl + ((ks - part * (ROWS / 16)) * 16 + 8 * hl + (jj >> 2)) * rowb + (32 * nb + 16 * mh + 4 * (jj & 3)) * 2;
                    const s16x4 lo = lds_read_tr(hp);
                    const s16x4 hi = lds_read_tr(hp + 4 * rowb);
                    const bf16x8 av = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
                    for (int tb = 0; tb < TB; ++tb) acc[tb][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv[tb], acc[tb][j], 0, 0, 0);
                }
            }
            if constexpr (TB == 1) xv[0] = *reinterpret_cast<const u32x4*>(xp[0] + kn * 16);
        }
    }
    // register e of block nb: output 32 nb + 8 (e/4) + 4 hl + e%4, token 32 tb + l32
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
        const int gt = tok0 + 32 * tb + l32;
        if (gt < a.t) {
            float* out = a.xw_part + ((int64_t)split * a.t + gt) * nw;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int nb = wave + 4 * j;
                if (nb < nblocks)
#pragma unroll
                    for (int e4 = 0; e4 < 4; ++e4)
                        *reinterpret_cast<f32x4*>(out + 32 * nb + 8 * e4 + 4 * hl) =
                            f32x4{acc[tb][j][4 * e4], acc[tb][j][4 * e4 + 1], acc[tb][j][4 * e4 + 2], acc[tb][j][4 * e4 + 3]};
            }
        }
    }
}

// The query path and x @ [w_k | w_proj] do not depend on each other: one launch runs them side by side.
// grid (heads + h / 256, token tiles of 32), 1024 lanes (the workgroups of the second kind use their first 256)
__global__ __launch_bounds__(1024) void prolog_qx_kernel(PrologArgs a)
{
    extern __shared__ __align__(16) uint8_t plds[];
    if ((int)blockIdx.x < a.n) {
        prolog_q_body(a, blockIdx.x, blockIdx.y * PTOK, plds);
    } else {
        if (threadIdx.x >= 256) return; // the barrier inside is among the remaining four waves
        prolog_xw_body<1>(a, blockIdx.x - a.n, blockIdx.y * PTOK, plds);
    }
}

// Prefill sizes: the query product per (head, 128 tokens) and x @ [w_k | w_proj] per (256 weight rows, 128 tokens) side
// by side in one launch, as at decode sizes.  grid (heads + h / 256, token tiles of 128), 256 lanes; the dynamic LDS is
// the larger of the two bodies' needs.
template <int DEPTH>
__global__ __launch_bounds__(256, 2) void prolog_qx_big_kernel(PrologArgs a)
{
    extern __shared__ __align__(16) uint8_t plds[];
    if ((int)blockIdx.x < a.n)
        prolog_q_big_body<DEPTH>(a, blockIdx.x, blockIdx.y * QB_TOK, plds);
    else
        prolog_xw_body<4, 2>(a, blockIdx.x - a.n, blockIdx.y * (4 * PTOK), plds);
}

} // namespace

bool prolog_supported(int64_t h, int64_t r, int64_t n, int64_t d, int64_t rope)
{
    return d == PD && rope == PROPE && n > 0 && n % 32 == 0 && n <= 128 && r > 0 && r % QK == 0 && r <= QMAX_R && h > 0 &&
           h % XW_K == 0;
}

uint64_t prolog_workspace_bytes(int64_t t, int64_t h, int64_t r, int64_t n)
{
    (void)r;
    return (uint64_t)(h / XW_K) * t * (PD + n) * sizeof(float);
}

void prolog_bind_workspace(PrologArgs& a, void* ws)
{
    a.xw_part = static_cast<float*>(ws);
    a.xw_stride = PD + a.n;
    a.xw_col0 = 0;
}

hipError_t prolog_launch(const PrologArgs& a, hipStream_t stream)
{
    if (a.t == 0) return hipSuccess;
    const int ttiles = (a.t + PTOK - 1) / PTOK;
    hipError_t e;
    static DeviceOnce attr_done;
    constexpr int xw_lds_max = XW_K * (PD + 128) * 2;
    e = attr_done.run([] {
        return hipFuncSetAttribute(reinterpret_cast<const void*>(prolog_qx_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   prolog_q_lds_bytes(QMAX_R) > xw_lds_max ? prolog_q_lds_bytes(QMAX_R) : xw_lds_max);
    });
    if (e != hipSuccess) return e;
    const int xw_lds = XW_K * (PD + a.n) * 2;
    if (a.t >= PROLOG_BIG_T) {
        static DeviceOnce big_attr_done;
        constexpr int big_lds_max = xw_lds_max / 2 > QB_LDS_BYTES ? xw_lds_max / 2 : QB_LDS_BYTES;
        e = big_attr_done.run([] {
            return hipFuncSetAttribute(reinterpret_cast<const void*>(prolog_qx_big_kernel<QB_DEPTH>), hipFuncAttributeMaxDynamicSharedMemorySize, big_lds_max);
        });
        if (e != hipSuccess) return e;
        ScopedKernelTimer tm(KID_PROLOG_Q, stream);
        const dim3 grid(a.n + a.ksplits, (a.t + QB_TOK - 1) / QB_TOK);
        const int smem = xw_lds / 2 > QB_LDS_BYTES ? xw_lds / 2 : QB_LDS_BYTES; // (the x product stages its rows in two halves here)
        hipLaunchKernelGGL(prolog_qx_big_kernel<QB_DEPTH>, grid, dim3(256), smem, stream, a);
    } else {
        const int smem = prolog_q_lds_bytes(a.r) > xw_lds ? prolog_q_lds_bytes(a.r) : xw_lds;
        ScopedKernelTimer tm(KID_PROLOG_Q, stream);
        hipLaunchKernelGGL(prolog_qx_kernel, dim3(a.n + a.ksplits, ttiles), dim3(1024), smem, stream, a);
    }
    if ((e = hipGetLastError()) != hipSuccess) return e;
    {
        ScopedKernelTimer tm(KID_PROLOG_K, stream);
        hipLaunchKernelGGL(prolog_k_kernel, dim3(a.t), dim3(128), 0, stream, a);
    }
    return hipGetLastError();
}

} // namespace pto
