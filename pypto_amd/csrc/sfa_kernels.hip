// Sparse flash attention over a paged, int8, MLA-compressed KV cache - gfx950 kernels.
//
// Replaces the device side of sparse_flash_attention_quant_compute / sparse_attention_antiquant_compute
// (models/deepseek_v32_exp/sparse_flash_attention_quant_impl.py:45-286,
//  models/deepseek_v32_exp/sparse_attention_antiquant_impl.py:44-266,422-720); the arithmetic follows the
// online-softmax golden (models/deepseek_v32_exp/deepseekv32_sparse_attention_antiquant.py:359-457):
//   K row = [ bf16(fp32(int8) * scale[col/128]) | rope bf16 ],  V = first 512 columns of K
//   S = q K^T in fp32 from bf16 operands, * softmax_scale
//   P~ = exp(S - m) rounded to bf16 un-normalised, l summed in fp32 from the unrounded values
//   O = (sum P~ V) / l, one rounding to bf16
//
// Work decomposition.  One workgroup (4 wavefronts) owns one (query token, KV split): it walks its share of
// the token's top-k list in tiles of 32 selected cache rows.  Per tile all 256 lanes gather the rows
// (8-byte loads, a wavefront covers the 512 int8 of one row per instruction), dequantise in registers and
// store the tile to LDS twice: row-major for the S = K Q^T product and token-minor ("V^T") for the O^T = V^T P
// product, so both MFMA A-operands are single 16-byte LDS reads.  Wavefront w owns query heads
// [32w, 32w+32): its slice of Q stays in registers (B operand of v_mfma_f32_32x32x16_bf16), S^T comes out
// with one head per lane (row statistics are in-lane reductions plus one cross-half exchange), and the
// rounded P~ registers are directly the B operand of the PV product.  O^T (512 x 32 per wavefront) lives in
// 256 accumulator registers.  The LDS tile is double buffered: tile i+1 is dequantised while tile i is in
// the matrix cores.
//
// KV splits write un-normalised fp32 partial outputs plus (m, l); sfa_combine_kernel merges them.
#include "common.h"
#include "kernels.h"
#include "timing.h"

namespace pto {
namespace {

constexpr int T = 32;                  // selected rows per tile
constexpr int DN = 512;                // nope / value width
constexpr int DR = 64;                 // rope width
constexpr int KSTEPS = (DN + DR) / 16; // 36 MFMA k-steps for S
constexpr int KROW = (DN + DR) * 2 + 16; // bytes per row of the row-major tile (16 B pad: conflict-free b128 reads)
constexpr int KBUF = T * KROW;           // 37376
constexpr int VBUF = DN * T * 2;         // 32768
constexpr int STAGE = KBUF + VBUF;       // 70144
constexpr int MAX_SPLIT_TOKENS = 2048;   // rows[] capacity
constexpr int SMEM_BYTES = 2 * STAGE + MAX_SPLIT_TOKENS * 4;
constexpr int HEADS_PER_WG = 128;

template <bool QUANT>
struct RawTile;
template <>
struct RawTile<true> {
    u32x2 nope[8]; // 8 tokens x 8 int8 (this lane's 8 columns)
    float scale[8];
    u32x4 rope;
};
template <>
struct RawTile<false> {
    u32x4 nope[8]; // 8 tokens x 8 bf16
    u32x4 rope;
};

// token-in-tile of element e (0..7) of 8-token chunk c (0..3): the k-slot order of the PV B operand
__device__ __forceinline__ int chunk_token(int c, int e) { return 16 * (c >> 1) + 8 * (e >> 2) + 4 * (c & 1) + (e & 3); }

template <bool QUANT>
__device__ __forceinline__ void load_raw(RawTile<QUANT>& r, const SfaArgs& a, const int* rows, int tile, int wave,
                                         int lane, int tid)
{
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int row = rows[tile * T + chunk_token(wave, e)];
        if constexpr (QUANT) {
            u32x2 v = {0u, 0u};
            float s = 0.f;
            if (row >= 0) {
                v = *reinterpret_cast<const u32x2*>(a.kn + (int64_t)row * a.kn_stride + lane * 8);
                s = *reinterpret_cast<const float*>(a.ks + (int64_t)row * a.ks_stride + (lane >> 4) * 4);
            }
            r.nope[e] = v;
            r.scale[e] = s;
        } else {
            u32x4 v = {0u, 0u, 0u, 0u};
            if (row >= 0) v = *reinterpret_cast<const u32x4*>(a.kn + (int64_t)row * a.kn_stride + lane * 16);
            r.nope[e] = v;
        }
    }
    {
        const int row = rows[tile * T + (tid >> 3)];
        u32x4 v = {0u, 0u, 0u, 0u};
        if (row >= 0) v = *reinterpret_cast<const u32x4*>(a.kr + (int64_t)row * a.kr_stride + (tid & 7) * 16);
        r.rope = v;
    }
}

__device__ __forceinline__ float i8_at(uint32_t w, int k) { return (float)(int8_t)(w >> (8 * k)); }

// Dequantise this lane's 8 tokens x 8 columns and store them to both LDS layouts of a stage.
template <bool QUANT>
__device__ __forceinline__ void dequant_store(const RawTile<QUANT>& r, uint8_t* stage, int wave, int lane, int tid)
{
    uint32_t kb[8][4]; // [token e][column pair]
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        if constexpr (QUANT) {
            const float s = r.scale[e];
            const uint32_t w0 = r.nope[e][0], w1 = r.nope[e][1];
            kb[e][0] = pack_bf16x2(i8_at(w0, 0) * s, i8_at(w0, 1) * s);
            kb[e][1] = pack_bf16x2(i8_at(w0, 2) * s, i8_at(w0, 3) * s);
            kb[e][2] = pack_bf16x2(i8_at(w1, 0) * s, i8_at(w1, 1) * s);
            kb[e][3] = pack_bf16x2(i8_at(w1, 2) * s, i8_at(w1, 3) * s);
        } else {
#pragma unroll
            for (int p = 0; p < 4; ++p) kb[e][p] = r.nope[e][p];
        }
        u32x4 v = {kb[e][0], kb[e][1], kb[e][2], kb[e][3]};
        *reinterpret_cast<u32x4*>(stage + chunk_token(wave, e) * KROW + lane * 16) = v;
    }
    // token-minor layout: block (column group of 8 = lane, chunk = wave) is 128 contiguous bytes holding
    // 8 columns x 8 tokens; the 16-byte slot of column d is swizzled with the column group.
    uint8_t* vt = stage + KBUF + (lane * 4 + wave) * 128;
#pragma unroll
    for (int d = 0; d < 8; ++d) {
        const uint32_t sel = (d & 1) ? 0x07060302u : 0x05040100u;
        u32x4 v;
#pragma unroll
        for (int p = 0; p < 4; ++p) v[p] = __builtin_amdgcn_perm(kb[2 * p + 1][d >> 1], kb[2 * p][d >> 1], sel);
        *reinterpret_cast<u32x4*>(vt + ((d ^ (lane & 7)) * 16)) = v;
    }
    *reinterpret_cast<u32x4*>(stage + (tid >> 3) * KROW + DN * 2 + (tid & 7) * 16) = r.rope;
}

template <bool QUANT>
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256), amdgpu_waves_per_eu(1, 1))) void sfa_decode_kernel(
    SfaArgs a)
{
    extern __shared__ __align__(16) uint8_t smem[];
    int* rows = reinterpret_cast<int*>(smem + 2 * STAGE);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hl = lane >> 5;
    const int sp = blockIdx.x, tq = blockIdx.y, hg = blockIdx.z;
    const int bi = tq / a.s1, si = tq - bi * a.s1;

    int cur = a.act_seq[bi] - a.s1 + 1 + si;
    cur = min(max(cur, 0), a.topk);
    const int ntiles_all = (cur + T - 1) / T;
    const int per = (ntiles_all + a.nsplit - 1) / a.nsplit;
    const int tile0 = sp * per;
    const int ntiles = max(min(ntiles_all, tile0 + per) - tile0, 0);
    const int tok0 = tile0 * T;

    // logical top-k entries of this split -> physical cache rows (or -1: absent)
    const int64_t max_logical = (int64_t)a.bt_stride * a.block_size;
    for (int i = tid; i < ntiles * T; i += 256) {
        const int g = tok0 + i;
        int row = -1;
        if (g < cur) {
            const int idx = a.topk_idx[(int64_t)tq * a.topk_stride + g];
            if (idx >= 0 && idx < max_logical) {
                const int page = a.block_table[(int64_t)bi * a.bt_stride + idx / a.block_size];
                const int64_t r = (int64_t)page * a.block_size + idx % a.block_size;
                if (page >= 0 && r < a.n_rows) row = (int)r;
            }
        }
        rows[i] = row;
    }

    // this lane's query head and its Q slice (B operand: head = column, 8 consecutive k per half-wave)
    const int head = hg * HEADS_PER_WG + wave * 32 + l32;
    const bool head_ok = head < a.nq;
    const bool wave_active = hg * HEADS_PER_WG + wave * 32 < a.nq;
    bf16x8 q[KSTEPS];
    {
        const int64_t qrow = (int64_t)tq * a.nq + (head_ok ? head : 0);
        const __bf16* qn = reinterpret_cast<const __bf16*>(a.q_nope) + qrow * DN + hl * 8;
        const __bf16* qr = reinterpret_cast<const __bf16*>(a.q_rope) + qrow * DR + hl * 8;
        const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            const __bf16* p = ks < DN / 16 ? qn + ks * 16 : qr + (ks - DN / 16) * 16;
            q[ks] = head_ok ? *reinterpret_cast<const bf16x8*>(p) : zero;
        }
    }

    f32x16 o[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
    float m_run = -INFINITY; // running max of S * scale * log2(e)
    float l_run = 0.f;       // this lane's share of sum exp
    const float c_log2 = a.softmax_scale * 1.4426950408889634f;

    __syncthreads(); // rows[] ready

    RawTile<QUANT> raw;
    if (ntiles > 0) {
        load_raw<QUANT>(raw, a, rows, 0, wave, lane, tid);
        dequant_store(raw, smem, wave, lane, tid);
        if (ntiles > 1) load_raw<QUANT>(raw, a, rows, 1, wave, lane, tid);
    }
    __syncthreads();

    for (int it = 0; it < ntiles; ++it) {
        uint8_t* stage = smem + (it & 1) * STAGE;
        if (it + 1 < ntiles) {
            dequant_store(raw, smem + ((it + 1) & 1) * STAGE, wave, lane, tid);
            if (it + 2 < ntiles) load_raw<QUANT>(raw, a, rows, it + 2, wave, lane, tid);
        }
        const uint32_t valid = (uint32_t)__ballot(rows[it * T + l32] >= 0);
        if (wave_active && valid != 0u) {
            // S^T[token, head] = K[token, :] . Q[head, :]
            f32x16 s;
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = 0.f;
            const uint8_t* ka = stage + l32 * KROW + hl * 16;
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                const bf16x8 kf = *reinterpret_cast<const bf16x8*>(ka + ks * 32);
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, q[ks], s, 0, 0, 0);
            }
            // register r holds token 8*(r/4) + 4*hl + r%4 for head l32
            float mx = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float z = s[r] * c_log2;
                if (valid != 0xffffffffu) {
                    const int tok = 8 * (r >> 2) + 4 * hl + (r & 3);
                    z = ((valid >> tok) & 1u) ? z : -INFINITY;
                }
                s[r] = z;
                mx = fmaxf(mx, z);
            }
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run, mx);
            if (__any(m_new > m_run)) {
                const float alpha = exp2f(m_run - m_new); // 0 on the first tile (m_run = -inf)
                l_run *= alpha;
#pragma unroll
                for (int i = 0; i < 16; ++i)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o[i][r] *= alpha;
                m_run = m_new;
            }
            uint32_t pb[8];
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                const float p0 = exp2f(s[r] - m_run), p1 = exp2f(s[r + 1] - m_run);
                l_run += p0 + p1;
                pb[r >> 1] = pack_bf16x2(p0, p1);
            }
            // O^T[dim, head] += V^T[dim, token] . P~[token, head]
            const uint8_t* vt = stage + KBUF;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                u32x4 pw = {pb[4 * j], pb[4 * j + 1], pb[4 * j + 2], pb[4 * j + 3]};
                const bf16x8 pf = __builtin_bit_cast(bf16x8, pw);
#pragma unroll
                for (int db = 0; db < 16; ++db) {
                    const int dg = 4 * db + (l32 >> 3), d = l32 & 7;
                    const bf16x8 vf =
                        *reinterpret_cast<const bf16x8*>(vt + (dg * 4 + 2 * j + hl) * 128 + ((d ^ (dg & 7)) * 16));
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf, o[db], 0, 0, 0);
                }
            }
        }
        __syncthreads();
    }

    if (!wave_active) return;
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    if (!head_ok) return;
    // register r of block db holds dim 32*db + 8*(r/4) + 4*hl + r%4 of head l32
    if (a.nsplit == 1) {
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        uint8_t* dst = reinterpret_cast<uint8_t*>(a.out) + ((int64_t)tq * a.nq + head) * DN * 2;
#pragma unroll
        for (int db = 0; db < 16; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                u32x2 v = {pack_bf16x2(o[db][4 * g] * inv, o[db][4 * g + 1] * inv),
                           pack_bf16x2(o[db][4 * g + 2] * inv, o[db][4 * g + 3] * inv)};
                *reinterpret_cast<u32x2*>(dst + (32 * db + 8 * g + 4 * hl) * 2) = v;
            }
    } else {
        const int64_t prow = ((int64_t)tq * a.nsplit + sp) * a.nq + head;
        float* dst = a.part_o + prow * DN;
#pragma unroll
        for (int db = 0; db < 16; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f32x4 v = {o[db][4 * g], o[db][4 * g + 1], o[db][4 * g + 2], o[db][4 * g + 3]};
                *reinterpret_cast<f32x4*>(dst + 32 * db + 8 * g + 4 * hl) = v;
            }
        if (hl == 0) {
            a.part_ml[prow * 2] = m_run;
            a.part_ml[prow * 2 + 1] = l_tot;
        }
    }
}

// out[row, :] = sum_s 2^(m_s - M) O_s[row, :] / sum_s 2^(m_s - M) l_s ; one block of 128 lanes per output row
__global__ __launch_bounds__(128) void sfa_combine_kernel(const float* __restrict__ part_o,
                                                          const float* __restrict__ part_ml, void* out, int nq,
                                                          int nsplit)
{
    const int row = blockIdx.x; // tq * nq + head
    const int tq = row / nq, head = row - tq * nq;
    float M = -INFINITY;
    for (int s = 0; s < nsplit; ++s) M = fmaxf(M, part_ml[(((int64_t)tq * nsplit + s) * nq + head) * 2]);
    float L = 0.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    if (M > -INFINITY) {
        for (int s = 0; s < nsplit; ++s) {
            const int64_t prow = ((int64_t)tq * nsplit + s) * nq + head;
            const float l = part_ml[prow * 2 + 1];
            if (l > 0.f) {
                const float w = exp2f(part_ml[prow * 2] - M);
                L += w * l;
                const f32x4 v = *reinterpret_cast<const f32x4*>(part_o + prow * DN + threadIdx.x * 4);
                acc += v * w;
            }
        }
    }
    const float inv = L > 0.f ? 1.f / L : 0.f;
    u32x2 v = {pack_bf16x2(acc[0] * inv, acc[1] * inv), pack_bf16x2(acc[2] * inv, acc[3] * inv)};
    *reinterpret_cast<u32x2*>(reinterpret_cast<uint8_t*>(out) + ((int64_t)row * DN + threadIdx.x * 4) * 2) = v;
}

int num_cus()
{
    static int cached = 0;
    if (cached == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        cached = n;
    }
    return cached;
}

} // namespace

int sfa_pick_splits(int t, int nq, int topk)
{
    const int hgroups = (nq + HEADS_PER_WG - 1) / HEADS_PER_WG;
    const int tiles = (topk + T - 1) / T;
    int n = num_cus() / (t * hgroups > 0 ? t * hgroups : 1);
    n = n < 1 ? 1 : n;
    n = n > tiles ? tiles : n;
    n = n > 16 ? 16 : n;
    return n;
}

uint64_t sfa_workspace_bytes(int t, int nq, int nsplit)
{
    if (nsplit <= 1) return 0;
    return (uint64_t)t * nsplit * nq * (DN + 2) * sizeof(float);
}

hipError_t sfa_launch(const SfaArgs& a, hipStream_t stream)
{
    const int t = a.b * a.s1;
    if (t == 0) return hipSuccess;
    static bool attr_done[2] = {false, false};
    auto kern = a.quant ? sfa_decode_kernel<true> : sfa_decode_kernel<false>;
    if (!attr_done[a.quant]) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES);
        if (e != hipSuccess) return e;
        attr_done[a.quant] = true;
    }
    const int hgroups = (a.nq + HEADS_PER_WG - 1) / HEADS_PER_WG;
    dim3 grid(a.nsplit, t, hgroups);
    {
        ScopedKernelTimer tm(KID_SFA_DECODE, stream);
        hipLaunchKernelGGL(kern, grid, dim3(256), SMEM_BYTES, stream, a);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (a.nsplit > 1) {
        ScopedKernelTimer tm(KID_SFA_COMBINE, stream);
        hipLaunchKernelGGL(sfa_combine_kernel, dim3(t * a.nq), dim3(128), 0, stream, a.part_o, a.part_ml, a.out, a.nq,
                           a.nsplit);
        e = hipGetLastError();
    }
    return e;
}

} // namespace pto
