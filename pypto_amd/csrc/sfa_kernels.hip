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
// Work decomposition.  One workgroup (4 wavefronts) owns one (query token, KV split, group of 64 heads): it
// walks its share of the token's top-k list in tiles of 32 selected cache rows.  Per tile all 256 lanes
// gather the rows (8-byte loads, a wavefront covers the 512 int8 of one row per instruction), dequantise in
// registers and store the tile row-major to LDS (16-byte chunks XOR-swizzled with the row, no padding).
// Wavefronts pair up on 32 heads: wave (hg, kh) holds the Q columns of the k-steps with parity kh (B operand
// of v_mfma_f32_32x32x16_bf16, 72 registers), computes its half of S^T = K Q^T, swaps the fp32 partial with
// its partner through LDS, and both run the same softmax (one head per lane: row statistics are in-lane
// reductions plus one cross-half exchange).  The rounded P~ registers are directly the B operand of
// O^T = V^T P~, of which wave kh accumulates the 32-column blocks of parity kh (128 accumulator registers).
// The V^T operand is read from the same row-major tile with ds_read_b64_tr_b16 (LDS transpose read: a 16-lane
// group fetches 4 rows x 16 columns and each lane receives 4 rows of one column).  The LDS tile is double
// buffered: tile i+1 is dequantised while tile i is in the matrix cores.  64 heads per workgroup (not 128)
// keeps Q + O at 200 of the 512 registers per lane, which leaves room to overlap loads, dequant and MFMA.
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
constexpr int KSTEPS = (DN + DR) / 16; // 36 MFMA k-steps for S, 18 per wave of a pair
constexpr int KROW = (DN + DR) * 2;    // 1152 bytes per tile row = 72 chunks of 16 bytes
constexpr int STAGE = T * KROW;        // 36864
constexpr int MAX_SPLIT_TOKENS = 2048; // capacity of rows[] / scales[]
constexpr int ROWS_OFF = 2 * STAGE;
constexpr int SCALES_OFF = ROWS_OFF + MAX_SPLIT_TOKENS * 4;
constexpr int XBUF_OFF = SCALES_OFF + MAX_SPLIT_TOKENS * 16;
constexpr int SMEM_BYTES = XBUF_OFF + 4 * 4096; // 131072
constexpr int HEADS_PER_WG = 64;

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

// ds_read_b64_tr_b16: within each group of 16 lanes, lane i receives element i%4 of the 8-byte chunks
// addressed by lanes i/4, 4 + i/4, 8 + i/4 and 12 + i/4 of the group.
__device__ __forceinline__ s16x4 lds_read_tr(uint8_t* p) { return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p); }

// chunk swizzle of tile row t: a bijection of t % 8, so that 8 consecutive rows (b128 column reads) and the
// 4 consecutive rows of a transpose read both land on distinct banks
__device__ __forceinline__ int swz(int t) { return ((t & 3) << 1) | ((t >> 2) & 1); }

template <bool QUANT>
struct RawTile;
template <>
struct RawTile<true> {
    u32x2 nope[8]; // 8 rows x 8 int8 (this lane's 8 columns)
    u32x4 rope;
    uint32_t absent;
};
template <>
struct RawTile<false> {
    u32x4 nope[8]; // 8 rows x 8 bf16
    u32x4 rope;
    uint32_t absent;
};

// Lane (wave w, lane l) fetches columns [8l, 8l+8) of tile rows 8w .. 8w+7 and one 16-byte piece of a rope row.
// Absent rows (-1) read row 0 instead; `absent` keeps one bit per load and the data is zeroed when it is
// consumed (dequant_store), so that no load has to be waited for here.
template <bool QUANT>
__device__ __forceinline__ void load_raw(RawTile<QUANT>& r, const SfaArgs& a, const int* rows, int tile, int wave,
                                         int lane, int tid)
{
    uint32_t absent = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int row = rows[tile * T + 8 * wave + e];
        const int64_t rr = row < 0 ? 0 : row;
        absent |= (row < 0 ? 1u : 0u) << e;
        if constexpr (QUANT)
            r.nope[e] = *reinterpret_cast<const u32x2*>(a.kn + rr * a.kn_stride + lane * 8);
        else
            r.nope[e] = *reinterpret_cast<const u32x4*>(a.kn + rr * a.kn_stride + lane * 16);
    }
    {
        const int row = rows[tile * T + (tid >> 3)];
        const int64_t rr = row < 0 ? 0 : row;
        absent |= (row < 0 ? 1u : 0u) << 8;
        r.rope = *reinterpret_cast<const u32x4*>(a.kr + rr * a.kr_stride + (tid & 7) * 16);
    }
    r.absent = absent;
}

__device__ __forceinline__ float i8_at(uint32_t w, int k) { return (float)(int8_t)(w >> (8 * k)); }

// Dequantise rows [E0, E1) of this lane's 8 rows x 8 columns and store them into an LDS stage; with ROPE also
// the lane's rope piece.
template <bool QUANT, int E0, int E1, bool ROPE>
__device__ __forceinline__ void dequant_store(const RawTile<QUANT>& r, uint8_t* stage, const float* scales, int tile,
                                              int wave, int lane, int tid)
{
#pragma unroll
    for (int e = E0; e < E1; ++e) {
        const int t = 8 * wave + e;
        u32x4 v;
        if constexpr (QUANT) {
            const float s = scales[(tile * T + t) * 4 + (lane >> 4)]; // 0 for an absent row
            uint32_t w0 = r.nope[e][0], w1 = r.nope[e][1];
            // keep the unpacking here: hoisted to the load, it would wait for the load right after issuing it
            asm volatile("" : "+v"(w0), "+v"(w1));
            v[0] = pack_bf16x2(i8_at(w0, 0) * s, i8_at(w0, 1) * s);
            v[1] = pack_bf16x2(i8_at(w0, 2) * s, i8_at(w0, 3) * s);
            v[2] = pack_bf16x2(i8_at(w1, 0) * s, i8_at(w1, 1) * s);
            v[3] = pack_bf16x2(i8_at(w1, 2) * s, i8_at(w1, 3) * s);
        } else {
            u32x4 w = r.nope[e];
            asm volatile("" : "+v"(w)); // as above: consume the load here, not where it was issued
            v = ((r.absent >> e) & 1u) ? u32x4{0u, 0u, 0u, 0u} : w;
        }
        *reinterpret_cast<u32x4*>(stage + t * KROW + ((lane ^ swz(t)) << 4)) = v;
    }
    if constexpr (ROPE) {
        const int t = tid >> 3;
        u32x4 rp = r.rope;
        asm volatile("" : "+v"(rp));
        rp = ((r.absent >> 8) & 1u) ? u32x4{0u, 0u, 0u, 0u} : rp;
        *reinterpret_cast<u32x4*>(stage + t * KROW + DN * 2 + (((tid & 7) ^ swz(t)) << 4)) = rp;
    }
}

template <bool QUANT>
__global__ __attribute__((amdgpu_flat_work_group_size(512, 512), amdgpu_waves_per_eu(2, 2))) void sfa_decode_kernel(
    SfaArgs a)
{
    extern __shared__ __align__(16) uint8_t smem[];
    int* rows = reinterpret_cast<int*>(smem + ROWS_OFF);
    float* scales = reinterpret_cast<float*>(smem + SCALES_OFF);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sp = blockIdx.x, tq = blockIdx.y, hz = blockIdx.z;
    const int bi = tq / a.s1, si = tq - bi * a.s1;

    int cur = a.act_seq[bi] - a.s1 + 1 + si;
    cur = min(max(cur, 0), a.topk);
    const int ntiles_all = (cur + T - 1) / T;
    const int per = (ntiles_all + a.nsplit - 1) / a.nsplit;
    const int tile0 = sp * per;
    const int ntiles_real = max(min(ntiles_all, tile0 + per) - tile0, 0);
    // an even number of tiles keeps the producer loop free of conditional loads (the odd one out is fully masked)
    const int ntiles = (ntiles_real + 1) & ~1;
    const int tok0 = tile0 * T;

    // logical top-k entries of this split -> physical cache rows (or -1: absent), and their 4 dequant scales
    const int64_t max_logical = (int64_t)a.bt_stride * a.block_size;
    for (int i = tid; i < ntiles * T; i += 512) {
        const int g = tok0 + i;
        int row = -1;
        if (g < cur && i < ntiles_real * T) { // the padding tile holds no token
            const int idx = a.topk_idx[(int64_t)tq * a.topk_stride + g];
            if (idx >= 0 && idx < max_logical) {
                const int page = a.block_table[(int64_t)bi * a.bt_stride + idx / a.block_size];
                const int64_t r = (int64_t)page * a.block_size + idx % a.block_size;
                if (page >= 0 && r < a.n_rows) row = (int)r;
            }
        }
        rows[i] = row;
        if constexpr (QUANT) {
            f32x4 sc = {0.f, 0.f, 0.f, 0.f};
            if (row >= 0) sc = *reinterpret_cast<const f32x4*>(a.ks + (int64_t)row * a.ks_stride);
            *reinterpret_cast<f32x4*>(scales + i * 4) = sc;
        }
    }
    __syncthreads(); // rows[] / scales[] ready

    // Both roles run the same barrier sequence: one before the first tile, then two per tile
    // (partial S exchanged; tile consumed and next tile stored).
    if (wave >= 4) {
        // ---------------------------------------------------------------- producer wavefronts
        // Gathered rows travel global -> registers -> LDS.  Two register tiles alternate so that the loads of
        // a tile are issued two tiles before it is dequantised.
        const int pw = wave - 4, ptid = tid - 256;
        const int last = ntiles - 1;
        RawTile<QUANT> raw0, raw1;
        if (ntiles > 0) {
            load_raw<QUANT>(raw0, a, rows, 0, pw, lane, ptid);
            load_raw<QUANT>(raw1, a, rows, 1, pw, lane, ptid);
            dequant_store<QUANT, 0, 8, true>(raw0, smem, scales, 0, pw, lane, ptid);
            load_raw<QUANT>(raw0, a, rows, min(2, last), pw, lane, ptid);
        }
        __syncthreads();
        // Every step stores one tile and issues the loads of another, unconditionally (past the end the last
        // tile is loaded again and stored into a stage nobody reads): with a fixed number of loads in flight
        // on every path the wait for a tile leaves the younger tile's loads outstanding.
        // The consumers spend about a third of a tile before their mid-tile barrier (half of S) and two thirds
        // after it (softmax, PV); the store of the next tile is split the same way around that barrier.
        auto produce = [&](int it, RawTile<QUANT>& next) {
            uint8_t* dst = smem + ((it + 1) & 1) * STAGE;
            dequant_store<QUANT, 0, 3, false>(next, dst, scales, min(it + 1, last), pw, lane, ptid);
            __syncthreads();
            dequant_store<QUANT, 3, 8, true>(next, dst, scales, min(it + 1, last), pw, lane, ptid);
            load_raw<QUANT>(next, a, rows, min(it + 3, last), pw, lane, ptid);
            __syncthreads();
        };
        for (int it = 0; it < ntiles; it += 2) {
            produce(it, raw1);
            produce(it + 1, raw0);
        }
        return;
    }

    // -------------------------------------------------------------------- consumer wavefronts
    const int l32 = lane & 31, hl = lane >> 5;
    const int hg = wave >> 1, kh = wave & 1; // head group of 32 within the workgroup; k-step / dim-block parity

    // this lane's query head and its Q slice: k-steps 2*i + kh, i = 0..17 (0..15 nope, 16..17 rope); B operand
    // layout: head = column, 8 consecutive k per half-wave.  Lanes past the last head reuse head 0's rows,
    // their results are never written.
    const int head = hz * HEADS_PER_WG + hg * 32 + l32;
    const bool head_ok = head < a.nq;
    const bool wave_active = hz * HEADS_PER_WG + hg * 32 < a.nq;
    bf16x8 q[KSTEPS / 2];
    {
        const int64_t qrow = (int64_t)tq * a.nq + (head_ok ? head : 0);
        const __bf16* qn = reinterpret_cast<const __bf16*>(a.q_nope) + qrow * DN + kh * 16 + hl * 8;
        const __bf16* qr = reinterpret_cast<const __bf16*>(a.q_rope) + qrow * DR + kh * 16 + hl * 8;
#pragma unroll
        for (int i = 0; i < DN / 32; ++i) q[i] = *reinterpret_cast<const bf16x8*>(qn + i * 32);
#pragma unroll
        for (int i = 0; i < DR / 32; ++i) q[DN / 32 + i] = *reinterpret_cast<const bf16x8*>(qr + i * 32);
    }

    f32x16 o[8]; // O^T blocks db = 2*i + kh: dims [32*db, 32*db + 32) x 32 heads
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
    float m_run = -INFINITY; // running max of S * scale * log2(e)
    float l_run = 0.f;       // this lane's share of sum exp
    const float c_log2 = a.softmax_scale * 1.4426950408889634f;

    // S operand (b128): row l32, chunk 2*ks + hl with ks = 2*i + kh -> chunk 4*i + 2*kh + hl; swizzled offsets
    // for even and odd i
    uint32_t s_off[2];
    {
        const int sw = swz(l32), c = 2 * kh + hl;
        s_off[0] = l32 * KROW + ((c ^ sw) << 4);
        s_off[1] = l32 * KROW + (((4 + c) ^ sw) << 4);
    }
    // V^T operand (transpose read): lane jj of 16-lane group G points at row 4*hl + jj/4 (+ 16*j + 8*h2),
    // columns 32*db + 16*(G&1) + 4*(jj&3) with db = 2*i + kh -> chunk 8*i + 4*kh + 2*(G&1) + (jj&3)/2
    uint32_t v_off;
    {
        const int jj = lane & 15, mh = (lane >> 4) & 1;
        const int cl = 4 * kh + 2 * mh + ((jj & 3) >> 1);
        const int sw = ((jj >> 2) << 1) | hl;
        v_off = (4 * hl + (jj >> 2)) * KROW + (jj & 1) * 8 + ((cl ^ sw) << 4);
    }
    uint8_t* xmine = smem + XBUF_OFF + wave * 4096 + lane * 16;
    uint8_t* xpeer = smem + XBUF_OFF + (wave ^ 1) * 4096 + lane * 16;

    __syncthreads(); // tile 0 stored

    for (int it = 0; it < ntiles; ++it) {
        uint8_t* stage = smem + (it & 1) * STAGE;
        const uint32_t valid = (uint32_t)__ballot(rows[it * T + l32] >= 0);
        // half of S^T[token, head] = K[token, :] . Q[head, :] (k-steps of parity kh)
        f32x16 s;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.f;
        {
            // operand reads run three k-steps ahead of the MFMAs that use them
            constexpr int AHEAD = 3;
            bf16x8 kf[KSTEPS / 2];
#pragma unroll
            for (int i = 0; i < AHEAD; ++i)
                kf[i] = *reinterpret_cast<const bf16x8*>(stage + s_off[i & 1] + (i >> 1) * 128);
#pragma unroll
            for (int i = 0; i < KSTEPS / 2; ++i) {
                if (i + AHEAD < KSTEPS / 2)
                    kf[i + AHEAD] =
                        *reinterpret_cast<const bf16x8*>(stage + s_off[(i + AHEAD) & 1] + ((i + AHEAD) >> 1) * 128);
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i], q[i], s, 0, 0, 0);
            }
            // issue order: AHEAD reads, then (MFMA, read) pairs, then the last MFMAs
            __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
#pragma unroll
            for (int i = 0; i < KSTEPS / 2 - AHEAD; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // one LDS read
            }
            __builtin_amdgcn_sched_group_barrier(0x008, AHEAD, 0);
        }
#pragma unroll
        for (int g = 0; g < 4; ++g)
            *reinterpret_cast<f32x4*>(xmine + g * 1024) = f32x4{s[4 * g], s[4 * g + 1], s[4 * g + 2], s[4 * g + 3]};
        __syncthreads(); // partial S of both waves of each pair is in LDS
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const f32x4 p = *reinterpret_cast<const f32x4*>(xpeer + g * 1024);
            s[4 * g] += p[0];
            s[4 * g + 1] += p[1];
            s[4 * g + 2] += p[2];
            s[4 * g + 3] += p[3];
        }
        if (wave_active && valid != 0u) {
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
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new); // 0 on the first tile (m_run = -inf)
                l_run *= alpha;
#pragma unroll
                for (int i = 0; i < 8; ++i)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o[i][r] *= alpha;
                m_run = m_new;
            }
            uint32_t pb[8];
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                const float p0 = __builtin_amdgcn_exp2f(s[r] - m_run), p1 = __builtin_amdgcn_exp2f(s[r + 1] - m_run);
                l_run += p0 + p1;
                pb[r >> 1] = pack_bf16x2(p0, p1);
            }
            // O^T[dim, head] += V^T[dim, token] . P~[token, head]; k-slot s of half hl in block j is token
            // 16*j + 8*(s/4) + 4*hl + s%4, the order in which the S^T registers hold the tokens
            {
                bf16x8 pf[2];
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    u32x4 pw = {pb[4 * j], pb[4 * j + 1], pb[4 * j + 2], pb[4 * j + 3]};
                    pf[j] = __builtin_bit_cast(bf16x8, pw);
                }
                // 16 MFMAs (j, i); their two transpose reads each run two MFMAs ahead
                constexpr int AHEAD = 2;
                s16x4 lo[16], hi[16];
                auto vread = [&](int n) {
                    uint8_t* vp = stage + v_off + (16 * (n >> 3)) * KROW + (n & 7) * 128;
                    lo[n] = lds_read_tr(vp);
                    hi[n] = lds_read_tr(vp + 8 * KROW);
                };
#pragma unroll
                for (int n = 0; n < AHEAD; ++n) vread(n);
#pragma unroll
                for (int n = 0; n < 16; ++n) {
                    if (n + AHEAD < 16) vread(n + AHEAD);
                    const s16x8 both = __builtin_shufflevector(lo[n], hi[n], 0, 1, 2, 3, 4, 5, 6, 7);
                    o[n & 7] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, both), pf[n >> 3],
                                                                       o[n & 7], 0, 0, 0);
                }
                __builtin_amdgcn_sched_group_barrier(0x100, 2 * AHEAD, 0);
#pragma unroll
                for (int n = 0; n < 16 - AHEAD; ++n) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // one MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0); // two LDS reads
                }
                __builtin_amdgcn_sched_group_barrier(0x008, AHEAD, 0);
            }
        }
        __syncthreads(); // tile consumed: its stage and the exchange buffer may be overwritten
    }

    if (!wave_active) return;
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    if (!head_ok) return;
    // register r of o[i] holds dim 32*(2*i + kh) + 8*(r/4) + 4*hl + r%4 of head l32
    if (a.nsplit == 1) {
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        uint8_t* dst = reinterpret_cast<uint8_t*>(a.out) + ((int64_t)tq * a.nq + head) * DN * 2;
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                u32x2 v = {pack_bf16x2(o[i][4 * g] * inv, o[i][4 * g + 1] * inv),
                           pack_bf16x2(o[i][4 * g + 2] * inv, o[i][4 * g + 3] * inv)};
                *reinterpret_cast<u32x2*>(dst + (32 * (2 * i + kh) + 8 * g + 4 * hl) * 2) = v;
            }
    } else {
        const int64_t prow = ((int64_t)tq * a.nsplit + sp) * a.nq + head;
        float* dst = a.part_o + prow * DN;
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f32x4 v = {o[i][4 * g], o[i][4 * g + 1], o[i][4 * g + 2], o[i][4 * g + 3]};
                *reinterpret_cast<f32x4*>(dst + 32 * (2 * i + kh) + 8 * g + 4 * hl) = v;
            }
        if (hl == 0 && kh == 0) {
            a.part_ml[prow * 2] = m_run;
            a.part_ml[prow * 2 + 1] = l_tot;
        }
    }
}

// attention_out <- 0 (cache without rows: every selected entry is absent)
__global__ void sfa_zero_kernel(uint32_t* out, int64_t n_words)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_words) out[i] = 0u;
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
    if (a.n_rows == 0) {
        const int64_t words = (int64_t)t * a.nq * DN / 2;
        hipLaunchKernelGGL(sfa_zero_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream,
                           static_cast<uint32_t*>(a.out), words);
        return hipGetLastError();
    }
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
        hipLaunchKernelGGL(kern, grid, dim3(512), SMEM_BYTES, stream, a);
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
