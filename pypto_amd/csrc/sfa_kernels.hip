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
constexpr int MAX_SPLIT_TOKENS = 2048; // largest share of a top-k list one workgroup may own
constexpr int NREG_KSTEPS = 12;        // of a wave's 18 k-steps of Q, these stay in registers ...
constexpr int NPARK = KSTEPS / 2 - NREG_KSTEPS; // ... and these are parked in LDS (16 bytes per lane each)
// LDS layout: two tile stages | S exchange | parked Q | per-split arrays sized by SfaArgs::split_cap
// (validity words, rows) | this sequence's page table (when it fits)
constexpr int XBUF_OFF = 2 * STAGE;
constexpr int QPARK_OFF = XBUF_OFF + 4 * 4096;
constexpr int SPLIT_OFF = QPARK_OFF + 4 * NPARK * 1024; // 114688
constexpr int LDS_LIMIT = 160 * 1024;
constexpr int OUT_ROW = DN * 4;  // epilogue staging: 64 heads x 512 fp32, reusing the front of LDS
__host__ __device__ constexpr int tmask_bytes(int cap) { return (cap / T + 2) * 4; }
__host__ __device__ constexpr int split_bytes(int cap) { return tmask_bytes(cap) + cap * 4; }
static_assert(64 * OUT_ROW <= LDS_LIMIT, "epilogue staging must fit");
constexpr int HEADS_PER_WG = 64;

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
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
    float sc[8];   // the rows' dequant scales for this lane's column group
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
// rows[] holds valid cache rows only (absent entries point at row 0); the tile's validity word says which
// rows are absent, and their data is zeroed when it is consumed (dequant_store), so that no load has to be
// waited for here.
template <bool QUANT>
__device__ __forceinline__ void load_raw(RawTile<QUANT>& r, const SfaArgs& a, const int* rows, const uint32_t* tmask,
                                         int tile, int wave, int lane, int tid)
{
    // the 8 rows are the same for every lane of the wavefront: two 16-byte LDS reads, then scalar address arithmetic
    // (the loads take a scalar base and the lane's column offset)
    const u32x4 ra = *reinterpret_cast<const u32x4*>(rows + tile * T + 8 * wave);
    const u32x4 rb = *reinterpret_cast<const u32x4*>(rows + tile * T + 8 * wave + 4);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t row = __builtin_amdgcn_readfirstlane(e < 4 ? ra[e & 3] : rb[e & 3]);
        if constexpr (QUANT) {
            r.nope[e] = *reinterpret_cast<const u32x2*>(a.kn + (uint64_t)row * a.kn_stride + lane * 8);
            r.sc[e] = *reinterpret_cast<const float*>(a.ks + (uint64_t)row * a.ks_stride + (lane >> 4) * 4);
        } else
            r.nope[e] = *reinterpret_cast<const u32x4*>(a.kn + (uint64_t)row * a.kn_stride + lane * 16);
    }
    const uint32_t row = (uint32_t)rows[tile * T + (tid >> 3)];
    r.rope = *reinterpret_cast<const u32x4*>(a.kr + (uint64_t)row * a.kr_stride + (tid & 7) * 16);
    const uint32_t present = tmask[tile];
    r.absent = ((~present >> (8 * wave)) & 0xffu) | (((~present >> (tid >> 3)) & 1u) << 8);
}

// int8 -> fp32 -> * scale with one conversion and one fma per element: byte k of w holds x + 128 (the caller
// flips the sign bits), so x * s = fma(float(byte), s, -128 s); -128 s is exact, hence one rounding, the same
// as rounding the product x * s.
__device__ __forceinline__ float dq(uint32_t w, int k, float s, float neg128s)
{
    return __builtin_fmaf((float)((w >> (8 * k)) & 0xffu), s, neg128s);
}

// Dequantise rows [E0, E1) of this lane's 8 rows x 8 columns and store them into an LDS stage; with ROPE also
// the lane's rope piece.
template <bool QUANT, int E0, int E1, bool ROPE>
__device__ __forceinline__ void dequant_store(const RawTile<QUANT>& r, uint8_t* stage, int wave, int lane, int tid)
{
#pragma unroll
    for (int e = E0; e < E1; ++e) {
        const int t = 8 * wave + e;
        u32x4 v;
        if constexpr (QUANT) {
            uint32_t w0 = r.nope[e][0], w1 = r.nope[e][1];
            float s = r.sc[e];
            // keep the unpacking here: hoisted to the load, it would wait for the load right after issuing it
            asm volatile("" : "+v"(w0), "+v"(w1), "+v"(s));
            s = ((r.absent >> e) & 1u) ? 0.f : s; // an absent row is stored as zeros
            w0 ^= 0x80808080u;
            w1 ^= 0x80808080u;
            const float c = -128.f * s;
            v[0] = pack_bf16x2(dq(w0, 0, s, c), dq(w0, 1, s, c));
            v[1] = pack_bf16x2(dq(w0, 2, s, c), dq(w0, 3, s, c));
            v[2] = pack_bf16x2(dq(w1, 0, s, c), dq(w1, 1, s, c));
            v[3] = pack_bf16x2(dq(w1, 2, s, c), dq(w1, 3, s, c));
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

// Resolves a workgroup's share of a token's top-k list: logical indices -> physical cache rows (absent entries: row 0
// and a cleared bit in the tile's validity word), in LDS.  NT lanes.
template <int NT>
__device__ __forceinline__ void resolve_split(const SfaArgs& a, int bi, int tq, int tok0, int cur, int ntiles_real,
                                              int ntiles, uint32_t* tmask, int* rows, int* bt_lds, int tid,
                                              int lane)
{
    // this sequence's page table -> LDS (saves one dependent global load per selected token)
    const bool bt_cached = a.bt_cached != 0;
    if (bt_cached)
        for (int i = tid; i < a.bt_stride; i += NT) bt_lds[i] = a.block_table[(int64_t)bi * a.bt_stride + i];
    // logical top-k entries of this split
    const int64_t max_logical = (int64_t)a.bt_stride * a.block_size;
    int my_idx[MAX_SPLIT_TOKENS / NT];
#pragma unroll
    for (int j = 0; j < MAX_SPLIT_TOKENS / NT; ++j) {
        const int i = tid + NT * j, g = tok0 + i;
        my_idx[j] = -1;
        if (i < ntiles_real * T && g < cur) my_idx[j] = a.topk_idx[(int64_t)tq * a.topk_stride + g];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < MAX_SPLIT_TOKENS / NT; ++j) {
        const int i = tid + NT * j;
        if (i >= ntiles * T) break; // wave-uniform: tiles are 32 wide, waves 64
        const int idx = my_idx[j];
        int row = -1;
        if (idx >= 0 && idx < max_logical) {
            const int page = bt_cached ? bt_lds[idx / a.block_size]
                                       : a.block_table[(int64_t)bi * a.bt_stride + idx / a.block_size];
            const int64_t r = (int64_t)page * a.block_size + idx % a.block_size;
            if (page >= 0 && r < a.n_rows) row = (int)r;
        }
        rows[i] = max(row, 0);
        const uint64_t present = __ballot(row >= 0);
        if (lane == 0) {
            tmask[i >> 5] = (uint32_t)present;
            tmask[(i >> 5) + 1] = (uint32_t)(present >> 32);
        }
    }
    __syncthreads(); // rows[] / tmask[] ready
}

template <bool QUANT>
__global__ __attribute__((amdgpu_flat_work_group_size(512, 512), amdgpu_waves_per_eu(2, 2))) void sfa_decode_kernel(
    SfaArgs a)
{
    extern __shared__ __align__(16) uint8_t smem[];
    uint32_t* tmask = reinterpret_cast<uint32_t*>(smem + SPLIT_OFF);
    int* rows = reinterpret_cast<int*>(smem + SPLIT_OFF + tmask_bytes(a.split_cap));
    int* bt_lds = reinterpret_cast<int*>(smem + SPLIT_OFF + split_bytes(a.split_cap));

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

    resolve_split<512>(a, bi, tq, tok0, cur, ntiles_real, ntiles, tmask, rows, bt_lds, tid, lane);

    // Both roles run the same barrier sequence: one before the first tile, then two per tile
    // (partial S exchanged; tile consumed and next tile stored).
    if (wave >= 4) {
        // ---------------------------------------------------------------- producer wavefronts
        // Gathered rows travel global -> registers -> LDS.  Two register tiles alternate so that the loads of
        // a tile are issued two tiles before it is dequantised.
        const int pw = wave - 4, ptid = tid - 256;
        const int last = ntiles - 1;
        RawTile<QUANT> raw0, raw1;
        // (tile 0 is gathered and stored by the consumer wavefronts, which would otherwise idle here: the cold first
        // gathers are slow to issue, and two sets of waves issue them side by side)
        if (ntiles > 0) {
            load_raw<QUANT>(raw1, a, rows, tmask, 1, pw, lane, ptid);
            load_raw<QUANT>(raw0, a, rows, tmask, min(2, last), pw, lane, ptid);
        }
        __syncthreads();
        // Every step stores one tile and issues the loads of another, unconditionally (past the end the last
        // tile is loaded again and stored into a stage nobody reads): with a fixed number of loads in flight
        // on every path the wait for a tile leaves the younger tile's loads outstanding.
        // The store of the next tile is split around the consumers' mid-tile barrier: most of it runs beside the
        // S MFMAs, the rest (and the loads of a later tile) beside softmax and PV.
        auto produce = [&](int it, RawTile<QUANT>& next) {
            uint8_t* dst = smem + ((it + 1) & 1) * STAGE;
            dequant_store<QUANT, 0, 5, false>(next, dst, pw, lane, ptid);
            __syncthreads();
            dequant_store<QUANT, 5, 8, true>(next, dst, pw, lane, ptid);
            load_raw<QUANT>(next, a, rows, tmask, min(it + 3, last), pw, lane, ptid);
            __syncthreads();
        };
        for (int it = 0; it < ntiles; it += 2) {
            produce(it, raw1);
            produce(it + 1, raw0);
        }
    } else {
    // -------------------------------------------------------------------- consumer wavefronts
    const int l32 = lane & 31, hl = lane >> 5;
    const int hg = wave >> 1, kh = wave & 1; // head group of 32 within the workgroup; k-step / dim-block parity

    // this lane's query head and its Q slice: k-steps 2*i + kh, i = 0..17 (0..15 nope, 16..17 rope); B operand
    // layout: head = column, 8 consecutive k per half-wave.  Lanes past the last head reuse head 0's rows,
    // their results are never written.
    const int head = hz * HEADS_PER_WG + hg * 32 + l32;
    const bool head_ok = head < a.nq;
    const bool wave_active = hz * HEADS_PER_WG + hg * 32 < a.nq;
    // 12 k-steps stay in registers; the other 6 (4 nope, 2 rope) are parked in LDS and read back by the same lane
    // every tile, which keeps the consumer inside its 256 registers.
    bf16x8 q[NREG_KSTEPS];
    uint8_t* qpark = smem + QPARK_OFF + wave * (NPARK * 1024) + lane * 16;
    RawTile<QUANT> first; // tile 0: wave w takes rows 8w .. 8w + 7, as producer wave w does for the later tiles
    if (ntiles > 0) load_raw<QUANT>(first, a, rows, tmask, 0, wave, lane, tid);
    {
        const int64_t qrow = (int64_t)tq * a.nq + (head_ok ? head : 0);
        const __bf16* qn = reinterpret_cast<const __bf16*>(a.q_nope) + qrow * DN + kh * 16 + hl * 8;
        const __bf16* qr = reinterpret_cast<const __bf16*>(a.q_rope) + qrow * DR + kh * 16 + hl * 8;
#pragma unroll
        for (int i = 0; i < KSTEPS / 2; ++i) {
            const bf16x8 v = *reinterpret_cast<const bf16x8*>(i < DN / 32 ? qn + i * 32 : qr + (i - DN / 32) * 32);
            if (i < NREG_KSTEPS)
                q[i < NREG_KSTEPS ? i : 0] = v;
            else
                *reinterpret_cast<bf16x8*>(qpark + (i - NREG_KSTEPS) * 1024) = v;
        }
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

    if (ntiles > 0) dequant_store<QUANT, 0, 8, true>(first, smem, wave, lane, tid);
    __syncthreads(); // tile 0 stored

    for (int it = 0; it < ntiles; ++it) {
        uint8_t* stage = smem + (it & 1) * STAGE;
        const uint32_t valid = tmask[it];
        // half of S^T[token, head] = K[token, :] . Q[head, :] (k-steps of parity kh)
        // One accumulation chain: a second one (even / odd k-steps) saves the few cycles a dependent MFMA waits for its
        // predecessor, but its 16 registers are worth more as two further operand reads in flight.
        f32x16 s;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.f;
        {
            // operand reads run AHEAD k-steps ahead of the MFMAs that use them
            constexpr int AHEAD = 4, N = KSTEPS / 2;
            bf16x8 kf[N], qp[N];
            auto fetch = [&](int i) {
                kf[i] = *reinterpret_cast<const bf16x8*>(stage + s_off[i & 1] + (i >> 1) * 128);
                if (i >= NREG_KSTEPS) qp[i] = *reinterpret_cast<const bf16x8*>(qpark + (i - NREG_KSTEPS) * 1024);
            };
#pragma unroll
            for (int i = 0; i < AHEAD; ++i) fetch(i);
#pragma unroll
            for (int i = 0; i < N; ++i) {
                if (i + AHEAD < N) fetch(i + AHEAD);
                const bf16x8 qi = i < NREG_KSTEPS ? q[i < NREG_KSTEPS ? i : 0] : qp[i];
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i], qi, s, 0, 0, 0);
            }
            // issue order: AHEAD fetches, then (MFMA, fetch) pairs, then the last MFMAs; a fetch is one LDS read
            // for a k-step whose Q fragment is in registers and two for a parked one
            __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
#pragma unroll
            for (int i = 0; i < NREG_KSTEPS - AHEAD; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
#pragma unroll
            for (int i = NREG_KSTEPS - AHEAD; i < N - AHEAD; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, AHEAD, 0);
        }
#pragma unroll
        for (int g = 0; g < 4; ++g)
            *reinterpret_cast<f32x4*>(xmine + g * 1024) = f32x4{s[4 * g], s[4 * g + 1], s[4 * g + 2], s[4 * g + 3]};
        __syncthreads(); // partial S of both waves of each pair is in LDS
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const f32x4 p = *reinterpret_cast<const f32x4*>(xmine + (kh ? -4096 : 4096) + g * 1024);
            s[4 * g] += p[0];
            s[4 * g + 1] += p[1];
            s[4 * g + 2] += p[2];
            s[4 * g + 3] += p[3];
        }
        if (wave_active && valid != 0u) {
            // register r holds token 8*(r/4) + 4*hl + r%4 for head l32; statistics on the raw scores
            // (softmax_scale > 0 commutes with max), exponent argument by one fma per score
            float mx = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                if (valid != 0xffffffffu) {
                    const int tok = 8 * (r >> 2) + 4 * hl + (r & 3);
                    s[r] = ((valid >> tok) & 1u) ? s[r] : -INFINITY;
                }
                mx = fmaxf(mx, s[r]);
            }
            {
                // maximum over both halves of the wavefront without a trip through LDS: v_permlane32_swap exchanges the
                // upper half of its first operand with the lower half of its second
                const auto sw = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, mx), __builtin_bit_cast(unsigned, mx), false, false);
                mx = fmaxf(__builtin_bit_cast(float, (unsigned)sw[0]), __builtin_bit_cast(float, (unsigned)sw[1])) * c_log2;
            }
            // The reference exponent only follows the running maximum when it has grown by more than 2^8: until
            // then P~ = 2^(z - m_run) may exceed 1 (by at most 2^8, no issue for bf16 or the fp32 sums), which
            // makes the rescale of the 128 accumulator registers a rare event.  Every P~, l and O stay relative to
            // the same m_run, so the result is unchanged.
            const float m_new = fmaxf(m_run, mx);
            if (__any(m_new > m_run + 8.f)) {
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
                const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], c_log2, -m_run));
                const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r + 1], c_log2, -m_run));
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
                // 16 MFMAs (j, i); their two transpose reads each run AHEAD MFMAs ahead
                constexpr int AHEAD = 3;
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

    // Epilogue, part 1: O^T blocks -> LDS as [head][512] fp32 rows (the tile stages are free now), 16-byte
    // chunks XOR-swizzled with the head so that the 8 lanes of a b128 write hit distinct banks.  Register r of
    // o[i] holds dim 32*(2*i + kh) + 8*(r/4) + 4*hl + r%4 of head l32.
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    const float mul = l_tot > 0.f ? 1.f / l_tot : 0.f; // splits hand over their normalised output as well
    const int hrow = hg * 32 + l32;
    uint8_t* orow = smem + hrow * OUT_ROW;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int c = 8 * (2 * i + kh) + 2 * g + hl;
            const f32x4 v = {o[i][4 * g] * mul, o[i][4 * g + 1] * mul, o[i][4 * g + 2] * mul, o[i][4 * g + 3] * mul};
            *reinterpret_cast<f32x4*>(orow + ((c ^ (hrow & 7)) << 4)) = v;
        }
    if (a.nsplit > 1 && head_ok && hl == 0 && kh == 0) {
        const int64_t prow = ((int64_t)tq * a.nsplit + sp) * a.nq + head;
        a.part_ml[prow * 2] = m_run;
        a.part_ml[prow * 2 + 1] = l_tot;
    }
    } // consumer
    __syncthreads();

    // Epilogue, part 2: all 512 lanes copy the 64 rows out, a wavefront writing 1 KB (fp32 partial) or 512 B
    // (bf16 output) of one row per instruction.
#pragma unroll 4
    for (int id = tid; id < HEADS_PER_WG * (DN / 4); id += 512) {
        const int hrow = id / (DN / 4), c = id % (DN / 4);
        const int head = hz * HEADS_PER_WG + hrow;
        if (head >= a.nq) continue;
        const f32x4 v = *reinterpret_cast<const f32x4*>(smem + hrow * OUT_ROW + ((c ^ (hrow & 7)) << 4));
        if (a.nsplit == 1) {
            const u32x2 w = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
            *reinterpret_cast<u32x2*>(reinterpret_cast<uint8_t*>(a.out) + (((int64_t)tq * a.nq + head) * DN + c * 4) * 2) = w;
        } else {
            // a split's share, normalised by its own sum, in fp16: |value| <= max |V| and 2^-11 relative rounding, a
            // quarter of the final bf16 rounding; half the bytes of fp32 for this kernel to write and the merge to read
            const int64_t prow = ((int64_t)tq * a.nsplit + sp) * a.nq + head;
            const f16x4 hv = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
            *reinterpret_cast<f16x4*>(a.part_o + prow * DN + c * 4) = hv;
        }
    }
}

// attention_out <- 0 (cache without rows: every selected entry is absent)
__global__ void sfa_zero_kernel(uint32_t* out, int64_t n_words)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_words) out[i] = 0u;
}

// out[row, :] = sum_s (2^(m_s - M) l_s / L) o_s[row, :] with L = sum_s 2^(m_s - M) l_s and o_s the split's normalised
// output; one block of 128 lanes per output row.  Splits are taken four at a time, every load of a group requested
// before any is used (splits past the last are the last again with weight 0).
__global__ __launch_bounds__(128) void sfa_combine_kernel(const void* __restrict__ part_o_fp16,
                                                          const float* __restrict__ part_ml, void* out, int nq,
                                                          int nsplit)
{
    const _Float16* part_o = static_cast<const _Float16*>(part_o_fp16); // (a plain pointer type keeps the symbol readable)
    const int row = blockIdx.x; // tq * nq + head
    const int tq = row / nq, head = row - tq * nq;
    float M = -INFINITY;
    for (int s = 0; s < nsplit; ++s) M = fmaxf(M, part_ml[(((int64_t)tq * nsplit + s) * nq + head) * 2]);
    float L = 0.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    if (M > -INFINITY) {
        for (int s0 = 0; s0 < nsplit; s0 += 4) {
            f16x4 v[4];
            float w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int64_t prow = ((int64_t)tq * nsplit + min(s0 + j, nsplit - 1)) * nq + head;
                v[j] = *reinterpret_cast<const f16x4*>(part_o + prow * DN + threadIdx.x * 4);
                const float m = part_ml[prow * 2], l = part_ml[prow * 2 + 1];
                w[j] = (s0 + j < nsplit && l > 0.f) ? exp2f(m - M) * l : 0.f;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                L += w[j];
                acc += f32x4{(float)v[j][0], (float)v[j][1], (float)v[j][2], (float)v[j][3]} * w[j];
            }
        }
    }
    const float inv = L > 0.f ? 1.f / L : 0.f;
    u32x2 v = {pack_bf16x2(acc[0] * inv, acc[1] * inv), pack_bf16x2(acc[2] * inv, acc[3] * inv)};
    *reinterpret_cast<u32x2*>(reinterpret_cast<uint8_t*>(out) + ((int64_t)row * DN + threadIdx.x * 4) * 2) = v;
}

int num_cus()
{
    static std::atomic<int> cached[64]; // per device ordinal; 0 = not asked yet
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    n = cached[dev & 63].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev & 63].store(n, std::memory_order_relaxed);
    }
    return n;
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
    return (uint64_t)t * nsplit * nq * (DN * sizeof(_Float16) + 2 * sizeof(float));
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
    SfaArgs args = a;
    const int tiles = (a.topk + T - 1) / T;
    args.split_cap = (((tiles + a.nsplit - 1) / a.nsplit + 1) & ~1) * T;
    int smem_bytes = SPLIT_OFF + split_bytes(args.split_cap);
    args.bt_cached = smem_bytes + a.bt_stride * 4 <= LDS_LIMIT ? 1 : 0;
    if (args.bt_cached) smem_bytes += a.bt_stride * 4;
    if (smem_bytes < HEADS_PER_WG * OUT_ROW) smem_bytes = HEADS_PER_WG * OUT_ROW; // epilogue staging
    static DeviceOnce attr_done[2];
    auto kern = a.quant ? sfa_decode_kernel<true> : sfa_decode_kernel<false>;
    {
        hipError_t e = attr_done[a.quant].run([&] {
            return hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       LDS_LIMIT);
        });
        if (e != hipSuccess) return e;
    }
    const int hgroups = (a.nq + HEADS_PER_WG - 1) / HEADS_PER_WG;
    dim3 grid(a.nsplit, t, hgroups);
    {
        ScopedKernelTimer tm(KID_SFA_DECODE, stream);
        hipLaunchKernelGGL(kern, grid, dim3(512), smem_bytes, stream, args);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (a.nsplit > 1) {
        ScopedKernelTimer tm(KID_SFA_COMBINE, stream);
        hipLaunchKernelGGL(sfa_combine_kernel, dim3(t * a.nq), dim3(128), 0, stream, static_cast<const void*>(a.part_o), a.part_ml, a.out, a.nq,
                           a.nsplit);
        e = hipGetLastError();
    }
    return e;
}

} // namespace pto
