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
// Work decomposition.  One workgroup of eight wavefronts owns one (query token, KV split, group of 128 heads) and
// walks its share of the token's top-k list in tiles of 32 selected cache rows; every gathered row is dequantised
// once for all 128 heads.  The dequantised tile sits row-major in LDS (16-byte chunks XOR-swizzled with the row),
// double buffered, and serves as K (row reads) and as V (transposing reads, ds_read_b64_tr_b16).  All eight
// wavefronts issue MFMAs (v_mfma_f32_32x32x16_bf16), two per SIMD, and each has two roles:
//   * scores: wave (hg, kh) computes S^T = K Q^T for the 32 heads of group hg over half of the 576-wide
//     contraction (nope columns [256 kh, 256 kh + 256) and rope columns [32 kh, 32 kh + 32)); its Q slice is the B
//     operand, resident in registers but for a few k-steps parked in LDS;
//   * values: wave (hh, dq) accumulates O^T = V^T P~ for the 64 heads of half hh and 128 of the 512 value
//     columns (128 accumulator registers); every V^T fragment read from LDS feeds two MFMAs.
// Between the two, per tile: the kh = 1 wave of a pair hands its partial S to the kh = 0 wave through LDS; the
// kh = 0 wave runs the online softmax (one head per lane) and leaves P~ (bf16, already in B-operand order), the
// rescale factors and a flag in LDS for the value role; and every wave produces its share of the next tile (four of
// the 32 rows): dequantises it out of the registers its gather landed in, stores it to the other LDS stage and issues
// the gather of the tile after.  Two workgroup barriers per tile.  All waves run the same phase at the same time on
// purpose: two waves of a SIMD issuing MFMAs keep the matrix pipe fed (one wave alone gets its LDS operands at half
// the rate), and two waves issuing vector work fill the vector port (one wave alone issues at about half its rate);
// running the phases of two wave groups one barrier interval apart was measured and is slower.
//
// KV splits write their output normalised by their own sum as fp16, in the accumulators' fragment order, plus (m, l);
// sfa_combine_kernel merges them and turns the result into rows.
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
constexpr int HEADS_PER_WG = 128;
// of a wave's 18 k-steps of Q, NREG stay in registers and the others are parked in LDS (16 bytes per lane each): with
// the 128 accumulator registers of the values role, the wave's share of a gathered tile and the operand fragments in
// flight this is what fits the 256 registers a wave has at two waves per SIMD without spilling
constexpr int NREG_SM = 12, NREG_PR = 12;
// of the 8 tile rows a pair of waves produces, the KH = 1 wave takes NR_PR and the softmax wave the others
constexpr int NR_PR = 4;
// operand fragments read ahead of the MFMA that uses them, in the scores and in the values phase (deeper costs
// registers the kernel does not have)
constexpr int S_AHEAD = 2, PV_AHEAD = 1;
constexpr int NPARK_SM = KSTEPS / 2 - NREG_SM, NPARK_PR = KSTEPS / 2 - NREG_PR;
// LDS layout: two tile stages | partial S, 4 KB per head group | P~, 2 KB per head group | rescale factors [4][32],
// flags [4] | parked Q | per-split arrays sized by SfaArgs::split_cap (validity words, rows) |
// this sequence's page table (when it fits)
constexpr int XBUF_OFF = 2 * STAGE;
constexpr int PBUF_OFF = XBUF_OFF + 4 * 4096;
constexpr int ALPHA_OFF = PBUF_OFF + 4 * 2048;
constexpr int FLAG_OFF = ALPHA_OFF + 4 * 32 * 4;
constexpr int QPARK_OFF = FLAG_OFF + 16;
constexpr int SPLIT_OFF = QPARK_OFF + 4 * (NPARK_SM + NPARK_PR) * 1024;
constexpr int LDS_LIMIT = 160 * 1024;
constexpr int OUT_ROW = DN * 2;  // epilogue staging: 128 heads x 512 values of 16 bits, reusing the front of LDS
constexpr int OUT_LSUM_OFF = HEADS_PER_WG * OUT_ROW; // the epilogue's row sums, behind the staging area (in the parked Q, dead by then)
constexpr int QROW = KROW;       // start-up staging of Q: 128 heads x 1152 bytes
static_assert(HEADS_PER_WG * QROW <= SPLIT_OFF, "the query of 128 heads fits below the per-split arrays");
__host__ __device__ constexpr int tmask_bytes(int cap) { return (cap / T + 2) * 4; }
__host__ __device__ constexpr int split_bytes(int cap) { return tmask_bytes(cap) + cap * 4; }
static_assert(OUT_LSUM_OFF >= QPARK_OFF && OUT_LSUM_OFF + HEADS_PER_WG * 4 <= SPLIT_OFF, "the epilogue's row sums lie in the parked Q, which nothing reads after the last tile's scores");
static_assert(QPARK_OFF % 16 == 0 && SPLIT_OFF % 16 == 0, "16-byte LDS accesses");
static_assert(SPLIT_OFF + split_bytes(MAX_SPLIT_TOKENS) <= LDS_LIMIT, "a whole top-k list must fit one workgroup");


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

// A wavefront's share of one gathered tile, in registers: NR of the tile's 32 rows (this lane's 8 columns of each), 8
// bytes of the tile's rope columns, and one of the share's 4 NR dequantisation scales.  The two waves of a pair (same
// head group hg) share rows 8 hg .. 8 hg + 7: the first NR_PR go to the KH = 1 wave, the others to the softmax wave.
template <bool QUANT, int NR>
struct RawTile;
template <int NR>
struct RawTile<true, NR> {
    u32x2 nope[NR]; // NR rows x 8 int8
    u32x2 rope;     // row tid/16, bytes 8 (tid%16) ..
    float sc;       // lanes 0 .. 4 NR - 1: scale of (row lane/4 of the share, column group lane%4)
};
template <int NR>
struct RawTile<false, NR> {
    u32x4 nope[NR]; // NR rows x 8 bf16
    u32x2 rope;
};

// Byte offset `row * stride` of a wave-uniform row, pinned in scalar registers so that the load that follows takes a
// scalar base and the lane's 32-bit offset (no 64-bit vector arithmetic per row).  An offset, not an address: the
// pointer it is added to keeps its address space, and the load stays a global one.
__device__ __forceinline__ uint64_t row_offset(uint32_t row, uint32_t stride)
{
    const uint64_t p = (uint64_t)row * stride;
    uint32_t lo = (uint32_t)p, hi = (uint32_t)(p >> 32);
    asm volatile("" : "+s"(lo), "+s"(hi));
    return ((uint64_t)hi << 32) | lo;
}

// rows[] holds valid cache rows only (absent entries point at row 0); the tile's validity word says which rows are
// absent, and their data is zeroed when it is consumed, so that no load depends on it.  All loads are unconditional.
// The share is rows pair0 + E0 .. pair0 + E0 + NR - 1 of the tile, pair0 a multiple of 8.
template <int NR>
struct RowRefs {
    uint64_t off[NR];  // byte offsets of the share's rows in the nope cache (scalar registers)
    uint32_t rope_row; // this lane's row for the rope columns
    uint32_t sc_row;   // this lane's row for the scales
};
template <bool QUANT, int NR, int E0>
__device__ __forceinline__ void prepare_rows(RowRefs<NR>& f, const SfaArgs& a, const int* rows, int tile, int pair0, int lane, int tid)
{
    // the pair's eight rows are the same for every lane: two 16-byte LDS reads, then scalar address arithmetic
    const u32x4 ra = *reinterpret_cast<const u32x4*>(rows + tile * T + pair0);
    const u32x4 rb = *reinterpret_cast<const u32x4*>(rows + tile * T + pair0 + 4);
    f.rope_row = (uint32_t)rows[tile * T + (tid >> 4)];
    if constexpr (QUANT) {
        const int l = lane < 4 * NR ? lane : 0;
        f.sc_row = (uint32_t)rows[tile * T + pair0 + E0 + (l >> 2)];
    }
#pragma unroll
    for (int e = 0; e < NR; ++e) {
        const uint32_t row = __builtin_amdgcn_readfirstlane(E0 + e < 4 ? ra[(E0 + e) & 3] : rb[(E0 + e) & 3]);
        f.off[e] = row_offset(row, a.kn_stride);
    }
}
template <bool QUANT, int NR>
__device__ __forceinline__ void issue_raw(RawTile<QUANT, NR>& r, const RowRefs<NR>& f, const SfaArgs& a, int lane, int tid)
{
#pragma unroll
    for (int e = 0; e < NR; ++e) {
        const uint8_t* rp = a.kn + f.off[e];
        if constexpr (QUANT)
            r.nope[e] = *reinterpret_cast<const u32x2*>(rp + lane * 8);
        else
            r.nope[e] = *reinterpret_cast<const u32x4*>(rp + lane * 16);
    }
    r.rope = *reinterpret_cast<const u32x2*>(a.kr + (uint64_t)f.rope_row * a.kr_stride + (tid & 15) * 8);
    if constexpr (QUANT) {
        const int l = lane < 4 * NR ? lane : 0;
        r.sc = *reinterpret_cast<const float*>(a.ks + (uint64_t)f.sc_row * a.ks_stride + (l & 3) * 4);
    }
}
template <bool QUANT, int NR, int E0>
__device__ __forceinline__ void load_raw(RawTile<QUANT, NR>& r, const SfaArgs& a, const int* rows, int tile, int pair0,
                                         int lane, int tid)
{
    RowRefs<NR> f;
    prepare_rows<QUANT, NR, E0>(f, a, rows, tile, pair0, lane, tid);
    issue_raw<QUANT, NR>(r, f, a, lane, tid);
}

// int8 -> fp32 -> * scale with one conversion and one fma per element: byte k of w holds x + 128 (the caller
// flips the sign bits), so x * s = fma(float(byte), s, -128 s); -128 s is exact, hence one rounding, the same
// as rounding the product x * s.
__device__ __forceinline__ float dq(uint32_t w, int k, float s, float neg128s)
{
    return __builtin_fmaf((float)((w >> (8 * k)) & 0xffu), s, neg128s);
}

// Dequantise the share and store it, and the lane's rope piece, into an LDS stage; `present` is the tile's validity word.
// Two rows at a time, instruction class by instruction class (16 conversions, 16 multiply-adds, 8 packs): a wave issues
// a vector instruction that depends on the one before it at half the rate of an independent one, and the scheduler,
// left alone, emits each element's conversion - multiply-add - pack chain back to back.
template <bool QUANT, int NR>
__device__ __forceinline__ void dequant_store(const RawTile<QUANT, NR>& r, uint8_t* stage, uint32_t present, int row0,
                                              int lane, int tid)
{
    float sc[NR];
    if constexpr (QUANT) {
        // the scale of (row e, this lane's group of 128 columns) sits in lane 4e + lane/16; an absent row is stored as
        // zeros (scale 0)
#pragma unroll
        for (int e = 0; e < NR; ++e)
            sc[e] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(4 * (4 * e + (lane >> 4)), __builtin_bit_cast(int, r.sc)));
#pragma unroll
        for (int e = 0; e < NR; ++e) sc[e] = ((present >> (row0 + e)) & 1u) ? sc[e] : 0.f;
    }
#pragma unroll
    for (int e0 = 0; e0 < NR; e0 += 2) {
        constexpr int G = 2;
        if constexpr (QUANT) {
            float f[G][8], c[G];
            uint32_t pk[G][4];
#pragma unroll
            for (int g = 0; g < G; ++g) {
                if (e0 + g >= NR) break;
                const uint32_t w0 = r.nope[e0 + g][0] ^ 0x80808080u, w1 = r.nope[e0 + g][1] ^ 0x80808080u;
                c[g] = -128.f * sc[e0 + g];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    f[g][k] = (float)((w0 >> (8 * k)) & 0xffu);
                    f[g][4 + k] = (float)((w1 >> (8 * k)) & 0xffu);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < G; ++g) {
                if (e0 + g >= NR) break;
#pragma unroll
                for (int k = 0; k < 8; ++k) f[g][k] = __builtin_fmaf(f[g][k], sc[e0 + g], c[g]);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < G; ++g) {
                if (e0 + g >= NR) break;
#pragma unroll
                for (int k = 0; k < 4; ++k) pk[g][k] = pack_bf16x2(f[g][2 * k], f[g][2 * k + 1]);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < G; ++g) {
                if (e0 + g >= NR) break;
                const int t = row0 + e0 + g;
                *reinterpret_cast<u32x4*>(stage + t * KROW + ((lane ^ swz(t)) << 4)) = u32x4{pk[g][0], pk[g][1], pk[g][2], pk[g][3]};
            }
        } else {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                if (e0 + g >= NR) break;
                const int t = row0 + e0 + g;
                const u32x4 v = ((present >> t) & 1u) ? r.nope[e0 + g] : u32x4{0u, 0u, 0u, 0u};
                *reinterpret_cast<u32x4*>(stage + t * KROW + ((lane ^ swz(t)) << 4)) = v;
            }
        }
    }
    {
        const int t = tid >> 4, piece = tid & 15;
        const u32x2 rp = ((present >> t) & 1u) ? r.rope : u32x2{0u, 0u};
        *reinterpret_cast<u32x2*>(stage + t * KROW + DN * 2 + (((piece >> 1) ^ swz(t)) << 4) + (piece & 1) * 8) = rp;
    }
}

// A workgroup's share of a token's top-k list: tiles [tile0, tile0 + ntiles) of the first `cur` entries.
struct SplitRange {
    int cur, tile0, ntiles;
};
__device__ __forceinline__ SplitRange split_range(int cur, int nsplit, int sp)
{
    const int ntiles_all = (cur + T - 1) / T;
    const int per = (ntiles_all + nsplit - 1) / nsplit;
    const int tile0 = sp * per;
    return {cur, tile0, max(min(ntiles_all, tile0 + per) - tile0, 0)};
}

// Resolves the workgroup's share: logical indices -> physical cache rows (absent entries: row 0 and a cleared bit in
// the tile's validity word), in LDS.  NT lanes.  The sequence's length, its page table and the share's top-k entries
// are requested together: the entries are fetched for the share a full list would give (the usual case) and only
// fetched again if the length, once known, moves the share.  `between` runs after those requests and before the first
// wait for them.  Returns the share.
template <int NT, class Between>
__device__ __forceinline__ SplitRange resolve_split(const SfaArgs& a, int bi, int si, int tq, int sp, uint32_t* tmask,
                                                    int* rows, int* bt_lds, int tid, int lane, Between&& between)
{
    constexpr int PER_LANE = MAX_SPLIT_TOKENS / NT;
    const int32_t* list = a.topk_idx + (int64_t)tq * a.topk_stride;
    const SplitRange guess = split_range(a.topk, a.nsplit, sp);
    int my_idx[PER_LANE];
    auto fetch = [&](int tok0) {
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j)
            if (NT * j < a.split_cap) my_idx[j] = list[min(tok0 + tid + NT * j, a.topk - 1)];
    };
    fetch(guess.tile0 * T);
    const int act = a.act_seq[bi];
    // this sequence's page table -> LDS (saves one dependent global load per selected token); a table that fits LDS
    // has at most BT_PER_LANE entries per lane
    constexpr int BT_PER_LANE = (LDS_LIMIT - SPLIT_OFF) / 4 / NT + 1;
    const bool bt_cached = a.bt_cached != 0;
    int btv[BT_PER_LANE];
    if (bt_cached) {
#pragma unroll
        for (int j = 0; j < BT_PER_LANE; ++j)
            if (tid + NT * j < a.bt_stride) btv[j] = a.block_table[(int64_t)bi * a.bt_stride + tid + NT * j];
    }
    between(); // the caller's own loads, behind the ones above and ahead of the first wait for them
    if (bt_cached) {
#pragma unroll
        for (int j = 0; j < BT_PER_LANE; ++j)
            if (tid + NT * j < a.bt_stride) bt_lds[tid + NT * j] = btv[j];
    }
    const SplitRange r = split_range(min(max(act - a.s1 + 1 + si, 0), a.topk), a.nsplit, sp);
    if (r.tile0 != guess.tile0) fetch(r.tile0 * T); // block-uniform
    const int tok0 = r.tile0 * T;
    const int ntiles_even = (r.ntiles + 1) & ~1; // whole wavefronts of entries
    const int64_t max_logical = (int64_t)a.bt_stride * a.block_size;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
        const int i = tid + NT * j;
        if (i >= ntiles_even * T) break; // wave-uniform: tiles are 32 wide, waves 64
        const int idx = (i < r.ntiles * T && tok0 + i < r.cur) ? my_idx[j] : -1;
        int row = -1;
        if (idx >= 0 && idx < max_logical) {
            int page; // (two loads under a branch, not one load from a selected pointer: that would be a generic-address load)
            if (bt_cached)
                page = bt_lds[idx / a.block_size];
            else
                page = a.block_table[(int64_t)bi * a.bt_stride + idx / a.block_size];
            const int64_t pr = (int64_t)page * a.block_size + idx % a.block_size;
            if (page >= 0 && pr < a.n_rows) row = (int)pr;
        }
        rows[i] = max(row, 0);
        const uint64_t present = __ballot(row >= 0);
        if (lane == 0) {
            tmask[i >> 5] = (uint32_t)present;
            tmask[(i >> 5) + 1] = (uint32_t)(present >> 32);
        }
    }
    __syncthreads(); // rows[] / tmask[] ready
    return r;
}

// Half of S^T[token, head] = K[token, :] . Q[head, :] for one wave: its 18 k-steps (kstep_of).  One accumulation
// chain; the K fragments (and the parked Q fragments) are read AHEAD k-steps before the MFMA that uses them.
template <int NREG, int KH>
__device__ __forceinline__ void s_partial(f32x16& s, const uint8_t* stage, const uint32_t (&s_off)[4], const bf16x8 (&q)[NREG],
                                          const uint8_t* qpark)
{
    constexpr int AHEAD = S_AHEAD, N = KSTEPS / 2;
    static_assert(NREG >= AHEAD && NREG <= N, "the first reads are of k-steps whose Q fragment is in registers");
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.f;
    bf16x8 kf[N], qp[N];
    auto fetch = [&](int i) {
        // nope k-step 16 KH + i: chunks 32 KH + 2 i + hl; rope k-step 32 + 2 KH + (i - 16): chunks 64 + 2 (2 KH + i - 16) + hl
        kf[i] = *reinterpret_cast<const bf16x8*>(i < 16 ? stage + s_off[i & 3] + KH * 512 + (i >> 2) * 128
                                                        : stage + s_off[2 * KH + i - 16] + DN * 2);
        if (i >= NREG) qp[i] = *reinterpret_cast<const bf16x8*>(qpark + (i - NREG) * 1024);
    };
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) fetch(i);
#pragma unroll
    for (int i = 0; i < N; ++i) {
        if (i + AHEAD < N) fetch(i + AHEAD);
        const bf16x8 qi = i < NREG ? q[i < NREG ? i : 0] : qp[i];
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i], qi, s, 0, 0, 0);
    }
    // issue order: AHEAD fetches, then (MFMA, fetch) pairs, then the last MFMAs; a fetch is one LDS read for a
    // k-step whose Q fragment is in registers and two for a parked one
    __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
#pragma unroll
    for (int i = 0; i < NREG - AHEAD; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
#pragma unroll
    for (int i = NREG - AHEAD; i < N - AHEAD; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, AHEAD, 0);
}

// The body of one wavefront.  KH = 0: the softmax wave of its pair; KH = 1: the wave that hands its partial S over.
template <bool QUANT, int KH>
__device__ __forceinline__ void sfa_wave(const SfaArgs& a, uint8_t* smem, uint32_t* tmask, int* rows, int* bt_lds, int tid)
{
    const int tq = blockIdx.x, sp = blockIdx.y, hz = blockIdx.z;
    const int bi = tq / a.s1, si = tq - bi * a.s1;
    constexpr int NREG = KH ? NREG_PR : NREG_SM;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6); // (scalar: what follows from it is too)
    const int l32 = lane & 31, hl = lane >> 5;
    const int hg = wave & 3;              // scores role: heads [32 hg, 32 hg + 32) of the workgroup's 128, contraction half KH = wave / 4
    const int hh = wave & 1, dq = wave >> 1; // values role: heads [64 hh, 64 hh + 64), value columns [128 dq, 128 dq + 128)
    const int head0 = hz * HEADS_PER_WG;
    const int head = head0 + hg * 32 + l32;
    const bool head_ok = head < a.nq;
    const bool s_active = head0 + hg * 32 < a.nq;
    const bool pv_active = head0 + hh * 64 < a.nq;

    // The query of the workgroup's 128 heads, requested right behind the few loads the look-up of the share starts with
    // (it is the largest piece of the start-up traffic and depends on nothing).  Fetched as whole cache lines - in each of four rounds of 128 nope
    // columns a lane takes four 16-byte pieces, 16 consecutive lanes one head's 256 bytes; then the rope columns, two
    // pieces per lane - because a load in operand layout (a lane pair per head) costs the texture addresser one line per
    // lane pair.  The operand layout is made on the way through LDS further down.
    u32x4 qraw[4][4], qraw_rope[2];
    auto request_q = [&]() {
        const int64_t qrow0 = (int64_t)tq * a.nq;
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int p = tid + 512 * j;
                const int64_t row = qrow0 + min(head0 + (p >> 4), a.nq - 1);
                qraw[r][j] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const __bf16*>(a.q_nope) + row * DN + 128 * r + 8 * (p & 15));
            }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int p = tid + 512 * j;
            const int64_t row = qrow0 + min(head0 + (p >> 3), a.nq - 1);
            qraw_rope[j] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const __bf16*>(a.q_rope) + row * DR + 8 * (p & 7));
        }
    };

    const SplitRange share = resolve_split<512>(a, bi, si, tq, sp, tmask, rows, bt_lds, tid, lane, request_q);
    const int ntiles = share.ntiles, last = ntiles - 1;

    // Production: this wave's share of every tile (rows row0 .. row0 + NR - 1 and 8 bytes of the rope columns).  The
    // share of tile i+1 is dequantised out of `raw` and stored between the two MFMA phases of tile i, and `raw` is
    // refilled at once with the share of tile i+2 (past the end the last tile is loaded again and stored into a stage
    // nobody reads: every path has the same loads in flight).
    constexpr int NR = KH ? NR_PR : 8 - NR_PR, E0 = KH ? 0 : NR_PR;
    const int pair0 = 8 * hg, row0 = pair0 + E0;
    RawTile<QUANT, NR> raw;
    if (ntiles > 0) load_raw<QUANT, NR, E0>(raw, a, rows, 0, pair0, lane, tid);

    // Q into operand layout: this lane's head (hg, l32) and its slice - the 16 k-steps of nope columns
    // [256 KH, 256 KH + 256) and the 2 of rope columns [32 KH, 32 KH + 32); B operand layout: head = column, 8
    // consecutive k per half-wave.  One trip through LDS (all of it below the per-split arrays is still unused).
    bf16x8 q[NREG];
    uint8_t* qpark = smem + QPARK_OFF + (KH ? 4 * NPARK_SM * 1024 + hg * (NPARK_PR * 1024) : hg * (NPARK_SM * 1024)) + lane * 16;
    {
        // (a negative softmax_scale is applied as its magnitude to the negated query: the row statistics below are
        // taken on the raw scores, which needs a factor that commutes with max)
        const uint32_t f = a.softmax_scale < 0.f ? 0x80008000u : 0u;
        const u32x4 qflip = {f, f, f, f};
        // all 128 heads' rows at once: row h at h * QROW, its 72 16-byte chunks (64 nope, 8 rope) XOR-swizzled with h
        // so that the 8 lanes of a b128 access hit distinct banks although a row is a multiple of 128 bytes
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int pp = tid + 512 * j, h = pp >> 4, c = 16 * r + (pp & 15);
                *reinterpret_cast<u32x4*>(smem + h * QROW + ((c ^ (h & 7)) << 4)) = qraw[r][j];
            }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int pp = tid + 512 * j, h = pp >> 3, c = 64 + (pp & 7);
            *reinterpret_cast<u32x4*>(smem + h * QROW + ((c ^ (h & 7)) << 4)) = qraw_rope[j];
        }
        __syncthreads();
        // k-step i of this wave's 18: nope chunks 2 (16 KH + i) + hl, rope chunks 64 + 2 (2 KH + i - 16) + hl
        u32x4 qa[KSTEPS / 2];
        {
            const int h = hg * 32 + l32;
            const uint8_t* row = smem + h * QROW;
#pragma unroll
            for (int i = 0; i < KSTEPS / 2; ++i) {
                const int c = (i < 16 ? 2 * (16 * KH + i) : 64 + 2 * (2 * KH + i - 16)) + hl;
                qa[i] = *reinterpret_cast<const u32x4*>(row + ((c ^ (h & 7)) << 4)) ^ qflip;
            }
        }
        __syncthreads(); // every wave has its fragments: the rows' space is free for the parked fragments and the tiles
#pragma unroll
        for (int i = 0; i < KSTEPS / 2; ++i) {
            const bf16x8 v = __builtin_bit_cast(bf16x8, qa[i]);
            if (i < NREG)
                q[i < NREG ? i : 0] = v;
            else
                *reinterpret_cast<bf16x8*>(qpark + (i - NREG) * 1024) = v;
        }
    }
    if (ntiles > 0) {
        dequant_store<QUANT, NR>(raw, smem, __builtin_amdgcn_readfirstlane(tmask[0]), row0, lane, tid);
        load_raw<QUANT, NR, E0>(raw, a, rows, min(1, last), pair0, lane, tid);
    }

    f32x16 o[4][2]; // O^T blocks [value columns 32 (4 dq + i) ..][heads 64 hh + 32 hb ..]
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int hb = 0; hb < 2; ++hb)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[i][hb][r] = 0.f;
    float m_run = -INFINITY; // running max of S * scale * log2(e)          (softmax wave)
    float l_run = 0.f;       // this lane's share of sum exp                (softmax wave)
    // (never exactly zero: a masked score is -inf, and -inf * 0 would be NaN; 2^(s * 1e-30) is 1 for every finite s, so
    // a zero scale still gives every attended row the same weight)
    const float c_log2 = fmaxf(fabsf(a.softmax_scale) * 1.4426950408889634f, 1e-30f);

    // S operand (b128): row l32, chunk 2*ks + hl of k-step ks; swizzled offsets of the four chunk positions 2 m + hl
    // inside a group of eight chunks
    uint32_t s_off[4];
    {
        const int sw = swz(l32);
#pragma unroll
        for (int m = 0; m < 4; ++m) s_off[m] = l32 * KROW + (((2 * m + hl) ^ sw) << 4);
    }
    // V^T operand (transpose read): lane jj of 16-lane group G points at row 4*hl + jj/4 (+ 16*j + 8*h2), columns
    // 32*db + 16*(G&1) + 4*(jj&3) with db = 4*dq + i -> chunk 16*dq + 4*i + 2*(G&1) + (jj&3)/2; swizzled offsets for even
    // and odd i
    uint32_t v_off[2];
    {
        const int jj = lane & 15, mh = (lane >> 4) & 1;
        const int cl = 2 * mh + ((jj & 3) >> 1);
        const int sw = ((jj >> 2) << 1) | hl;
        const uint32_t base = (4 * hl + (jj >> 2)) * KROW + (jj & 1) * 8 + dq * 256;
        v_off[0] = base + ((cl ^ sw) << 4);
        v_off[1] = base + (((4 + cl) ^ sw) << 4);
    }
    uint8_t* xbuf = smem + XBUF_OFF + hg * 4096 + lane * 16;
    uint8_t* pbuf = smem + PBUF_OFF + hg * 2048 + lane * 16;
    float* alpha_lds = reinterpret_cast<float*>(smem + ALPHA_OFF);
    uint32_t* flag_lds = reinterpret_cast<uint32_t*>(smem + FLAG_OFF);
    if (tid < 4) flag_lds[tid] = 0u;
    __syncthreads(); // tile 0 stored, Q parked

    // Two barriers per tile: partial S handed over | P~ and the next tile ready.
    for (int it = 0; it < ntiles; ++it) {
        uint8_t* stage = smem + (it & 1) * STAGE;
        const uint32_t valid = __builtin_amdgcn_readfirstlane(tmask[it]);
        RowRefs<NR> next_rows; // of the tile after next, looked up under the score MFMAs
        prepare_rows<QUANT, NR, E0>(next_rows, a, rows, min(it + 2, last), pair0, lane, tid);
        f32x16 s;
        if (s_active) s_partial<NREG, KH>(s, stage, s_off, q, qpark);
        if (KH == 1 && s_active) {
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *reinterpret_cast<f32x4*>(xbuf + g * 1024) = f32x4{s[4 * g], s[4 * g + 1], s[4 * g + 2], s[4 * g + 3]};
        }
        __syncthreads(); // the partial S of the KH = 1 waves is in LDS
        if (KH == 0 && s_active && valid != 0u) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 p = *reinterpret_cast<const f32x4*>(xbuf + g * 1024);
                s[4 * g] += p[0];
                s[4 * g + 1] += p[1];
                s[4 * g + 2] += p[2];
                s[4 * g + 3] += p[3];
            }
            // register r holds token 8*(r/4) + 4*hl + r%4 for head l32; statistics on the raw scores (the factor
            // is not negative, so it commutes with max), exponent argument by one fma per score
            float mx = -INFINITY;
            if (valid != 0xffffffffu) {
                // (the half-wave's shift first: the bit positions left are compile-time constants)
                const uint32_t vh = valid >> (4 * hl);
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = ((vh >> (8 * (r >> 2) + (r & 3))) & 1u) ? s[r] : -INFINITY;
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[r]);
            {
                // maximum over both halves of the wavefront without a trip through LDS: v_permlane32_swap exchanges the
                // upper half of its first operand with the lower half of its second
                const auto sw = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, mx), __builtin_bit_cast(unsigned, mx), false, false);
                mx = fmaxf(__builtin_bit_cast(float, (unsigned)sw[0]), __builtin_bit_cast(float, (unsigned)sw[1])) * c_log2;
            }
            // The reference exponent only follows the running maximum when it has grown by more than 2^8: until
            // then P~ = 2^(z - m_run) may exceed 1 (by at most 2^8, no issue for bf16 or the fp32 sums), which
            // makes the rescale of the accumulator registers a rare event.  Every P~, l and O stay relative to
            // the same m_run, so the result is unchanged.
            const float m_new = fmaxf(m_run, mx);
            const bool rescale = __any(m_new > m_run + 8.f);
            if (rescale) {
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new); // 0 on the first tile (m_run = -inf)
                l_run *= alpha;
                m_run = m_new;
                if (hl == 0) alpha_lds[hg * 32 + l32] = alpha;
            }
            if (lane == 0) flag_lds[hg] = rescale ? 1u : 0u;
            uint32_t pb[8];
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], c_log2, -m_run));
                const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r + 1], c_log2, -m_run));
                l_run += p0 + p1;
                pb[r >> 1] = pack_bf16x2(p0, p1);
            }
            // P~ in the order the S^T registers hold the tokens: k-slot s of half hl in block j is token
            // 16*j + 8*(s/4) + 4*hl + s%4 - which is also how the V^T fragments are read
#pragma unroll
            for (int j = 0; j < 2; ++j)
                *reinterpret_cast<u32x4*>(pbuf + j * 1024) = u32x4{pb[4 * j], pb[4 * j + 1], pb[4 * j + 2], pb[4 * j + 3]};
        }
        {
            // the next tile: out of the registers into the other stage, then the gather of the tile after
            const int nx = min(it + 1, last);
            dequant_store<QUANT, NR>(raw, smem + ((it + 1) & 1) * STAGE, __builtin_amdgcn_readfirstlane(tmask[nx]), row0, lane, tid);
            issue_raw<QUANT, NR>(raw, next_rows, a, lane, tid);
        }
        __syncthreads(); // P~ and the next tile are in LDS
        if (pv_active && valid != 0u) {
            // O^T[dim, head] += V^T[dim, token] . P~[token, head]
#pragma unroll
            for (int hb = 0; hb < 2; ++hb) {
                const uint32_t f = __builtin_amdgcn_readfirstlane(flag_lds[2 * hh + hb]);
                if (f) {
                    const float alpha = alpha_lds[(2 * hh + hb) * 32 + l32];
#pragma unroll
                    for (int i = 0; i < 4; ++i)
#pragma unroll
                        for (int r = 0; r < 16; ++r) o[i][hb][r] *= alpha;
                }
            }
            bf16x8 pf[2][2];
#pragma unroll
            for (int hb = 0; hb < 2; ++hb)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    pf[hb][j] = *reinterpret_cast<const bf16x8*>(smem + PBUF_OFF + (2 * hh + hb) * 2048 + j * 1024 + lane * 16);
            // 8 V^T fragments (token block j, column block i), two transpose reads each, feeding two MFMAs each;
            // the reads run AHEAD fragments ahead
            constexpr int AHEAD = PV_AHEAD;
            s16x4 lo[8], hi[8];
            auto vread = [&](int n) {
                const int j = n >> 2, i = n & 3;
                uint8_t* vp = stage + v_off[i & 1] + (16 * j) * KROW + (i >> 1) * 128;
                lo[n] = lds_read_tr(vp);
                hi[n] = lds_read_tr(vp + 8 * KROW);
            };
#pragma unroll
            for (int n = 0; n < AHEAD; ++n) vread(n);
#pragma unroll
            for (int n = 0; n < 8; ++n) {
                if (n + AHEAD < 8) vread(n + AHEAD);
                const s16x8 both = __builtin_shufflevector(lo[n], hi[n], 0, 1, 2, 3, 4, 5, 6, 7);
                const bf16x8 vf = __builtin_bit_cast(bf16x8, both);
#pragma unroll
                for (int hb = 0; hb < 2; ++hb)
                    o[n & 3][hb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[hb][n >> 2], o[n & 3][hb], 0, 0, 0);
            }
        }
    }

    // Epilogue.  The softmax waves publish the row sums (in a part of LDS the staging area below does not reach) and every
    // wave normalises its O^T blocks.  Register r of o[i][hb] holds dim 32*(4*dq + i) + 8*(r/4) + 4*hl + r%4 of head
    // 64*hh + 32*hb + l32: four consecutive dims, and the other half-wave holds the four next to them.
    float* lsum = reinterpret_cast<float*>(smem + OUT_LSUM_OFF);
    if (KH == 0) {
        const float l_tot = l_run + __shfl_xor(l_run, 32);
        if (hl == 0) lsum[hg * 32 + l32] = s_active ? l_tot : 0.f;
        if (a.nsplit > 1 && head_ok && hl == 0) {
            const int64_t prow = ((int64_t)tq * a.nsplit + sp) * a.nq + head;
            a.part_ml[prow * 2] = m_run;
            a.part_ml[prow * 2 + 1] = l_tot;
        }
    }
    __syncthreads(); // row sums published; nobody reads a tile, P~ or parked Q any more
    if (a.nsplit > 1) {
        // A split's share, normalised by its own sum, in fp16 (|value| <= max |V| and 2^-11 relative rounding, a quarter
        // of the final bf16 rounding, half the bytes of fp32 for this kernel to write and the merge to read).  It leaves
        // in fragment order, straight from the accumulators: [token][split][head group][wave 8][hb 2][i 4][half 2]
        // [lane 64] x 8 fp16 - every store instruction writes 1 KB of consecutive bytes, and nothing is staged.  The
        // merge kernel reads the same order and does the transposition to rows once, for the output, instead of once
        // per split here.  (Streaming stores: 34 MB leave the chip's 256 workgroups at once and are read back once.)
        if (pv_active) {
            const int wave = tid >> 6;
            _Float16* wbase = a.part_o + ((((int64_t)tq * a.nsplit + sp) * gridDim.z + hz) * 8 + wave) * 8192 + lane * 8;
#pragma unroll
            for (int hb = 0; hb < 2; ++hb) {
                const float l = lsum[64 * hh + 32 * hb + l32];
                const float mul = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
                        uint32_t w[4];
#pragma unroll
                        for (int k = 0; k < 4; ++k)
                            w[k] = __builtin_bit_cast(uint32_t, f16x2{(_Float16)(o[i][hb][8 * h + 2 * k] * mul), (_Float16)(o[i][hb][8 * h + 2 * k + 1] * mul)});
                        __builtin_nontemporal_store(u32x4{w[0], w[1], w[2], w[3]}, reinterpret_cast<u32x4*>(wbase + ((hb * 4 + i) * 2 + h) * 512));
                    }
            }
        }
        return;
    }
    // One split: the output itself, bf16 rows.  v_permlane32_swap pairs up the two half-waves' four-dim pieces - the lower
    // half-wave ends up with the 8 dims of block g = 2 gp, the upper one with those of block 2 gp + 1 - so that a lane
    // stores 16 bytes; all 128 heads' rows are staged in LDS as [head][512] rows of 1024 bytes (everything below
    // OUT_LSUM_OFF is free now), the 16-byte chunks of a row XOR-swizzled with the head so that the 8 lanes of a b128
    // access hit distinct banks, and all 512 lanes copy the rows out, a wavefront writing one whole row per instruction.
    if (pv_active) {
#pragma unroll
        for (int hb = 0; hb < 2; ++hb) {
            const int hrow = 64 * hh + 32 * hb + l32;
            const float l = lsum[hrow];
            const float mul = l > 0.f ? 1.f / l : 0.f;
            uint8_t* orow = smem + hrow * OUT_ROW;
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int gp = 0; gp < 2; ++gp) {
                    uint32_t w[2][2]; // [block 2 gp, 2 gp + 1][pair of dims]
#pragma unroll
                    for (int g = 0; g < 2; ++g)
#pragma unroll
                        for (int k = 0; k < 2; ++k)
                            w[g][k] = pack_bf16x2(o[i][hb][4 * (2 * gp + g) + 2 * k] * mul, o[i][hb][4 * (2 * gp + g) + 2 * k + 1] * mul);
                    // the swap exchanges the upper half-wave of its first operand with the lower half-wave of its second
                    const auto s0 = __builtin_amdgcn_permlane32_swap(w[0][0], w[1][0], false, false);
                    const auto s1 = __builtin_amdgcn_permlane32_swap(w[0][1], w[1][1], false, false);
                    const int c = 4 * (4 * dq + i) + 2 * gp + hl;
                    *reinterpret_cast<u32x4*>(orow + ((c ^ (hrow & 7)) << 4)) = u32x4{(uint32_t)s0[0], (uint32_t)s1[0], (uint32_t)s0[1], (uint32_t)s1[1]};
                }
        }
    }
    __syncthreads();
#pragma unroll 4
    for (int id = tid; id < HEADS_PER_WG * (DN / 8); id += 512) {
        const int hrow = id / (DN / 8), c = id % (DN / 8);
        const int oh = head0 + hrow;
        if (oh >= a.nq) break; // (wave-uniform: a wavefront copies one row)
        const u32x4 v = *reinterpret_cast<const u32x4*>(smem + hrow * OUT_ROW + ((c ^ (hrow & 7)) << 4));
        *reinterpret_cast<u32x4*>(reinterpret_cast<uint8_t*>(a.out) + (((int64_t)tq * a.nq + oh) * DN + c * 8) * 2) = v;
    }
}

// grid (query token, KV split, group of 128 heads).  Workgroups go to the XCDs round-robin in launch order, so with the
// token as the fastest grid dimension the splits of one token run on one XCD (when the token count is a multiple of 8)
// and share its L2 for the token's queries.
template <bool QUANT>
__global__ __attribute__((amdgpu_flat_work_group_size(512, 512), amdgpu_waves_per_eu(2, 2))) void sfa_decode_kernel(
    SfaArgs a)
{
    extern __shared__ __align__(16) uint8_t smem[];
    uint32_t* tmask = reinterpret_cast<uint32_t*>(smem + SPLIT_OFF);
    int* rows = reinterpret_cast<int*>(smem + SPLIT_OFF + tmask_bytes(a.split_cap));
    int* bt_lds = reinterpret_cast<int*>(smem + SPLIT_OFF + split_bytes(a.split_cap));

    const int tid = threadIdx.x;

    // Both kinds of wavefront run the same barrier sequence: one before the first tile, two per tile, the epilogue's.
    if (tid < 256)
        sfa_wave<QUANT, 0>(a, smem, tmask, rows, bt_lds, tid);
    else
        sfa_wave<QUANT, 1>(a, smem, tmask, rows, bt_lds, tid);
}

// attention_out <- 0 (cache without rows: every selected entry is absent)
__global__ void sfa_zero_kernel(uint32_t* out, int64_t n_words)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_words) out[i] = 0u;
}

// out[row, :] = sum_s (2^(m_s - M) l_s / L) o_s[row, :] with L = sum_s 2^(m_s - M) l_s and o_s the split's normalised
// output.  The partials lie in the fragment order the attention kernel's accumulators have (see its epilogue).  One
// workgroup merges, for one token, what wave wv of the attention workgroups left for head block hb: 32 heads x 128
// value columns; its wavefront i takes column block i, a lane owning for its head (l32) the four 4-column runs at
// 32 i + 16 h + 8 g + 4 hl.  Splits are taken G at a time (G = 2, 4 or 8: the smallest that covers the split count,
// eight for more than eight splits), every load of a group requested before any is used (splits past the last are the
// last again with weight 0).  The workgroup then turns its 32 x 128 block through LDS
// and writes the 256-byte row pieces, 16 lanes a piece.
constexpr int CROW = 128 * 2 + 16; // LDS row of the merge's transposition: 128 bf16 plus one 16-byte chunk of padding
template <int G>
__global__ __launch_bounds__(256) void sfa_combine_kernel(const void* __restrict__ part_o_fp16,
                                                          const float* __restrict__ part_ml, void* out, int nq,
                                                          int nsplit, int hgroups)
{
    __shared__ __align__(16) uint8_t tr[32 * CROW];
    const _Float16* part_o = static_cast<const _Float16*>(part_o_fp16); // (a plain pointer type keeps the symbol readable)
    const int lane = threadIdx.x & 63, l32 = lane & 31, hl = lane >> 5;
    const int i = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int task = blockIdx.x; // ((tq * hgroups + hz) * 8 + wv) * 2 + hb
    const int hb = task & 1, wv = (task >> 1) & 7;
    const int th = task >> 4, hz = th % hgroups, tq = th / hgroups;
    const int hh = wv & 1, dq = wv >> 1;
    const int head_base = hz * HEADS_PER_WG + 64 * hh + 32 * hb;
    if (head_base >= nq) return; // (a head block past the last head: nothing was written for it)
    const int headc = min(head_base + l32, nq - 1);
    float acc[2][8];
#pragma unroll
    for (int x = 0; x < 16; ++x) (&acc[0][0])[x] = 0.f;
    float M = -INFINITY, L = 0.f;
    const int64_t split_stride = (int64_t)hgroups * 8 * 8192; // fp16 elements between two splits of a token
    const _Float16* frag0 = part_o + (((int64_t)tq * nsplit * hgroups + hz) * 8 + wv) * 8192 + (hb * 4 + i) * 1024; // (the workgroup's four wavefronts read 8 KB in a row per split)
    const float* ml0 = part_ml + (int64_t)tq * nsplit * nq * 2;
    for (int s0 = 0; s0 < nsplit; s0 += G) {
        f16x8 v[G][2];
        float m[G], l[G];
#pragma unroll
        for (int j = 0; j < G; ++j) {
            const int s = min(s0 + j, nsplit - 1);
            const _Float16* base = frag0 + s * split_stride;
#pragma unroll
            for (int h = 0; h < 2; ++h) v[j][h] = *reinterpret_cast<const f16x8*>(base + h * 512 + lane * 8);
            m[j] = ml0[((int64_t)s * nq + headc) * 2];
            l[j] = s0 + j < nsplit ? ml0[((int64_t)s * nq + headc) * 2 + 1] : 0.f;
        }
        // the group's maximum joins the running one: what was summed so far is rescaled once per group
        float Mg = M;
#pragma unroll
        for (int j = 0; j < G; ++j) Mg = l[j] > 0.f ? fmaxf(Mg, m[j]) : Mg;
        if (Mg != -INFINITY) { // (otherwise nothing attended in these splits)
            if (s0 > 0) {
                const float back = exp2f(M - Mg); // 0 while nothing has been summed (M = -inf)
                L *= back;
#pragma unroll
                for (int x = 0; x < 16; ++x) (&acc[0][0])[x] *= back;
            }
            M = Mg;
#pragma unroll
            for (int j = 0; j < G; ++j) {
                const float w = l[j] > 0.f ? exp2f(m[j] - M) * l[j] : 0.f;
                L += w;
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc[h][e] += (float)v[j][h][e] * w;
            }
        }
    }
    const float inv = L > 0.f ? 1.f / L : 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const float* x = &acc[h][4 * g];
            const u32x2 w = {pack_bf16x2(x[0] * inv, x[1] * inv), pack_bf16x2(x[2] * inv, x[3] * inv)};
            *reinterpret_cast<u32x2*>(tr + l32 * CROW + (32 * i + 16 * h + 8 * g + 4 * hl) * 2) = w;
        }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int r = 16 * k + (threadIdx.x >> 4), c = threadIdx.x & 15;
        const u32x4 w = *reinterpret_cast<const u32x4*>(tr + r * CROW + c * 16);
        if (head_base + r < nq)
            *reinterpret_cast<u32x4*>(reinterpret_cast<uint8_t*>(out) + (((int64_t)tq * nq + head_base + r) * DN + 128 * dq + 8 * c) * 2) = w;
    }
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

uint64_t sfa_partials_bytes(int t, int nq, int nsplit)
{
    if (nsplit <= 1) return 0;
    const int hgroups = (nq + HEADS_PER_WG - 1) / HEADS_PER_WG; // (whole 128-head groups: the partials lie in fragment order)
    return (uint64_t)t * nsplit * hgroups * HEADS_PER_WG * DN * sizeof(_Float16);
}

uint64_t sfa_workspace_bytes(int t, int nq, int nsplit)
{
    if (nsplit <= 1) return 0;
    return sfa_partials_bytes(t, nq, nsplit) + (uint64_t)t * nsplit * nq * 2 * sizeof(float);
}

// Scratch for callers that cannot allocate (sfa_static_scratch): one array per GPU the library runs on, held until the
// process ends.  In host code the array's name is only a handle for hipGetSymbolAddress - the device address it returns
// is what kernels and copies are given.
static __device__ __align__(256) unsigned char scratch[SFA_STATIC_SCRATCH_BYTES];

hipError_t sfa_static_scratch(void** ptr)
{
    static std::atomic<void*> cached[64]; // per device ordinal: every GPU has its own copy of the array at its own address
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    void* p = cached[dev & 63].load(std::memory_order_acquire);
    if (p == nullptr) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (p == nullptr) return hipErrorInvalidSymbol;
        cached[dev & 63].store(p, std::memory_order_release);
    }
    *ptr = p;
    return hipSuccess;
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
    dim3 grid(t, a.nsplit, hgroups);
    {
        ScopedKernelTimer tm(KID_SFA_DECODE, stream);
        hipLaunchKernelGGL(kern, grid, dim3(512), smem_bytes, stream, args);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (a.nsplit > 1) {
        ScopedKernelTimer tm(KID_SFA_COMBINE, stream);
        auto merge = a.nsplit <= 2 ? sfa_combine_kernel<2> : a.nsplit <= 4 ? sfa_combine_kernel<4> : sfa_combine_kernel<8>;
        hipLaunchKernelGGL(merge, dim3(t * hgroups * 16), dim3(256), 0, stream, static_cast<const void*>(a.part_o),
                           a.part_ml, a.out, a.nq, a.nsplit, hgroups);
        e = hipGetLastError();
    }
    return e;
}

} // namespace pto
