// Lightning indexer (int8 index scores + top-k) - gfx950 kernels.
//
// Replaces the device side of lightning_indexer_decode_compute
// (models/deepseek_v32_exp/lightning_indexer_quant_impl.py:38-216); arithmetic follows the golden
// (models/deepseek_v32_exp/deepseekv32_lightning_indexer_quant.py:178-263):
//   w_scale[h] = fp16(q_scale[h] * weight[h])
//   y[h, n]    = fp16(relu(int32 dot(q[h], k[n])) * 2^-11)
//   score[n]   = (sum_h fp32(w_scale[h]) * fp32(y[h, n])) * fp32(k_scale[n])
//   top-k over score[0 : eff_seq), eff_seq = act_seq - (s1 - 1 - i); best first, equal scores by ascending
//   index (framework/src/interface/interpreter/calculator/calc_torch.cpp:2481-2494); unused slots = -1.
//
// indexer_score_kernel: v_mfma_i32_16x16x64_i8 with the query heads as rows (A, resident in registers)
// and 16 cached keys as columns (B, loaded from the paged cache straight in operand layout: lane l reads
// 16 bytes of key l%16).  The result has one key per lane and 16 heads per lane; relu, the 2^-11 scaling and
// the fp16 rounding are 4 VALU operations per (head, key), and the weighted head sum is a second MFMA
// (v_mfma_f32_16x16x32_f16: row 0 of A holds w_scale, B is the fp16 tile just produced; every product of two
// fp16 values is exact in fp32, so this is the golden's fp32 sum up to the order of additions).  Scores go to
// a dense fp32 row per query token, and their order-preserving keys into a 256-bin histogram in LDS (score_bin:
// quarter octaves).  Every workgroup owns a 2048-key span of its sequence and leaves its histogram in a slot of
// its own in the workspace (16-bit counts): plain stores, nothing to clear beforehand and no global atomics.
//
// indexer_select_kernel: every workgroup adds up the spans' histograms of its query token, finds the bin B that
// holds the k-th largest key, and files its 4096 scores: bins above B are winners, bin B goes to a tie list (both
// lists in the workspace, appended with one global atomic per workgroup; the counters are cleared by the score
// kernel).
//
// indexer_topk_kernel: one workgroup per query token takes the winners, picks the missing krem entries out of
// the tie list by radix-selecting on the 64-bit words (key << 32 | ~index) (so equal keys resolve to the
// smaller index), and bitonic-sorts the k words.  A tie list that overflowed its capacity (e.g. all scores
// equal) falls back to radix-selecting over the whole score row.
#include "common.h"
#include "kernels.h"
#include "timing.h"

namespace pto {
namespace {

constexpr int D = 128;          // index head dim
constexpr int CHUNK = 512;      // keys per pass of a workgroup of the score kernel (8 groups of 16 per wavefront)
constexpr int PASSES = 4;       // passes per workgroup (amortise the Q / w_scale set-up)
constexpr int MAX_K = 2048;     // top-k capacity
constexpr int NBINS = 2048;     // digit bins of the radix select and of the final ordering (11 bits)
constexpr int SBINS = 256;      // bins of the selection histogram (score_bin)
constexpr int SUBBINS = 64;     // second level inside the threshold bin: the next six key bits (tie_sub_bin)
constexpr int SUB_RANK_CAP = 128; // ties of one second-level step that are ranked by direct comparison (more: digit by digit)
constexpr int SEL_CHUNK = 4096; // scores per workgroup of the select kernel
constexpr int TIE_CAP = 8192;   // capacity of the per-row tie list

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
// A scale as it lies in memory (fp16 bits, or fp32 in the fp32-scale variant) and as the fp32 factor it stands for.
template <bool F32> struct ScaleOf { typedef uint16_t raw; static __device__ __forceinline__ float f32(raw v) { return f16_bits_to_f32(v); } };
template <> struct ScaleOf<true> { typedef float raw; static __device__ __forceinline__ float f32(raw v) { return v; } };
// fp16(fp32(a * b)): the product is rounded to fp32 first and that value to fp16, as the golden's tensor operations do.
// (The compiler would otherwise fuse the multiplication and the conversion into one mixed-precision instruction that
// rounds the exact product once - a different fp16 value about once in 8000 products.)
__device__ __forceinline__ _Float16 round_f32_product_to_f16(float a, float b)
{
    float p = a * b;
    asm volatile("" : "+v"(p));
    return (_Float16)p;
}
// w_scale = q_scale * weight rounded once to fp16: the fp16 product of two fp16 values, or - fp32 scales - the fp32
// product of the scale and the widened weight
template <bool F32>
__device__ __forceinline__ _Float16 w_scale_of(const void* q_scale, const uint16_t* weights, int64_t h)
{
    const _Float16 w = __builtin_bit_cast(_Float16, weights[h]);
    if constexpr (F32)
        return round_f32_product_to_f16(static_cast<const float*>(q_scale)[h], (float)w);
    else
        return (_Float16)(__builtin_bit_cast(_Float16, static_cast<const uint16_t*>(q_scale)[h]) * w);
}
__device__ __forceinline__ uint32_t score_key(float f) { return f32_to_ordered(f + 0.0f); } // -0 -> +0
// Bin of a score key in the selection histogram, non-decreasing in the key: quarter octaves (sign, exponent, two
// mantissa bits - the top 11 key bits) of the magnitudes 2^-20 .. 2^12, 128 bins for either sign; smaller and larger
// magnitudes fall into the first and last bin of their sign.  Keys of one interior bin share their top 11 bits.
__device__ __forceinline__ uint32_t score_bin(uint32_t key)
{
    constexpr int LO = (127 - 20) * 4; // exponent field and two mantissa bits of 2^-20
    const int t = (int)(key >> 21);
    return t >= 1024 ? 128u + (uint32_t)min(max(t - 1024 - LO, 0), 127) : (uint32_t)min(max(t - (1023 - LO - 127), 0), 127);
}
__device__ __forceinline__ bool score_bin_is_interior(uint32_t bin) { return (bin & 127u) != 0u && (bin & 127u) != 127u; }
// The keys of an interior bin share their top 11 bits; the next six split the bin into 64 equal steps, in key order.
__device__ __forceinline__ uint32_t tie_sub_bin(uint32_t key) { return (key >> 15) & (SUBBINS - 1u); }
// Smallest and largest key of a bin (the first and last bin of a sign reach to the end of the sign's keys).
__device__ __forceinline__ void score_bin_range(uint32_t bin, uint32_t& lo, uint32_t& hi)
{
    constexpr int LO = (127 - 20) * 4;
    const uint32_t j = bin & 127u;
    const uint32_t t = bin >= 128u ? 1024u + LO + j : j + (1023u - LO - 127u);
    lo = j == 0u ? (bin & 128u) << 24 : t << 21;
    hi = j == 127u ? ((bin & 128u) << 24) | 0x7fffffffu : (t << 21) | 0x1fffffu;
}

__device__ __forceinline__ uint64_t make_cand(uint32_t key, int idx)
{
    return ((uint64_t)key << 32) | (uint32_t)(0xffffffffu - (uint32_t)idx);
}

// One step of a wavefront scan in the vector unit's own lane network (no trip through LDS): the value of the lane
// CTRL names (row_shr:n = 0x110 + n within a row of 16 lanes, row_bcast15 = 0x142 / row_bcast31 = 0x143 across rows,
// limited to the rows of ROW_MASK), IDENT where there is no such lane.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_from(uint32_t v, uint32_t ident)
{
    return (uint32_t)__builtin_amdgcn_update_dpp((int)ident, (int)v, CTRL, ROW_MASK, 0xf, false);
}

// wavefront-wide inclusive prefix sum: lane l gets v[0] + .. + v[l]
__device__ __forceinline__ uint32_t wave_prefix_sum(uint32_t v)
{
    v += dpp_from<0x111, 0xf>(v, 0u);
    v += dpp_from<0x112, 0xf>(v, 0u);
    v += dpp_from<0x114, 0xf>(v, 0u);
    v += dpp_from<0x118, 0xf>(v, 0u);
    v += dpp_from<0x142, 0xa>(v, 0u); // rows 1 and 3 add the totals of rows 0 and 2
    v += dpp_from<0x143, 0xc>(v, 0u); // rows 2 and 3 add the total of rows 0 and 1
    return v;
}

// wavefront-wide minimum / maximum, the same value in every lane
__device__ __forceinline__ uint32_t wave_min(uint32_t v)
{
    v = min(v, dpp_from<0x111, 0xf>(v, 0xffffffffu));
    v = min(v, dpp_from<0x112, 0xf>(v, 0xffffffffu));
    v = min(v, dpp_from<0x114, 0xf>(v, 0xffffffffu));
    v = min(v, dpp_from<0x118, 0xf>(v, 0xffffffffu));
    v = min(v, dpp_from<0x142, 0xa>(v, 0xffffffffu));
    v = min(v, dpp_from<0x143, 0xc>(v, 0xffffffffu));
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

__device__ __forceinline__ uint32_t wave_max(uint32_t v)
{
    v = max(v, dpp_from<0x111, 0xf>(v, 0u));
    v = max(v, dpp_from<0x112, 0xf>(v, 0u));
    v = max(v, dpp_from<0x114, 0xf>(v, 0u));
    v = max(v, dpp_from<0x118, 0xf>(v, 0u));
    v = max(v, dpp_from<0x142, 0xa>(v, 0u));
    v = max(v, dpp_from<0x143, 0xc>(v, 0u));
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

// The workgroup's histograms (S1 query tokens, one 2048-key span) go to its own slots, as 16-bit counts (at most 2048
// each), two per lane.  The span-0 workgroup also clears the select kernel's list counters of its query tokens.  256 lanes.
template <int S1>
__device__ __forceinline__ void flush_span_hist(const IndexerArgs& a, const uint32_t (*hist)[SBINS], int row0, int span, int tid)
{
    if (tid < SBINS / 2) {
#pragma unroll
        for (int s = 0; s < S1; ++s) {
            const int64_t slot = (int64_t)(row0 + s) * a.pchunks + span;
            reinterpret_cast<uint32_t*>(a.span_hist + slot * SBINS)[tid] = hist[s][2 * tid] | (hist[s][2 * tid + 1] << 16);
        }
    }
    if (span == 0 && tid < 4 * S1) a.counters[(int64_t)row0 * 4 + tid] = 0u;
}

// S1 query tokens of one sequence share every key fragment.
// POW2: block_size is a power of two (page index by shift instead of an integer division per key).
template <int S1, bool POW2, bool F32>
__global__ __launch_bounds__(256) void indexer_score_kernel(IndexerArgs a)
{
    __shared__ __align__(16) uint32_t hist[S1][SBINS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int bi = blockIdx.y;
    const int sgrp = blockIdx.z; // group of S1 consecutive query tokens of the sequence
    const int L = min(a.act_seq[bi], a.max_ctx); // keys past the page table's reach do not exist
    if (blockIdx.x * (CHUNK * PASSES) >= L) return;
    const int row0 = bi * a.s1 + sgrp * S1;

    for (int i = tid; i < S1 * SBINS; i += 256) (&hist[0][0])[i] = 0;

    // int8 A fragments: head hb*16 + l16, bytes 64*ks + 16*g .. +15
    i32x4 qf[S1][4][2];
    // fp16 A fragments of the head sum: row 0 (lanes with l16 == 0) holds w_scale, k-slot (g, e) of MFMA mm is
    // head 32*mm + 16*(e/4) + 4*g + e%4 - the head whose int32 result this lane group holds in that slot
    f16x8 wa[S1][2];
#pragma unroll
    for (int s = 0; s < S1; ++s) {
#pragma unroll
        for (int hb = 0; hb < 4; ++hb) {
            const int8_t* qp = a.q + ((int64_t)(row0 + s) * a.nh + hb * 16 + l16) * D + 16 * g;
            qf[s][hb][0] = *reinterpret_cast<const i32x4*>(qp);
            qf[s][hb][1] = *reinterpret_cast<const i32x4*>(qp + 64);
        }
#pragma unroll
        for (int mm = 0; mm < 2; ++mm)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int64_t h = (int64_t)(row0 + s) * a.nh + 32 * mm + 16 * (e >> 2) + 4 * g + (e & 3);
                wa[s][mm][e] = l16 == 0 ? w_scale_of<F32>(a.q_scale, a.weights, h) : (_Float16)0.f; // one fp16 rounding
            }
    }
    __syncthreads(); // histogram zeroed

    for (int pass = 0; pass < PASSES; ++pass) {
    const int tok_begin = (blockIdx.x * PASSES + pass) * CHUNK;
    if (tok_begin >= L) break;
    const int tok_end = min(L, tok_begin + CHUNK);
    // Each wavefront owns 8 groups of 16 keys.  All page-table lookups are issued first, then all key loads
    // (absent keys read row 0 and get scale 0), so that 4 KB per wavefront are in flight before the first MFMA.
    constexpr int STEPS = CHUNK / 64;
    const int bs = a.block_size, bs_shift = __builtin_ctz(bs);
    int page[STEPS], tk[STEPS];
#pragma unroll
    for (int j = 0; j < STEPS; ++j) {
        tk[j] = min(tok_begin + wave * 16 + 64 * j + l16, tok_end - 1);
        const int pi = POW2 ? tk[j] >> bs_shift : tk[j] / bs;
        page[j] = a.block_table[(int64_t)bi * a.bt_stride + pi];
    }
    int64_t krow[STEPS];
    bool present[STEPS];
#pragma unroll
    for (int j = 0; j < STEPS; ++j) {
        const int in_page = POW2 ? tk[j] & (bs - 1) : tk[j] % bs;
        present[j] = tok_begin + wave * 16 + 64 * j + l16 < tok_end && page[j] >= 0 && page[j] < a.n_blocks;
        krow[j] = present[j] ? (int64_t)page[j] * bs + in_page : 0;
    }
    i32x4 kf0[STEPS], kf1[STEPS];
    typename ScaleOf<F32>::raw ksb[STEPS];
#pragma unroll
    for (int j = 0; j < STEPS; ++j) {
        const int8_t* kp = a.k_cache + krow[j] * D + 16 * g;
        kf0[j] = *reinterpret_cast<const i32x4*>(kp);
        kf1[j] = *reinterpret_cast<const i32x4*>(kp + 64);
        ksb[j] = static_cast<const typename ScaleOf<F32>::raw*>(a.k_scale)[krow[j]];
    }
#pragma unroll
    for (int j = 0; j < STEPS; ++j) {
        const int tok = tok_begin + wave * 16 + 64 * j + l16;
        const bool ok = tok < tok_end;
#pragma unroll
        for (int s = 0; s < S1; ++s) {
            f16x8 y[2];
#pragma unroll
            for (int hb = 0; hb < 4; ++hb) {
                i32x4 acc = {0, 0, 0, 0};
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(qf[s][hb][0], kf0[j], acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(qf[s][hb][1], kf1[j], acc, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    y[hb >> 1][4 * (hb & 1) + r] = (_Float16)((float)max(acc[r], 0) * (1.0f / 2048.0f));
            }
            f32x4 sum = {0.f, 0.f, 0.f, 0.f};
            sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(wa[s][0], y[0], sum, 0, 0, 0);
            sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(wa[s][1], y[1], sum, 0, 0, 0);
            // row 0 of the result: register 0 of lanes 0..15, one key each
            const int eff = L - (a.s1 - 1 - (sgrp * S1 + s));
            if (ok && g == 0) {
                const float sc = sum[0] * (present[j] ? ScaleOf<F32>::f32(ksb[j]) : 0.f);
                a.scores[(int64_t)(row0 + s) * a.score_stride + tok] = sc;
                if (tok < eff) atomicAdd(&hist[s][score_bin(score_key(sc))], 1u);
            }
        }
    }
    } // pass
    __syncthreads();
    flush_span_hist<S1>(a, hist, row0, (int)blockIdx.x, tid);
}

// relu(a) * 2^-11 and relu(b) * 2^-11, each rounded once to fp16, packed (a in the low half).  The int32 sums arrive
// biased: the MFMA accumulators start at SCORE_BIAS = the bit pattern of the float 1.5 * 2^23, and since |a| < 2^21 the
// accumulator's bits, read as a float, are exactly 12582912 + a - the integer-to-float conversion costs nothing.  One
// fused multiply-add takes the bias off and scales (exact in fp32: a * 2^-11 has at most 21 significant bits); relu
// commutes with the rounding to fp16, so it is taken on the packed pair.  (Written in plain C on purpose: the
// compiler's hazard recognizer does not look inside inline assembly, and a hand-placed VALU write into a register that
// an MFMA is still writing goes wrong.)
constexpr int SCORE_BIAS = 0x4B400000;
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t relu_scale_pack(int a, int b)
{
    f16x2 v = {(_Float16)__builtin_fmaf(__int_as_float(a), 0x1p-11f, -6144.0f),
               (_Float16)__builtin_fmaf(__int_as_float(b), 0x1p-11f, -6144.0f)};
    const f16x2 z = {(_Float16)0.f, (_Float16)0.f};
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(v, z));
}

// Score kernel for block sizes that are multiples of 128: a wavefront owns 128 consecutive keys of one page per pass
// (one page-table entry; the entries of all its passes are fetched up front with one load, lane p holding pass p's),
// keeps the loads of the next NBUF-1 half passes (64 keys, 8 KB each) in flight while it scores the current one, and
// files its results 64 at a time: w_scale sits in every row of the head-sum operand, so every lane group holds the 16
// scores of a key group and lane group g keeps those of key group g - after four key groups lane l holds the score of
// key l of the 64, next to that key's scale (loaded with one 128-byte instruction per 64 keys).
constexpr int PPASSES = 4; // passes (of 512 keys) per workgroup of the paged kernel
constexpr int SPAN = CHUNK * PPASSES; // keys per workgroup of either score kernel: one histogram slot
static_assert(SPAN == CHUNK * PASSES, "both score kernels own spans of the same size");
template <int S1, bool F32>
__global__ __launch_bounds__(256, S1 == 1 ? 3 : 2) void indexer_score_paged_kernel(IndexerArgs a)
{
    constexpr int NBUF = 2; // half-pass buffers: NBUF-1 halves ahead (deeper prefetch measured no faster)
    constexpr int NHALF = 2 * PPASSES;
    __shared__ __align__(16) uint32_t hist[S1][SBINS];
    __shared__ __align__(16) float s_sc[S1][CHUNK * PPASSES]; // the workgroup's scores, written out in one burst at the end
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int sgrp = blockIdx.z;
    const int bs = a.block_size;
    // The (sequence, 2048-key span) of this workgroup: by its place in the grid when every sequence fills its spans.
    // With ragged lengths the workgroups that have work should be the first ones of the launch order, so that they
    // spread evenly over the CUs: workgroup w (its place in launch order, sequence-major) takes the w-th span that
    // holds keys.  Every wavefront finds it on its own from the sequence lengths (lane l holds sequences l, l + 64, ..;
    // a wavefront prefix sum of the spans per sequence), which are fetched together with the page-table entries of the
    // grid place; only if the span is another one (ragged lengths) are those fetched again.  Batches beyond
    // SCAN_SEQS sequences keep the grid place.
    // Lane p takes the page-table entry of pass p and the sequence's first entry, and picks once the length is known:
    // it then holds the first cache row of pass p (-1: unmapped page); a pass past the end re-reads the sequence's
    // first page and is discarded.
    int bi = blockIdx.y, span = blockIdx.x;
    const uint32_t w = blockIdx.x + gridDim.x * blockIdx.y;
    constexpr int SCAN_SEQS = 256;
    const bool balanced = a.b <= SCAN_SEQS;
    int lens[SCAN_SEQS / 64];
    // (unconditional loads, so that they travel with the ones below)
#pragma unroll
    for (int j = 0; j < SCAN_SEQS / 64; ++j) lens[j] = a.act_seq[min(lane + 64 * j, a.b - 1)];
    int pg_mine, pg_first, L, mytok;
    auto fetch = [&]() {
        mytok = span * (CHUNK * PPASSES) + wave * 128 + (lane < PPASSES ? lane : 0) * CHUNK;
        const int32_t* bt = a.block_table + (int64_t)bi * a.bt_stride;
        pg_mine = bt[min(mytok / bs, a.bt_stride - 1)];
        pg_first = bt[0];
        L = min(a.act_seq[bi], a.max_ctx); // keys past the page table's reach do not exist
    };
    fetch();
    if (balanced) {
        uint32_t base = 0;
        int fseq = -1, fspan = 0;
#pragma unroll
        for (int j = 0; j < SCAN_SEQS / 64; ++j) {
            const int len = min(lens[j], a.max_ctx);
            const uint32_t cnt = (lane + 64 * j < a.b && len > 0) ? (uint32_t)((len + CHUNK * PPASSES - 1) / (CHUNK * PPASSES)) : 0u;
            const uint32_t incl = wave_prefix_sum(cnt), excl = incl - cnt;
            const uint64_t hit = __ballot(w >= base + excl && w < base + incl); // at most one lane, in one round
            if (hit != 0ull && fseq < 0) {
                const int l = __builtin_ctzll(hit);
                fseq = 64 * j + l;
                fspan = (int)(w - base - (uint32_t)__builtin_amdgcn_readlane((int)excl, l));
            }
            base += (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
        }
        if (fseq < 0) return; // more workgroups than spans with keys
        if (fseq != bi || fspan != span) {
            bi = fseq;
            span = fspan;
            fetch();
        }
    }
    if (span * (CHUNK * PPASSES) >= L) return;
    const int row0 = bi * a.s1 + sgrp * S1;
    const int wtok = span * (CHUNK * PPASSES) + wave * 128; // first key of this wave's pass 0
    int64_t myrow;
    {
        const int tc = mytok < L ? mytok : 0;
        const int pg = mytok < L ? pg_mine : pg_first;
        myrow = (pg >= 0 && pg < a.n_blocks) ? (int64_t)pg * bs + tc % bs : -1;
    }
    auto pass_row = [&](int pass) {
        const uint32_t lo = __builtin_amdgcn_readlane((uint32_t)myrow, pass);
        const uint32_t hi = __builtin_amdgcn_readlane((uint32_t)(myrow >> 32), pass);
        return (int64_t)(((uint64_t)hi << 32) | lo);
    };

    i32x4 kf[NBUF][4][2];
    typename ScaleOf<F32>::raw ksc[NBUF][2]; // [buffer][unused for odd halves]: the scales of a pass travel with its first half
    auto load_half = [&](int hh, int buf) {
        const int64_t r = pass_row(hh >> 1);
        const int64_t rb = r < 0 ? 0 : r;
        const int8_t* kp = a.k_cache + (rb + 64 * (hh & 1) + l16) * D + 16 * g;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            kf[buf][jj][0] = *reinterpret_cast<const i32x4*>(kp + jj * 16 * D);
            kf[buf][jj][1] = *reinterpret_cast<const i32x4*>(kp + jj * 16 * D + 64);
        }
        ksc[buf][0] = static_cast<const typename ScaleOf<F32>::raw*>(a.k_scale)[rb + 64 * (hh & 1) + lane];
    };
    // The key loads go out first; the query and its scales follow them (memory operations complete in order, and the
    // first MFMA needs all of them).  Every memory operation from here on is unconditional, so that the number in
    // flight is the same on every path into the loop and the waits can count them.
#pragma unroll
    for (int u = 0; u < NBUF - 1; ++u) load_half(u, u);
    // int8 A fragments: head hb*16 + l16, bytes 64*ks + 16*g .. +15
    i32x4 qf[S1][4][2];
#pragma unroll
    for (int s = 0; s < S1; ++s)
#pragma unroll
        for (int hb = 0; hb < 4; ++hb) {
            const int8_t* qp = a.q + ((int64_t)(row0 + s) * a.nh + hb * 16 + l16) * D + 16 * g;
            qf[s][hb][0] = *reinterpret_cast<const i32x4*>(qp);
            qf[s][hb][1] = *reinterpret_cast<const i32x4*>(qp + 64);
        }
    // fp16 A fragments of the head sum, the same in every row: k-slot (g, e) of MFMA mm is head
    // 32*mm + 16*(e/4) + 4*g + e%4 - the head whose int32 result this lane group holds in that slot; the value is
    // q_scale * weights in one fp16 rounding
    f16x8 wa[S1][2];
#pragma unroll
    for (int s = 0; s < S1; ++s)
#pragma unroll
        for (int mm = 0; mm < 2; ++mm) {
            typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
            const int64_t h = (int64_t)(row0 + s) * a.nh + 32 * mm + 4 * g;
            const f16x4 wlo = *reinterpret_cast<const f16x4*>(a.weights + h), whi = *reinterpret_cast<const f16x4*>(a.weights + h + 16);
            if constexpr (F32) {
                const f32x4 qlo = *reinterpret_cast<const f32x4*>(static_cast<const float*>(a.q_scale) + h);
                const f32x4 qhi = *reinterpret_cast<const f32x4*>(static_cast<const float*>(a.q_scale) + h + 16);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    wa[s][mm][e] = round_f32_product_to_f16(qlo[e], (float)wlo[e]);
                    wa[s][mm][4 + e] = round_f32_product_to_f16(qhi[e], (float)whi[e]);
                }
            } else {
                const uint16_t* qs = static_cast<const uint16_t*>(a.q_scale);
                const f16x4 qlo = *reinterpret_cast<const f16x4*>(qs + h), qhi = *reinterpret_cast<const f16x4*>(qs + h + 16);
                wa[s][mm] = __builtin_shufflevector(qlo * wlo, qhi * whi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
        }
    for (int i = tid; i < S1 * SBINS; i += 256) (&hist[0][0])[i] = 0;
    __syncthreads();

    auto compute_half = [&](int hh, int buf) {
        float res[S1];
#pragma unroll
        for (int s = 0; s < S1; ++s) res[s] = 0.f;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
#pragma unroll
            for (int s = 0; s < S1; ++s) {
                u32x4 y[2];
#pragma unroll
                for (int hb = 0; hb < 4; ++hb) {
                    i32x4 acc = {SCORE_BIAS, SCORE_BIAS, SCORE_BIAS, SCORE_BIAS};
                    acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(qf[s][hb][0], kf[buf][jj][0], acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(qf[s][hb][1], kf[buf][jj][1], acc, 0, 0, 0);
                    y[hb >> 1][2 * (hb & 1)] = relu_scale_pack(acc[0], acc[1]);
                    y[hb >> 1][2 * (hb & 1) + 1] = relu_scale_pack(acc[2], acc[3]);
                }
                f32x4 sum = {0.f, 0.f, 0.f, 0.f};
                sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(wa[s][0], __builtin_bit_cast(f16x8, y[0]), sum, 0, 0, 0);
                sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(wa[s][1], __builtin_bit_cast(f16x8, y[1]), sum, 0, 0, 0);
                res[s] = jj == g ? sum[0] : res[s];
            }
        }
        const int tok = wtok + (hh >> 1) * CHUNK + 64 * (hh & 1) + lane;
        const float ks = pass_row(hh >> 1) >= 0 ? ScaleOf<F32>::f32(ksc[buf][0]) : 0.f;
#pragma unroll
        for (int s = 0; s < S1; ++s) {
            const float sc = res[s] * ks;
            s_sc[s][tok - span * (CHUNK * PPASSES)] = sc;
            const int eff = L - (a.s1 - 1 - (sgrp * S1 + s));
            if (tok < eff) atomicAdd(&hist[s][score_bin(score_key(sc))], 1u);
        }
    };

    // NBUF halves per trip, so that buffer indices are compile-time constants; past the end the last half is loaded
    // again (a cache hit whose data is never used) so that the loads stay unconditional
    static_assert(NHALF % NBUF == 0, "whole trips");
    for (int base = 0; base < NHALF; base += NBUF) {
#pragma unroll
        for (int u = 0; u < NBUF; ++u) {
            const int hh = base + u;
            if (hh < NHALF) {
                const int nx = hh + NBUF - 1;
                load_half(nx < NHALF ? nx : NHALF - 1, (u + NBUF - 1) % NBUF);
                compute_half(hh, u);
            }
        }
    }
    __syncthreads();
    // one contiguous 8 KB write per query token (256-byte stores from inside the loop, between the key loads, cost
    // 2 us more); score rows are padded to whole workgroup spans, so no bounds check
#pragma unroll
    for (int s = 0; s < S1; ++s) {
        float* dst = a.scores + (int64_t)(row0 + s) * a.score_stride + (int64_t)span * (CHUNK * PPASSES);
#pragma unroll
        for (int i = 0; i < CHUNK * PPASSES / 1024; ++i)
            *reinterpret_cast<f32x4*>(dst + 4 * (tid + 256 * i)) = *reinterpret_cast<const f32x4*>(&s_sc[s][4 * (tid + 256 * i)]);
    }
    flush_span_hist<S1>(a, hist, row0, span, tid);
}

__global__ void indexer_fill_kernel(int32_t* p, int n, int32_t v)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// inclusive suffix sum over a wavefront (lane l gets the sum of v[l .. 63]); all 64 lanes active
__device__ __forceinline__ uint32_t wave_suffix_sum(uint32_t v)
{
    const uint32_t incl = wave_prefix_sum(v);
    return (uint32_t)__builtin_amdgcn_readlane((int)incl, 63) - incl + v;
}

// block-wide inclusive suffix sum (lane t gets sum of v[t .. nthreads-1]); tmp holds one word per wavefront
template <int NWAVES>
__device__ __forceinline__ uint32_t block_suffix_sum(uint32_t v, uint32_t* tmp)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    {
        // suffix = wavefront total - exclusive prefix (unsigned arithmetic, exact)
        const uint32_t incl = wave_prefix_sum(v);
        const uint32_t total = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
        v = total - incl + v;
    }
    __syncthreads();
    if (lane == 0) tmp[wave] = v;
    __syncthreads();
    uint32_t add = 0;
    for (int w = wave + 1; w < NWAVES; ++w) add += tmp[w];
    return v + add;
}

// Valid length of query token `row`'s score row: the sequence's length, cut to what the page table can address
// (the score kernels write no score beyond that), less the query tokens that come after this one.
__device__ __forceinline__ int row_length(const int32_t* act_seq, int row, int s1, int max_ctx)
{
    const int bi = row / s1, si = row - bi * s1;
    return max(min(act_seq[bi], max_ctx) - (s1 - 1 - si), 0);
}

// grid (chunks of SEL_CHUNK scores, query tokens), 256 lanes
__global__ __launch_bounds__(256) void indexer_select_kernel(IndexerArgs a)
{
    __shared__ uint32_t tmp[4];
    __shared__ uint32_t s_bin, s_base_gt, s_base_tie;
    __shared__ __align__(16) uint32_t s_hist[4][SBINS];
    const int tid = threadIdx.x, row = blockIdx.y;
    const int i_begin = blockIdx.x * SEL_CHUNK;
    // everything this workgroup reads is requested at once - the row's length, the histograms of the first GROUP spans
    // and the workgroup's 16 scores per lane (addresses clamped to the padded row) - one round trip.  The histograms
    // are read as they lie in memory, 16 bytes per lane: lane l takes bins 8 (l % 32) .. + 7 of spans l / 32,
    // l / 32 + 8, ..  A slot of a span without keys was never written: it is requested all the same (workspace
    // memory) and left out of the sum once the length is known.
    constexpr int GROUP = 32;
    const int sg = tid >> 5, oct = tid & 31;
    const uint16_t* sh = a.span_hist + (int64_t)row * a.pchunks * SBINS + 8 * oct;
    u32x4 cv[GROUP / 8];
#pragma unroll
    for (int j = 0; j < GROUP / 8; ++j) cv[j] = *reinterpret_cast<const u32x4*>(sh + (int64_t)min(sg + 8 * j, a.pchunks - 1) * SBINS);
    const float* x = a.scores + (int64_t)row * a.score_stride;
    f32x4 v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = *reinterpret_cast<const f32x4*>(x + min(i_begin + 4 * (j * 256 + tid), a.score_stride - 4));
    const int bi = row / a.s1;
    const int len = min(a.act_seq[bi], a.max_ctx);
    const int n = max(len - (a.s1 - 1 - (row - bi * a.s1)), 0);
    // (a workgroup past the row's end leaves further down, behind the first use of what was requested above: an exit
    // here would let the compiler move those requests behind the wait for the length - two round trips instead of one)
    const int nsp = min((len + SPAN - 1) / SPAN, a.pchunks); // spans whose workgroup ran
    if (tid == 0) s_bin = 0xffffffffu; // n <= k: no threshold bin, everything is a winner

    uint32_t acc[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
    for (int g0 = 0; g0 < nsp; g0 += GROUP) { // (one trip but for contexts beyond GROUP spans; block-uniform)
        if (g0 > 0) {
#pragma unroll
            for (int j = 0; j < GROUP / 8; ++j)
                cv[j] = *reinterpret_cast<const u32x4*>(sh + (int64_t)min(g0 + sg + 8 * j, a.pchunks - 1) * SBINS);
        }
#pragma unroll
        for (int j = 0; j < GROUP / 8; ++j) {
            const bool in = g0 + sg + 8 * j < nsp;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                acc[2 * c] += in ? cv[j][c] & 0xffffu : 0u;
                acc[2 * c + 1] += in ? cv[j][c] >> 16 : 0u;
            }
        }
    }
    // the two span groups of a wavefront (lanes l and l + 32 hold the same bins), then the four wavefronts through LDS
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const auto sw = __builtin_amdgcn_permlane32_swap(acc[c], acc[c], false, false);
        acc[c] = (uint32_t)sw[0] + (uint32_t)sw[1];
    }
    if ((tid & 32) == 0) {
        uint32_t* dst = &s_hist[tid >> 6][8 * oct];
        *reinterpret_cast<u32x4*>(dst) = u32x4{acc[0], acc[1], acc[2], acc[3]};
        *reinterpret_cast<u32x4*>(dst + 4) = u32x4{acc[4], acc[5], acc[6], acc[7]};
    }
    __syncthreads();
    if (i_begin >= n) return;
    // bin of the k-th largest key: lane t owns bin t
    const uint32_t own = s_hist[0][tid] + s_hist[1][tid] + s_hist[2][tid] + s_hist[3][tid];
    const uint32_t k = (uint32_t)a.k;
    {
        const uint32_t above = block_suffix_sum<4>(own, tmp) - own; // elements in the bins above
        if (above < k && k <= above + own) s_bin = (uint32_t)tid;
    }
    __syncthreads();
    const uint32_t bin = s_bin;

    // file this workgroup's scores: 16 per lane.  A score's side of the threshold bin is read off its key: winners lie
    // above the bin's largest key, ties between its smallest and largest.  Without a threshold bin every key is a winner.
    uint32_t key_lo = 0u, key_hi = 0u;
    const bool all_win = bin == 0xffffffffu;
    if (!all_win) score_bin_range(bin, key_lo, key_hi);
    uint32_t key[16];
    uint32_t c_gt = 0, c_tie = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int i = i_begin + 4 * (j * 256 + tid) + c;
            const uint32_t u = score_key(v[j][c]);
            key[4 * j + c] = u;
            const bool in = i < n;
            c_gt += in && (all_win || u > key_hi) ? 1u : 0u;
            c_tie += in && !all_win && u >= key_lo && u <= key_hi ? 1u : 0u;
        }
    const uint32_t packed = block_suffix_sum<4>(c_gt | (c_tie << 16), tmp);
    if (tid == 0) {
        uint32_t* cnt = a.counters + (int64_t)row * 4;
        s_base_gt = atomicAdd(cnt, packed & 0xffffu);
        s_base_tie = atomicAdd(cnt + 1, packed >> 16);
    }
    __syncthreads();
    uint32_t p_gt = s_base_gt + (packed & 0xffffu) - c_gt;
    uint32_t p_tie = s_base_tie + (packed >> 16) - c_tie;
    uint64_t* winners = a.winners + (int64_t)row * MAX_K;
    uint64_t* ties = a.ties + (int64_t)row * TIE_CAP;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int i = i_begin + 4 * (j * 256 + tid) + c;
            const uint32_t u = key[4 * j + c];
            const bool in = i < n;
            const bool gt = in && (all_win || u > key_hi), tie = in && !all_win && u >= key_lo && u <= key_hi;
            // (one store per element, to whichever list takes it)
            uint64_t* dst = gt ? winners + p_gt : ties + p_tie;
            if ((gt && p_gt < MAX_K) || (tie && p_tie < TIE_CAP)) *dst = make_cand(u, i);
            p_gt += gt ? 1u : 0u;
            p_tie += tie ? 1u : 0u;
        }
}

// Radix-select the `need` largest of the 64-bit words f enumerates (all share the bits above `top`), top-down
// in digits of 11 bits; every selected word is handed to emit().  Words are distinct, so the walk ends with a
// bin that is taken whole.  Workgroup of 1024 lanes; hist has 2048 words, tmp 16.
template <class Each, class Emit>
__device__ __forceinline__ void radix_select64(Each&& for_each, Emit&& emit, uint32_t need, int top, uint32_t* hist,
                                               uint32_t* tmp, uint32_t* s_bin, uint32_t* s_krem, uint32_t* s_cnt)
{
    const int tid = threadIdx.x;
    uint64_t prefix = 0, known = 0; // bits fixed so far and their mask
    while (need > 0 && top > 0) {
        const int bits = top >= 11 ? 11 : top;
        const int shift = top - bits;
        const uint64_t dmask = (1ull << bits) - 1ull;
        hist[tid] = 0;
        hist[tid + 1024] = 0;
        __syncthreads();
        for_each([&](uint64_t w) {
            if ((w & known) == prefix) atomicAdd(&hist[(uint32_t)((w >> shift) & dmask)], 1u);
        });
        __syncthreads();
        const uint32_t h_lo = hist[2 * tid], h_hi = hist[2 * tid + 1]; // lane t owns bins 2t and 2t+1
        const uint32_t incl = block_suffix_sum<16>(h_lo + h_hi, tmp);
        const uint32_t above_hi = incl - h_lo - h_hi, above_lo = above_hi + h_hi;
        if (above_hi < need && need <= above_hi + h_hi) {
            *s_bin = 2 * tid + 1;
            *s_krem = need - above_hi;
            *s_cnt = h_hi;
        } else if (above_lo < need && need <= above_lo + h_lo) {
            *s_bin = 2 * tid;
            *s_krem = need - above_lo;
            *s_cnt = h_lo;
        }
        __syncthreads();
        const uint64_t b = *s_bin;
        const uint32_t krem = *s_krem, cnt = *s_cnt;
        // everything in the bins above b is selected; bin b whole if it is exactly what is missing
        const bool whole = cnt == krem;
        for_each([&](uint64_t w) {
            if ((w & known) != prefix) return;
            const uint64_t d = (w >> shift) & dmask;
            if (d > b || (whole && d == b)) emit(w);
        });
        __syncthreads();
        if (whole) return;
        prefix |= b << shift;
        known |= dmask << shift;
        need = krem;
        top = shift;
    }
}

// cand[0 .. m) holds the selected words in any order (the rest of its 2048 slots is zero): write their indices in
// descending word order, then -1 up to k.  The words are first grouped by key into at most 2048 equal steps of the
// selected keys' range, so a counting pass (histogram, suffix scan, scatter) puts every word within a few slots of
// its place - and then ranked inside their group by direct comparison.  A bin with more than 64 words (heavily tied scores)
// would make that ranking quadratic; then a bitonic sort of all 2048 words is used instead.
// Workgroup of 1024 lanes; hist has 2048 words, scratch 8192 words (start | cursor | grouped words), tmp 16.
__device__ __forceinline__ void order_and_write(uint64_t* cand, uint32_t m, uint32_t* hist, uint32_t* scratch,
                                                uint32_t* tmp, uint32_t* s_flag, int32_t* out, int k)
{
    const int tid = threadIdx.x;
    uint32_t* start = scratch;          // [2048] slots taken by the higher bins
    uint32_t* cursor = scratch + NBINS; // [2048]
    uint64_t* grouped = reinterpret_cast<uint64_t*>(scratch + 2 * NBINS); // [2048]
    hist[tid] = 0;
    hist[tid + 1024] = 0;
    cursor[tid] = 0;
    cursor[tid + 1024] = 0;
    if (tid == 0) {
        *s_flag = 0;
        tmp[14] = 0xffffffffu; // smallest selected key
        tmp[15] = 0u;          // largest selected key
    }
    __syncthreads();
    uint64_t w[2];
    uint32_t bin[2];
    bool valid[2];
    uint32_t kmin = 0xffffffffu, kmax = 0u;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int i = tid + 1024 * h;
        valid[h] = (uint32_t)i < m;
        w[h] = cand[i];
        if (valid[h]) {
            kmin = min(kmin, (uint32_t)(w[h] >> 32));
            kmax = max(kmax, (uint32_t)(w[h] >> 32));
        }
    }
    kmin = wave_min(kmin);
    kmax = wave_max(kmax);
    if ((tid & 63) == 0) {
        atomicMin(&tmp[14], kmin);
        atomicMax(&tmp[15], kmax);
    }
    __syncthreads();
    // bins: the selected keys' range cut into at most 2048 equal steps (the keys are order-preserving images of the
    // scores, dense enough over the top-k range that a step holds a handful of words)
    kmin = tmp[14];
    const uint32_t range = tmp[15] - kmin;
    const int shift = max(0, 21 - (int)__builtin_clz(range | 1u));
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        bin[h] = ((uint32_t)(w[h] >> 32) - kmin) >> shift;
        if (valid[h]) atomicAdd(&hist[bin[h]], 1u);
    }
    __syncthreads();
    {
        const uint32_t h_lo = hist[2 * tid], h_hi = hist[2 * tid + 1]; // lane t owns bins 2t and 2t+1
        if (h_lo > 64u || h_hi > 64u) *s_flag = 1;
        const uint32_t incl = block_suffix_sum<16>(h_lo + h_hi, tmp);
        start[2 * tid + 1] = incl - h_lo - h_hi;
        start[2 * tid] = incl - h_lo;
    }
    __syncthreads();
    if (*s_flag == 0) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
            if (valid[h]) grouped[start[bin[h]] + atomicAdd(&cursor[bin[h]], 1u)] = w[h];
        __syncthreads();
#pragma unroll
        for (int h = 0; h < 2; ++h)
            if (valid[h]) {
                const uint32_t s0 = start[bin[h]], c = hist[bin[h]];
                uint32_t rank = 0;
                for (uint32_t j = 0; j < c; ++j) rank += grouped[s0 + j] > w[h] ? 1u : 0u;
                if ((int)(s0 + rank) < k) out[s0 + rank] = (int32_t)(0xffffffffu - (uint32_t)(w[h] & 0xffffffffull));
            }
        for (int j = (int)m + tid; j < k; j += 1024) out[j] = -1;
        return;
    }
    // bitonic sort, descending, 2048 words, two per lane.  A compare-exchange step of stride <= 64 stays inside
    // the 128 words owned by one wavefront (lane i of wave w handles the pair (128w + 2i - i%stride, + stride)),
    // so only the steps of stride >= 128 need a workgroup barrier; the others rely on LDS operations of one
    // wavefront completing in order.
    for (int size = 2; size <= MAX_K; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            if (stride >= 128) __syncthreads();
            const int pos = 2 * tid - (tid & (stride - 1)); // lower index of the pair
            const bool desc = (pos & size) == 0;
            const uint64_t lo = cand[pos], hi = cand[pos + stride];
            if ((lo < hi) == desc) {
                cand[pos] = hi;
                cand[pos + stride] = lo;
            }
            if (stride >= 128) __syncthreads();
            else __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        }
    }
    __syncthreads();
    for (int j = tid; j < k; j += 1024) out[j] = (int32_t)(0xffffffffu - (uint32_t)(cand[j] & 0xffffffffull));
}

__global__ __launch_bounds__(1024) void indexer_topk_kernel(IndexerArgs a)
{
    __shared__ uint32_t hist[NBINS];
    __shared__ uint64_t cand[MAX_K];
    __shared__ uint64_t tie[TIE_CAP];
    __shared__ uint32_t tmp[16];
    __shared__ uint32_t s_bin, s_krem, s_cnt, s_out;

    const int tid = threadIdx.x, row = blockIdx.x;
    // the winners and the first 2048 ties are requested together with the counts that say how many of them are real
    // (the lists are workspace memory: reading past their fill is harmless), one round trip instead of three
    const uint64_t* wsrc = a.winners + (int64_t)row * MAX_K;
    const uint64_t* tsrc = a.ties + (int64_t)row * TIE_CAP;
    static_assert(MAX_K == 2048 && TIE_CAP >= 2048, "two winners and two early ties per lane");
    const uint64_t w0 = wsrc[tid], w1 = wsrc[tid + 1024];
    const uint64_t t0 = tsrc[tid], t1 = tsrc[tid + 1024];
    const int n = row_length(a.act_seq, row, a.s1, a.max_ctx);
    const int k = a.k;
    // (the counters of a query token are cleared by its sequence's first score workgroup: a sequence without keys has none)
    const uint32_t c_gt = a.counters[(int64_t)row * 4], c_tie = a.counters[(int64_t)row * 4 + 1];
    const uint32_t n_gt = n > 0 ? min(c_gt, (uint32_t)MAX_K) : 0u;
    const uint32_t n_tie = n > 0 ? c_tie : 0u;
    const uint32_t need = (uint32_t)min(n, k) - min(n_gt, (uint32_t)min(n, k));

    cand[tid] = tid < (int)n_gt ? w0 : 0ull;
    cand[tid + 1024] = tid + 1024 < (int)n_gt ? w1 : 0ull;
    tie[tid] = t0;
    tie[tid + 1024] = t1;
    if (tid == 0) s_out = n_gt;
    __syncthreads();
    auto emit = [&](uint64_t w) {
        const uint32_t p = atomicAdd(&s_out, 1u);
        if (p < MAX_K) cand[p] = w;
    };

    if (need > 0 && n_tie <= TIE_CAP) {
        // the usual case: the tie list (one histogram bin) fits in LDS
        if (n_tie > 2048) { // block-uniform
            for (int i = tid + 2048; i < (int)n_tie; i += 1024) tie[i] = tsrc[i];
            __syncthreads();
        }
        auto each = [&](auto&& f) {
            for (int i = tid; i < (int)n_tie; i += 1024) f(tie[i]);
        };
        if (score_bin_is_interior(score_bin((uint32_t)(tie[0] >> 32)))) {
            // The ties of an interior bin share their top 11 key bits.  They are counted by the next six (64 steps in
            // key order, one LDS counter each); a suffix scan of the 64 counts by one wavefront finds the step that holds
            // the last wanted tie.  Ties in the steps above it are taken, those inside it (a few dozen) are set aside
            // and ranked against each other.  (Against a digit of the radix select: 64 counters instead of 2048 to clear
            // and scan, and no second digit.)
            uint32_t* subc = hist + NBINS - SUBBINS; // (the far end of hist: its front holds the ties set aside)
            if (tid < SUBBINS) subc[tid] = 0u;
            if (tid == 0) { // (overwritten below by the lane whose step it is)
                s_bin = 0u;
                s_krem = need;
                s_cnt = 0xffffffffu;
                tmp[0] = 0u;
            }
            __syncthreads();
            each([&](uint64_t w) { atomicAdd(&subc[tie_sub_bin((uint32_t)(w >> 32))], 1u); });
            __syncthreads();
            if (tid < SUBBINS) {
                const uint32_t c_sub = subc[tid];
                const uint32_t above = wave_suffix_sum(c_sub) - c_sub;
                if (above < need && need <= above + c_sub) {
                    s_bin = (uint32_t)tid;
                    s_krem = need - above;
                    s_cnt = c_sub;
                }
            }
            __syncthreads();
            const uint32_t sb = s_bin, krem = s_krem, cnt = s_cnt;
            const bool whole = cnt == krem, small = cnt <= SUB_RANK_CAP;
            uint64_t* aside = reinterpret_cast<uint64_t*>(hist);
            each([&](uint64_t w) {
                const uint32_t d = tie_sub_bin((uint32_t)(w >> 32));
                if (d > sb || (whole && d == sb))
                    emit(w);
                else if (d == sb && small) {
                    const uint32_t p = atomicAdd(&tmp[0], 1u);
                    if (p < SUB_RANK_CAP) aside[p] = w;
                }
            });
            __syncthreads();
            if (!whole && small) {
                // (words are distinct: the rank of one among the others is the number of larger ones)
                if (tid < (int)cnt) {
                    const uint64_t w = aside[tid];
                    uint32_t larger = 0;
                    for (uint32_t j = 0; j < cnt; ++j) larger += aside[j] > w ? 1u : 0u;
                    if (larger < krem) emit(w);
                }
            } else if (!whole) {
                // a crowded step (heavily tied scores): digit by digit over its 15 remaining key bits and the index
                __syncthreads();
                auto each_in = [&](auto&& f) {
                    each([&](uint64_t w) {
                        if (tie_sub_bin((uint32_t)(w >> 32)) == sb) f(w);
                    });
                };
                radix_select64(each_in, emit, krem, 47, hist, tmp, &s_bin, &s_krem, &s_cnt);
            }
        } else {
            // a first or last bin (magnitudes outside the histogram's range): its keys need not share any bits
            radix_select64(each, emit, need, 64, hist, tmp, &s_bin, &s_krem, &s_cnt);
        }
    } else if (need > 0) {
        // overflowed tie list: select over the whole row instead (winners are found again, so start empty)
        if (tid == 0) s_out = 0;
        __syncthreads();
        const float* x = a.scores + (int64_t)row * a.score_stride;
        auto each = [&](auto&& f) {
            for (int i0 = 4 * tid; i0 < n; i0 += 4096) {
                const f32x4 v = *reinterpret_cast<const f32x4*>(x + i0);
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    if (i0 + c < n) f(make_cand(score_key(v[c]), i0 + c));
            }
        };
        radix_select64(each, emit, (uint32_t)min(n, k), 64, hist, tmp, &s_bin, &s_krem, &s_cnt);
    }
    __syncthreads();

    order_and_write(cand, (uint32_t)min(n, k), hist, reinterpret_cast<uint32_t*>(tie), tmp, &s_bin,
                    a.topk_res + (int64_t)row * k, k);
}

// Standalone top-k of fp32 rows (pypto.topk: python/pypto/op/comparison.py:302-344; order of equal values - smaller
// index first - framework/src/interface/interpreter/calculator/calc_torch.cpp:2481-2494,2734-2749): values and int32
// indices of the k largest (or smallest) elements of every row, best first.  One workgroup of 1024 lanes per row.  Rows
// of up to TOPK_SORT_CAP elements are sorted whole in LDS; longer rows (then k <= MAX_K) go through the radix select
// first.  Words are (key << 32 | ~index) with the order-preserving key of the value (of its negation for the smallest),
// so descending word order is the rule above; -0 and +0 count as equal.
constexpr int TOPK_SORT_CAP = 8192;

// bitonic sort of a[0 .. p), p a power of two <= TOPK_SORT_CAP, descending; 1024 lanes
__device__ __forceinline__ void bitonic_desc(uint64_t* a, int p)
{
    const int tid = threadIdx.x;
    for (int size = 2; size <= p; size <<= 1)
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (int i = tid; i < p / 2; i += 1024) {
                const int pos = 2 * i - (i & (stride - 1)); // lower index of the pair
                const bool desc = (pos & size) == 0;
                const uint64_t lo = a[pos], hi = a[pos + stride];
                if ((lo < hi) == desc) {
                    a[pos] = hi;
                    a[pos + stride] = lo;
                }
            }
        }
    __syncthreads();
}

__global__ __launch_bounds__(1024) void topk_rows_kernel(const float* __restrict__ x, float* __restrict__ values,
                                                         int32_t* __restrict__ indices, int n, int k, int largest)
{
    __shared__ uint64_t buf[TOPK_SORT_CAP];
    __shared__ uint32_t hist[NBINS];
    __shared__ uint32_t tmp[16];
    __shared__ uint32_t s_bin, s_krem, s_cnt, s_out;
    const int tid = threadIdx.x;
    const float* row = x + (int64_t)blockIdx.x * n;
    auto word = [&](int i) { return make_cand(score_key(largest ? row[i] : -row[i]), i); };
    int p;
    if (n <= TOPK_SORT_CAP) {
        p = 2;
        while (p < n) p <<= 1;
        for (int i = tid; i < p; i += 1024) buf[i] = i < n ? word(i) : 0ull; // (every real word is > 0: its index part is)
    } else {
        p = MAX_K;
        for (int i = tid; i < MAX_K; i += 1024) buf[i] = 0ull;
        if (tid == 0) s_out = 0;
        __syncthreads();
        auto each = [&](auto&& f) {
            for (int i = tid; i < n; i += 1024) f(word(i));
        };
        auto emit = [&](uint64_t w) {
            const uint32_t q = atomicAdd(&s_out, 1u);
            if (q < MAX_K) buf[q] = w;
        };
        radix_select64(each, emit, (uint32_t)k, 64, hist, tmp, &s_bin, &s_krem, &s_cnt);
    }
    bitonic_desc(buf, p);
    for (int j = tid; j < k; j += 1024) {
        const int i = (int)(0xffffffffu - (uint32_t)(buf[j] & 0xffffffffull));
        indices[(int64_t)blockIdx.x * k + j] = i;
        values[(int64_t)blockIdx.x * k + j] = row[i];
    }
}

} // namespace

bool topk_supported(int64_t n, int64_t k) { return n >= 1 && k >= 1 && k <= n && n <= (1 << 24) && (n <= TOPK_SORT_CAP || k <= MAX_K); }

hipError_t topk_launch(const float* x, float* values, int32_t* indices, int64_t rows, int n, int k, bool largest, hipStream_t stream)
{
    if (rows == 0) return hipSuccess;
    hipLaunchKernelGGL(topk_rows_kernel, dim3((unsigned)rows), dim3(1024), 0, stream, x, values, indices, n, k, largest ? 1 : 0);
    return hipGetLastError();
}

// workspace: scores [t, stride] f32 | span_hist [t, spans, 256] u16 | counters [t, 4] u32 | winners [t, 2048] u64 |
// ties [t, 8192] u64; spans = stride / 2048
static uint64_t align256(uint64_t x) { return (x + 255) & ~(uint64_t)255; }

uint64_t indexer_workspace_bytes(int t, int stride)
{
    const uint64_t spans = (uint64_t)stride / SPAN;
    return align256((uint64_t)t * stride * 4) + align256((uint64_t)t * spans * SBINS * 2) + align256((uint64_t)t * 4 * 4) +
           align256((uint64_t)t * (MAX_K + TIE_CAP) * 8);
}

void indexer_bind_workspace(IndexerArgs& a, void* ws)
{
    const int t = a.b * a.s1;
    const uint64_t spans = (uint64_t)a.score_stride / SPAN;
    uint8_t* p = static_cast<uint8_t*>(ws);
    a.scores = reinterpret_cast<float*>(p);
    p += align256((uint64_t)t * a.score_stride * 4);
    a.span_hist = reinterpret_cast<uint16_t*>(p);
    p += align256((uint64_t)t * spans * SBINS * 2);
    a.counters = reinterpret_cast<uint32_t*>(p);
    p += align256((uint64_t)t * 4 * 4);
    a.winners = reinterpret_cast<uint64_t*>(p);
    a.ties = a.winners + (uint64_t)t * MAX_K;
    a.pchunks = (int32_t)spans;
}

hipError_t indexer_launch(const IndexerArgs& a, hipStream_t stream)
{
    const int t = a.b * a.s1;
    if (t == 0) return hipSuccess;
    const int max_ctx = a.bt_stride * a.block_size;
    if (max_ctx == 0 || a.n_blocks == 0) { // a page table without columns, or a cache without pages: no key exists, every slot is -1
        const int n = t * a.k;
        hipLaunchKernelGGL(indexer_fill_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, a.topk_res, n, -1);
        return hipGetLastError();
    }
    // one workgroup per 2048-key span the page table can address (a.pchunks slots per query token hold at least as many)
    const int chunks = (max_ctx + SPAN - 1) / SPAN;
    const int pchunks = chunks;
    IndexerArgs args = a;
    args.max_ctx = max_ctx;
    {
        ScopedKernelTimer tm(KID_INDEXER_SCORE, stream);
        const bool pow2 = (a.block_size & (a.block_size - 1)) == 0;
        const bool s2 = a.s1 % 2 == 0, f32 = a.scales_f32;
        if (a.block_size % 128 == 0) {
            auto kern = s2 ? (f32 ? indexer_score_paged_kernel<2, true> : indexer_score_paged_kernel<2, false>)
                           : (f32 ? indexer_score_paged_kernel<1, true> : indexer_score_paged_kernel<1, false>);
            hipLaunchKernelGGL(kern, dim3(pchunks, a.b, s2 ? a.s1 / 2 : a.s1), dim3(256), 0, stream, args);
        } else {
            auto kern = s2 ? (pow2 ? (f32 ? indexer_score_kernel<2, true, true> : indexer_score_kernel<2, true, false>)
                                   : (f32 ? indexer_score_kernel<2, false, true> : indexer_score_kernel<2, false, false>))
                           : (pow2 ? (f32 ? indexer_score_kernel<1, true, true> : indexer_score_kernel<1, true, false>)
                                   : (f32 ? indexer_score_kernel<1, false, true> : indexer_score_kernel<1, false, false>));
            hipLaunchKernelGGL(kern, dim3(chunks, a.b, s2 ? a.s1 / 2 : a.s1), dim3(256), 0, stream, args);
        }
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    {
        ScopedKernelTimer tm(KID_INDEXER_SELECT, stream);
        hipLaunchKernelGGL(indexer_select_kernel, dim3((max_ctx + SEL_CHUNK - 1) / SEL_CHUNK, t), dim3(256), 0, stream, args);
    }
    {
        ScopedKernelTimer tm(KID_INDEXER_TOPK, stream);
        hipLaunchKernelGGL(indexer_topk_kernel, dim3(t), dim3(1024), 0, stream, args);
    }
    return hipGetLastError();
}

} // namespace pto
