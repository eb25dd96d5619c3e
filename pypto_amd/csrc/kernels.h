// Host-side launch interface between the C ABI (api.cpp) and the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pto {

// ---------------------------------------------------------------- sparse flash attention
struct SfaArgs {
    const void* q_nope; // [t*nq, 512] bf16
    const void* q_rope; // [t*nq, 64]  bf16
    // Cache streams, each addressed as base + row * stride (bytes): three tensors, or three
    // offsets into one packed 656-byte row.
    const uint8_t* kn; // 512 x int8 (or 512 x bf16 when !quant)
    const uint8_t* kr; // 64 x bf16
    const uint8_t* ks; // 4 x fp32
    uint32_t kn_stride, kr_stride, ks_stride;
    int64_t n_rows;
    const int32_t* topk_idx;    // [t, topk_stride]
    const int32_t* block_table; // [b, bt_stride]
    const int32_t* act_seq;     // [b]
    void* out;                  // [t*nq, 512] bf16
    _Float16* part_o;           // [t, nsplit, head groups, 128 x 512] fp16 in the accumulators' fragment order: each split's output normalised by its own sum (nsplit > 1)
    float* part_ml;             // [t, nsplit, nq, 2]  fp32 (running max in log2 units, sum)
    int32_t b, s1, nq, topk, topk_stride, block_size, bt_stride, nsplit;
    int32_t split_cap; // set by sfa_launch: capacity (tokens) of the per-split LDS arrays
    int32_t bt_cached; // set by sfa_launch: the sequence's page table fits in LDS
    float softmax_scale;
    bool quant;
};

int sfa_pick_splits(int t, int nq, int topk);
uint64_t sfa_workspace_bytes(int t, int nq, int nsplit);
uint64_t sfa_partials_bytes(int t, int nq, int nsplit); // the fp16 partials at the front of that workspace; (m, l) follow
hipError_t sfa_launch(const SfaArgs& a, hipStream_t stream);
// Device address, on the current device, of the library's own scratch array of SFA_STATIC_SCRATCH_BYTES bytes (looked up
// once per device).  Every call on a GPU shares that GPU's array.
constexpr uint64_t SFA_STATIC_SCRATCH_BYTES = 40ull << 20;
hipError_t sfa_static_scratch(void** ptr);

// ---------------------------------------------------------------- lightning indexer
struct IndexerArgs {
    const int8_t* q;             // [t, nh, 128]
    const void* q_scale;         // [t, nh] fp16, or fp32 when scales_f32
    const int8_t* k_cache;       // [blocks*bs, 128]
    const void* k_scale;         // [blocks*bs] fp16, or fp32 when scales_f32
    const uint16_t* weights;     // [t, nh] fp16
    const int32_t* act_seq;      // [b]
    const int32_t* block_table;  // [b, bt_stride]
    int32_t* topk_res;           // [t, k]
    float* scores;               // workspace [t, score_stride]
    uint16_t* span_hist;         // workspace [t, pchunks, 256]: per 2048-key span, histogram of the score keys (quarter octaves)
    uint32_t* counters;          // workspace [t, 4]: winners, ties (cleared by the score kernel)
    uint64_t* winners;           // workspace [t, 2048]
    uint64_t* ties;              // workspace [t, 8192]
    int64_t n_blocks;
    int32_t b, s1, nh, block_size, bt_stride, k, score_stride;
    int32_t max_ctx; // set by indexer_launch: bt_stride * block_size, the longest sequence the page table can address
    bool scales_f32; // q_scale and k_scale are fp32: w_scale = fp16(q_scale * fp32(weight)), k_scale enters the score as it is
    int32_t pchunks; // set by indexer_bind_workspace: histogram slots (2048-key spans) per query token = score_stride / 2048
};

uint64_t indexer_workspace_bytes(int t, int score_stride);
void indexer_bind_workspace(IndexerArgs& a, void* workspace);
hipError_t indexer_launch(const IndexerArgs& a, hipStream_t stream);

// ---------------------------------------------------------------- standalone top-k of fp32 rows
bool topk_supported(int64_t n, int64_t k); // rows of up to 8192 elements with any k <= n; longer rows with k <= 2048
hipError_t topk_launch(const float* x, float* values, int32_t* indices, int64_t rows, int n, int k, bool largest,
                       hipStream_t stream);

// ---------------------------------------------------------------- grouped expert selection
struct SelectExpertsArgs {
    const void* logits; // [t, ne] fp32 or bf16
    const void* bias;   // [ne] bf16 or fp32
    float* topk_weights; // [t, top_k]
    int32_t* topk_ids;   // [t, top_k]
    int64_t t;
    int32_t ne, top_k, topk_group, n_group;
    float routed_scaling_factor;
    bool renormalize, fill_neg_inf, logits_bf16, bias_bf16;
};

bool select_experts_supported(int ne, int n_group, int top_k);
hipError_t select_experts_launch(const SelectExpertsArgs& a, hipStream_t stream);

// ---------------------------------------------------------------- paged GQA decode attention
struct GqaArgs {
    const void* q;  // [t, nq, 128] bf16
    const void* k;  // [blocks, block_size, nkv, 128] bf16
    const void* v;  // same shape
    const int32_t* block_table; // [b, bt_stride]
    const int32_t* act_seq;     // [b]
    void* out;                  // [t, nq, 128] bf16
    float* part_o;              // workspace [t*nq, nsplit, 128] fp32 (nsplit > 1)
    float* part_ml;             // workspace [t*nq, nsplit, 2]: running max (log2 units), sum
    int64_t n_blocks;
    int32_t b, s1, nq, nkv, hsub, block_size, bt_stride, nsplit, chunk;
    float softmax_scale;
};

void gqa_pick_chunk(int max_ctx, int forced_chunk, int* chunk, int* nsplit);
uint64_t gqa_workspace_bytes(int64_t t, int nq, int nsplit);
hipError_t gqa_launch(const GqaArgs& a, hipStream_t stream);

// ---------------------------------------------------------------- lightning indexer prolog
struct PrologArgs {
    const uint16_t* x;         // [t, h] bf16
    const int8_t* q_norm;      // [t, r]
    const float* q_norm_scale; // [t]
    const int8_t* w_qb;        // [r, n*128]
    const float* w_qb_scale;   // [n*128]
    const uint16_t* w_k;       // [h, 128] bf16
    const uint16_t* w_proj;    // [h, n] bf16
    const uint16_t* ln_gamma;  // [128] bf16
    const uint16_t* ln_beta;   // [128] bf16
    const uint16_t* cos;       // [t, 64] bf16
    const uint16_t* sin;       // [t, 64] bf16
    const uint16_t* had_q;     // [128, 128] bf16
    const uint16_t* had_k;     // [128, 128] bf16
    int8_t* k_cache;           // [cache_rows, 128], updated in place
    uint16_t* k_scale_cache;   // [cache_rows] fp16, updated in place
    const int64_t* k_cache_index; // [t]
    int8_t* q_int8;            // [t, n, 128]
    uint16_t* q_scale;         // [t, n] fp16
    uint16_t* weights;         // [t, n] fp16
    float* xw_part;            // fp32 partial sums of x @ [w_k | w_proj]: element (split, token, col) at
                               // xw_part[(split * t + token) * xw_stride + xw_col0 + col]
    int32_t xw_stride, xw_col0;
    int64_t cache_rows;
    int32_t t, h, r, n, ksplits;
    float eps, wscale_n, wscale_d;
};

bool prolog_supported(int64_t h, int64_t r, int64_t n, int64_t d, int64_t rope);
uint64_t prolog_workspace_bytes(int64_t t, int64_t h, int64_t r, int64_t n);
void prolog_bind_workspace(PrologArgs& a, void* workspace);
hipError_t prolog_launch(const PrologArgs& a, hipStream_t stream);

// ---------------------------------------------------------------- MLA prolog (int8 form)
struct MlaPrologArgs {
    const uint16_t* x;          // [t, h] bf16
    const uint16_t* w_dq;       // [h, r] bf16
    const void* w_uq_qr;        // [r, n*192] int8 (bf16 in the bf16 form)
    const float* w_qb_scale;    // [n*192]
    const uint16_t* w_uk;       // [n, 128, 512] bf16
    const uint16_t* w_dkv_kr;   // [h, 576] bf16
    const uint16_t* gamma_cq;   // [r] bf16
    const uint16_t* gamma_ckv;  // [512] bf16
    const uint16_t* cos;        // [t, 64] bf16
    const uint16_t* sin;        // [t, 64] bf16
    const int64_t* cache_index; // [t]
    int8_t* kv_cache;           // [cache_rows, 512] int8 (bf16 in the bf16 form), updated in place
    uint16_t* kr_cache;         // [cache_rows, 64] bf16, updated in place
    float* k_scale_cache;       // [cache_rows, 4], updated in place
    int8_t* q_norm;             // [t, r] int8 (bf16 in the bf16 form)
    float* q_norm_scale;        // [t]
    uint16_t* q_nope;           // [t, n, 512] bf16
    uint16_t* q_rope;           // [t, n, 64] bf16
    const uint16_t* w_k;        // fused with the indexer prolog only: its [h, 128] and [h, n_idx] bf16 weights, whose
    const uint16_t* w_proj;     // products with x ride along in the first kernel
    float* xa_part;             // workspace [ksplits, t, ncols]
    uint16_t* qb_nope;          // workspace [t, n, 128] bf16
    float* qb_part;             // workspace, bf16 form only: [ceil(r / 1024), t, n*192] partial sums of q_norm @ w_uq_qr
    int64_t cache_rows;
    int32_t t, h, r, n, ksplits;
    int32_t n_idx, ncols;       // index heads (0: not fused); columns of a partial-sum row: r + 576 (+ 128 + n_idx)
    float eps_cq, eps_ckv;
    bool quant;                 // int8 form (w_uq_qr int8 + scales, int8 cache) or bf16 form
};

bool mla_prolog_supported(int64_t h, int64_t r, int64_t n, int64_t d_nope, int64_t d_rope, int64_t c);
uint64_t mla_prolog_workspace_bytes(int64_t t, int64_t h, int64_t r, int64_t n, int64_t n_idx, bool quant);
void mla_prolog_bind_workspace(MlaPrologArgs& a, void* workspace);
hipError_t mla_prolog_launch(const MlaPrologArgs& a, hipStream_t stream);
// The fused MLA + indexer prolog as four launches (needs n_idx a multiple of 64); fused_prolog_bind points the indexer's
// partial sums into the MLA prolog's and sizes are those of mla_prolog_workspace_bytes(.., n_idx).
bool fused_prolog_supported(int64_t n_idx);
void fused_prolog_bind(MlaPrologArgs& m, PrologArgs& p, void* workspace);
hipError_t fused_prolog_launch(const MlaPrologArgs& m, const PrologArgs& p, hipStream_t stream);

// ---------------------------------------------------------------- GLM-4.5 attention_pre_quant
struct AttnPreArgs {
    const uint16_t* x;          // [t, h] bf16 hidden states
    const uint16_t* residual;   // [t, h] bf16
    const uint16_t* gamma;      // [h] bf16 input norm weight
    const uint16_t* bias;       // [h] bf16 input norm bias
    const uint16_t* in_scale;   // [h] bf16 quantisation scale (multiplied)
    const uint16_t* in_offset;  // [h] bf16 quantisation offset (added)
    const int8_t* w;            // [h, n_out] int8
    const int32_t* qbias;       // [n_out]
    const float* deq;           // [n_out]
    const uint16_t* q_gamma;    // [128] bf16
    const uint16_t* q_bias;
    const uint16_t* k_gamma;
    const uint16_t* k_bias;
    const uint16_t* cos;        // [t, 1, half] bf16
    const uint16_t* sin;
    uint16_t* q;                // [t, q_heads * 128] bf16
    uint16_t* k;                // [t, kv_heads * 128]
    uint16_t* v;                // [t, kv_heads * 128]
    uint16_t* residual_out;     // [t, h]
    int8_t* x_q;                // workspace [t, h]: the quantised normalised rows
    int32_t* part;              // workspace [ksplits, t, n_out]: int32 partial sums of the projection
    int32_t t, h, n_out, q_heads, kv_heads, half, ksplits;
    float eps, mean_coff;       // mean_coff = fp32(1 / h)
};

bool attention_pre_supported(int64_t h, int64_t d, int64_t half);
int attention_pre_ksplits(int64_t t, int64_t h, int64_t n_out); // partial sums per output of the projection
uint64_t attention_pre_workspace_bytes(int64_t t, int64_t h, int64_t n_out);
void attention_pre_bind_workspace(AttnPreArgs& a, void* workspace);
hipError_t attention_pre_launch(const AttnPreArgs& a, hipStream_t stream);

// ---------------------------------------------------------------- paged row gather
struct GatherArgs {
    const void* src;         // [n_src, hidden], any element type
    const void* indices;     // [b, k] int32 or int64 logical token indices
    const void* block_table; // [b, nblk] int32 or int64 physical page of each logical page
    void* out;               // [b * k, size]
    int32_t* status;         // optional: incremented once per entry that addresses no source row
    int64_t rows, k, nblk, block_size, n_src;
    int64_t src_pitch, row_bytes; // bytes between source rows; bytes copied per row (= output pitch)
    bool idx64, bt64;
};

hipError_t paged_gather_launch(const GatherArgs& a, hipStream_t stream);

} // namespace pto
