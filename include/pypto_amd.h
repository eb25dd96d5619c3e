/*
 * pypto_amd.h - C ABI of the MI355X-native DeepSeek-V3.2 sparse decode-attention operators.
 *
 * The library (libpypto_amd.so, built from pypto_amd/csrc with hipcc for gfx950) is the drop-in
 * boundary for three operator families of the reference's models/deepseek_v32_exp directory.  Each
 * operator is a workspace-query / launch pair over one flat tensor list, the calling convention of the
 * reference's ahead-of-time kernel bundle ABI (framework/include/tile_fwk_bundle/pypto_bundle_api.h:30-51):
 * the tensor list holds every operand, outputs included, in the positional order of the Python entry
 * point it replaces; the launch is asynchronous on the caller's HIP stream unless `sync` is non-zero, in which case
 * it returns after the stream has drained (pypto_bundle_api.h:41-44: "sync!=0 waits for completion"); 0 means success.
 * Besides the reference's (workspace, stream, sync) a launch takes `workspace_bytes`, so that a short workspace is
 * refused instead of overrun.
 *
 * Tensor descriptors use the reference's layout (pypto_bundle_api.h:30-35) and its DataType numbering
 * (framework/include/tilefwk/data_type.h:33-65).  All tensors are dense row-major device memory on the
 * current device.  With sync = 0 no entry point synchronises the stream (a launch can be captured into a HIP graph);
 * none allocates device memory: scratch comes
 * from the caller through `workspace` (reference: python/src/bindings/runtime.cpp:697-702, where the
 * workspace is a torch allocation made by the caller's side of the binding).
 */
#ifndef PYPTO_AMD_H
#define PYPTO_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* framework/include/tile_fwk_bundle/pypto_bundle_api.h:30-35 */
typedef struct {
    void* addr;       /* device address */
    int32_t dataType; /* PtoDataType */
    int32_t rank;
    int64_t shape[8];
} PtoTensorDesc;

/* framework/include/tilefwk/data_type.h:33-65 (positions in the DataType enum) */
enum PtoDataType { PTO_DT_INT8 = 1, PTO_DT_INT32 = 3, PTO_DT_INT64 = 4, PTO_DT_FP16 = 6, PTO_DT_FP32 = 7, PTO_DT_BF16 = 8 };

/* Error codes (negative).  pto_last_error() gives the message of the calling thread's last failure. */
enum PtoStatus {
    PTO_OK = 0,
    PTO_ERR_ARG_COUNT = -1, /* wrong number of tensors */
    PTO_ERR_DTYPE = -2,     /* a tensor has the wrong dtype */
    PTO_ERR_SHAPE = -3,     /* rank/shape mismatch between operands or with the parameters */
    PTO_ERR_PARAM = -4,     /* unsupported scalar parameter */
    PTO_ERR_WORKSPACE = -5, /* workspace missing or too small */
    PTO_ERR_NULL = -6,      /* null device address */
    PTO_ERR_HIP = -7,       /* the HIP runtime reported an error on launch */
    PTO_ERR_ALIGN = -8      /* a device address is not aligned as the operator needs (16 bytes; paged_gather and topk: one element) */
};

/* Scalar arguments of sparse_flash_attention_quant_* / sparse_attention_antiquant_*
 * (models/deepseek_v32_exp/sparse_flash_attention_quant_impl.py:655-674: nq, n_kv, softmax_scale, topk,
 * block_size, max_blocknum_perbatch; the trailing tile_config holds Ascend tiling knobs and has no
 * counterpart here). */
typedef struct {
    int32_t nq;
    int32_t n_kv;
    float softmax_scale;
    int32_t topk;
    int32_t block_size;
    int32_t max_blocknum_perbatch;
    int32_t kv_splits; /* 0 = choose from the problem size; >0 forces the number of KV splits per query token */
} PtoSfaParams;

/* Scalar arguments of lightning_indexer_decode
 * (models/deepseek_v32_exp/lightning_indexer_quant_impl.py:226-238: selected_count; unroll_list and
 * configs are Ascend tiling knobs - the only semantic field, extend_param scale = 1/2048 with ReLU,
 * models/deepseek_v32_exp/deepseekv32_lightning_indexer_quant.py:43, is fixed in the kernels). */
typedef struct {
    int32_t selected_count;
} PtoIndexerParams;

/*
 * sparse_flash_attention_quant_d / _p / _d_950
 * (models/deepseek_v32_exp/sparse_flash_attention_quant_impl.py:572-591,655-674,734-753).
 * tensors[9], in order:
 *   0 query_nope    [t*nq, 512]      BF16
 *   1 query_rope    [t*nq, 64]       BF16
 *   2 key_nope_2d   [N, 512]         INT8 (quantised cache) or BF16
 *   3 key_rope_2d   [N, 64]          BF16
 *   4 k_nope_scales [N, 4]           FP32 (one scale per 128 nope columns; ignored for a BF16 cache)
 *   5 topk_indices  [t, n_kv*topk]   INT32 (entries past a token's valid length are ignored)
 *   6 block_table   [b, max_blocknum_perbatch] INT32 (-1 = unused)
 *   7 kv_act_seqs   [b]              INT32
 *   8 attention_out [b, s1, nq, 512] BF16 (output)
 */
uint64_t pto_sfa_quant_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoSfaParams* params);
int pto_sfa_quant_launch(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoSfaParams* params,
                         void* workspace, uint64_t workspace_bytes, void* hip_stream, int sync);

/*
 * The allocation-free launch of sparse_flash_attention_quant: pto_sfa_quant_launch without the workspace arguments.
 * It has no counterpart in the reference.  It is for callers that cannot allocate device memory - code under HIP graph
 * capture, tight serving loops, harnesses that forbid it: the scratch the KV splits need (what
 * pto_sfa_quant_workspace reports) lives in an array inside the library, 40 MiB on every GPU the library runs on, held
 * until the process ends.  A problem that needs more is refused with PTO_ERR_WORKSPACE.  Every call on a GPU shares that
 * GPU's array: calls that overlap in time on one GPU (two streams, two threads) race; calls on one stream do not.
 * Tensors and parameters as for pto_sfa_quant_launch.
 */
int pto_sfa_quant_launch_noalloc(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoSfaParams* params,
                                 void* hip_stream, int sync);

/*
 * sparse_attention_antiquant_d / _p / _d_950
 * (models/deepseek_v32_exp/sparse_attention_antiquant_impl.py:287-302,358-373,739-749).
 * tensors[7], in order:
 *   0 query_nope    [t*nq, 512] BF16
 *   1 query_rope    [t*nq, 64]  BF16
 *   2 nope_cache    [N, 656]    INT8: bytes 0..511 int8 nope | 512..639 64 x bf16 rope | 640..655 4 x fp32 scales
 *   3 topk_indices  [t, n_kv*topk] INT32
 *   4 block_table   [b, max_blocknum_perbatch] INT32
 *   5 kv_act_seqs   [b] INT32
 *   6 attention_out [t*nq, 512] BF16 (output)
 */
uint64_t pto_sfa_antiquant_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoSfaParams* params);
int pto_sfa_antiquant_launch(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoSfaParams* params,
                             void* workspace, uint64_t workspace_bytes, void* hip_stream, int sync);

/*
 * lightning_indexer_decode (models/deepseek_v32_exp/lightning_indexer_quant_impl.py:226-238).
 * tensors[8], in order:
 *   0 idx_query       [t, 64, 128]            INT8
 *   1 idx_query_scale [t, 64]                 FP16 (FP32: see below)
 *   2 idx_key_cache   [blocks, block_size, 1, 128] INT8
 *   3 idx_key_scale   [blocks, block_size, 1] FP16 (FP32: see below)
 *   4 idx_weight      [t, 64]                 FP16
 *   5 act_seq_key     [b]                     INT32
 *   6 block_table     [b, max_blocks]         INT32
 *   7 topk_res        [t, 1, selected_count]  INT32 (output; -1 beyond a token's valid length)
 * The reference's operator takes fp16 scales.  Both scale tensors may instead be FP32 (per-token scales kept in fp32):
 * then the per-head factor is fp16(idx_query_scale * fp32(idx_weight)) - the golden's fp16 rounding point, taken from the
 * fp32 product - and idx_key_scale enters the final fp32 product unrounded; one FP16 and one FP32 scale tensor is an error.
 */
uint64_t pto_lightning_indexer_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors,
                                         const PtoIndexerParams* params);
int pto_lightning_indexer_launch(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoIndexerParams* params,
                                 void* workspace, uint64_t workspace_bytes, void* hip_stream, int sync);

/* Scalar arguments of topk (python/pypto/op/comparison.py:302-344: k, largest; dim is the last one - the Python mirror
 * moves any other dimension there). */
typedef struct {
    int32_t k;
    int32_t largest; /* non-zero: the k largest; zero: the k smallest */
} PtoTopkParams;

/*
 * topk (python/pypto/op/comparison.py:302-344; interpreter semantics
 * framework/src/interface/interpreter/calculator/calc_torch.cpp:2481-2494,2734-2749; golden torch.topk(sorted=True),
 * framework/tests/st/operation/python/vector_operator_golden.py:2247-2259): the k largest (smallest) elements of every
 * row, best first, equal values by ascending index (-0 and +0 are equal).
 * tensors[3], in order:
 *   0 input    [rows, n] FP32 (finite values)
 *   1 values   [rows, k] FP32  (output)
 *   2 indices  [rows, k] INT32 (output)
 * 1 <= k <= n; rows longer than 8192 elements need k <= 2048.  No workspace.
 */
uint64_t pto_topk_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoTopkParams* params);
int pto_topk_launch(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoTopkParams* params, void* workspace,
                    uint64_t workspace_bytes, void* hip_stream, int sync);

/* Scalar arguments of select_experts (models/glm_v4_5/glm_select_experts.py:317-330: top_k, renormalize, topk_group,
 * num_expert_group).  routed_scaling_factor and fill_neg_inf come from the reference's generalised gating golden
 * (python/tests/ut/interpreter/_ops/moe_gating_topk.py:272,285): the weights are multiplied by the factor, and the experts
 * of unselected groups are filled with -inf instead of the GLM kernel's 0.0 (glm_select_experts.py:169). */
typedef struct {
    int32_t top_k;
    int32_t renormalize;
    int32_t topk_group;
    int32_t num_expert_group;
    float routed_scaling_factor;
    int32_t fill_neg_inf;
} PtoSelectExpertsParams;

/*
 * select_experts (models/glm_v4_5/glm_select_experts.py:316-364; kernel :193-228).
 * tensors[4], in order:
 *   0 router_logits            [T, ne]    FP32 (the reference's dtype) or BF16; ne <= 256
 *   1 e_score_correction_bias  [ne]       BF16 (the reference's dtype) or FP32
 *   2 topk_weights             [T, top_k] FP32  (output)
 *   3 topk_ids                 [T, top_k] INT32 (output; descending biased score, equal scores by ascending id)
 * Inputs must be finite.  Needs no workspace (the query returns 0 for valid and for invalid arguments alike; use the
 * launch's status).
 */
uint64_t pto_select_experts_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors,
                                      const PtoSelectExpertsParams* params);
int pto_select_experts_launch(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoSelectExpertsParams* params,
                              void* workspace, uint64_t workspace_bytes, void* hip_stream, int sync);

/* Scalar arguments of the GLM-4.5 paged decode attention (models/glm_v4_5/glm_attention.py:1585-1594: softmax_scale; the
 * trailing tile_config holds Ascend tiling knobs and has no counterpart here). */
typedef struct {
    float softmax_scale;
    int32_t kv_chunk; /* 0 = choose; >0 forces the number of cached tokens one workgroup walks (rounded up to 128) */
} PtoGqaParams;

/*
 * attention / attention_for_950 / attention_for_950_high_through / attention_for_910_high_performance /
 * attention_for_910_s1_range_high_performance (models/glm_v4_5/glm_attention.py:1584-1700; kernel :427-568).
 * tensors[6], in order:
 *   0 query        [t, nq, 128]                    BF16 (t = b * s1; rotary embedding already applied)
 *   1 key_cache    [blocks, block_size, nkv, 128]  BF16 (block_size a multiple of 32; nq a multiple of nkv)
 *   2 value_cache  [blocks, block_size, nkv, 128]  BF16
 *   3 block_tables [b, max_blocks]                 INT32 (-1 = unused)
 *   4 actual_seqs  [b]                             INT32
 *   5 attn_res     [t, nq, 128]                    BF16 (output; query token j of a sequence attends to the first
 *                                                  actual_seq - (s1 - 1 - j) cached tokens, zeros if that is <= 0)
 */
uint64_t pto_gqa_decode_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoGqaParams* params);
int pto_gqa_decode_launch(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoGqaParams* params, void* workspace,
                          uint64_t workspace_bytes, void* hip_stream, int sync);

/* Scalar arguments of lightning_indexer_prolog_quant: attrs.eps of the LayerNorm
 * (models/deepseek_v32_exp/lightning_indexer_prolog_quant_impl.py:84-88; the layout strings are fixed "TND" / "PA_BSND",
 * the configs argument holds Ascend tiling knobs). */
typedef struct {
    float eps;
} PtoIndexerPrologParams;

/*
 * lightning_indexer_prolog_quant (models/deepseek_v32_exp/lightning_indexer_prolog_quant_impl.py:203-243; tensors in the
 * order of IndexerPrologQuantInput :63-80 followed by IndexerPrologQuantOutput :83-89).  tensors[21], in order:
 *    0 x              [t, h]                 BF16   (h a multiple of 256)
 *    1 q_norm         [t, r]                 INT8   (r a multiple of 128, at most 2048)
 *    2 q_norm_scale   [t, 1]                 FP32
 *    3 w_qb           [r, n*128]             INT8   (plain row-major; the reference's Ascend NZ tiling is a device format)
 *    4 w_qb_scale     [n*128, 1]             FP32
 *    5 wk             [h, 128]               BF16
 *    6 w_proj         [h, n]                 BF16   (n a multiple of 32, at most 128)
 *    7 ln_gamma_k     [128]                  BF16
 *    8 ln_beta_k      [128]                  BF16
 *    9 cos_idx_rope   [t, 64]                BF16
 *   10 sin_idx_rope   [t, 64]                BF16
 *   11 hadamard_q     [128, 128]             BF16
 *   12 hadamard_k     [128, 128]             BF16
 *   13 k_cache        [blocks, bs, 1, 128]   INT8   (updated in place at the rows k_cache_index names)
 *   14 k_cache_scale  [blocks, bs, 1, 1]     FP16   (updated in place)
 *   15 k_cache_index  [t]                    INT64  (cache row of each token; rows outside the cache are skipped)
 *   16 q_int8         [t, n, 128]            INT8   (output)
 *   17 q_scale        [t, n, 1]              FP16   (output)
 *   18 k_int8         = tensor 13 (the reference passes the cache again as the output; it must be the same buffer)
 *   19 k_scale        = tensor 14
 *   20 weights        [t, n]                 FP16   (output)
 */
uint64_t pto_indexer_prolog_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors,
                                      const PtoIndexerPrologParams* params);
int pto_indexer_prolog_launch(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoIndexerPrologParams* params,
                              void* workspace, uint64_t workspace_bytes, void* hip_stream, int sync);

/* Scalar argument of attention_pre_quant: the epsilon of its three RmsNorms, a constant 1e-5 inside the reference kernel
 * (models/glm_v4_5/glm_attention_pre_quant.py:301). */
typedef struct {
    float eps;
} PtoAttentionPreQuantParams;

/*
 * attention_pre_quant (models/glm_v4_5/glm_attention_pre_quant.py:633-747; kernel :235-505, argument checks :50-129):
 * residual add + RmsNorm with bias, per-channel int8 quantisation, int8 QKV projection with int32 bias and per-output
 * dequantisation, per-head RmsNorm with bias on the query and key heads, rotary embedding on each head's first
 * 2 * half_rotary_dim dims.  tensors[19], in the order of the reference signature:
 *    0 hidden_states                     [t, h]        BF16   (h a multiple of 256, at most 16384)
 *    1 residual                          [t, h]        BF16
 *    2 input_layernorm_weight            [h]           BF16
 *    3 input_layernorm_bias              [h]           BF16
 *    4 atten_qkv_input_scale_reciprocal  [h]           BF16   (multiplied onto the normalised row)
 *    5 atten_qkv_input_offset            [h]           BF16   (added after the scale)
 *    6 atten_qkv_weight                  [h, n_out]    INT8   (plain row-major; the reference's Ascend NZ tiling is a
 *                                                              device format; n_out = q_size + 2 kv_size)
 *    7 atten_qkv_quant_bias              [n_out]       INT32
 *    8 atten_qkv_deq_scale               [n_out]       FP32
 *    9 atten_q_norm_weight               [128]         BF16
 *   10 atten_q_norm_bias                 [128]         BF16
 *   11 atten_k_norm_weight               [128]         BF16
 *   12 atten_k_norm_bias                 [128]         BF16
 *   13 cos                               [t, 1, half]  BF16   (1 <= half <= 64)
 *   14 sin                               [t, 1, half]  BF16
 *   15 query                             [t, q_size]   BF16   (output; q_size a multiple of 128)
 *   16 key                               [t, kv_size]  BF16   (output; kv_size a multiple of 128)
 *   17 value                             [t, kv_size]  BF16   (output)
 *   18 residual_res                      [t, h]        BF16   (output: hidden_states + residual)
 */
uint64_t pto_attention_pre_quant_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors,
                                           const PtoAttentionPreQuantParams* params);
int pto_attention_pre_quant_launch(const PtoTensorDesc* tensors, uint32_t n_tensors,
                                   const PtoAttentionPreQuantParams* params, void* workspace, uint64_t workspace_bytes,
                                   void* hip_stream, int sync);

/* Scalar arguments of mla_prolog_quant_d / mla_prolog_quant_p: the two RmsNorm epsilons and the cache mode
 * (models/deepseek_v32_exp/mla_prolog_quant_impl.py:866-871; tile_config and rope_cfg hold Ascend tiling knobs). */
#define PTO_CACHE_PA_BSND 0 /* "PA_BSND": paged caches [block_num, block_size, 1, dim] */
typedef struct {
    float epsilon_cq;
    float epsilon_ckv;
    int32_t cache_mode;
} PtoMlaPrologParams;

/*
 * mla_prolog_quant_d and mla_prolog_quant_p (models/deepseek_v32_exp/mla_prolog_quant_impl.py:745-951, compute :520-727;
 * the decode and the prefill entry of the reference differ in Ascend pass options only).  tensors[21] in the reference's
 * argument order, int8 form:
 *    0 token_x           [t, h]                  BF16   (h a multiple of 256)
 *    1 w_dq              [h, r]                  BF16   (r a multiple of 128, at most 2048; plain row-major - the
 *                                                        reference's Ascend NZ tiling is a device format)
 *    2 w_uq_qr           [r, n*192]              INT8   (n even)
 *    3 dequant_scale     [n*192, 1]              FP32
 *    4 w_uk              [n, 128, 512]           BF16
 *    5 w_dkv_kr          [h, 576]                BF16
 *    6 gamma_cq          [r]                     BF16
 *    7 gamma_ckv         [512]                   BF16
 *    8 cos               [t, 64]                 BF16
 *    9 sin               [t, 64]                 BF16
 *   10 cache_index       [t]                     INT64  (flat cache row of each token; rows outside the cache are skipped)
 *   11 kv_cache          [blocks, bs, 1, 512]    INT8   (updated in place)
 *   12 kr_cache          [blocks, bs, 1, 64]     BF16   (updated in place)
 *   13 k_scale_cache     [blocks, bs, 1, 4]      FP32   (updated in place)
 *   14 q_norm_out        [t, r]                  INT8   (output)
 *   15 q_norm_scale_out  [t, 1]                  FP32   (output)
 *   16 query_nope_out    [t, n, 512]             BF16   (output)
 *   17 query_rope_out    [t, n, 64]              BF16   (output)
 *   18-20 kv_cache_out, kr_cache_out, k_scale_cache_out: the buffers of 11-13 again
 * bf16 form (the reference's "is_quant" False, :578-581): dequant_scale with no elements (rank 1 or 2), and w_uq_qr,
 * kv_cache, q_norm_out, kv_cache_out all BF16 - no quantisation anywhere: q_norm_out is the RmsNorm output, the kv cache row
 * the normalised key; k_scale_cache and q_norm_scale_out are not touched; q_lora_rank must then be a multiple of 256.
 */
uint64_t pto_mla_prolog_quant_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors,
                                        const PtoMlaPrologParams* params);
int pto_mla_prolog_quant_launch(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoMlaPrologParams* params,
                                void* workspace, uint64_t workspace_bytes, void* hip_stream, int sync);

/* Scalar arguments of mla_indexer_prolog_quant_d / _p: the MLA prolog's two epsilons and cache mode, and ip_attrs.eps of
 * the indexer's LayerNorm (models/deepseek_v32_exp/mla_indexer_prolog_quant_impl.py:521-527). */
typedef struct {
    float epsilon_cq;
    float epsilon_ckv;
    int32_t cache_mode;
    float indexer_eps;
} PtoMlaIndexerPrologParams;

/*
 * mla_indexer_prolog_quant_d and mla_indexer_prolog_quant_p
 * (models/deepseek_v32_exp/mla_indexer_prolog_quant_impl.py:320-477 and :479-634, compute :45-318): the MLA prolog
 * followed by the lightning-indexer prolog on the MLA prolog's q_norm / q_norm_scale, which stay internal (workspace), with
 * token_x, cos, sin and cache_index shared by both.  tensors[34] in the reference's argument order:
 *    0-13  token_x, mla_w_dq, mla_w_uq_qr, mla_dequant_scale, mla_w_uk, mla_w_dkv_kr, mla_gamma_cq, mla_gamma_ckv, cos, sin,
 *          cache_index, mla_kv_cache, mla_kr_cache, mla_k_scale_cache             (as tensors 0-13 of pto_mla_prolog_quant_*)
 *    14-23 ip_w_qb_in, ip_w_qb_scale_in, ip_wk_in, ip_w_proj_in, ip_ln_gamma_k_in, ip_ln_beta_k_in, ip_hadamard_q_in,
 *          ip_hadamard_k_in, ip_k_cache, ip_k_cache_scale                         (as tensors 3-8, 11-14 of pto_indexer_prolog_*)
 *    24-28 mla_query_nope_out, mla_query_rope_out, mla_kv_cache_out, mla_kr_cache_out, mla_k_scale_cache_out
 *    29-33 ip_q_int8_out, ip_q_scale_out, ip_k_int8_out, ip_k_scale_out, ip_weights_out
 * The cache outputs are the cache inputs themselves (updated in place).  Shape limits are those of the two operators.
 */
uint64_t pto_mla_indexer_prolog_quant_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors,
                                                const PtoMlaIndexerPrologParams* params);
int pto_mla_indexer_prolog_quant_launch(const PtoTensorDesc* tensors, uint32_t n_tensors,
                                        const PtoMlaIndexerPrologParams* params, void* workspace,
                                        uint64_t workspace_bytes, void* hip_stream, int sync);

/*
 * gather_in_ub(param, indices, block_table, block_size, axis=-2) and
 * gather_in_l1(src, indices, block_table, block_size, size, is_b_matrix, is_trans)
 * (python/pypto/experimental/gather.py:18-84; semantics
 * framework/src/interface/interpreter/calculator/calc_torch.cpp:1870-1981):
 *   out[j, :size] = src[ block_table[idx[j] / block_size] * block_size + idx[j] % block_size , :size ].
 * The reference operators take one index row and one page-table row ([1, k], [1, nblk]); here b such pairs are
 * gathered in one launch, row i of indices through row i of block_table, output rows in index order.
 * tensors[4] or tensors[5], in order:
 *   0 src         [N, hidden]   INT8 | INT32 | INT64 | FP16 | FP32 | BF16
 *   1 indices     [b, k]        INT32 | INT64
 *   2 block_table [b, nblk]     INT32 | INT64
 *   3 out         [b*k, size]   dtype of src (output)
 *   4 status      [1]           INT32 (optional, in/out): incremented once per entry the reference's interpreter would
 *                               reject (index outside [0, nblk*block_size), negative page, row outside src;
 *                               calc_torch.cpp:1916-1950).  Such an entry's output row is written as zeros.
 * `size` (gather_in_l1's column count; operation_impl.cpp:1705-1712) must be <= hidden; 0 means all columns.
 * The layout hints is_b_matrix / is_trans and `axis` describe Ascend buffers and have no counterpart.  No workspace.
 */
typedef struct {
    int32_t block_size;
    int32_t size;
} PtoPagedGatherParams;
uint64_t pto_paged_gather_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoPagedGatherParams* params);
int pto_paged_gather_launch(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoPagedGatherParams* params,
                            void* workspace, uint64_t workspace_bytes, void* hip_stream, int sync);

/* Message of the calling thread's most recent failed call ("" if none).  Replaces the message strings
 * the reference's binding layer returns (python/src/bindings/runtime.cpp:270-335). */
const char* pto_last_error(void);

/*
 * Measurement hooks (no counterpart in the reference, whose profiling is Ascend-specific:
 * framework/src/machine/device/dynamic/aicore_prof.cpp).  While enabled, every kernel launch of the library
 * is bracketed by a HIP event pair recorded on the launch stream; pto_kernel_timing_read waits for the
 * events recorded so far for one kernel, returns their summed duration and count, and forgets them.
 * Kernel ids: 0 indexer_score_kernel, 1 indexer_topk_kernel, 2 sfa_decode_kernel, 3 sfa_combine_kernel,
 * 4 indexer_select_kernel, 5 select_experts_kernel, 6 gqa_decode_kernel, 7 gqa_combine_kernel, 8 apq_norm_kernel,
 * 9 prolog_qx_kernel, 10 apq_gemm_kernel, 11 prolog_k_kernel, 12 mla_xa_kernel, 13 mla_norm_kernel (fused_norm_kernel in the fused
 * prolog), 14 mla_qb_kernel (fused_qb_kernel in the fused prolog), 15 mla_wuk_kernel, 16 apq_head_kernel,
 * 17 paged_gather_kernel
 * (pto_kernel_name returns "" past the last id).
 * Off by default; not for use under graph capture.
 */
int pto_kernel_timing_enable(int on);
int pto_kernel_timing_read(int kernel_id, double* total_ms, uint64_t* launches);
/* The offset of the instrument: what an event pair around an empty kernel reads on `hip_stream`, less that kernel's own
 * duration (averaged over a few pairs; synchronises the stream).  Take it off every per-launch figure of
 * pto_kernel_timing_read to get dispatch begin-to-end durations. */
int pto_kernel_timing_overhead(void* hip_stream, double* ms);
const char* pto_kernel_name(int kernel_id);

/* ABI version of this header. */
int pto_abi_version(void);

#ifdef __cplusplus
}
#endif

#endif /* PYPTO_AMD_H */
