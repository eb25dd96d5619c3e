// C ABI of libpypto_amd (declared in include/pypto_amd.h): operand validation and kernel dispatch.
//
// Validation mirrors what the reference's binding layer checks before a launch
// (python/pypto/frontend/parser/entry.py:351-365,664-747 and
//  python/src/bindings/torch_tensor_converter.cpp:157-214): tensor count, dtypes, ranks, static dims.
#include "pypto_amd.h"

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "kernels.h"
#include "timing.h"

namespace {

thread_local std::string g_last_error;

int fail(int code, const char* fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

const char* dtype_name(int dt)
{
    switch (dt) {
        case PTO_DT_INT8: return "int8";
        case PTO_DT_INT32: return "int32";
        case PTO_DT_INT64: return "int64";
        case PTO_DT_FP16: return "fp16";
        case PTO_DT_FP32: return "fp32";
        case PTO_DT_BF16: return "bf16";
        default: return "unsupported";
    }
}

// `align`: the alignment the kernels' vector accesses assume of the tensor's address (16 bytes: what any torch allocation
// and any view of whole rows has).  A misaligned address is refused here rather than left to the memory system.
int check_tensor(const char* op, const PtoTensorDesc& t, const char* name, int dtype, int rank, int align = 16)
{
    if (t.dataType != dtype)
        return fail(PTO_ERR_DTYPE, "%s: %s must be %s, got %s", op, name, dtype_name(dtype), dtype_name(t.dataType));
    if (t.rank != rank) return fail(PTO_ERR_SHAPE, "%s: %s must have rank %d, got %d", op, name, rank, t.rank);
    int64_t numel = 1;
    for (int i = 0; i < rank; ++i) {
        if (t.shape[i] < 0) return fail(PTO_ERR_SHAPE, "%s: %s has a negative dimension", op, name);
        numel *= t.shape[i];
    }
    if (numel > 0 && t.addr == nullptr) return fail(PTO_ERR_NULL, "%s: %s has a null address", op, name);
    if (numel > 0 && reinterpret_cast<uintptr_t>(t.addr) % (uintptr_t)align != 0)
        return fail(PTO_ERR_ALIGN, "%s: the address of %s must be a multiple of %d bytes", op, name, align);
    return PTO_OK;
}

struct SfaPlan {
    pto::SfaArgs args;
    uint64_t ws_bytes;
};

// Common checks of both attention entry points once the cache streams are resolved.
int plan_sfa(const char* op, const PtoTensorDesc& qn, const PtoTensorDesc& qr, const PtoTensorDesc& tk,
             const PtoTensorDesc& bt, const PtoTensorDesc& act, const PtoTensorDesc& out, int64_t out_rows,
             const PtoSfaParams* p, SfaPlan* plan)
{
    if (p == nullptr) return fail(PTO_ERR_PARAM, "%s: params is null", op);
    if (p->nq <= 0) return fail(PTO_ERR_PARAM, "%s: nq must be positive, got %d", op, p->nq);
    if (p->n_kv != 1) return fail(PTO_ERR_PARAM, "%s: n_kv must be 1 (MLA shares one compressed KV head), got %d", op, p->n_kv);
    if (p->topk <= 0 || p->topk > 2048) return fail(PTO_ERR_PARAM, "%s: topk must be in [1, 2048], got %d", op, p->topk);
    if (p->block_size <= 0) return fail(PTO_ERR_PARAM, "%s: block_size must be positive, got %d", op, p->block_size);
    if (p->kv_splits < 0 || p->kv_splits > 64) return fail(PTO_ERR_PARAM, "%s: kv_splits must be in [0, 64]", op);
    if (!(p->softmax_scale == p->softmax_scale)) return fail(PTO_ERR_PARAM, "%s: softmax_scale is NaN", op);
    if (qn.shape[1] != 512) return fail(PTO_ERR_SHAPE, "%s: query_nope last dim must be 512, got %lld", op, (long long)qn.shape[1]);
    if (qr.shape[1] != 64) return fail(PTO_ERR_SHAPE, "%s: query_rope last dim must be 64, got %lld", op, (long long)qr.shape[1]);
    if (qr.shape[0] != qn.shape[0]) return fail(PTO_ERR_SHAPE, "%s: query_nope and query_rope row counts differ", op);
    if (qn.shape[0] % p->nq != 0) return fail(PTO_ERR_SHAPE, "%s: query rows (%lld) not a multiple of nq (%d)", op, (long long)qn.shape[0], p->nq);
    const int64_t t = qn.shape[0] / p->nq;
    const int64_t b = act.shape[0];
    if (b == 0 ? t != 0 : t % b != 0)
        return fail(PTO_ERR_SHAPE, "%s: query tokens (%lld) not a multiple of the batch (%lld)", op, (long long)t, (long long)b);
    if (tk.shape[0] != t) return fail(PTO_ERR_SHAPE, "%s: topk_indices has %lld rows, expected %lld", op, (long long)tk.shape[0], (long long)t);
    if (tk.shape[1] < (int64_t)p->n_kv * p->topk)
        return fail(PTO_ERR_SHAPE, "%s: topk_indices has %lld columns, expected n_kv*topk = %d", op, (long long)tk.shape[1], p->n_kv * p->topk);
    if (bt.shape[0] != b) return fail(PTO_ERR_SHAPE, "%s: block_table has %lld rows, expected %lld", op, (long long)bt.shape[0], (long long)b);
    if (bt.shape[1] != p->max_blocknum_perbatch)
        return fail(PTO_ERR_SHAPE, "%s: block_table has %lld columns, max_blocknum_perbatch is %d", op, (long long)bt.shape[1], p->max_blocknum_perbatch);
    if (out_rows != qn.shape[0]) return fail(PTO_ERR_SHAPE, "%s: attention_out holds %lld head rows, expected %lld", op, (long long)out_rows, (long long)qn.shape[0]);
    if (t > 0x7fffffff / 2048 || qn.shape[0] > 0x7fffffff) return fail(PTO_ERR_SHAPE, "%s: too many query tokens", op);

    pto::SfaArgs& a = plan->args;
    a.q_nope = qn.addr;
    a.q_rope = qr.addr;
    a.topk_idx = static_cast<const int32_t*>(tk.addr);
    a.block_table = static_cast<const int32_t*>(bt.addr);
    a.act_seq = static_cast<const int32_t*>(act.addr);
    a.out = out.addr;
    a.b = (int32_t)b;
    a.s1 = b ? (int32_t)(t / b) : 0;
    a.nq = p->nq;
    a.topk = p->topk;
    a.topk_stride = (int32_t)tk.shape[1];
    a.block_size = p->block_size;
    a.bt_stride = (int32_t)bt.shape[1];
    a.softmax_scale = p->softmax_scale;
    a.nsplit = p->kv_splits > 0 ? p->kv_splits : pto::sfa_pick_splits((int)t, p->nq, p->topk);
    a.part_o = nullptr;
    a.part_ml = nullptr;
    plan->ws_bytes = pto::sfa_workspace_bytes((int)t, p->nq, a.nsplit);
    return PTO_OK;
}

int bind_workspace(const char* op, SfaPlan* plan, void* ws, uint64_t ws_bytes)
{
    if (plan->ws_bytes == 0) return PTO_OK;
    if (ws == nullptr || ws_bytes < plan->ws_bytes)
        return fail(PTO_ERR_WORKSPACE, "%s: workspace of %llu bytes required, got %llu", op,
                    (unsigned long long)plan->ws_bytes, (unsigned long long)(ws ? ws_bytes : 0));
    pto::SfaArgs& a = plan->args;
    a.part_o = static_cast<_Float16*>(ws);
    a.part_ml = reinterpret_cast<float*>(static_cast<char*>(ws) + pto::sfa_partials_bytes(a.b * a.s1, a.nq, a.nsplit));
    return PTO_OK;
}

int plan_sfa_quant(const PtoTensorDesc* ts, uint32_t n, const PtoSfaParams* p, SfaPlan* plan)
{
    const char* op = "sparse_flash_attention_quant";
    if (ts == nullptr || n != 9) return fail(PTO_ERR_ARG_COUNT, "%s: expected 9 tensors, got %u", op, n);
    int rc;
    if ((rc = check_tensor(op, ts[0], "query_nope", PTO_DT_BF16, 2))) return rc;
    if ((rc = check_tensor(op, ts[1], "query_rope", PTO_DT_BF16, 2))) return rc;
    const bool quant = ts[2].dataType == PTO_DT_INT8;
    if (!quant && ts[2].dataType != PTO_DT_BF16)
        return fail(PTO_ERR_DTYPE, "%s: key_nope_2d must be int8 or bf16, got %s", op, dtype_name(ts[2].dataType));
    if ((rc = check_tensor(op, ts[2], "key_nope_2d", ts[2].dataType, 2))) return rc;
    if ((rc = check_tensor(op, ts[3], "key_rope_2d", PTO_DT_BF16, 2))) return rc;
    if ((rc = check_tensor(op, ts[4], "k_nope_scales", PTO_DT_FP32, 2))) return rc;
    if ((rc = check_tensor(op, ts[5], "topk_indices", PTO_DT_INT32, 2))) return rc;
    if ((rc = check_tensor(op, ts[6], "block_table", PTO_DT_INT32, 2))) return rc;
    if ((rc = check_tensor(op, ts[7], "kv_act_seqs", PTO_DT_INT32, 1))) return rc;
    if ((rc = check_tensor(op, ts[8], "attention_out", PTO_DT_BF16, 4))) return rc;
    const int64_t n_rows = ts[2].shape[0];
    if (ts[2].shape[1] != 512) return fail(PTO_ERR_SHAPE, "%s: key_nope_2d last dim must be 512", op);
    if (ts[3].shape[0] != n_rows || ts[3].shape[1] != 64) return fail(PTO_ERR_SHAPE, "%s: key_rope_2d must be [%lld, 64]", op, (long long)n_rows);
    if (quant && (ts[4].shape[0] != n_rows || ts[4].shape[1] != 4)) return fail(PTO_ERR_SHAPE, "%s: k_nope_scales must be [%lld, 4]", op, (long long)n_rows);
    if (ts[8].shape[3] != 512) return fail(PTO_ERR_SHAPE, "%s: attention_out last dim must be 512", op);
    if (n_rows > 0x7fffffff) return fail(PTO_ERR_SHAPE, "%s: cache has too many rows", op);
    if (p && ts[8].shape[2] != p->nq) return fail(PTO_ERR_SHAPE, "%s: attention_out dim 2 must equal nq", op);
    const int64_t out_rows = ts[8].shape[0] * ts[8].shape[1] * ts[8].shape[2];
    if ((rc = plan_sfa(op, ts[0], ts[1], ts[5], ts[6], ts[7], ts[8], out_rows, p, plan))) return rc;
    if (ts[8].shape[0] != plan->args.b) return fail(PTO_ERR_SHAPE, "%s: attention_out dim 0 must equal the batch", op);
    pto::SfaArgs& a = plan->args;
    a.quant = quant;
    a.kn = static_cast<const uint8_t*>(ts[2].addr);
    a.kr = static_cast<const uint8_t*>(ts[3].addr);
    a.ks = static_cast<const uint8_t*>(ts[4].addr);
    a.kn_stride = quant ? 512 : 1024;
    a.kr_stride = 128;
    a.ks_stride = 16;
    a.n_rows = n_rows;
    return PTO_OK;
}

int plan_sfa_antiquant(const PtoTensorDesc* ts, uint32_t n, const PtoSfaParams* p, SfaPlan* plan)
{
    const char* op = "sparse_attention_antiquant";
    if (ts == nullptr || n != 7) return fail(PTO_ERR_ARG_COUNT, "%s: expected 7 tensors, got %u", op, n);
    int rc;
    if ((rc = check_tensor(op, ts[0], "query_nope", PTO_DT_BF16, 2))) return rc;
    if ((rc = check_tensor(op, ts[1], "query_rope", PTO_DT_BF16, 2))) return rc;
    if ((rc = check_tensor(op, ts[2], "nope_cache", PTO_DT_INT8, 2))) return rc;
    if ((rc = check_tensor(op, ts[3], "topk_indices", PTO_DT_INT32, 2))) return rc;
    if ((rc = check_tensor(op, ts[4], "block_table", PTO_DT_INT32, 2))) return rc;
    if ((rc = check_tensor(op, ts[5], "kv_act_seqs", PTO_DT_INT32, 1))) return rc;
    if ((rc = check_tensor(op, ts[6], "attention_out", PTO_DT_BF16, 2))) return rc;
    if (ts[2].shape[1] != 656) return fail(PTO_ERR_SHAPE, "%s: nope_cache rows must be 656 bytes, got %lld", op, (long long)ts[2].shape[1]);
    if (ts[6].shape[1] != 512) return fail(PTO_ERR_SHAPE, "%s: attention_out last dim must be 512", op);
    if (ts[2].shape[0] > 0x7fffffff) return fail(PTO_ERR_SHAPE, "%s: cache has too many rows", op);
    if ((rc = plan_sfa(op, ts[0], ts[1], ts[3], ts[4], ts[5], ts[6], ts[6].shape[0], p, plan))) return rc;
    pto::SfaArgs& a = plan->args;
    a.quant = true;
    a.kn = static_cast<const uint8_t*>(ts[2].addr);
    a.kr = a.kn + 512;
    a.ks = a.kn + 640;
    a.kn_stride = a.kr_stride = a.ks_stride = 656;
    a.n_rows = ts[2].shape[0];
    return PTO_OK;
}

int launch_sfa(const char* op, SfaPlan* plan, void* ws, uint64_t ws_bytes, void* stream)
{
    int rc = bind_workspace(op, plan, ws, ws_bytes);
    if (rc) return rc;
    hipError_t e = pto::sfa_launch(plan->args, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(PTO_ERR_HIP, "%s: HIP launch failed: %s", op, hipGetErrorString(e));
    return PTO_OK;
}

struct IndexerPlan {
    pto::IndexerArgs args;
    uint64_t ws_bytes;
};

int plan_indexer(const PtoTensorDesc* ts, uint32_t n, const PtoIndexerParams* p, IndexerPlan* plan)
{
    const char* op = "lightning_indexer_decode";
    if (ts == nullptr || n != 8) return fail(PTO_ERR_ARG_COUNT, "%s: expected 8 tensors, got %u", op, n);
    if (p == nullptr) return fail(PTO_ERR_PARAM, "%s: params is null", op);
    int rc;
    if ((rc = check_tensor(op, ts[0], "idx_query", PTO_DT_INT8, 3))) return rc;
    // the scales are fp16 (the reference's signature) or both fp32 (per-token scales kept in fp32)
    const bool scales_f32 = ts[1].dataType == PTO_DT_FP32;
    const int scale_dt = scales_f32 ? PTO_DT_FP32 : PTO_DT_FP16;
    if ((rc = check_tensor(op, ts[1], "idx_query_scale", scale_dt, 2))) return rc;
    if ((rc = check_tensor(op, ts[2], "idx_key_cache", PTO_DT_INT8, 4))) return rc;
    if ((rc = check_tensor(op, ts[3], "idx_key_scale", scale_dt, 3))) return rc;
    if ((rc = check_tensor(op, ts[4], "idx_weight", PTO_DT_FP16, 2))) return rc;
    if ((rc = check_tensor(op, ts[5], "act_seq_key", PTO_DT_INT32, 1))) return rc;
    if ((rc = check_tensor(op, ts[6], "block_table", PTO_DT_INT32, 2))) return rc;
    if ((rc = check_tensor(op, ts[7], "topk_res", PTO_DT_INT32, 3))) return rc;
    if (p->selected_count <= 0 || p->selected_count > 2048)
        return fail(PTO_ERR_PARAM, "%s: selected_count must be in [1, 2048], got %d", op, p->selected_count);
    const int64_t t = ts[0].shape[0], nh = ts[0].shape[1], d = ts[0].shape[2];
    const int64_t blocks = ts[2].shape[0], bs = ts[2].shape[1];
    const int64_t b = ts[5].shape[0];
    if (nh != 64 || d != 128) return fail(PTO_ERR_SHAPE, "%s: idx_query must be [t, 64, 128], got [%lld, %lld, %lld]", op, (long long)t, (long long)nh, (long long)d);
    if (ts[2].shape[2] != 1 || ts[2].shape[3] != d) return fail(PTO_ERR_SHAPE, "%s: idx_key_cache must be [blocks, block_size, 1, 128]", op);
    if (bs <= 0) return fail(PTO_ERR_SHAPE, "%s: block_size must be positive", op);
    if (ts[3].shape[0] != blocks || ts[3].shape[1] != bs || ts[3].shape[2] != 1) return fail(PTO_ERR_SHAPE, "%s: idx_key_scale must be [blocks, block_size, 1]", op);
    if (ts[1].shape[0] != t || ts[1].shape[1] != nh) return fail(PTO_ERR_SHAPE, "%s: idx_query_scale must be [t, 64]", op);
    if (ts[4].shape[0] != t || ts[4].shape[1] != nh) return fail(PTO_ERR_SHAPE, "%s: idx_weight must be [t, 64]", op);
    if (b == 0 ? t != 0 : t % b != 0) return fail(PTO_ERR_SHAPE, "%s: query tokens (%lld) not a multiple of the batch (%lld)", op, (long long)t, (long long)b);
    if (b && t / b > 4) return fail(PTO_ERR_SHAPE, "%s: at most 4 query tokens per sequence, got %lld", op, (long long)(t / b));
    if (ts[6].shape[0] != b) return fail(PTO_ERR_SHAPE, "%s: block_table has %lld rows, expected %lld", op, (long long)ts[6].shape[0], (long long)b);
    if (ts[7].shape[0] != t || ts[7].shape[1] != 1 || ts[7].shape[2] != p->selected_count)
        return fail(PTO_ERR_SHAPE, "%s: topk_res must be [t, 1, selected_count]", op);
    const int64_t max_ctx = ts[6].shape[1] * bs;
    if (max_ctx > (1 << 20) || blocks * bs > 0x7fffffff || t > 65535) return fail(PTO_ERR_SHAPE, "%s: problem too large", op);
    pto::IndexerArgs& a = plan->args;
    a.q = static_cast<const int8_t*>(ts[0].addr);
    a.q_scale = ts[1].addr;
    a.scales_f32 = scales_f32;
    a.k_cache = static_cast<const int8_t*>(ts[2].addr);
    a.k_scale = ts[3].addr;
    a.weights = static_cast<const uint16_t*>(ts[4].addr);
    a.act_seq = static_cast<const int32_t*>(ts[5].addr);
    a.block_table = static_cast<const int32_t*>(ts[6].addr);
    a.topk_res = static_cast<int32_t*>(ts[7].addr);
    a.scores = nullptr;
    a.n_blocks = blocks;
    a.b = (int32_t)b;
    a.s1 = b ? (int32_t)(t / b) : 0;
    a.nh = (int32_t)nh;
    a.block_size = (int32_t)bs;
    a.bt_stride = (int32_t)ts[6].shape[1];
    a.k = p->selected_count;
    a.score_stride = (int32_t)((max_ctx + 4095) & ~(int64_t)4095); // whole workgroup spans of the score kernel
    plan->ws_bytes = pto::indexer_workspace_bytes((int)t, a.score_stride);
    return PTO_OK;
}

struct AttnPrePlan {
    pto::AttnPreArgs args;
    uint64_t ws_bytes;
};

int plan_attention_pre(const PtoTensorDesc* ts, uint32_t n, const PtoAttentionPreQuantParams* p, AttnPrePlan* plan)
{
    const char* op = "attention_pre_quant";
    if (ts == nullptr || n != 19) return fail(PTO_ERR_ARG_COUNT, "%s: expected 19 tensors, got %u", op, n);
    if (p == nullptr) return fail(PTO_ERR_PARAM, "%s: params is null", op);
    if (!(p->eps >= 0.f)) return fail(PTO_ERR_PARAM, "%s: eps must be a non-negative number", op);
    static const struct { const char* name; int dtype, rank; } spec[19] = {
        {"hidden_states", PTO_DT_BF16, 2}, {"residual", PTO_DT_BF16, 2}, {"input_layernorm_weight", PTO_DT_BF16, 1},
        {"input_layernorm_bias", PTO_DT_BF16, 1}, {"atten_qkv_input_scale_reciprocal", PTO_DT_BF16, 1},
        {"atten_qkv_input_offset", PTO_DT_BF16, 1}, {"atten_qkv_weight", PTO_DT_INT8, 2},
        {"atten_qkv_quant_bias", PTO_DT_INT32, 1}, {"atten_qkv_deq_scale", PTO_DT_FP32, 1},
        {"atten_q_norm_weight", PTO_DT_BF16, 1}, {"atten_q_norm_bias", PTO_DT_BF16, 1},
        {"atten_k_norm_weight", PTO_DT_BF16, 1}, {"atten_k_norm_bias", PTO_DT_BF16, 1}, {"cos", PTO_DT_BF16, 3},
        {"sin", PTO_DT_BF16, 3}, {"query", PTO_DT_BF16, 2}, {"key", PTO_DT_BF16, 2}, {"value", PTO_DT_BF16, 2},
        {"residual_res", PTO_DT_BF16, 2}};
    int rc;
    for (int i = 0; i < 19; ++i)
        if ((rc = check_tensor(op, ts[i], spec[i].name, spec[i].dtype, spec[i].rank))) return rc;
    const int64_t t = ts[0].shape[0], h = ts[0].shape[1], n_out = ts[6].shape[1], d = ts[9].shape[0];
    const int64_t half = ts[13].shape[2], q_size = ts[15].shape[1], kv_size = ts[16].shape[1];
    if (ts[1].shape[0] != t || ts[1].shape[1] != h || ts[18].shape[0] != t || ts[18].shape[1] != h)
        return fail(PTO_ERR_SHAPE, "%s: residual and residual_res must be [%lld, %lld] like hidden_states", op, (long long)t, (long long)h);
    for (int i = 2; i <= 5; ++i)
        if (ts[i].shape[0] != h) return fail(PTO_ERR_SHAPE, "%s: %s must have %lld entries, got %lld", op, spec[i].name, (long long)h, (long long)ts[i].shape[0]);
    if (ts[6].shape[0] != h) return fail(PTO_ERR_SHAPE, "%s: atten_qkv_weight must be [%lld, total_head_size], got %lld rows", op, (long long)h, (long long)ts[6].shape[0]);
    if (ts[7].shape[0] != n_out || ts[8].shape[0] != n_out)
        return fail(PTO_ERR_SHAPE, "%s: atten_qkv_quant_bias and atten_qkv_deq_scale must have %lld entries", op, (long long)n_out);
    for (int i = 10; i <= 12; ++i)
        if (ts[i].shape[0] != d) return fail(PTO_ERR_SHAPE, "%s: %s must have %lld entries like atten_q_norm_weight", op, spec[i].name, (long long)d);
    if (!pto::attention_pre_supported(h, d, half))
        return fail(PTO_ERR_SHAPE, "%s: need head size 128, hidden size a multiple of 256 up to 16384 and 1 <= half_rotary_dim <= 64; got head size %lld, hidden size %lld, half_rotary_dim %lld",
                    op, (long long)d, (long long)h, (long long)half);
    for (int i = 13; i <= 14; ++i)
        if (ts[i].shape[0] != t || ts[i].shape[1] != 1 || ts[i].shape[2] != half)
            return fail(PTO_ERR_SHAPE, "%s: %s must be [%lld, 1, %lld]", op, spec[i].name, (long long)t, (long long)half);
    if (ts[15].shape[0] != t || ts[16].shape[0] != t || ts[17].shape[0] != t || ts[17].shape[1] != kv_size)
        return fail(PTO_ERR_SHAPE, "%s: query, key and value must have %lld rows, key and value the same width", op, (long long)t);
    if (q_size <= 0 || kv_size <= 0 || q_size % d != 0 || kv_size % d != 0 || q_size + 2 * kv_size != n_out)
        return fail(PTO_ERR_SHAPE, "%s: query width %lld and key / value width %lld must be multiples of the head size adding up to total_head_size %lld",
                    op, (long long)q_size, (long long)kv_size, (long long)n_out);
    if (t > 65535 || n_out > (1 << 20)) return fail(PTO_ERR_SHAPE, "%s: problem too large", op);
    pto::AttnPreArgs& a = plan->args;
    a.x = static_cast<const uint16_t*>(ts[0].addr);
    a.residual = static_cast<const uint16_t*>(ts[1].addr);
    a.gamma = static_cast<const uint16_t*>(ts[2].addr);
    a.bias = static_cast<const uint16_t*>(ts[3].addr);
    a.in_scale = static_cast<const uint16_t*>(ts[4].addr);
    a.in_offset = static_cast<const uint16_t*>(ts[5].addr);
    a.w = static_cast<const int8_t*>(ts[6].addr);
    a.qbias = static_cast<const int32_t*>(ts[7].addr);
    a.deq = static_cast<const float*>(ts[8].addr);
    a.q_gamma = static_cast<const uint16_t*>(ts[9].addr);
    a.q_bias = static_cast<const uint16_t*>(ts[10].addr);
    a.k_gamma = static_cast<const uint16_t*>(ts[11].addr);
    a.k_bias = static_cast<const uint16_t*>(ts[12].addr);
    a.cos = static_cast<const uint16_t*>(ts[13].addr);
    a.sin = static_cast<const uint16_t*>(ts[14].addr);
    a.q = static_cast<uint16_t*>(ts[15].addr);
    a.k = static_cast<uint16_t*>(ts[16].addr);
    a.v = static_cast<uint16_t*>(ts[17].addr);
    a.residual_out = static_cast<uint16_t*>(ts[18].addr);
    a.x_q = nullptr;
    a.part = nullptr;
    a.t = (int32_t)t;
    a.h = (int32_t)h;
    a.n_out = (int32_t)n_out;
    a.q_heads = (int32_t)(q_size / d);
    a.kv_heads = (int32_t)(kv_size / d);
    a.half = (int32_t)half;
    a.ksplits = pto::attention_pre_ksplits(t, h, n_out);
    a.eps = p->eps;
    a.mean_coff = (float)(1.0 / (double)h);
    plan->ws_bytes = pto::attention_pre_workspace_bytes(t, h, n_out);
    return PTO_OK;
}

int plan_paged_gather(const PtoTensorDesc* ts, uint32_t n, const PtoPagedGatherParams* p, pto::GatherArgs* a)
{
    const char* op = "paged_gather";
    if (ts == nullptr || (n != 4 && n != 5)) return fail(PTO_ERR_ARG_COUNT, "%s: expected 4 or 5 tensors, got %u", op, n);
    if (p == nullptr) return fail(PTO_ERR_PARAM, "%s: params is null", op);
    if (p->block_size <= 0) return fail(PTO_ERR_PARAM, "%s: block_size must be positive, got %d", op, p->block_size);
    if (p->size < 0) return fail(PTO_ERR_PARAM, "%s: size must not be negative, got %d", op, p->size);
    int64_t esize;
    switch (ts[0].dataType) {
        case PTO_DT_INT8: esize = 1; break;
        case PTO_DT_FP16: case PTO_DT_BF16: esize = 2; break;
        case PTO_DT_INT32: case PTO_DT_FP32: esize = 4; break;
        case PTO_DT_INT64: esize = 8; break;
        default: return fail(PTO_ERR_DTYPE, "%s: src has an unsupported dtype (%d)", op, ts[0].dataType);
    }
    for (int i = 1; i <= 2; ++i)
        if (ts[i].dataType != PTO_DT_INT32 && ts[i].dataType != PTO_DT_INT64)
            return fail(PTO_ERR_DTYPE, "%s: %s must be int32 or int64, got %s", op, i == 1 ? "indices" : "block_table",
                        dtype_name(ts[i].dataType));
    int rc;
    // (this operator moves rows in pieces as wide as the addresses allow: element alignment is all it asks for)
    if ((rc = check_tensor(op, ts[0], "src", ts[0].dataType, 2, (int)esize))) return rc;
    if ((rc = check_tensor(op, ts[1], "indices", ts[1].dataType, 2, ts[1].dataType == PTO_DT_INT64 ? 8 : 4))) return rc;
    if ((rc = check_tensor(op, ts[2], "block_table", ts[2].dataType, 2, ts[2].dataType == PTO_DT_INT64 ? 8 : 4))) return rc;
    if ((rc = check_tensor(op, ts[3], "out", ts[0].dataType, 2, (int)esize))) return rc; // out and src share a dtype
    if (n == 5) {
        if ((rc = check_tensor(op, ts[4], "status", PTO_DT_INT32, 1, 4))) return rc;
        if (ts[4].shape[0] != 1) return fail(PTO_ERR_SHAPE, "%s: status must hold one word", op);
    }
    const int64_t hidden = ts[0].shape[1], b = ts[1].shape[0], k = ts[1].shape[1];
    const int64_t size = p->size > 0 ? p->size : hidden;
    if (size > hidden) return fail(PTO_ERR_PARAM, "%s: size (%lld) exceeds the source row width (%lld)", op, (long long)size, (long long)hidden);
    if (ts[2].shape[0] != b) return fail(PTO_ERR_SHAPE, "%s: block_table has %lld rows, indices has %lld", op, (long long)ts[2].shape[0], (long long)b);
    if (k > 0 && b > 0x7fffffffffffLL / k) return fail(PTO_ERR_SHAPE, "%s: too many indices", op);
    if (ts[3].shape[0] != b * k || ts[3].shape[1] != size)
        return fail(PTO_ERR_SHAPE, "%s: out must be [%lld, %lld], got [%lld, %lld]", op, (long long)(b * k), (long long)size,
                    (long long)ts[3].shape[0], (long long)ts[3].shape[1]);
    a->src = ts[0].addr;
    a->indices = ts[1].addr;
    a->block_table = ts[2].addr;
    a->out = ts[3].addr;
    a->status = n == 5 ? static_cast<int32_t*>(ts[4].addr) : nullptr;
    a->rows = b * k;
    a->k = k > 0 ? k : 1;
    a->nblk = ts[2].shape[1];
    a->block_size = p->block_size;
    a->n_src = ts[0].shape[0];
    a->src_pitch = hidden * esize;
    a->row_bytes = size * esize;
    a->idx64 = ts[1].dataType == PTO_DT_INT64;
    a->bt64 = ts[2].dataType == PTO_DT_INT64;
    return PTO_OK;
}

int plan_select_experts(const PtoTensorDesc* ts, uint32_t n, const PtoSelectExpertsParams* p, pto::SelectExpertsArgs* a)
{
    const char* op = "select_experts";
    if (ts == nullptr || n != 4) return fail(PTO_ERR_ARG_COUNT, "%s: expected 4 tensors, got %u", op, n);
    if (p == nullptr) return fail(PTO_ERR_PARAM, "%s: params is null", op);
    if (ts[0].dataType != PTO_DT_FP32 && ts[0].dataType != PTO_DT_BF16)
        return fail(PTO_ERR_DTYPE, "%s: router_logits must be fp32 or bf16, got %s", op, dtype_name(ts[0].dataType));
    if (ts[1].dataType != PTO_DT_BF16 && ts[1].dataType != PTO_DT_FP32)
        return fail(PTO_ERR_DTYPE, "%s: e_score_correction_bias must be bf16 or fp32, got %s", op, dtype_name(ts[1].dataType));
    int rc;
    if ((rc = check_tensor(op, ts[0], "router_logits", ts[0].dataType, 2))) return rc;
    if ((rc = check_tensor(op, ts[1], "e_score_correction_bias", ts[1].dataType, 1))) return rc;
    if ((rc = check_tensor(op, ts[2], "topk_weights", PTO_DT_FP32, 2))) return rc;
    if ((rc = check_tensor(op, ts[3], "topk_ids", PTO_DT_INT32, 2))) return rc;
    const int64_t t = ts[0].shape[0], ne = ts[0].shape[1];
    if (ts[1].shape[0] != ne) return fail(PTO_ERR_SHAPE, "%s: bias has %lld entries, router_logits has %lld experts", op, (long long)ts[1].shape[0], (long long)ne);
    if (ts[2].shape[0] != t || ts[3].shape[0] != t || ts[2].shape[1] != p->top_k || ts[3].shape[1] != p->top_k)
        return fail(PTO_ERR_SHAPE, "%s: topk_weights and topk_ids must be [%lld, %d]", op, (long long)t, p->top_k);
    if (ne > 0x7fffffff || !pto::select_experts_supported((int)ne, p->num_expert_group, p->top_k))
        return fail(PTO_ERR_PARAM, "%s: need 1 <= experts <= 256, 1 <= groups <= 64 dividing the experts, 1 <= top_k <= min(32, experts); got experts %lld, groups %d, top_k %d",
                    op, (long long)ne, p->num_expert_group, p->top_k);
    if (p->topk_group < 1 || p->topk_group > p->num_expert_group)
        return fail(PTO_ERR_PARAM, "%s: topk_group must be in [1, num_expert_group], got %d", op, p->topk_group);
    if (!(p->routed_scaling_factor == p->routed_scaling_factor)) return fail(PTO_ERR_PARAM, "%s: routed_scaling_factor is NaN", op);
    a->logits = ts[0].addr;
    a->bias = ts[1].addr;
    a->topk_weights = static_cast<float*>(ts[2].addr);
    a->topk_ids = static_cast<int32_t*>(ts[3].addr);
    a->t = t;
    a->ne = (int32_t)ne;
    a->top_k = p->top_k;
    a->topk_group = p->topk_group;
    a->n_group = p->num_expert_group;
    a->routed_scaling_factor = p->routed_scaling_factor;
    a->renormalize = p->renormalize != 0;
    a->fill_neg_inf = p->fill_neg_inf != 0;
    a->logits_bf16 = ts[0].dataType == PTO_DT_BF16;
    a->bias_bf16 = ts[1].dataType == PTO_DT_BF16;
    return PTO_OK;
}

struct GqaPlan {
    pto::GqaArgs args;
    uint64_t ws_bytes;
};

int plan_gqa(const PtoTensorDesc* ts, uint32_t n, const PtoGqaParams* p, GqaPlan* plan)
{
    const char* op = "attention";
    if (ts == nullptr || n != 6) return fail(PTO_ERR_ARG_COUNT, "%s: expected 6 tensors, got %u", op, n);
    if (p == nullptr) return fail(PTO_ERR_PARAM, "%s: params is null", op);
    int rc;
    if ((rc = check_tensor(op, ts[0], "query", PTO_DT_BF16, 3))) return rc;
    if ((rc = check_tensor(op, ts[1], "key_cache", PTO_DT_BF16, 4))) return rc;
    if ((rc = check_tensor(op, ts[2], "value_cache", PTO_DT_BF16, 4))) return rc;
    if ((rc = check_tensor(op, ts[3], "block_tables", PTO_DT_INT32, 2))) return rc;
    if ((rc = check_tensor(op, ts[4], "actual_seqs", PTO_DT_INT32, 1))) return rc;
    if ((rc = check_tensor(op, ts[5], "attn_res", PTO_DT_BF16, 3))) return rc;
    if (!(p->softmax_scale == p->softmax_scale)) return fail(PTO_ERR_PARAM, "%s: softmax_scale is NaN", op);
    if (p->kv_chunk < 0 || p->kv_chunk > (1 << 20)) return fail(PTO_ERR_PARAM, "%s: kv_chunk must be in [0, 2^20]", op);
    const int64_t t = ts[0].shape[0], nq = ts[0].shape[1], d = ts[0].shape[2];
    const int64_t blocks = ts[1].shape[0], bs = ts[1].shape[1], nkv = ts[1].shape[2];
    const int64_t b = ts[4].shape[0];
    if (d != 128 || ts[1].shape[3] != 128) return fail(PTO_ERR_SHAPE, "%s: head dim must be 128", op);
    for (int i = 0; i < 4; ++i)
        if (ts[2].shape[i] != ts[1].shape[i]) return fail(PTO_ERR_SHAPE, "%s: key_cache and value_cache shapes differ", op);
    for (int i = 0; i < 3; ++i)
        if (ts[5].shape[i] != ts[0].shape[i]) return fail(PTO_ERR_SHAPE, "%s: attn_res and query shapes differ", op);
    if (bs <= 0 || bs % 32 != 0) return fail(PTO_ERR_SHAPE, "%s: block_size must be a positive multiple of 32, got %lld", op, (long long)bs);
    if (nkv <= 0 || nq <= 0 || nq % nkv != 0) return fail(PTO_ERR_SHAPE, "%s: nq (%lld) must be a positive multiple of nkv (%lld)", op, (long long)nq, (long long)nkv);
    if (b == 0 ? t != 0 : t % b != 0) return fail(PTO_ERR_SHAPE, "%s: query tokens (%lld) not a multiple of the batch (%lld)", op, (long long)t, (long long)b);
    if (ts[3].shape[0] != b) return fail(PTO_ERR_SHAPE, "%s: block_tables has %lld rows, expected %lld", op, (long long)ts[3].shape[0], (long long)b);
    const int64_t max_ctx = ts[3].shape[1] * bs;
    const int64_t hsub = (nq / nkv + 15) / 16;
    if (max_ctx > 0x3fffffff || t > 65535 || nkv * hsub > 65535 || nq > 0x7fff || blocks > 0x7fffffff)
        return fail(PTO_ERR_SHAPE, "%s: problem too large", op);
    pto::GqaArgs& a = plan->args;
    a.q = ts[0].addr;
    a.k = ts[1].addr;
    a.v = ts[2].addr;
    a.block_table = static_cast<const int32_t*>(ts[3].addr);
    a.act_seq = static_cast<const int32_t*>(ts[4].addr);
    a.out = ts[5].addr;
    a.part_o = nullptr;
    a.part_ml = nullptr;
    a.n_blocks = blocks;
    a.b = (int32_t)b;
    a.s1 = b ? (int32_t)(t / b) : 0;
    a.nq = (int32_t)nq;
    a.nkv = (int32_t)nkv;
    a.hsub = (int32_t)hsub;
    a.block_size = (int32_t)bs;
    a.bt_stride = (int32_t)ts[3].shape[1];
    a.softmax_scale = p->softmax_scale;
    pto::gqa_pick_chunk((int)max_ctx, p->kv_chunk, &a.chunk, &a.nsplit);
    plan->ws_bytes = pto::gqa_workspace_bytes(t, (int)nq, a.nsplit);
    return PTO_OK;
}

struct PrologPlan {
    pto::PrologArgs args;
    uint64_t ws_bytes;
};

int plan_prolog(const PtoTensorDesc* ts, uint32_t n, const PtoIndexerPrologParams* p, PrologPlan* plan)
{
    const char* op = "lightning_indexer_prolog_quant";
    if (ts == nullptr || n != 21) return fail(PTO_ERR_ARG_COUNT, "%s: expected 21 tensors, got %u", op, n);
    if (p == nullptr) return fail(PTO_ERR_PARAM, "%s: params is null", op);
    static const struct { const char* name; int dtype; int rank; } spec[21] = {
        {"x", PTO_DT_BF16, 2}, {"q_norm", PTO_DT_INT8, 2}, {"q_norm_scale", PTO_DT_FP32, 2}, {"w_qb", PTO_DT_INT8, 2},
        {"w_qb_scale", PTO_DT_FP32, 2}, {"wk", PTO_DT_BF16, 2}, {"w_proj", PTO_DT_BF16, 2}, {"ln_gamma_k", PTO_DT_BF16, 1},
        {"ln_beta_k", PTO_DT_BF16, 1}, {"cos_idx_rope", PTO_DT_BF16, 2}, {"sin_idx_rope", PTO_DT_BF16, 2},
        {"hadamard_q", PTO_DT_BF16, 2}, {"hadamard_k", PTO_DT_BF16, 2}, {"k_cache", PTO_DT_INT8, 4},
        {"k_cache_scale", PTO_DT_FP16, 4}, {"k_cache_index", PTO_DT_INT64, 1}, {"q_int8", PTO_DT_INT8, 3},
        {"q_scale", PTO_DT_FP16, 3}, {"k_int8", PTO_DT_INT8, 4}, {"k_scale", PTO_DT_FP16, 4}, {"weights", PTO_DT_FP16, 2}};
    int rc;
    for (int i = 0; i < 21; ++i)
        if ((rc = check_tensor(op, ts[i], spec[i].name, spec[i].dtype, spec[i].rank))) return rc;
    if (!(p->eps >= 0.f)) return fail(PTO_ERR_PARAM, "%s: eps must be non-negative", op);
    const int64_t t = ts[0].shape[0], h = ts[0].shape[1], r = ts[1].shape[1], nd = ts[3].shape[1];
    const int64_t d = ts[11].shape[0], rope = ts[9].shape[1], nh = ts[6].shape[1];
    if (d != 128 || nd != nh * d || !pto::prolog_supported(h, r, nh, d, rope))
        return fail(PTO_ERR_SHAPE, "%s: need head dim 128, rotary dim 64, heads a multiple of 32 (at most 128), w_qb [r, heads*128] with r a multiple of 128 (at most 2048) and h a multiple of 256; got h %lld r %lld heads %lld dim %lld rotary %lld w_qb cols %lld",
                    op, (long long)h, (long long)r, (long long)nh, (long long)d, (long long)rope, (long long)nd);
    const bool ok = ts[1].shape[0] == t && ts[2].shape[0] == t && ts[2].shape[1] == 1 && ts[3].shape[0] == r &&
                    ts[4].shape[0] == nd && ts[4].shape[1] == 1 && ts[5].shape[0] == h && ts[5].shape[1] == d &&
                    ts[6].shape[0] == h && ts[7].shape[0] == d && ts[8].shape[0] == d && ts[9].shape[0] == t &&
                    ts[10].shape[0] == t && ts[10].shape[1] == rope && ts[11].shape[1] == d && ts[12].shape[0] == d &&
                    ts[12].shape[1] == d && ts[13].shape[2] == 1 && ts[13].shape[3] == d &&
                    ts[14].shape[0] == ts[13].shape[0] && ts[14].shape[1] == ts[13].shape[1] && ts[14].shape[2] == 1 &&
                    ts[14].shape[3] == 1 && ts[15].shape[0] == t && ts[16].shape[0] == t && ts[16].shape[1] == nh &&
                    ts[16].shape[2] == d && ts[17].shape[0] == t && ts[17].shape[1] == nh && ts[17].shape[2] == 1 &&
                    ts[20].shape[0] == t && ts[20].shape[1] == nh;
    if (!ok) return fail(PTO_ERR_SHAPE, "%s: operand shapes do not fit together (t %lld, h %lld, r %lld, heads %lld)", op, (long long)t, (long long)h, (long long)r, (long long)nh);
    if (ts[18].addr != ts[13].addr || ts[19].addr != ts[14].addr)
        return fail(PTO_ERR_PARAM, "%s: k_int8 / k_scale must be the k_cache / k_cache_scale buffers (the cache is updated in place)", op);
    if (t > 0x7fffffff / 256) return fail(PTO_ERR_SHAPE, "%s: too many tokens", op);
    pto::PrologArgs& a = plan->args;
    a.x = static_cast<const uint16_t*>(ts[0].addr);
    a.q_norm = static_cast<const int8_t*>(ts[1].addr);
    a.q_norm_scale = static_cast<const float*>(ts[2].addr);
    a.w_qb = static_cast<const int8_t*>(ts[3].addr);
    a.w_qb_scale = static_cast<const float*>(ts[4].addr);
    a.w_k = static_cast<const uint16_t*>(ts[5].addr);
    a.w_proj = static_cast<const uint16_t*>(ts[6].addr);
    a.ln_gamma = static_cast<const uint16_t*>(ts[7].addr);
    a.ln_beta = static_cast<const uint16_t*>(ts[8].addr);
    a.cos = static_cast<const uint16_t*>(ts[9].addr);
    a.sin = static_cast<const uint16_t*>(ts[10].addr);
    a.had_q = static_cast<const uint16_t*>(ts[11].addr);
    a.had_k = static_cast<const uint16_t*>(ts[12].addr);
    a.k_cache = static_cast<int8_t*>(ts[13].addr);
    a.k_scale_cache = static_cast<uint16_t*>(ts[14].addr);
    a.k_cache_index = static_cast<const int64_t*>(ts[15].addr);
    a.q_int8 = static_cast<int8_t*>(ts[16].addr);
    a.q_scale = static_cast<uint16_t*>(ts[17].addr);
    a.weights = static_cast<uint16_t*>(ts[20].addr);
    a.xw_part = nullptr;
    a.cache_rows = ts[13].shape[0] * ts[13].shape[1];
    a.t = (int32_t)t;
    a.h = (int32_t)h;
    a.r = (int32_t)r;
    a.n = (int32_t)nh;
    a.ksplits = (int32_t)(h / 256);
    a.eps = p->eps;
    a.wscale_n = (float)(1.0 / __builtin_sqrt((double)nh));
    a.wscale_d = (float)(1.0 / __builtin_sqrt((double)d));
    plan->ws_bytes = pto::prolog_workspace_bytes(t, h, r, nh);
    return PTO_OK;
}

struct MlaPrologPlan {
    pto::MlaPrologArgs args;
    uint64_t ws_bytes;
};

int plan_mla_prolog(const PtoTensorDesc* ts, uint32_t n, const PtoMlaPrologParams* p, MlaPrologPlan* plan)
{
    const char* op = "mla_prolog_quant";
    if (ts == nullptr || n != 21) return fail(PTO_ERR_ARG_COUNT, "%s: expected 21 tensors, got %u", op, n);
    if (p == nullptr) return fail(PTO_ERR_PARAM, "%s: params is null", op);
    if (p->cache_mode != PTO_CACHE_PA_BSND)
        return fail(PTO_ERR_PARAM, "%s: only cache mode PA_BSND (%d) is built, got %d", op, PTO_CACHE_PA_BSND, p->cache_mode);
    // int8 form: INT8 w_uq_qr with its dequant_scale, INT8 kv_cache and q_norm_out.  bf16 form: an empty dequant_scale,
    // BF16 w_uq_qr, kv_cache and q_norm_out (k_scale_cache and q_norm_scale_out are then left untouched).
    const bool quant = !(ts[3].rank >= 1 && ts[3].shape[0] == 0);
    const int wdt = quant ? PTO_DT_INT8 : PTO_DT_BF16;
    if (ts[3].rank < 1 || ts[3].rank > 2) return fail(PTO_ERR_SHAPE, "%s: dequant_scale must have rank 1 or 2", op);
    if (ts[3].dataType != PTO_DT_FP32) return fail(PTO_ERR_DTYPE, "%s: dequant_scale must be fp32", op);
    if (ts[2].dataType != wdt || ts[11].dataType != wdt || ts[14].dataType != wdt || ts[18].dataType != wdt)
        return fail(PTO_ERR_DTYPE, "%s: with %s dequant_scale, w_uq_qr, kv_cache and q_norm_out must all be %s (int8 form: INT8 w_uq_qr with its dequant_scale, INT8 kv_cache; bf16 form: empty dequant_scale, BF16 throughout)",
                    op, quant ? "a non-empty" : "an empty", dtype_name(wdt));
    const struct { const char* name; int dtype; int rank; } spec[21] = {
        {"token_x", PTO_DT_BF16, 2}, {"w_dq", PTO_DT_BF16, 2}, {"w_uq_qr", wdt, 2}, {"dequant_scale", PTO_DT_FP32, ts[3].rank},
        {"w_uk", PTO_DT_BF16, 3}, {"w_dkv_kr", PTO_DT_BF16, 2}, {"gamma_cq", PTO_DT_BF16, 1}, {"gamma_ckv", PTO_DT_BF16, 1},
        {"cos", PTO_DT_BF16, 2}, {"sin", PTO_DT_BF16, 2}, {"cache_index", PTO_DT_INT64, 1}, {"kv_cache", wdt, 4},
        {"kr_cache", PTO_DT_BF16, 4}, {"k_scale_cache", PTO_DT_FP32, 4}, {"q_norm_out", wdt, 2},
        {"q_norm_scale_out", PTO_DT_FP32, 2}, {"query_nope_out", PTO_DT_BF16, 3}, {"query_rope_out", PTO_DT_BF16, 3},
        {"kv_cache_out", wdt, 4}, {"kr_cache_out", PTO_DT_BF16, 4}, {"k_scale_cache_out", PTO_DT_FP32, 4}};
    int rc;
    for (int i = 0; i < 21; ++i)
        if ((rc = check_tensor(op, ts[i], spec[i].name, spec[i].dtype, spec[i].rank))) return rc;
    if (!(p->epsilon_cq >= 0.f) || !(p->epsilon_ckv >= 0.f)) return fail(PTO_ERR_PARAM, "%s: epsilons must be non-negative", op);
    const int64_t t = ts[0].shape[0], h = ts[0].shape[1], r = ts[1].shape[1];
    const int64_t nh = ts[4].shape[0], dn = ts[4].shape[1], c = ts[4].shape[2], rope = ts[9].shape[1];
    if (!pto::mla_prolog_supported(h, r, nh, dn, rope, c))
        return fail(PTO_ERR_SHAPE, "%s: need w_uk [heads, 128, 512] with an even number of heads, rotary dim 64, q_lora_rank a multiple of 128 (at most 2048) and h a multiple of 256; got h %lld r %lld heads %lld nope %lld rotary %lld kv rank %lld",
                    op, (long long)h, (long long)r, (long long)nh, (long long)dn, (long long)rope, (long long)c);
    if (!quant && r % 256 != 0)
        return fail(PTO_ERR_SHAPE, "%s: the bf16 form needs q_lora_rank a multiple of 256, got %lld", op, (long long)r);
    const int64_t nq = nh * (dn + rope);
    const bool ok = ts[1].shape[0] == h && ts[2].shape[0] == r && ts[2].shape[1] == nq &&
                    (!quant || (ts[3].rank == 2 && ts[3].shape[0] == nq && ts[3].shape[1] == 1)) && ts[5].shape[0] == h && ts[5].shape[1] == c + rope && ts[6].shape[0] == r &&
                    ts[7].shape[0] == c && ts[8].shape[0] == t && ts[8].shape[1] == rope && ts[9].shape[0] == t &&
                    ts[10].shape[0] == t && ts[11].shape[2] == 1 && ts[11].shape[3] == c &&
                    ts[12].shape[0] == ts[11].shape[0] && ts[12].shape[1] == ts[11].shape[1] && ts[12].shape[2] == 1 &&
                    ts[12].shape[3] == rope && ts[13].shape[0] == ts[11].shape[0] && ts[13].shape[1] == ts[11].shape[1] &&
                    ts[13].shape[2] == 1 && ts[13].shape[3] == 4 && ts[14].shape[0] == t && ts[14].shape[1] == r &&
                    ts[15].shape[0] == t && ts[15].shape[1] == 1 && ts[16].shape[0] == t && ts[16].shape[1] == nh &&
                    ts[16].shape[2] == c && ts[17].shape[0] == t && ts[17].shape[1] == nh && ts[17].shape[2] == rope;
    if (!ok) return fail(PTO_ERR_SHAPE, "%s: operand shapes do not fit together (t %lld, h %lld, r %lld, heads %lld)", op, (long long)t, (long long)h, (long long)r, (long long)nh);
    if (ts[18].addr != ts[11].addr || ts[19].addr != ts[12].addr || ts[20].addr != ts[13].addr)
        return fail(PTO_ERR_PARAM, "%s: kv_cache_out / kr_cache_out / k_scale_cache_out must be the kv_cache / kr_cache / k_scale_cache buffers (the caches are updated in place)", op);
    if (t > 0x7fffffff / 4096) return fail(PTO_ERR_SHAPE, "%s: too many tokens", op);
    pto::MlaPrologArgs& a = plan->args;
    a.x = static_cast<const uint16_t*>(ts[0].addr);
    a.w_dq = static_cast<const uint16_t*>(ts[1].addr);
    a.w_uq_qr = ts[2].addr;
    a.quant = quant;
    a.qb_part = nullptr;
    a.w_qb_scale = static_cast<const float*>(ts[3].addr);
    a.w_uk = static_cast<const uint16_t*>(ts[4].addr);
    a.w_dkv_kr = static_cast<const uint16_t*>(ts[5].addr);
    a.gamma_cq = static_cast<const uint16_t*>(ts[6].addr);
    a.gamma_ckv = static_cast<const uint16_t*>(ts[7].addr);
    a.cos = static_cast<const uint16_t*>(ts[8].addr);
    a.sin = static_cast<const uint16_t*>(ts[9].addr);
    a.cache_index = static_cast<const int64_t*>(ts[10].addr);
    a.kv_cache = static_cast<int8_t*>(ts[11].addr);
    a.kr_cache = static_cast<uint16_t*>(ts[12].addr);
    a.k_scale_cache = static_cast<float*>(ts[13].addr);
    a.q_norm = static_cast<int8_t*>(ts[14].addr);
    a.q_norm_scale = static_cast<float*>(ts[15].addr);
    a.q_nope = static_cast<uint16_t*>(ts[16].addr);
    a.q_rope = static_cast<uint16_t*>(ts[17].addr);
    a.xa_part = nullptr;
    a.qb_nope = nullptr;
    a.w_k = nullptr;
    a.w_proj = nullptr;
    a.n_idx = 0;
    a.ncols = (int32_t)(r + c + rope);
    a.cache_rows = ts[11].shape[0] * ts[11].shape[1];
    a.t = (int32_t)t;
    a.h = (int32_t)h;
    a.r = (int32_t)r;
    a.n = (int32_t)nh;
    a.ksplits = (int32_t)((h + 1023) / 1024);
    a.eps_cq = p->epsilon_cq;
    a.eps_ckv = p->epsilon_ckv;
    plan->ws_bytes = pto::mla_prolog_workspace_bytes(t, h, r, nh, 0, quant);
    return PTO_OK;
}

// mla_indexer_prolog_quant: the MLA prolog followed by the lightning-indexer prolog, which reads the MLA prolog's
// q_norm / q_norm_scale (held in the workspace) and shares token_x, cos, sin and cache_index with it.
struct FusedPrologPlan {
    MlaPrologPlan mla;
    PrologPlan ip;
    uint64_t off_ip_ws, off_q_norm, off_q_norm_scale, ws_bytes;
    bool fused; // four launches (the two operators' kernels side by side) instead of seven
};

uint64_t up256(uint64_t x) { return (x + 255) & ~(uint64_t)255; }

int plan_fused_prolog(const PtoTensorDesc* ts, uint32_t n, const PtoMlaIndexerPrologParams* p, void* ws, FusedPrologPlan* plan)
{
    const char* op = "mla_indexer_prolog_quant";
    if (ts == nullptr || n != 34) return fail(PTO_ERR_ARG_COUNT, "%s: expected 34 tensors, got %u", op, n);
    if (p == nullptr) return fail(PTO_ERR_PARAM, "%s: params is null", op);
    if (ts[0].rank != 2 || ts[1].rank != 2) return fail(PTO_ERR_SHAPE, "%s: token_x and mla_w_dq must have rank 2", op);
    const int64_t t = ts[0].shape[0], r = ts[1].shape[1];
    if (t < 0 || r <= 0) return fail(PTO_ERR_SHAPE, "%s: bad token count or q_lora_rank", op);
    // the intermediate tensors; their addresses are placeholders until the workspace is known
    uint8_t* base = ws ? static_cast<uint8_t*>(ws) : reinterpret_cast<uint8_t*>(uintptr_t(256));
    PtoTensorDesc qn = {}, qs = {};
    qn.dataType = PTO_DT_INT8;
    qn.rank = 2;
    qn.shape[0] = t;
    qn.shape[1] = r;
    qs.dataType = PTO_DT_FP32;
    qs.rank = 2;
    qs.shape[0] = t;
    qs.shape[1] = 1;
    qn.addr = base;
    qs.addr = base;
    PtoTensorDesc m[21], q[21];
    for (int i = 0; i < 14; ++i) m[i] = ts[i];
    m[14] = qn;
    m[15] = qs;
    for (int i = 0; i < 5; ++i) m[16 + i] = ts[24 + i];
    const PtoMlaPrologParams mp = {p->epsilon_cq, p->epsilon_ckv, p->cache_mode};
    int rc = plan_mla_prolog(m, 21, &mp, &plan->mla);
    if (rc) return rc;
    if (!plan->mla.args.quant)
        return fail(PTO_ERR_DTYPE, "%s: the fused operator exists in the int8 form only (INT8 mla_w_uq_qr with its dequant_scale)", op);
    q[0] = ts[0];
    q[1] = qn;
    q[2] = qs;
    for (int i = 0; i < 6; ++i) q[3 + i] = ts[14 + i];
    q[9] = ts[8];
    q[10] = ts[9];
    q[11] = ts[20];
    q[12] = ts[21];
    q[13] = ts[22];
    q[14] = ts[23];
    q[15] = ts[10];
    for (int i = 0; i < 5; ++i) q[16 + i] = ts[29 + i];
    const PtoIndexerPrologParams ipp = {p->indexer_eps};
    rc = plan_prolog(q, 21, &ipp, &plan->ip);
    if (rc) return rc;
    plan->fused = pto::fused_prolog_supported(plan->ip.args.n);
    if (plan->fused) { // the indexer's partial sums live inside the MLA prolog's: no workspace of its own
        plan->mla.ws_bytes = pto::mla_prolog_workspace_bytes(t, plan->mla.args.h, r, plan->mla.args.n, plan->ip.args.n, true);
        plan->ip.ws_bytes = 0;
    }
    plan->off_ip_ws = up256(plan->mla.ws_bytes);
    plan->off_q_norm = plan->off_ip_ws + up256(plan->ip.ws_bytes);
    plan->off_q_norm_scale = plan->off_q_norm + up256((uint64_t)t * r);
    plan->ws_bytes = plan->off_q_norm_scale + up256((uint64_t)t * 4);
    if (ws) {
        plan->mla.args.q_norm = reinterpret_cast<int8_t*>(base + plan->off_q_norm);
        plan->mla.args.q_norm_scale = reinterpret_cast<float*>(base + plan->off_q_norm_scale);
        plan->ip.args.q_norm = plan->mla.args.q_norm;
        plan->ip.args.q_norm_scale = plan->mla.args.q_norm_scale;
    }
    return PTO_OK;
}

// The exported launches: the asynchronous launch, then - when the caller asks for it, as the reference's bundle launch
// allows (framework/include/tile_fwk_bundle/pypto_bundle_api.h:41-44, "sync != 0 waits for completion") - a wait for
// the stream.
int finish_launch(const char* op, int rc, void* hip_stream, int sync)
{
    if (rc != PTO_OK || sync == 0) return rc;
    hipError_t e = hipStreamSynchronize(static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(PTO_ERR_HIP, "%s: waiting for the stream failed: %s", op, hipGetErrorString(e));
    return PTO_OK;
}

} // namespace

extern "C" {

uint64_t pto_mla_indexer_prolog_quant_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors,
                                                const PtoMlaIndexerPrologParams* params)
{
    FusedPrologPlan plan;
    return plan_fused_prolog(tensors, n_tensors, params, nullptr, &plan) == PTO_OK ? plan.ws_bytes : 0;
}

static int mla_indexer_prolog_quant_launch_async(const PtoTensorDesc* tensors, uint32_t n_tensors,
                                        const PtoMlaIndexerPrologParams* params, void* workspace,
                                        uint64_t workspace_bytes, void* hip_stream)
{
    const char* op = "mla_indexer_prolog_quant";
    FusedPrologPlan plan;
    int rc = plan_fused_prolog(tensors, n_tensors, params, nullptr, &plan);
    if (rc) return rc;
    if (plan.mla.args.t == 0) return PTO_OK;
    if (workspace == nullptr || workspace_bytes < plan.ws_bytes)
        return fail(PTO_ERR_WORKSPACE, "%s: workspace of %llu bytes required, got %llu", op,
                    (unsigned long long)plan.ws_bytes, (unsigned long long)(workspace ? workspace_bytes : 0));
    if ((rc = plan_fused_prolog(tensors, n_tensors, params, workspace, &plan))) return rc;
    uint8_t* base = static_cast<uint8_t*>(workspace);
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    hipError_t e;
    if (plan.fused) {
        pto::fused_prolog_bind(plan.mla.args, plan.ip.args, base);
        e = pto::fused_prolog_launch(plan.mla.args, plan.ip.args, stream);
    } else {
        pto::mla_prolog_bind_workspace(plan.mla.args, base);
        pto::prolog_bind_workspace(plan.ip.args, base + plan.off_ip_ws);
        e = pto::mla_prolog_launch(plan.mla.args, stream);
        if (e == hipSuccess) e = pto::prolog_launch(plan.ip.args, stream);
    }
    if (e != hipSuccess) return fail(PTO_ERR_HIP, "%s: HIP launch failed: %s", op, hipGetErrorString(e));
    return PTO_OK;
}

uint64_t pto_mla_prolog_quant_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoMlaPrologParams* params)
{
    MlaPrologPlan plan;
    return plan_mla_prolog(tensors, n_tensors, params, &plan) == PTO_OK ? plan.ws_bytes : 0;
}

static int mla_prolog_quant_launch_async(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoMlaPrologParams* params,
                                void* workspace, uint64_t workspace_bytes, void* hip_stream)
{
    const char* op = "mla_prolog_quant";
    MlaPrologPlan plan;
    int rc = plan_mla_prolog(tensors, n_tensors, params, &plan);
    if (rc) return rc;
    if (plan.args.t == 0) return PTO_OK;
    if (workspace == nullptr || workspace_bytes < plan.ws_bytes)
        return fail(PTO_ERR_WORKSPACE, "%s: workspace of %llu bytes required, got %llu", op,
                    (unsigned long long)plan.ws_bytes, (unsigned long long)(workspace ? workspace_bytes : 0));
    pto::mla_prolog_bind_workspace(plan.args, workspace);
    hipError_t e = pto::mla_prolog_launch(plan.args, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(PTO_ERR_HIP, "%s: HIP launch failed: %s", op, hipGetErrorString(e));
    return PTO_OK;
}

uint64_t pto_indexer_prolog_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors,
                                      const PtoIndexerPrologParams* params)
{
    PrologPlan plan;
    return plan_prolog(tensors, n_tensors, params, &plan) == PTO_OK ? plan.ws_bytes : 0;
}

static int indexer_prolog_launch_async(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoIndexerPrologParams* params,
                              void* workspace, uint64_t workspace_bytes, void* hip_stream)
{
    const char* op = "lightning_indexer_prolog_quant";
    PrologPlan plan;
    int rc = plan_prolog(tensors, n_tensors, params, &plan);
    if (rc) return rc;
    if (plan.args.t == 0) return PTO_OK;
    if (workspace == nullptr || workspace_bytes < plan.ws_bytes)
        return fail(PTO_ERR_WORKSPACE, "%s: workspace of %llu bytes required, got %llu", op,
                    (unsigned long long)plan.ws_bytes, (unsigned long long)(workspace ? workspace_bytes : 0));
    pto::prolog_bind_workspace(plan.args, workspace);
    hipError_t e = pto::prolog_launch(plan.args, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(PTO_ERR_HIP, "%s: HIP launch failed: %s", op, hipGetErrorString(e));
    return PTO_OK;
}

uint64_t pto_attention_pre_quant_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors,
                                           const PtoAttentionPreQuantParams* params)
{
    AttnPrePlan plan;
    return plan_attention_pre(tensors, n_tensors, params, &plan) == PTO_OK ? plan.ws_bytes : 0;
}

static int attention_pre_quant_launch_async(const PtoTensorDesc* tensors, uint32_t n_tensors,
                                   const PtoAttentionPreQuantParams* params, void* workspace, uint64_t workspace_bytes,
                                   void* hip_stream)
{
    const char* op = "attention_pre_quant";
    AttnPrePlan plan;
    int rc = plan_attention_pre(tensors, n_tensors, params, &plan);
    if (rc) return rc;
    if (plan.args.t == 0) return PTO_OK;
    if (workspace == nullptr || workspace_bytes < plan.ws_bytes)
        return fail(PTO_ERR_WORKSPACE, "%s: workspace of %llu bytes required, got %llu", op,
                    (unsigned long long)plan.ws_bytes, (unsigned long long)(workspace ? workspace_bytes : 0));
    pto::attention_pre_bind_workspace(plan.args, workspace);
    hipError_t e = pto::attention_pre_launch(plan.args, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(PTO_ERR_HIP, "%s: HIP launch failed: %s", op, hipGetErrorString(e));
    return PTO_OK;
}

uint64_t pto_gqa_decode_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoGqaParams* params)
{
    GqaPlan plan;
    return plan_gqa(tensors, n_tensors, params, &plan) == PTO_OK ? plan.ws_bytes : 0;
}

static int gqa_decode_launch_async(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoGqaParams* params, void* workspace,
                          uint64_t workspace_bytes, void* hip_stream)
{
    const char* op = "attention";
    GqaPlan plan;
    int rc = plan_gqa(tensors, n_tensors, params, &plan);
    if (rc) return rc;
    if (plan.ws_bytes > 0) {
        if (workspace == nullptr || workspace_bytes < plan.ws_bytes)
            return fail(PTO_ERR_WORKSPACE, "%s: workspace of %llu bytes required, got %llu", op,
                        (unsigned long long)plan.ws_bytes, (unsigned long long)(workspace ? workspace_bytes : 0));
        pto::GqaArgs& a = plan.args;
        const uint64_t rows = (uint64_t)a.b * a.s1 * a.nq;
        a.part_o = static_cast<float*>(workspace);
        a.part_ml = a.part_o + rows * a.nsplit * 128;
    }
    hipError_t e = pto::gqa_launch(plan.args, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(PTO_ERR_HIP, "%s: HIP launch failed: %s", op, hipGetErrorString(e));
    return PTO_OK;
}

uint64_t pto_paged_gather_workspace(const PtoTensorDesc*, uint32_t, const PtoPagedGatherParams*) { return 0; }

static int paged_gather_launch_async(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoPagedGatherParams* params, void*,
                            uint64_t, void* hip_stream)
{
    pto::GatherArgs a;
    int rc = plan_paged_gather(tensors, n_tensors, params, &a);
    if (rc) return rc;
    hipError_t e = pto::paged_gather_launch(a, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(PTO_ERR_HIP, "paged_gather: HIP launch failed: %s", hipGetErrorString(e));
    return PTO_OK;
}

uint64_t pto_topk_workspace(const PtoTensorDesc*, uint32_t, const PtoTopkParams*) { return 0; }

static int topk_launch_async(const PtoTensorDesc* ts, uint32_t n, const PtoTopkParams* p, void*, uint64_t, void* hip_stream)
{
    const char* op = "topk";
    if (ts == nullptr || n != 3) return fail(PTO_ERR_ARG_COUNT, "%s: expected 3 tensors, got %u", op, n);
    if (p == nullptr) return fail(PTO_ERR_PARAM, "%s: params is null", op);
    int rc;
    // (the kernel reads and writes single elements: element alignment is all it asks for, so a view that starts at any
    // row of a tensor is a valid operand)
    if ((rc = check_tensor(op, ts[0], "input", PTO_DT_FP32, 2, 4))) return rc;
    if ((rc = check_tensor(op, ts[1], "values", PTO_DT_FP32, 2, 4))) return rc;
    if ((rc = check_tensor(op, ts[2], "indices", PTO_DT_INT32, 2, 4))) return rc;
    const int64_t rows = ts[0].shape[0], len = ts[0].shape[1];
    if (ts[1].shape[0] != rows || ts[2].shape[0] != rows || ts[1].shape[1] != p->k || ts[2].shape[1] != p->k)
        return fail(PTO_ERR_SHAPE, "%s: values and indices must be [%lld, %d]", op, (long long)rows, p->k);
    if (rows > 0x7fffffff) return fail(PTO_ERR_SHAPE, "%s: too many rows", op);
    if (!pto::topk_supported(len, p->k))
        return fail(PTO_ERR_PARAM, "%s: need 1 <= k <= row length; rows longer than 8192 elements need k <= 2048; got row length %lld, k %d",
                    op, (long long)len, p->k);
    hipError_t e = pto::topk_launch(static_cast<const float*>(ts[0].addr), static_cast<float*>(ts[1].addr),
                                    static_cast<int32_t*>(ts[2].addr), rows, (int)len, p->k, p->largest != 0,
                                    static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(PTO_ERR_HIP, "%s: HIP launch failed: %s", op, hipGetErrorString(e));
    return PTO_OK;
}

uint64_t pto_select_experts_workspace(const PtoTensorDesc*, uint32_t, const PtoSelectExpertsParams*) { return 0; }

static int select_experts_launch_async(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoSelectExpertsParams* params,
                              void*, uint64_t, void* hip_stream)
{
    pto::SelectExpertsArgs a;
    int rc = plan_select_experts(tensors, n_tensors, params, &a);
    if (rc) return rc;
    hipError_t e = pto::select_experts_launch(a, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(PTO_ERR_HIP, "select_experts: HIP launch failed: %s", hipGetErrorString(e));
    return PTO_OK;
}

uint64_t pto_sfa_quant_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoSfaParams* params)
{
    SfaPlan plan;
    return plan_sfa_quant(tensors, n_tensors, params, &plan) == PTO_OK ? plan.ws_bytes : 0;
}

static int sfa_quant_launch_async(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoSfaParams* params, void* workspace,
                         uint64_t workspace_bytes, void* hip_stream)
{
    SfaPlan plan;
    int rc = plan_sfa_quant(tensors, n_tensors, params, &plan);
    if (rc) return rc;
    return launch_sfa("sparse_flash_attention_quant", &plan, workspace, workspace_bytes, hip_stream);
}

int pto_sfa_quant_launch_noalloc(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoSfaParams* params,
                                 void* hip_stream, int sync)
{
    const char* op = "sparse_flash_attention_quant (no-allocation entry)";
    SfaPlan plan;
    int rc = plan_sfa_quant(tensors, n_tensors, params, &plan);
    if (rc) return rc;
    if (plan.ws_bytes > pto::SFA_STATIC_SCRATCH_BYTES)
        return fail(PTO_ERR_WORKSPACE, "%s: this problem needs %llu bytes of scratch, the library's own scratch array holds %llu; use pto_sfa_quant_launch with a workspace",
                    op, (unsigned long long)plan.ws_bytes, (unsigned long long)pto::SFA_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    if (plan.ws_bytes > 0) {
        hipError_t e = pto::sfa_static_scratch(&ws);
        if (e != hipSuccess) return fail(PTO_ERR_HIP, "%s: the scratch array's address is not available: %s", op, hipGetErrorString(e));
    }
    return finish_launch(op, launch_sfa(op, &plan, ws, plan.ws_bytes, hip_stream), hip_stream, sync);
}

uint64_t pto_sfa_antiquant_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoSfaParams* params)
{
    SfaPlan plan;
    return plan_sfa_antiquant(tensors, n_tensors, params, &plan) == PTO_OK ? plan.ws_bytes : 0;
}

static int sfa_antiquant_launch_async(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoSfaParams* params,
                             void* workspace, uint64_t workspace_bytes, void* hip_stream)
{
    SfaPlan plan;
    int rc = plan_sfa_antiquant(tensors, n_tensors, params, &plan);
    if (rc) return rc;
    return launch_sfa("sparse_attention_antiquant", &plan, workspace, workspace_bytes, hip_stream);
}

uint64_t pto_lightning_indexer_workspace(const PtoTensorDesc* tensors, uint32_t n_tensors,
                                         const PtoIndexerParams* params)
{
    IndexerPlan plan;
    return plan_indexer(tensors, n_tensors, params, &plan) == PTO_OK ? plan.ws_bytes : 0;
}

static int lightning_indexer_launch_async(const PtoTensorDesc* tensors, uint32_t n_tensors, const PtoIndexerParams* params,
                                 void* workspace, uint64_t workspace_bytes, void* hip_stream)
{
    const char* op = "lightning_indexer_decode";
    IndexerPlan plan;
    int rc = plan_indexer(tensors, n_tensors, params, &plan);
    if (rc) return rc;
    if (plan.ws_bytes > 0 && (workspace == nullptr || workspace_bytes < plan.ws_bytes))
        return fail(PTO_ERR_WORKSPACE, "%s: workspace of %llu bytes required, got %llu", op,
                    (unsigned long long)plan.ws_bytes, (unsigned long long)(workspace ? workspace_bytes : 0));
    pto::indexer_bind_workspace(plan.args, workspace);
    hipError_t e = pto::indexer_launch(plan.args, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(PTO_ERR_HIP, "%s: HIP launch failed: %s", op, hipGetErrorString(e));
    return PTO_OK;
}

#define PTO_EXPORT_LAUNCH(op, ParamsT)                                                                                \
    int pto_##op##_launch(const PtoTensorDesc* tensors, uint32_t n_tensors, const ParamsT* params, void* workspace,  \
                          uint64_t workspace_bytes, void* hip_stream, int sync)                                      \
    {                                                                                                                 \
        return finish_launch(#op, op##_launch_async(tensors, n_tensors, params, workspace, workspace_bytes, hip_stream), \
                             hip_stream, sync);                                                                       \
    }
PTO_EXPORT_LAUNCH(mla_indexer_prolog_quant, PtoMlaIndexerPrologParams)
PTO_EXPORT_LAUNCH(mla_prolog_quant, PtoMlaPrologParams)
PTO_EXPORT_LAUNCH(indexer_prolog, PtoIndexerPrologParams)
PTO_EXPORT_LAUNCH(attention_pre_quant, PtoAttentionPreQuantParams)
PTO_EXPORT_LAUNCH(gqa_decode, PtoGqaParams)
PTO_EXPORT_LAUNCH(paged_gather, PtoPagedGatherParams)
PTO_EXPORT_LAUNCH(select_experts, PtoSelectExpertsParams)
PTO_EXPORT_LAUNCH(topk, PtoTopkParams)
PTO_EXPORT_LAUNCH(sfa_quant, PtoSfaParams)
PTO_EXPORT_LAUNCH(sfa_antiquant, PtoSfaParams)
PTO_EXPORT_LAUNCH(lightning_indexer, PtoIndexerParams)
#undef PTO_EXPORT_LAUNCH

int pto_kernel_timing_enable(int on)
{
    pto::timing_set(on != 0);
    return PTO_OK;
}

int pto_kernel_timing_read(int kernel_id, double* total_ms, uint64_t* launches)
{
    if (kernel_id < 0 || kernel_id >= pto::KID_COUNT || total_ms == nullptr || launches == nullptr)
        return fail(PTO_ERR_PARAM, "pto_kernel_timing_read: bad kernel id or null output");
    hipError_t e = pto::timing_collect(kernel_id, total_ms, launches);
    if (e != hipSuccess) return fail(PTO_ERR_HIP, "pto_kernel_timing_read: %s", hipGetErrorString(e));
    return PTO_OK;
}

int pto_kernel_timing_overhead(void* hip_stream, double* ms)
{
    if (ms == nullptr) return fail(PTO_ERR_PARAM, "pto_kernel_timing_overhead: null output");
    hipError_t e = pto::timing_pair_overhead(static_cast<hipStream_t>(hip_stream), ms);
    if (e != hipSuccess) return fail(PTO_ERR_HIP, "pto_kernel_timing_overhead: %s", hipGetErrorString(e));
    return PTO_OK;
}

const char* pto_kernel_name(int kernel_id)
{
    static const char* names[] = {"indexer_score_kernel", "indexer_topk_kernel", "sfa_decode_kernel",
                                  "sfa_combine_kernel", "indexer_select_kernel", "select_experts_kernel",
                                  "gqa_decode_kernel", "gqa_combine_kernel", "apq_norm_kernel", "prolog_qx_kernel", "apq_gemm_kernel",
                                  "prolog_k_kernel", "mla_xa_kernel", "mla_norm_kernel", "mla_qb_kernel",
                                  "mla_wuk_kernel", "apq_head_kernel", "paged_gather_kernel"};
    return kernel_id >= 0 && kernel_id < pto::KID_COUNT ? names[kernel_id] : "";
}

const char* pto_last_error(void) { return g_last_error.c_str(); }

int pto_abi_version(void) { return 2; }

} // extern "C"
