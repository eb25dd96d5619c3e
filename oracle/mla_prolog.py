"""CPU restatement of the reference's MLA prolog golden (test infrastructure only).

Follows ``mla_prolog_quant_v32_compute`` and its helpers in models/deepseek_v32_exp/deepseekv32_mla_prolog_quant.py
(:32-124 helpers, :131-283 compute, :285-441 generators) with is_quant_a False, no smoothing, and is_quant_b True (the
int8 form of the reference's quantised tests, :700-812, described below) or False (the bf16 form of its tests
:815-938: no quantisation anywhere - q_norm is the RmsNorm output itself, w_uq_qr is bf16, the kv cache holds the
normalised key in bf16 and the scale tensors are not touched).  The operator turns hidden states into everything sparse
flash attention reads:
  query : x @ w_dq (fp32 -> bf16) -> RmsNorm(gamma_cq) -> per-token int8 quantisation (q_norm, q_norm_scale: also the
          inputs of the lightning-indexer prolog) -> int8 GEMM with w_uq_qr (exact int32) * token scale * channel scale
          -> bf16 [t, n, 192]; the first 128 dims of a head times w_uk[head] (fp32 -> bf16) = q_nope [t, n, 512]; the
          last 64 through the rotary embedding = q_rope [t, n, 64]
  key   : x @ w_dkv_kr (fp32 -> bf16) [t, 576]; the first 512 -> RmsNorm(gamma_ckv) -> four groups of 128, each
          quantised to int8 with its own fp32 dequant scale; the last 64 through the rotary embedding; all three
          written into the paged caches (kv int8 [.., 512], scale fp32 [.., 4], rope bf16 [.., 64]) at cache_index
The rotary embedding takes interleaved pairs: element pairs (2i, 2i+1) are first moved to positions (i, 32+i).
"""
import torch


def rms_norm(x, gamma, eps=None):
    """:32-48 - fp32; the golden has no epsilon (eps None).  With eps: the operator's own order of operations
    (models/deepseek_v32_exp/mla_prolog_quant_impl.py:127-163): x * (1 / sqrt(sum(x*x/n) + eps)) * gamma."""
    xd = x.dtype
    xf = x.float()
    ms = torch.sum(xf * xf * (1.0 / x.shape[-1]), dim=-1, keepdim=True)
    if eps is None:
        res = xf / torch.sqrt(ms) * gamma.float()
    else:
        res = gamma.float() * (xf * (1.0 / torch.sqrt(ms + eps)))
    return res.to(xd)


def quant(x, per_token=True):
    """:104-122 - symmetric int8: scale 127 / absmax over the last dim (per_token) or over dim -2 (per channel);
    returns the int8 values and the fp32 dequant scale."""
    xf = x.float()
    mx = torch.amax(torch.abs(xf), dim=-1 if per_token else -2, keepdim=True)
    scale_quant = 127 / mx
    y = torch.round(xf * scale_quant).to(torch.int32)
    y = torch.trunc(y.to(torch.float16)).to(torch.int8)
    return y, 1 / scale_quant


def rotate_half(x):
    x1, x2 = x.chunk(2, dim=-1)
    return torch.cat((-x2, x1), dim=-1)


def rope_interleaved(x, cos, sin):
    """:74-101 for one operand - x [t, n, r] with interleaved pairs, cos/sin [t, r]; fp32, result in x's dtype."""
    xf = x.float()
    t, n, r = xf.shape
    xf = xf.reshape(t, n, r // 2, 2).permute(0, 1, 3, 2).reshape(t, n, r)
    c, s = cos.float().unsqueeze(1), sin.float().unsqueeze(1)
    return ((xf * c) + (rotate_half(xf) * s)).to(x.dtype)


def _scatter(cache, rows, index):
    """:51-67 - rows written at the flat cache rows index (later rows win, as in the loop)."""
    out = cache.clone()
    flat = out.view(-1, cache.shape[-1])
    for i in range(index.numel()):
        flat[int(index.reshape(-1)[i])] = rows[i]
    return out


def query_tail(inp, q_norm, q_norm_scale):
    """The query path downstream of the (quantised) RmsNorm: q_nope [t, n, 512] and q_rope [t, n, 64] from q_norm,
    q_norm_scale (tests also call it with the product's own q_norm to check the downstream stages on their own).
    q_norm_scale None: the bf16 form."""
    t = q_norm.shape[0]
    n, d_nope, c = inp["w_uk"].shape
    d_rope = inp["cos"].shape[1]
    dt = inp["x"].dtype
    if q_norm_scale is None:
        qb = torch.matmul(q_norm.float(), inp["w_uq_qr"].float())                              # :214
    else:
        qb = torch.matmul(q_norm.to(torch.int32), inp["w_uq_qr"].to(torch.int32)).float()      # :205-210
        qb = (qb * q_norm_scale) * inp["w_qb_scale"].reshape(1, -1)                            # :211-212
    qb = qb.to(dt).reshape(t, n, d_nope + d_rope)                                              # :216-218
    q_nope = torch.matmul(qb[:, :, :d_nope].permute(1, 0, 2).float(), inp["w_uk"].float())     # :220-225
    q_nope = q_nope.to(dt).permute(1, 0, 2).contiguous()                                       # :226-228
    q_rope = rope_interleaved(qb[:, :, d_nope:], inp["cos"], inp["sin"])                       # :265-272
    return q_nope, q_rope


def mla_prolog(inp, eps_cq=None, eps_ckv=None):
    """inp: the tensors of make_case().  Returns q_norm int8 [t, r], q_norm_scale fp32 [t, 1], q_nope bf16 [t, n, 512],
    q_rope bf16 [t, n, 64] and updated copies kv_cache, kr_cache, k_scale_cache."""
    x = inp["x"]                                                    # [t, h] bf16
    t = x.shape[0]
    n, d_nope, c = inp["w_uk"].shape
    d_rope = inp["cos"].shape[1]
    quant_b = inp["w_uq_qr"].dtype == torch.int8
    qa = torch.matmul(x.float(), inp["w_dq"].float()).to(torch.bfloat16)                       # :192-194
    qn = rms_norm(qa, inp["gamma_cq"], eps_cq)                                                 # :196
    q_norm, q_norm_scale = quant(qn, True) if quant_b else (qn, None)                          # :204
    q_nope, q_rope = query_tail(inp, q_norm, q_norm_scale)

    kv = torch.matmul(x.float(), inp["w_dkv_kr"].float()).to(x.dtype)                          # :243-247
    ckv = rms_norm(kv[:, :c], inp["gamma_ckv"], eps_ckv)                                       # :250-251
    if quant_b:
        k_nope, k_scale = quant(ckv.reshape(t, 4, c // 4), True)                               # :254-256
    else:
        k_nope, k_scale = ckv, None
    k_rope = rope_interleaved(kv[:, c:].reshape(t, 1, d_rope), inp["cos"], inp["sin"]).reshape(t, d_rope)
    idx = inp["cache_index"]
    return {
        "q_norm": q_norm, "q_norm_scale": q_norm_scale, "q_nope": q_nope, "q_rope": q_rope,
        "kv_cache": _scatter(inp["kv_cache"], k_nope.reshape(t, c), idx),                      # :275-276
        "kr_cache": _scatter(inp["kr_cache"], k_rope, idx),                                    # :279-280
        "k_scale_cache": (_scatter(inp["k_scale_cache"], k_scale.reshape(t, 4), idx)           # :282-287
                          if quant_b else inp["k_scale_cache"].clone()),
    }


def intermediates(inp, eps_cq=None, eps_ckv=None):
    """bf16 / fp32 tensors just before the roundings that can flip (tests use them to tell a rounding-boundary
    difference from an error): RmsNorm output of the query path [t, r], bf16 q_b [t, n, 192], RmsNorm output of the
    key path [t, 512]."""
    x = inp["x"]
    t = x.shape[0]
    n, d_nope, c = inp["w_uk"].shape
    qa = torch.matmul(x.float(), inp["w_dq"].float()).to(torch.bfloat16)
    qn = rms_norm(qa, inp["gamma_cq"], eps_cq)
    if inp["w_uq_qr"].dtype == torch.int8:
        q_norm, q_norm_scale = quant(qn, True)
        qb = torch.matmul(q_norm.to(torch.int32), inp["w_uq_qr"].to(torch.int32)).float()
        qb = ((qb * q_norm_scale) * inp["w_qb_scale"].reshape(1, -1)).to(x.dtype).reshape(t, n, -1)
    else:
        qb = torch.matmul(qn.float(), inp["w_uq_qr"].float()).to(x.dtype).reshape(t, n, -1)
    kv = torch.matmul(x.float(), inp["w_dkv_kr"].float()).to(x.dtype)
    ckv = rms_norm(kv[:, :c], inp["gamma_ckv"], eps_ckv)
    return {"q_a": qa, "q_rms": qn, "q_b": qb, "kv": kv, "kv_rms": ckv}


def make_case(b, s1, s2, seed=5, h=7168, q_lora_rank=1536, n=128, d_nope=128, d_rope=64, c=512, block_size=128,
              quant_b=True):
    """The reference generator's distributions (:331-441): x U[-1,1), weights U[-0.1,0.1) (w_uq_qr then quantised per
    output channel), gammas U[-1,1), cos/sin U[-0.1,0.1), caches filled from U[-1,1) data (the kv part quantised per
    group of 128); the last s1 positions of each length-s2 sequence are the new tokens (:299-313)."""
    g = torch.Generator().manual_seed(seed)
    t = b * s1
    bf = torch.bfloat16

    def uni(lo, hi, *shape):
        return torch.rand(shape, generator=g) * (hi - lo) + lo

    w_uq_qr = uni(-0.1, 0.1, q_lora_rank, n * (d_nope + d_rope)).to(bf)
    w_qb_scale = torch.zeros((0,), dtype=torch.float32)          # the bf16 form passes an empty dequant_scale (:613)
    if quant_b:
        w_uq_qr, w_qb_scale = quant(w_uq_qr, False)
    inp = {
        "x": uni(-1, 1, t, h).to(bf),
        "w_dq": uni(-0.1, 0.1, h, q_lora_rank).to(bf),
        "w_uq_qr": w_uq_qr,
        "w_qb_scale": w_qb_scale.reshape(-1, 1).contiguous(),
        "w_uk": uni(-0.1, 0.1, n, d_nope, c).to(bf),
        "w_dkv_kr": uni(-0.1, 0.1, h, c + d_rope).to(bf),
        "gamma_cq": uni(-1, 1, q_lora_rank).to(bf),
        "gamma_ckv": uni(-1, 1, c).to(bf),
        "cos": uni(-0.1, 0.1, t, d_rope).to(bf),
        "sin": uni(-0.1, 0.1, t, d_rope).to(bf),
    }
    pages_per_seq = (s2 + block_size - 1) // block_size
    n_pages = b * pages_per_seq
    table = torch.randperm(n_pages, generator=g).to(torch.int32).reshape(b, pages_per_seq)
    inp["block_table"] = table
    kv_old = uni(-1, 1, n_pages * block_size, 4, c // 4).to(bf)
    if quant_b:
        kv_q, kv_s = quant(kv_old, True)
        inp["kv_cache"] = kv_q.reshape(n_pages, block_size, 1, c)
        inp["k_scale_cache"] = kv_s.reshape(n_pages, block_size, 1, 4).contiguous()
    else:
        inp["kv_cache"] = kv_old.reshape(n_pages, block_size, 1, c).contiguous()
        inp["k_scale_cache"] = torch.zeros((n_pages, block_size, 1, 4), dtype=torch.float32)          # :603-606
    inp["kr_cache"] = uni(-1, 1, n_pages, block_size, 1, d_rope).to(bf)
    idx = torch.empty((b, s1), dtype=torch.int64)
    for i in range(b):
        for j in range(s1):
            pos = s2 - s1 + j
            idx[i, j] = int(table[i, pos // block_size]) * block_size + pos % block_size
    inp["cache_index"] = idx.reshape(t)
    return inp


def make_fused_case(b, s1, s2, seed=5, n_idx=64, **kw):
    """Inputs of the fused MLA + indexer prolog (models/deepseek_v32_exp/deepseekv32_mla_indexer_prolog_quant.py:336-393,
    :613-800): the MLA prolog's case plus the indexer's own weights and caches; token_x, cos, sin and cache_index are
    shared.  Returns (mla_case, indexer_case) - the indexer case still lacks q_norm / q_norm_scale, which the MLA
    prolog produces."""
    from . import indexer_prolog as ip
    mla = make_case(b, s1, s2, seed=seed, **kw)
    h, r = mla["x"].shape[1], mla["w_dq"].shape[1]
    idx = ip.make_case(b, s1, s2, seed=seed + 1000, h=h, q_lora_rank=r, n=n_idx)
    for k in ("q_norm", "q_norm_scale", "block_table"):
        del idx[k]
    idx.update(x=mla["x"], cos=mla["cos"], sin=mla["sin"], k_cache_index=mla["cache_index"])
    return mla, idx


def mla_indexer_prolog(mla_case, idx_case, eps_cq=None, eps_ckv=None, eps_idx=1e-6):
    """The fused golden is the composition (fused driver :336-393 and :711-713): the indexer prolog golden runs on the
    MLA prolog golden's q_norm / q_norm_scale."""
    from . import indexer_prolog as ip
    m = mla_prolog(mla_case, eps_cq, eps_ckv)
    i = ip.indexer_prolog(dict(idx_case, q_norm=m["q_norm"], q_norm_scale=m["q_norm_scale"]), eps=eps_idx)
    return m, i
