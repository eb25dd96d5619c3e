"""CPU restatement of the reference's lightning-indexer prolog golden (test infrastructure only).

Follows ``indexer_prolog`` and its helpers in models/deepseek_v32_exp/deepseekv32_lightning_indexer_prolog_quant.py
(:163-288; generators :30-160): the producer of everything the lightning indexer reads.
  query   : int8 GEMM q_norm @ w_qb (exact int32) * q_norm_scale * w_qb_scale -> bf16 -> rotary embedding on the first
            64 of each head's 128 dims -> right-multiply by the 128x128 "hadamard_q" matrix (fp32 matmul, -> bf16)
            -> per-(token, head) int8 quantisation (127 / absmax, round to nearest even) + fp16 dequant scale
  key     : x @ w_k (fp32) -> LayerNorm (fp32, eps) -> bf16 -> rotary -> hadamard_k -> bf16 -> quantisation ->
            written into the paged int8 index cache (and its fp16 scale cache) at k_cache_index
  weights : x @ w_proj (fp32 -> bf16) * 64^-0.5 * 128^-0.5 -> fp16
"""
import math

import torch


def layer_norm(x, gamma, beta, eps=1e-6):
    """:163-170 - in fp32, biased variance, result in the input dtype."""
    xd = x.dtype
    x = x.float()
    mean = x.mean(dim=-1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
    x = (x - mean) / torch.sqrt(var + eps)
    return (x * gamma.float() + beta.float()).to(xd)


def quant_int8(x):
    """:173-185 - per last-dim row: int8 values and the fp32 dequant scale."""
    xf = x.float()
    mx = torch.amax(torch.abs(xf), dim=-1, keepdim=True)
    scale_quant = 127.0 / mx
    y = torch.round(xf * scale_quant).to(torch.int32)            # rint
    y = torch.trunc(y.to(x.dtype)).to(torch.int8)
    return y, 1.0 / scale_quant


def rotate_half(x):
    x1, x2 = x.chunk(2, dim=-1)
    return torch.cat((-x2, x1), dim=-1)


def single_rope(x, cos, sin):
    """:194-206 - x [t, n, r], cos/sin [t, r]; fp32 arithmetic, result in x's dtype."""
    xf = x.float()
    out = xf * cos.float().unsqueeze(1) + rotate_half(xf) * sin.float().unsqueeze(1)
    return out.to(x.dtype)


def indexer_prolog(inp, rope_dim=64, eps=1e-6):
    """inp: the tensors of make_case().  Returns q_int8 [t, n, d], q_scale [t, n, 1] fp16, k_cache, k_scale_cache
    (updated copies), weights [t, n] fp16."""
    x = inp["x"]                                     # [t, h] bf16
    t = x.shape[0]
    n_d = inp["w_qb"].shape[1]
    d = inp["hadamard_q"].shape[0]
    n = n_d // d
    q = torch.matmul(inp["q_norm"].to(torch.int32), inp["w_qb"].to(torch.int32)).float()          # :232-233
    q = q * inp["q_norm_scale"].reshape(t, 1)                                                      # :234
    q = q * inp["w_qb_scale"].reshape(1, n_d)                                                      # :235
    q = q.reshape(t, n, d).to(torch.bfloat16)                                                      # :236
    q = torch.cat([single_rope(q[..., :rope_dim], inp["cos"], inp["sin"]), q[..., rope_dim:]], dim=-1)   # :237-239
    q = torch.matmul(q.float(), inp["hadamard_q"].float()).to(x.dtype)                            # :243
    q_int8, q_scale = quant_int8(q)                                                                # :244
    q_scale = q_scale.to(torch.float16)                                                            # :245

    k = torch.matmul(x.float(), inp["w_k"].float())                                                # :247
    k = layer_norm(k, inp["ln_gamma"], inp["ln_beta"], eps).to(x.dtype)                            # :248
    k = torch.cat([single_rope(k[:, :rope_dim].unsqueeze(1), inp["cos"], inp["sin"]).squeeze(1), k[:, rope_dim:]], dim=-1)
    k = torch.matmul(k.float(), inp["hadamard_k"].float()).to(x.dtype)                             # :255
    k_int8, k_scale = quant_int8(k)                                                                # :256
    k_scale = k_scale.to(torch.float16)                                                            # :257
    k_cache = inp["k_cache"].clone()
    k_scale_cache = inp["k_scale_cache"].clone()
    idx = inp["k_cache_index"].long()
    k_cache.view(-1, d)[idx] = k_int8                                                              # :261-262
    k_scale_cache.view(-1, 1)[idx] = k_scale

    w = torch.matmul(x.float(), inp["w_proj"].float()).to(x.dtype).float()                         # :265
    w = (w * (n ** -0.5) * (d ** -0.5)).to(torch.float16)                                          # :266-267
    return {"q_int8": q_int8, "q_scale": q_scale, "k_cache": k_cache, "k_scale_cache": k_scale_cache, "weights": w}


def intermediates(inp, rope_dim=64, eps=1e-6):
    """The bf16 tensors just before quantisation (q [t, n, d], k [t, d]) - tests use them to tell a rounding-boundary
    difference from an error."""
    x = inp["x"]
    t = x.shape[0]
    n_d = inp["w_qb"].shape[1]
    d = inp["hadamard_q"].shape[0]
    n = n_d // d
    q = torch.matmul(inp["q_norm"].to(torch.int32), inp["w_qb"].to(torch.int32)).float()
    q = (q * inp["q_norm_scale"].reshape(t, 1) * inp["w_qb_scale"].reshape(1, n_d)).reshape(t, n, d).to(torch.bfloat16)
    q = torch.cat([single_rope(q[..., :rope_dim], inp["cos"], inp["sin"]), q[..., rope_dim:]], dim=-1)
    q = torch.matmul(q.float(), inp["hadamard_q"].float()).to(x.dtype)
    k = layer_norm(torch.matmul(x.float(), inp["w_k"].float()), inp["ln_gamma"], inp["ln_beta"], eps).to(x.dtype)
    k = torch.cat([single_rope(k[:, :rope_dim].unsqueeze(1), inp["cos"], inp["sin"]).squeeze(1), k[:, rope_dim:]], dim=-1)
    k = torch.matmul(k.float(), inp["hadamard_k"].float()).to(x.dtype)
    return q, k


def make_case(b, s1, s2, seed=7, h=7168, q_lora_rank=1536, n=64, d=128, rope_dim=64, block_size=128,
              hadamard="uniform"):
    """The reference generator's distributions (:105-160): everything U[-1,1) (int8 tensors U{-128..127}), LayerNorm
    gamma 1 / beta 0, random rotary angles, the last s1 tokens of each sequence of length s2 are the new ones.
    hadamard "uniform" is the reference's stand-in (a random matrix); "walsh" is a scaled Walsh-Hadamard matrix."""
    g = torch.Generator().manual_seed(seed)
    t = b * s1
    bf = torch.bfloat16

    def uni(*shape):
        return torch.rand(shape, generator=g) * 2 - 1

    inp = {
        "x": uni(t, h).to(bf),
        "q_norm": torch.randint(-128, 128, (t, q_lora_rank), generator=g, dtype=torch.int8),
        "q_norm_scale": uni(t, 1),
        "w_qb": torch.randint(-128, 128, (q_lora_rank, n * d), generator=g, dtype=torch.int8),
        "w_qb_scale": uni(n * d, 1),
        "w_k": uni(h, d).to(bf),
        "w_proj": uni(h, n).to(bf),
        "ln_gamma": torch.ones(d, dtype=bf),
        "ln_beta": torch.zeros(d, dtype=bf),
    }
    ang = torch.rand((t, rope_dim), generator=g) * 2 * math.pi
    inp["cos"], inp["sin"] = torch.cos(ang).to(bf), torch.sin(ang).to(bf)
    if hadamard == "walsh":
        hm = torch.ones((1, 1))
        while hm.shape[0] < d:
            hm = torch.cat([torch.cat([hm, hm], 1), torch.cat([hm, -hm], 1)], 0)
        inp["hadamard_q"] = inp["hadamard_k"] = (hm * d ** -0.5).to(bf)
    else:
        inp["hadamard_q"], inp["hadamard_k"] = uni(d, d).to(bf), uni(d, d).to(bf)
    pages_per_seq = (s2 + block_size - 1) // block_size
    n_pages = b * pages_per_seq
    table = torch.randperm(n_pages, generator=g).to(torch.int32).reshape(b, pages_per_seq)
    inp["block_table"] = table
    inp["k_cache"] = torch.randint(-128, 128, (n_pages, block_size, 1, d), generator=g, dtype=torch.int8)
    inp["k_scale_cache"] = uni(n_pages, block_size, 1, 1).to(torch.float16)
    idx = torch.empty((b, s1), dtype=torch.int64)
    for i in range(b):
        for j in range(s1):
            pos = s2 - s1 + j                                                          # :60-69
            idx[i, j] = int(table[i, pos // block_size]) * block_size + pos % block_size
    inp["k_cache_index"] = idx.reshape(t)
    return inp
