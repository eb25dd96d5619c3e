"""CPU restatement of the reference's paged GQA decode attention goldens (test infrastructure only).

attention_flash follows ``ifa_flash_torch`` (models/glm_v4_5/glm_attention.py:1374-1483): one tile per cache page, fp32
scores, tile-local maximum, P~ = exp(S - m_tile) rounded to the input dtype (bf16) un-normalised before the PV product,
fp32 running (m, l, O), one division at the end.  attention_fp64 follows the "high precision" golden
(models/glm_v4_5/utils/golden/attn_golden.py:97-130): plain softmax attention in float64 over the gathered rows.
Causal length of query token j of a sequence with s1 query tokens: act - (s1 - 1 - j), clamped at 0
(glm_attention.py:1411-1412).  The reference's flash golden hard-codes the scale d**-0.5 (:1437), which is what its
drivers pass as softmax_scale (glm_attention.py:310); here the scale is the argument.
"""
import math

import torch

from .paged import gen_block_table


def cur_seq_of(act, s1, j):
    return max(int(act) - (s1 - 1 - j), 0)


def attention_flash(q, k_cache, v_cache, block_table, act_seqs, softmax_scale, tile=None):
    """q [t, nq, d] bf16; k_cache / v_cache [blocks, bs, nkv, d] bf16 -> [t, nq, d] bf16 (zeros where nothing is attended).
    ``tile``: tokens per tile; None is the reference's choice, one tile per cache page.  (Another tile size is the same
    algorithm with its roundings of P~ taken relative to other maxima: tests use it as a yardstick of what the
    algorithm's accuracy is when the tile is not the page.)"""
    t, nq, d = q.shape
    _, bs, nkv, _ = k_cache.shape
    b = len(act_seqs)
    s1 = t // b
    g = nq // nkv
    out = torch.zeros_like(q)
    step = bs if tile is None else int(tile)
    for bi in range(b):
        for j in range(s1):
            cur = cur_seq_of(act_seqs[bi], s1, j)
            if cur == 0:
                continue
            qi = q[bi * s1 + j].view(nkv, g, d).float()
            m = l = o = None
            for p in range(math.ceil(cur / step)):
                n = min(step, cur - p * step)
                if tile is None:
                    blk = int(block_table[bi, p])
                    kj = k_cache[blk, :n].permute(1, 0, 2).float()                   # [nkv, n, d]
                    vj = v_cache[blk, :n].permute(1, 0, 2).float()
                else:
                    pos = torch.arange(p * step, p * step + n)
                    rows = block_table[bi, pos // bs].long() * bs + pos % bs
                    kj = k_cache.reshape(-1, nkv, d)[rows].permute(1, 0, 2).float()
                    vj = v_cache.reshape(-1, nkv, d)[rows].permute(1, 0, 2).float()
                s = torch.matmul(qi, kj.transpose(1, 2)) * softmax_scale              # :1436-1437
                mt = s.max(dim=-1, keepdim=True).values                              # :1438
                pt = torch.exp(s - mt)                                               # :1439-1440
                lt = pt.sum(dim=-1, keepdim=True)                                    # :1441
                pv = torch.matmul(pt.to(q.dtype).float(), vj)                        # :1444 / :1466
                if m is None:
                    m, l, o = mt, lt, pv                                             # :1444-1451
                else:
                    m_new = torch.maximum(m, mt)                                     # :1457
                    t2 = torch.exp(m - m_new)                                        # :1458-1459
                    t4 = torch.exp(mt - m_new)                                       # :1460-1461
                    l = t2 * l + t4 * lt                                             # :1462-1464
                    o = o * t2 + pv * t4                                             # :1465-1468
                    m = m_new
            out[bi * s1 + j] = (o / l).to(q.dtype).view(nq, d)                        # :1447 / :1471
    return out


def attention_fp64(q, k_cache, v_cache, block_table, act_seqs, softmax_scale):
    t, nq, d = q.shape
    _, bs, nkv, _ = k_cache.shape
    b = len(act_seqs)
    s1 = t // b
    g = nq // nkv
    out = torch.zeros((t, nq, d), dtype=torch.float64)
    for bi in range(b):
        for j in range(s1):
            cur = cur_seq_of(act_seqs[bi], s1, j)
            if cur == 0:
                continue
            pos = torch.arange(cur)
            rows = block_table[bi, pos // bs].long() * bs + pos % bs
            k = k_cache.reshape(-1, nkv, d)[rows].double().permute(1, 0, 2)          # [nkv, cur, d]
            v = v_cache.reshape(-1, nkv, d)[rows].double().permute(1, 0, 2)
            qi = q[bi * s1 + j].view(nkv, g, d).double()
            p = torch.softmax(torch.matmul(qi, k.transpose(1, 2)) * softmax_scale, dim=-1)
            out[bi * s1 + j] = torch.matmul(p, v).view(nq, d)
    return out


def rope_neox(x, positions, theta=1e6, rotary_dim=64):
    """Half-split rotary embedding on the first rotary_dim dims: o1 = x1 cos - x2 sin, o2 = x2 cos + x1 sin
    (models/glm_v4_5/utils/golden/attn_golden.py:300-321).  x [n, heads, d], positions [n].  Used to make inputs only:
    the attention operator receives q and the cache already rotated."""
    half = rotary_dim // 2
    inv = theta ** (-torch.arange(half, dtype=torch.float32) / half)
    ang = positions.float().unsqueeze(-1) * inv
    cos, sin = ang.cos().unsqueeze(1), ang.sin().unsqueeze(1)
    xf = x.float()
    x1, x2 = xf[..., :half], xf[..., half:rotary_dim]
    return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin, xf[..., rotary_dim:]], dim=-1).to(x.dtype)


def make_case(b, s1, nq, nkv, act_seqs, block_size=128, seed=0, dist="normal", d=128, extra_blocks=2):
    """dist "normal": the benchmark's GQA configuration (q, k, v ~ N(0,1), rotary embedding theta 1e6 on the first 64 dims of
    q and k); dist "uniform": the reference driver's inputs (U[-1,1), glm_attention.py:1313-1315)."""
    g = torch.Generator().manual_seed(seed)
    max_blocks = max((max(act_seqs) + block_size - 1) // block_size, 1)
    total, table = gen_block_table(act_seqs, block_size, g, max_blocks)
    n_blocks = total + extra_blocks
    t = b * s1
    if dist == "uniform":
        q = torch.rand((t, nq, d), generator=g) * 2 - 1
        k = torch.rand((n_blocks, block_size, nkv, d), generator=g) * 2 - 1
        v = torch.rand((n_blocks, block_size, nkv, d), generator=g) * 2 - 1
    else:
        q = torch.randn((t, nq, d), generator=g)
        k = torch.randn((n_blocks, block_size, nkv, d), generator=g)
        v = torch.randn((n_blocks, block_size, nkv, d), generator=g)
        # rotate q at its own position and every cached key at the position its page-table slot gives it
        qpos = torch.tensor([cur_seq_of(act_seqs[i // s1], s1, i % s1) - 1 for i in range(t)]).clamp(min=0)
        q = rope_neox(q, qpos)
        kpos = torch.zeros(n_blocks * block_size, dtype=torch.long)
        for bi in range(b):
            for p in range((act_seqs[bi] + block_size - 1) // block_size):
                blk = int(table[bi, p])
                kpos[blk * block_size:(blk + 1) * block_size] = torch.arange(p * block_size, (p + 1) * block_size)
        k = rope_neox(k.view(-1, nkv, d), kpos).view(n_blocks, block_size, nkv, d)
    return {"q": q.to(torch.bfloat16), "k": k.to(torch.bfloat16), "v": v.to(torch.bfloat16), "block_table": table,
            "act_seq": list(act_seqs), "b": b, "s1": s1, "nq": nq, "nkv": nkv, "block_size": block_size,
            "softmax_scale": d ** -0.5}
