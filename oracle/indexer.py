"""Lightning indexer (int8 index scores + top-k) - CPU golden (test infrastructure).

Restates ``lightning_indexer_compute``
(models/deepseek_v32_exp/deepseekv32_lightning_indexer_quant.py:178-263) and
its data generators (same file, :46-175).  Arithmetic the golden fixes:

  w_scale[h]   = fp16( q_scale[h] * weight[h] )                     one fp16 multiply (:216)
  y[h, n]      = fp16( relu(int32 dot(q[h], k[n])) * 2^-11 )        exact int dot, exact fp32 scaling, RNE to fp16 (:226-228)
  score[n]     = ( sum_h fp32(w_scale[h]) * fp32(y[h, n]) ) * fp32(k_scale[n])     fp32 (:238-241)
  top-k        = torch.topk over score[:eff_seq], eff_seq = act - (s1 - 1 - i); -1 fills unused slots (:244-261)

fp32-scale variant (the benchmark's configuration with fp32 per-token scales; the reference's operator takes fp16):
q_scale and k_scale may be fp32 tensors.  Then w_scale[h] = fp16(fp32(q_scale[h] * fp32(weight[h]))) and k_scale
enters the last product as it is; everything else is unchanged.  With fp32 scales that hold fp16 values the two
variants give the same bits.

Every product in the head sum is exact in fp32 (11-bit x 11-bit significands);
only the order of the 64 fp32 additions is left to the BLAS that torch calls,
so scores are defined up to fp32 summation order.  ``scores_exact`` gives the
same quantity with the sum carried in float64 for tolerance checks.  Ordering
of equal scores follows oracle.topk (smaller index first).
"""
import math

import numpy as np
import torch

from .paged import gen_block_table
from .topk import topk_sorted_stable

SCORE_SHIFT = 1.0 / 2048.0


def w_scale_of(q_scale, weights):
    """[t,nh] fp16 x [t,nh] fp16 -> fp16 product (one rounding).

    fp32-scale variant (not in the reference, whose operator takes fp16 scales only): an fp32 q_scale is multiplied
    with the fp16 weight in fp32 and the product is rounded to fp16 - the golden's rounding point, reached from the
    fp32 product instead of the exact one (two roundings where the 35-bit product does not fit fp32's 24 bits)."""
    if q_scale.dtype == torch.float32:
        return (q_scale * weights.to(torch.float32)).to(torch.float16)
    return (q_scale.to(torch.float16) * weights.to(torch.float16)).to(torch.float16)


def scores(query, q_scale, key_cache, k_scale, weights, act_seq, block_table, s1, acc_dtype=torch.float32):
    """Dense score matrix [t, max_blocks*bs] (fp32 unless acc_dtype says otherwise),
    zero beyond each sequence's length, computed page by page like the golden."""
    t, nh, d = query.shape
    b = len(act_seq)
    n_blocks, bs = key_cache.shape[0], key_cache.shape[1]
    keys = key_cache.reshape(n_blocks * bs, d)
    ks = k_scale.reshape(n_blocks, bs)
    ws = w_scale_of(q_scale.reshape(t, nh), weights.reshape(t, nh))
    out = torch.zeros((t, block_table.shape[1] * bs), dtype=acc_dtype)
    for bi in range(b):
        L = int(act_seq[bi])
        q_i = query[bi * s1:(bi + 1) * s1].reshape(s1 * nh, d).to(torch.int32)
        w_i = ws[bi * s1:(bi + 1) * s1].to(acc_dtype)  # [s1, nh]
        for j in range(math.ceil(L / bs)):
            page = int(block_table[bi, j])
            n = min(bs, L - j * bs)
            k_j = keys[page * bs:page * bs + n].to(torch.int32)
            dot = torch.matmul(q_i, k_j.t())
            y = (dot.to(torch.float32).relu() * SCORE_SHIFT).to(torch.float16)
            y = y.reshape(s1, nh, n).to(acc_dtype)
            wy = torch.bmm(w_i.reshape(s1, 1, nh), y).reshape(s1, n)
            out[bi * s1:(bi + 1) * s1, j * bs:j * bs + n] = wy * ks[page, :n].to(acc_dtype)
    return out


def scores_exact(query, q_scale, key_cache, k_scale, weights, act_seq, block_table, s1):
    """Scores with the head sum and the k_scale product carried in float64."""
    return scores(query, q_scale, key_cache, k_scale, weights, act_seq, block_table, s1, acc_dtype=torch.float64)


def eff_seq_of(act_seq, s1, s1_idx):
    return int(act_seq) - (s1 - 1 - s1_idx)


def select(score_rows, act_seq, s1, selected_count):
    """Top-k per query token from a dense score matrix -> int32 [t, 1, selected_count]."""
    t = score_rows.shape[0]
    out = torch.full((t, 1, selected_count), -1, dtype=torch.int32)
    for r in range(t):
        n = eff_seq_of(act_seq[r // s1], s1, r % s1)
        if n <= 0:
            continue
        k = min(n, selected_count)
        _, idx = topk_sorted_stable(score_rows[r, :n], k)
        out[r, 0, :k] = idx
    return out


def lightning_indexer(query, q_scale, key_cache, k_scale, weights, act_seq, block_table, s1, selected_count=2048):
    sc = scores(query, q_scale, key_cache, k_scale, weights, act_seq, block_table, s1)
    return select(sc, act_seq, s1, selected_count)


def scatter_to_cache(k_bsd, block_table, n_blocks, block_size):
    """[b, s, d] logical keys -> paged cache [n_blocks, bs, d] through the page table."""
    b, s, d = k_bsd.shape
    cache = torch.zeros((n_blocks, block_size, d), dtype=k_bsd.dtype)
    padded = torch.zeros((b, block_table.shape[1] * block_size, d), dtype=k_bsd.dtype)
    padded[:, :s] = k_bsd
    for bi in range(b):
        for j, page in enumerate(block_table[bi].tolist()):
            if page >= 0:
                cache[page] = padded[bi, j * block_size:(j + 1) * block_size]
    return cache


def make_case(b, s1, act_seq, nh=64, d=128, block_size=128, selected_count=2048, seed=0, dist="bench",
              spare_pages=0, scale_dtype=torch.float16):
    """Synthetic indexer inputs with the reference's tensor signature.

    dist="bench":  q/k int8 U{-127..127}, scales ~U(0.005,0.02) in scale_dtype (fp16: the reference's operator;
                   fp32: the benchmark's configuration as written), weights fp16 ~N(0,1)/8.
    dist="driver": the reference driver's recipe - randn cast to int8, scale = absmax/127
                   in fp16 (floored at 1e-3), requantised; weights fp16 ~N(0,1).
    """
    g = torch.Generator().manual_seed(seed)
    act = [int(a) for a in act_seq]
    n_blocks, table = gen_block_table(act, block_size, generator=g)
    n_blocks += spare_pages
    t = b * s1
    if dist == "bench":
        query = torch.randint(-127, 128, (t, nh, d), generator=g, dtype=torch.int8)
        key_cache = torch.randint(-127, 128, (n_blocks, block_size, 1, d), generator=g, dtype=torch.int8)
        q_scale = (0.005 + 0.015 * torch.rand((t, nh), generator=g)).to(scale_dtype)
        k_scale = (0.005 + 0.015 * torch.rand((n_blocks, block_size, 1), generator=g)).to(scale_dtype)
        weights = (torch.randn((t, nh), generator=g) / 8).to(torch.float16)
    else:
        s2 = max(act)
        query = torch.randn((t, nh, d), generator=g).to(torch.int8)
        weights = torch.randn((t, nh), generator=g).to(torch.float16)
        k_log = torch.randn((b, s2, d), generator=g).to(torch.int8)
        key_cache = scatter_to_cache(k_log, table, n_blocks, block_size).reshape(n_blocks, block_size, 1, d)
        floor = torch.tensor(1e-3, dtype=torch.float16)
        q_scale = (query.abs().max(dim=-1, keepdim=True).values / 127).to(torch.float16).maximum(floor)
        k_scale = (key_cache.abs().max(dim=-1, keepdim=True).values / 127).to(torch.float16).maximum(floor)
        query = torch.round(query / q_scale).clip(-127, 127).to(torch.int8)
        key_cache = torch.round(key_cache / k_scale).clip(-127, 127).to(torch.int8)
        q_scale = q_scale.reshape(t, nh)
        k_scale = k_scale.reshape(n_blocks, block_size, 1)
    return {
        "b": b, "s1": s1, "nh": nh, "d": d, "block_size": block_size, "selected_count": selected_count,
        "act_seq": act, "query": query, "q_scale": q_scale, "key_cache": key_cache, "k_scale": k_scale,
        "weights": weights, "block_table": table,
    }
