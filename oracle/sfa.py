"""Sparse flash attention over an int8 paged MLA cache - CPU goldens (test infrastructure).

Restates, on the CPU in torch fp32, the goldens the reference keeps in its
operator drivers (paths relative to the reference checkout):

  attention_no_flash    models/deepseek_v32_exp/deepseekv32_sparse_flash_attention_quant.py:174-259
                        (one softmax over all selected tokens; P normalised, then rounded to bf16)
  attention_flash       models/deepseek_v32_exp/deepseekv32_sparse_flash_attention_quant.py:54-171 and
                        models/deepseek_v32_exp/deepseekv32_sparse_attention_antiquant.py:359-457
                        (online softmax over s2_tile chunks; exp(S - m_tile) rounded to bf16 unnormalised)
  pack_cache_rows /     models/deepseek_v32_exp/deepseekv32_sparse_attention_antiquant.py:262-272,112-122
  unpack_cache_rows     (656-byte row: 512 int8 | 64 bf16 | 4 fp32)
  quantize_nope         models/deepseek_v32_exp/deepseekv32_sparse_flash_attention_quant.py:361-365
  make_case             models/deepseek_v32_exp/deepseekv32_sparse_flash_attention_quant.py:303-404

Rounding points that the goldens fix and that every function here keeps:
  dequant  : bf16( fp32(int8) * fp32 scale[row, col // 128] )
  scores   : fp32 matmul of bf16-valued operands, then * softmax_scale in fp32
  P        : no-flash  bf16( exp(s - m) / l );   flash  bf16( exp(s - m_tile) ) with l summed in fp32 before rounding
  output   : fp32 accumulate, one final rounding to bf16

A query token whose clamped length ``cur_seq`` is 0 never enters the golden's
inner loop (its output row keeps the initial zeros); the restatement keeps
that: such rows are all-zero.
"""
import math

import torch

from .paged import gen_block_table, logical_to_physical

NOPE_DIM = 512
ROPE_DIM = 64
SCALE_GROUP = 128
PACKED_ROW_BYTES = NOPE_DIM + 2 * ROPE_DIM + 4 * (NOPE_DIM // SCALE_GROUP)  # 656


def cur_seq_of(act_seq, s1, s1_idx, topk):
    """Number of selected tokens query token s1_idx of a sequence attends to."""
    return min(max(int(act_seq) - s1 + 1 + s1_idx, 0), topk)


def dequant_nope(kn_int8, scales):
    """[n,512] int8, [n,4] fp32 -> [n,512] bf16."""
    n = kn_int8.shape[0]
    x = kn_int8.reshape(n * 4, SCALE_GROUP).to(torch.float32) * scales.reshape(n * 4, 1).to(torch.float32)
    return x.reshape(n, NOPE_DIM).to(torch.bfloat16)


def quantize_nope(kn_bf16_2d):
    """Per-token, per-128-column symmetric int8 quantisation. Returns (int8 [n,512], fp32 [n,4])."""
    n = kn_bf16_2d.shape[0]
    g = kn_bf16_2d.reshape(n, 4, SCALE_GROUP)
    scales = g.to(torch.float32).abs().amax(dim=-1, keepdim=True).clamp(min=1e-8) / 127.0
    q = torch.round(g / scales).clamp(-128, 127).to(torch.int8)
    return q.reshape(n, NOPE_DIM), scales.reshape(n, 4)


def pack_cache_rows(kn_int8, kr_bf16, scales):
    n = kn_int8.shape[0]
    rows = torch.zeros((n, PACKED_ROW_BYTES), dtype=torch.int8)
    rows[:, :NOPE_DIM] = kn_int8
    rows[:, NOPE_DIM:NOPE_DIM + 2 * ROPE_DIM] = kr_bf16.contiguous().view(torch.int8)
    rows[:, NOPE_DIM + 2 * ROPE_DIM:] = scales.contiguous().view(torch.int8)
    return rows


def unpack_cache_rows(rows):
    kn = rows[:, :NOPE_DIM].contiguous()
    kr = rows[:, NOPE_DIM:NOPE_DIM + 2 * ROPE_DIM].contiguous().view(torch.bfloat16)
    sc = rows[:, NOPE_DIM + 2 * ROPE_DIM:].contiguous().view(torch.float32)
    return kn, kr, sc


def _gather_tile(kn, kr, kn_scales, idx, block_table_row, block_size):
    """Selected cache rows as (K [n,576], V [n,512]) with the golden's dequant rounding."""
    rows = logical_to_physical(idx, block_table_row, block_size)
    if kn.dtype == torch.int8:
        nope = dequant_nope(kn[rows], kn_scales[rows])
    else:
        nope = kn[rows]
    k = torch.cat([nope, kr[rows]], dim=-1)
    return k, nope


def attention_no_flash(q, kn, kr, kn_scales, topk_indices, block_table, act_seq, block_size, softmax_scale, topk):
    """q [b,s1,nq,576] bf16 -> [b,s1,nq,512] bf16 (single-pass softmax golden)."""
    b, s1, nq, _ = q.shape
    out = torch.zeros((b, s1, nq, NOPE_DIM), dtype=q.dtype)
    tk = topk_indices.reshape(b * s1, -1)
    for bi in range(b):
        for si in range(s1):
            n = cur_seq_of(act_seq[bi], s1, si, topk)
            if n == 0:
                continue
            k, v = _gather_tile(kn, kr, kn_scales, tk[bi * s1 + si, :n], block_table[bi], block_size)
            s = torch.matmul(q[bi, si].to(torch.float32), k.to(torch.float32).t()) * softmax_scale
            p = torch.exp(s - s.amax(dim=-1, keepdim=True))
            p = (p / p.sum(dim=-1, keepdim=True)).to(q.dtype)
            out[bi, si] = torch.matmul(p.to(torch.float32), v.to(torch.float32)).to(q.dtype)
    return out


def attention_no_flash_token_loop(q, kn, kr, kn_scales, topk_indices, block_table, act_seq, block_size, softmax_scale, topk):
    """The single-pass golden the way the reference writes it: Python loops over batch, query token and selected
    token, one cache row looked up, dequantised and copied at a time
    (models/deepseek_v32_exp/deepseekv32_sparse_flash_attention_quant.py:203-257).  Same arithmetic as
    attention_no_flash, which gathers with index tensors; kept for the pin that the two agree bit for bit and as the
    "as written" CPU timing."""
    b, s1, nq, _ = q.shape
    out = torch.zeros((b, s1, nq, NOPE_DIM), dtype=torch.bfloat16)
    for bi in range(b):
        for si in range(s1):
            n = cur_seq_of(act_seq[bi], s1, si, topk)
            if n == 0:
                continue
            k_rows = torch.zeros((n, NOPE_DIM + ROPE_DIM), dtype=torch.bfloat16)
            for j in range(n):
                idx = int(topk_indices[bi * s1 + si, j])
                off = int(block_table[bi, idx // block_size]) * block_size + idx % block_size
                deq = (kn[off].reshape(4, SCALE_GROUP).float() * kn_scales[off].reshape(4, 1)).reshape(NOPE_DIM)
                k_rows[j, :NOPE_DIM] = deq.to(torch.bfloat16)
                k_rows[j, NOPE_DIM:] = kr[off]
            s = torch.matmul(q[bi, si].float(), k_rows.float().t()) * softmax_scale
            p = torch.exp(s - s.amax(dim=-1, keepdim=True))
            p = (p / p.sum(dim=-1, keepdim=True)).to(torch.bfloat16)
            out[bi, si] = torch.matmul(p.float(), k_rows[:, :NOPE_DIM].float()).to(torch.bfloat16)
    return out


def attention_flash(q, kn, kr, kn_scales, topk_indices, block_table, act_seq, block_size, softmax_scale, topk,
                    s2_tile=512):
    """Online-softmax golden: per s2_tile chunk, P~ = exp(s - m_tile) is rounded to
    bf16 *unnormalised* for the PV product while l is summed in fp32 from the
    unrounded values; chunks are merged with the usual (m, l, O) recurrence."""
    b, s1, nq, _ = q.shape
    out = torch.zeros((b, s1, nq, NOPE_DIM), dtype=q.dtype)
    tk = topk_indices.reshape(b * s1, -1)
    for bi in range(b):
        for si in range(s1):
            n = cur_seq_of(act_seq[bi], s1, si, topk)
            if n == 0:
                continue
            qi = q[bi, si].to(torch.float32)
            m = l = o = None
            for t0 in range(0, n, s2_tile):
                k, v = _gather_tile(kn, kr, kn_scales, tk[bi * s1 + si, t0:min(t0 + s2_tile, n)], block_table[bi],
                                    block_size)
                s = torch.matmul(qi, k.to(torch.float32).t()) * softmax_scale
                m_t = s.amax(dim=-1, keepdim=True)
                p = torch.exp(s - m_t)
                l_t = p.sum(dim=-1, keepdim=True)
                o_t = torch.matmul(p.to(q.dtype).to(torch.float32), v.to(torch.float32))
                if m is None:
                    m, l, o = m_t, l_t, o_t
                else:
                    m_new = torch.maximum(m, m_t)
                    a_old, a_new = torch.exp(m - m_new), torch.exp(m_t - m_new)
                    l = l * a_old + l_t * a_new
                    o = o * a_old + o_t * a_new
                    m = m_new
            out[bi, si] = (o / l).to(q.dtype)
    return out


def attention_packed(q_nope, q_rope, cache_rows, topk_indices, block_table, act_seq, nq, block_size, softmax_scale,
                     topk, flash=False, s2_tile=512):
    """Packed 656-byte-row variant; q_nope [t*nq,512], q_rope [t*nq,64]; returns [b,s1,nq,512]."""
    b = len(act_seq)
    s1 = q_nope.shape[0] // nq // b
    q = torch.cat([q_nope.reshape(b, s1, nq, NOPE_DIM), q_rope.reshape(b, s1, nq, ROPE_DIM)], dim=-1)
    kn, kr, sc = unpack_cache_rows(cache_rows)
    if flash:
        return attention_flash(q, kn, kr, sc, topk_indices, block_table, act_seq, block_size, softmax_scale, topk,
                               s2_tile)
    return attention_no_flash(q, kn, kr, sc, topk_indices, block_table, act_seq, block_size, softmax_scale, topk)


def attention_fp64(q, kn, kr, kn_scales, topk_indices, block_table, act_seq, block_size, softmax_scale, topk):
    """Independent textbook attention in float64 over the same selected rows.
    Only the input dequantisation keeps its bf16 rounding (it defines the
    operand values); no intermediate is rounded.  Used to pin the goldens."""
    b, s1, nq, _ = q.shape
    out = torch.zeros((b, s1, nq, NOPE_DIM), dtype=torch.float64)
    tk = topk_indices.reshape(b * s1, -1)
    for bi in range(b):
        for si in range(s1):
            n = cur_seq_of(act_seq[bi], s1, si, topk)
            if n == 0:
                continue
            k, v = _gather_tile(kn, kr, kn_scales, tk[bi * s1 + si, :n], block_table[bi], block_size)
            s = (q[bi, si].double() @ k.double().t()) * softmax_scale
            out[bi, si] = torch.softmax(s, dim=-1) @ v.double()
    return out


def make_case(b, nq, s1, act_seq, topk=2048, block_size=128, seed=42, quant=True, softmax_scale=None,
              dist="uniform", spare_pages=0):
    """Synthetic case in the style of the reference's generator: shuffled page
    table, top-k list = arange(len) when the sequence is shorter than topk else
    a random subset, q / cache ~ U[-1,1) bf16 ("uniform") or the benchmark
    distribution ("bench": q, rope ~ N(0,1), int8 nope U{-127..127},
    scales ~ U(0.005, 0.02))."""
    g = torch.Generator().manual_seed(seed)
    act = [int(a) for a in (act_seq if isinstance(act_seq, (list, tuple)) else [act_seq] * b)]
    assert len(act) == b
    n_pages, table = gen_block_table(act, block_size, generator=g)
    n_pages += spare_pages
    n_rows = n_pages * block_size
    tk = torch.zeros((b, s1, topk), dtype=torch.int32)
    for bi in range(b):
        for si in range(s1):
            if act[bi] < topk:
                tk[bi, si, :act[bi]] = torch.arange(act[bi], dtype=torch.int32)
            else:
                tk[bi, si] = torch.randperm(act[bi], generator=g)[:topk].to(torch.int32)
    if dist == "uniform":
        q = (torch.rand((b, s1, nq, NOPE_DIM + ROPE_DIM), generator=g) * 2 - 1).to(torch.bfloat16)
        kn_f = (torch.rand((n_rows, NOPE_DIM), generator=g) * 2 - 1).to(torch.bfloat16)
        kr = (torch.rand((n_rows, ROPE_DIM), generator=g) * 2 - 1).to(torch.bfloat16)
        if quant:
            kn, scales = quantize_nope(kn_f)
        else:
            kn, scales = kn_f, torch.ones((n_rows, 4), dtype=torch.float32)
    else:
        q = torch.randn((b, s1, nq, NOPE_DIM + ROPE_DIM), generator=g).to(torch.bfloat16)
        kr = torch.randn((n_rows, ROPE_DIM), generator=g).to(torch.bfloat16)
        kn = torch.randint(-127, 128, (n_rows, NOPE_DIM), generator=g, dtype=torch.int8)
        scales = 0.005 + 0.015 * torch.rand((n_rows, 4), generator=g)
    if softmax_scale is None:
        softmax_scale = (NOPE_DIM + ROPE_DIM) ** -0.5
    return {
        "b": b, "s1": s1, "nq": nq, "topk": topk, "block_size": block_size, "softmax_scale": float(softmax_scale),
        "act_seq": act, "q": q, "kn": kn, "kr": kr, "kn_scales": scales,
        "topk_indices": tk.reshape(b * s1, topk), "block_table": table,
    }
