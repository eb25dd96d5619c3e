"""Page-table index math of the paged KV caches (CPU oracle, test infrastructure).

Follows the semantics of the reference's paged gather
(python/pypto/experimental/gather.py:27-82; interpreter bounds checks
framework/src/interface/interpreter/calculator/calc_torch.cpp:1916-1950) and of
its page-table generators
(models/deepseek_v32_exp/deepseekv32_sparse_flash_attention_quant.py:262-300,
models/deepseek_v32_exp/deepseekv32_lightning_indexer_quant.py:76-109).
"""
import math

import numpy as np
import torch


def logical_to_physical(indices, page_table_row, block_size):
    """Cache row of each logical token index: page[idx // bs] * bs + idx % bs."""
    idx = torch.as_tensor(indices).to(torch.int64)
    page = torch.as_tensor(page_table_row).to(torch.int64).reshape(-1)
    if idx.numel() and (idx.min() < 0 or idx.max() >= page.numel() * block_size):
        raise IndexError("logical index outside the page table")
    phys = page[idx // block_size] * block_size + idx % block_size
    if phys.numel() and phys.min() < 0:
        raise IndexError("logical index maps to an unused (-1) page")
    return phys


def paged_gather(src_2d, indices, page_table_row, block_size):
    """out[j, :] = src[page[idx[j] // bs] * bs + idx[j] % bs, :]."""
    phys = logical_to_physical(torch.as_tensor(indices).reshape(-1), page_table_row, block_size)
    if phys.numel() and phys.max() >= src_2d.shape[0]:
        raise IndexError("physical row outside the cache")
    return src_2d[phys]


def gen_block_table(act_seq, block_size, generator=None, max_blocks=None):
    """Random page table: every sequence gets ceil(len/bs) distinct physical
    pages dealt from one shuffled pool; unused slots hold -1.

    Returns (total_pages, table int32 [b, max ceil(len/bs)]).
    """
    act = [int(x) for x in act_seq]
    per_seq = [math.ceil(s / block_size) for s in act]
    total = sum(per_seq)
    width = max(per_seq) if per_seq else 0
    if max_blocks is not None:
        width = max(width, max_blocks)
    pool = torch.randperm(total, generator=generator).to(torch.int32)
    table = torch.full((len(act), width), -1, dtype=torch.int32)
    pos = 0
    for b, n in enumerate(per_seq):
        table[b, :n] = pool[pos:pos + n]
        pos += n
    return total, table


def cache_rows_of_new_tokens(act_seq, block_table, block_size, s1):
    """Physical cache row of each of the last s1 tokens of every sequence
    (the rows the producer stage writes), int64 [b, s1]."""
    b = len(act_seq)
    out = torch.full((b, s1), -1, dtype=torch.int64)
    for i in range(b):
        for j in range(s1):
            pos = int(act_seq[i]) - s1 + j
            out[i, j] = int(block_table[i, pos // block_size]) * block_size + pos % block_size
    return out
