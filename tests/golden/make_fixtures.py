#!/usr/bin/env python3
"""Writes the golden fixtures of this directory from the CPU oracle (run from the repo root:
``python tests/golden/make_fixtures.py``).

The reference's goldens live inside operator drivers that import ``pypto`` and ``torch_npu`` at module level
and cannot be imported here, and the reference stores no vectors of its own, so the fixtures are produced by
the restatement in ``oracle/`` (which tests/test_oracle_*.py pin against the reference's known answers and
closed forms).  They freeze inputs and expected outputs so that later changes of the oracle, of torch, or of
the kernels are caught against fixed data.  bf16 / fp16 tensors are stored as their 16-bit patterns.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import indexer as oi  # noqa: E402
from oracle import sfa as osfa  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def bits16(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def sfa_fixture():
    # config-1 shape scaled to fixture size: 1 sequence + a short one (cur_seq < topk), 16 heads, 4+1 pages
    c = osfa.make_case(2, 16, 2, [500, 70], topk=128, seed=1234, dist="bench", softmax_scale=192 ** -0.5)
    args = (c["q"], c["kn"], c["kr"], c["kn_scales"], c["topk_indices"], c["block_table"], c["act_seq"],
            c["block_size"], c["softmax_scale"], c["topk"])
    np.savez_compressed(
        os.path.join(HERE, "sfa_small.npz"),
        q=bits16(c["q"]), kn=c["kn"].numpy(), kr=bits16(c["kr"]), kn_scales=c["kn_scales"].numpy(),
        topk_indices=c["topk_indices"].numpy(), block_table=c["block_table"].numpy(),
        act_seq=np.array(c["act_seq"], dtype=np.int32), softmax_scale=np.float32(c["softmax_scale"]),
        out_no_flash=bits16(osfa.attention_no_flash(*args)),
        out_flash64=bits16(osfa.attention_flash(*args, s2_tile=64)))


def indexer_fixture():
    # four sequences around the selection size 64: longer, longer, equal+, shorter; two query tokens each
    c = oi.make_case(4, 2, [300, 97, 66, 15], seed=4321, selected_count=64)
    # engineered exact ties: duplicate some cached keys (and their scales) inside sequence 0
    keys = c["key_cache"].reshape(-1, 128)
    ks = c["k_scale"].reshape(-1)
    bt = c["block_table"]
    def row(b, n):
        return int(bt[b, n // 128]) * 128 + n % 128
    for src, dst in ((3, 200), (3, 77), (150, 151), (10, 299)):
        keys[row(0, dst)] = keys[row(0, src)]
        ks[row(0, dst)] = ks[row(0, src)]
    out = oi.lightning_indexer(c["query"], c["q_scale"], c["key_cache"], c["k_scale"], c["weights"], c["act_seq"],
                               c["block_table"], 2, 64)
    scores = oi.scores_exact(c["query"], c["q_scale"], c["key_cache"], c["k_scale"], c["weights"], c["act_seq"],
                             c["block_table"], 2)
    np.savez_compressed(
        os.path.join(HERE, "indexer_small.npz"),
        query=c["query"].numpy(), q_scale=bits16(c["q_scale"]), key_cache=c["key_cache"].numpy(),
        k_scale=bits16(c["k_scale"]), weights=bits16(c["weights"]), act_seq=np.array(c["act_seq"], dtype=np.int32),
        block_table=c["block_table"].numpy(), topk_res=out.numpy(), scores_f64=scores.numpy())


if __name__ == "__main__":
    sfa_fixture()
    indexer_fixture()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
