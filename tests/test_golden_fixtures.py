"""The oracle must keep reproducing the committed fixtures bit for bit (guards against drift of the oracle or of
the torch build underneath it)."""
import torch

from oracle import indexer as oi
from oracle import sfa as osfa

from _fixtures import load_indexer_small, load_sfa_small


def test_sfa_fixture_reproduced():
    c, expect = load_sfa_small()
    args = (c["q"], c["kn"], c["kr"], c["kn_scales"], c["topk_indices"], c["block_table"], c["act_seq"],
            c["block_size"], c["softmax_scale"], c["topk"])
    assert torch.equal(osfa.attention_no_flash(*args), expect["no_flash"])
    assert torch.equal(osfa.attention_flash(*args, s2_tile=64), expect["flash64"])
    assert expect["no_flash"].shape == (2, 2, 16, 512)
    assert osfa.cur_seq_of(70, 2, 0, 128) == 69  # second sequence is shorter than the selection size


def test_indexer_fixture_reproduced_and_ties_resolved_by_index():
    c, topk, scores = load_indexer_small()
    out = oi.lightning_indexer(c["query"], c["q_scale"], c["key_cache"], c["k_scale"], c["weights"], c["act_seq"],
                               c["block_table"], 2, 64)
    assert torch.equal(out, topk)
    # duplicated keys give exactly equal scores; where both copies are selected the smaller index comes first
    for r in (0, 1):
        for a, b in ((3, 77), (3, 200), (150, 151), (10, 299)):
            assert float(scores[r, a]) == float(scores[r, b])
            row = topk[r, 0].tolist()
            if a in row and b in row:
                assert row.index(a) < row.index(b)
    assert (topk[7, 0, 15:] == -1).all() and (topk[6, 0, 14:] == -1).all()  # sequence of 15 tokens, 2 query tokens
