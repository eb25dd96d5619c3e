"""Pins oracle.select_experts: brute force on small inputs, reductions to library routines, engineered ties."""
import math

import torch

from oracle import select_experts as ose


def brute(logits, bias, top_k, renorm, topk_group, n_group, scale, neg_inf):
    t, ne = logits.shape
    gs = ne // n_group
    ws, ids = [], []
    for r in range(t):
        sig = [1.0 / (1.0 + math.exp(-float(v))) for v in logits[r].float()]
        sig = [float(torch.tensor(v, dtype=torch.float32)) for v in sig]
        x = [float(torch.tensor(s, dtype=torch.float32) + bias[e].float()) for e, s in enumerate(sig)]
        gmax = [max(x[g * gs:(g + 1) * gs]) for g in range(n_group)]
        gorder = sorted(range(n_group), key=lambda g: (-gmax[g], g))[:topk_group]
        xm = [x[e] if e // gs in gorder else (-math.inf if neg_inf else 0.0) for e in range(ne)]
        order = sorted(range(ne), key=lambda e: (-xm[e], e))[:top_k]
        w = [sig[e] for e in order]
        if renorm:
            tot = float(torch.tensor(w, dtype=torch.float32).sum())
            w = [v / tot for v in w]
        ws.append([v * scale for v in w])
        ids.append(order)
    return torch.tensor(ws, dtype=torch.float32), torch.tensor(ids, dtype=torch.int32)


def test_brute_force_small():
    for seed, (ne, ng, tg, k, neg) in enumerate([(16, 4, 2, 3, False), (16, 4, 2, 3, True), (160, 8, 4, 8, True),
                                                  (160, 1, 1, 8, False), (12, 3, 1, 4, False)]):
        logits, bias = ose.make_case(7, ne, seed)
        w, ids = ose.select_experts(logits, k, True, tg, ng, bias, 2.5, neg)
        bw, bids = brute(logits, bias, k, True, tg, ng, 2.5, neg)
        assert torch.equal(ids, bids)
        assert torch.allclose(w, bw, rtol=2e-6, atol=0)


def test_one_group_is_plain_topk():
    logits, bias = ose.make_case(64, 160, 3, dist="uniform")
    w, ids = ose.select_experts(logits, 8, False, 1, 1, bias)
    x = ose.biased_scores(logits, bias)
    vals, lib_ids = torch.topk(x, 8, dim=-1)
    assert torch.equal(x.gather(1, ids.long()), vals)      # same values in the same (descending) order
    assert torch.equal(w, logits.float().sigmoid().gather(1, ids.long()))


def test_reference_inline_golden_same_set():
    # the golden of the reference test uses torch.topk(sorted=False): same set of experts, any order
    logits, bias = ose.make_case(32, 160, 0, dist="uniform")
    _, ids = ose.select_experts(logits, 8, True, 1, 1, bias)
    x = logits.float().sigmoid() + bias.float().unsqueeze(0)
    ref = torch.topk(x, k=8, dim=-1, sorted=False)[1]
    assert torch.equal(ids.long().sort(dim=-1).values, ref.sort(dim=-1).values)


def test_ties_take_the_smaller_index_and_zero_fill_competes():
    logits = torch.zeros((1, 8))
    bias = torch.zeros(8, dtype=torch.bfloat16)
    w, ids = ose.select_experts(logits, 3, True, 1, 1, bias)
    assert ids.tolist() == [[0, 1, 2]] and torch.allclose(w, torch.full((1, 3), 1 / 3))
    # two groups of 4, one kept: the kept group's biased scores are negative, so with the 0.0 fill the masked experts
    # (score 0.0, lowest ids first) beat them; with -inf they cannot
    bias = torch.tensor([-2.0] * 4 + [-3.0] * 4, dtype=torch.bfloat16)
    _, ids0 = ose.select_experts(logits, 3, False, 1, 2, bias, fill_neg_inf=False)
    _, ids1 = ose.select_experts(logits, 3, False, 1, 2, bias, fill_neg_inf=True)
    assert ids0.tolist() == [[4, 5, 6]] and ids1.tolist() == [[0, 1, 2]]


def test_renormalised_weights_sum_to_the_scale():
    logits, bias = ose.make_case(128, 160, 5, logits_dtype=torch.bfloat16, bias_dtype=torch.float32)
    w, ids = ose.select_experts(logits, 8, True, 4, 8, bias, 2.5, True)
    assert torch.allclose(w.sum(-1), torch.full((128,), 2.5), rtol=1e-6)
    assert (w[:, :-1] > 0).all() and ids.min() >= 0 and ids.max() < 160
    # every selected expert lies in one of at most 4 groups
    assert all(len(set((row // 20).tolist())) <= 4 for row in ids)
