"""Pins oracle.gqa: the flash golden against float64 textbook attention and against closed-form special cases."""
import torch

from oracle import gqa


def test_flash_matches_fp64_within_bf16():
    c = gqa.make_case(3, 2, 12, 2, [300, 129, 1], seed=1, block_size=64)
    o = gqa.attention_flash(c["q"], c["k"], c["v"], c["block_table"], c["act_seq"], c["softmax_scale"])
    r = gqa.attention_fp64(c["q"], c["k"], c["v"], c["block_table"], c["act_seq"], c["softmax_scale"])
    assert (o.double() - r).abs().max() < 2.0 ** -7 * r.abs().max() + 1e-3
    # act_seq 1 with two query tokens: token 0 sees nothing (zeros), token 1 sees exactly one row -> equals that V row
    assert (o[4] == 0).all()
    blk = int(c["block_table"][2, 0])
    assert torch.equal(o[5].view(2, 6, 128), c["v"][blk, 0].unsqueeze(1).expand(2, 6, 128))


def test_tile_argument_regroups_the_same_rows():
    """tile = page size walks the page table by positions instead of by pages: the same rows, so the same bits; one tile
    per sequence is plain softmax attention with one bf16 rounding of P~."""
    c = gqa.make_case(2, 2, 4, 2, [150, 33], seed=4, block_size=32)
    args = (c["q"], c["k"], c["v"], c["block_table"], c["act_seq"], c["softmax_scale"])
    assert torch.equal(gqa.attention_flash(*args, tile=32), gqa.attention_flash(*args))
    whole = gqa.attention_flash(*args, tile=150)
    r = gqa.attention_fp64(*args)
    assert (whole.double() - r).abs().max() < 2.0 ** -7 * r.abs().max() + 1e-3


def test_zero_query_gives_the_mean_of_v():
    c = gqa.make_case(1, 1, 8, 2, [200], seed=2, block_size=32, dist="uniform")
    q = torch.zeros_like(c["q"])
    o = gqa.attention_flash(q, c["k"], c["v"], c["block_table"], c["act_seq"], 1.0)
    pos = torch.arange(200)
    rows = c["block_table"][0, pos // 32].long() * 32 + pos % 32
    mean = c["v"].reshape(-1, 2, 128)[rows].double().mean(0)            # [nkv, d]
    assert (o[0].view(2, 4, 128).double() - mean.unsqueeze(1)).abs().max() < 2e-3


def test_heads_map_to_kv_heads_in_blocks():
    # head h uses KV head h // (nq // nkv): make KV head 1 all zeros in V -> heads 4..7 output zero
    c = gqa.make_case(1, 1, 8, 2, [70], seed=3, block_size=32)
    v = c["v"].clone()
    v[:, :, 1] = 0
    o = gqa.attention_flash(c["q"], c["k"], v, c["block_table"], c["act_seq"], c["softmax_scale"])
    assert (o[0, 4:] == 0).all() and (o[0, :4] != 0).any()


def test_rope_is_a_rotation_and_relative():
    g = torch.Generator().manual_seed(0)
    x = torch.randn((5, 3, 128), generator=g)
    pos = torch.tensor([0, 1, 7, 100, 4095])
    y = gqa.rope_neox(x, pos)
    assert torch.equal(y[0], x[0])                                         # position 0: identity
    assert torch.equal(y[..., 64:], x[..., 64:])                           # only the first 64 dims rotate
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), rtol=1e-5)       # rotation keeps the norm
    # dot products depend on the position difference only
    a, b = torch.randn((1, 1, 128), generator=g), torch.randn((1, 1, 128), generator=g)
    d1 = (gqa.rope_neox(a, torch.tensor([10])) * gqa.rope_neox(b, torch.tensor([3]))).sum()
    d2 = (gqa.rope_neox(a, torch.tensor([507])) * gqa.rope_neox(b, torch.tensor([500]))).sum()
    assert torch.allclose(d1, d2, rtol=1e-3, atol=1e-3)
