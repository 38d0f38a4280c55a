"""Pins the ring-attention oracle (oracle/ring.py) against things that are not the oracle:
fp64 softmax/logsumexp closed forms, F.scaled_dot_product_attention, autograd, torch.logaddexp,
and brute force over every rank of every ring size up to 8."""
import itertools
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import ring


def rnd(*shape, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=dtype)


# ------------------------------------------------------------------ integer work: exact
def test_causal_mask_closed_form():
    for n in (1, 2, 7, 64):
        m = ring.causal_mask(n)
        assert m.dtype == torch.bool
        assert torch.equal(m, torch.triu(torch.ones(n, n, dtype=torch.bool), diagonal=1))
        for i, j in itertools.product(range(min(n, 5)), repeat=2):
            assert bool(m[i, j]) == (j > i)


@pytest.mark.parametrize("world", range(1, 9))
def test_schedule_table_exhaustive(world):
    for rank in range(world):
        for causal in (True, False):
            sched = ring.schedule(world, rank, causal)
            assert [s for s, *_ in sched] == list(range(world))
            held = [c for _, c, _, _ in sched]
            # each chunk is visited exactly once, starting with the rank's own and walking backwards
            assert sorted(held) == list(range(world))
            assert held[0] == rank
            for s, c, run, blk_causal in sched:
                assert c == (rank - s) % world
                if causal:
                    # executed blocks are exactly the chunks at or before the rank's own
                    assert run == (c <= rank)
                    assert blk_causal == (c == rank)
                else:
                    assert run and not blk_causal


def test_rope_slice_and_positions_exact():
    S, D, W = 48, 8, 4
    cos = torch.arange(S * D, dtype=torch.float32).view(S, D)
    sin = -cos
    for r in range(W):
        c, s = ring.rope_slice(cos, sin, r, W)
        assert torch.equal(c, cos[r * 12:(r + 1) * 12]) and torch.equal(s, sin[r * 12:(r + 1) * 12])
        pos = ring.position_ids(r, S, W, batch_size=3)
        assert pos.dtype == torch.long and pos.shape == (3, 12)
        assert torch.equal(pos[1], torch.arange(r * 12, (r + 1) * 12))
    with pytest.raises(AssertionError):
        ring.rope_slice(cos, sin, 0, 5)


# ------------------------------------------------------------------ block forward
@pytest.mark.parametrize("causal", [False, True])
def test_block_forward_vs_softmax_closed_form(causal):
    q, k, v = rnd(2, 3, 16, 8, seed=1), rnd(2, 3, 16, 8, seed=2), rnd(2, 3, 16, 8, seed=3)
    scale = 0.37
    o, lse = ring.block_forward(q, k, v, scale, causal)
    s = torch.einsum("bhid,bhjd->bhij", q, k) * scale
    if causal:
        s = s + torch.full((16, 16), float("-inf"), dtype=s.dtype).triu(1)
    assert torch.allclose(o, torch.softmax(s, -1) @ v, atol=1e-12)
    assert torch.allclose(lse, torch.logsumexp(s, -1), atol=1e-12)
    assert lse.shape == (2, 3, 16)


@pytest.mark.parametrize("causal", [False, True])
def test_block_forward_vs_sdpa(causal):
    q, k, v = (rnd(1, 2, 32, 16, seed=s, dtype=torch.float32) for s in (4, 5, 6))
    o, _ = ring.block_forward(q, k, v, 1 / math.sqrt(16), causal)
    ref = F.scaled_dot_product_attention(q, k, v, is_causal=causal)
    assert torch.allclose(o, ref, atol=2e-6)


def test_block_forward_rectangular_dense():
    q, k, v = rnd(1, 1, 5, 4, seed=7), rnd(1, 1, 11, 4, seed=8), rnd(1, 1, 11, 4, seed=9)
    o, lse = ring.block_forward(q, k, v, 0.5, False)
    s = (q @ k.transpose(-1, -2)) * 0.5
    assert torch.allclose(o, torch.softmax(s, -1) @ v, atol=1e-12)
    assert torch.allclose(lse, torch.logsumexp(s, -1), atol=1e-12)


# ------------------------------------------------------------------ block backward
@pytest.mark.parametrize("causal", [False, True])
def test_block_backward_vs_autograd(causal):
    q, k, v = (rnd(2, 2, 12, 8, seed=s).requires_grad_() for s in (10, 11, 12))
    do = rnd(2, 2, 12, 8, seed=13)
    scale = 0.41
    s = (q @ k.transpose(-1, -2)) * scale
    if causal:
        s = s + torch.full((12, 12), float("-inf"), dtype=s.dtype).triu(1)
    o = torch.softmax(s, -1) @ v
    gq, gk, gv = torch.autograd.grad(o, (q, k, v), do)
    with torch.no_grad():
        o2, lse = ring.block_forward(q, k, v, scale, causal)
        dq, dk, dv = ring.block_backward(do, q, k, v, o2, lse, scale, causal)
    for a, b in ((dq, gq), (dk, gk), (dv, gv)):
        assert torch.allclose(a, b, atol=1e-11)


def test_block_forward_gradcheck():
    q, k, v = (rnd(1, 1, 4, 3, seed=s).requires_grad_() for s in (14, 15, 16))
    assert torch.autograd.gradcheck(lambda a, b, c: ring.block_forward(a, b, c, 0.7, True)[0], (q, k, v))


# ------------------------------------------------------------------ merge
def test_merge_vs_logaddexp_and_weighted_mean():
    o1, o2 = rnd(2, 2, 6, 4, seed=20, dtype=torch.float32), rnd(2, 2, 6, 4, seed=21, dtype=torch.float32)
    l1, l2 = rnd(2, 2, 6, seed=22, dtype=torch.float32) * 3, rnd(2, 2, 6, seed=23, dtype=torch.float32) * 3
    out, lse = ring.merge(None, None, o1, l1)
    assert torch.equal(out, o1) and torch.equal(lse, l1.unsqueeze(-1))
    out, lse = ring.merge(out, lse, o2, l2)
    want_lse = torch.logaddexp(l1, l2)
    w1, w2 = torch.exp(l1 - want_lse).unsqueeze(-1), torch.exp(l2 - want_lse).unsqueeze(-1)
    assert torch.allclose(lse.squeeze(-1), want_lse, atol=1e-6)
    assert torch.allclose(out, w1 * o1 + w2 * o2, atol=1e-6)


def test_merge_properties():
    o = [rnd(1, 1, 5, 4, seed=30 + i) for i in range(3)]
    l = [rnd(1, 1, 5, seed=40 + i) * 2 for i in range(3)]

    def fold(order):
        out = lse = None
        for i in order:
            out, lse = ring.merge(out, lse, o[i], l[i])
        return out, lse

    a, b = fold([0, 1, 2]), fold([2, 0, 1])
    assert torch.allclose(a[0], b[0], atol=1e-12) and torch.allclose(a[1], b[1], atol=1e-12)
    # merging a block that saw no keys (lse = -inf) is the identity
    out, lse = ring.merge(a[0], a[1], torch.zeros_like(o[0]), torch.full_like(l[0], float("-inf")))
    assert torch.equal(out, a[0]) and torch.equal(lse, a[1])
    # dtypes: bf16 block is promoted to fp32 on the first call
    out, lse = ring.merge(None, None, o[0].to(torch.bfloat16), l[0].to(torch.bfloat16))
    assert out.dtype == torch.float32 and lse.dtype == torch.bfloat16 and lse.shape[-1] == 1


def test_merge_slice_error_and_slice_path():
    o, l = rnd(1, 1, 4, 2, seed=50), rnd(1, 1, 4, seed=51)
    with pytest.raises(RuntimeError):
        ring.merge(None, None, o, l, slice_=(slice(None),))
    out, lse = ring.merge(None, None, o.clone(), l.clone())
    sl = (slice(None), slice(None), slice(0, 2))
    bo, bl = rnd(1, 1, 2, 2, seed=52), rnd(1, 1, 2, seed=53)
    out2, lse2 = ring.merge(out.clone(), lse.clone(), bo, bl, slice_=sl)
    ref_o, ref_l = ring.merge(out[sl], lse[sl], bo, bl)
    assert torch.allclose(out2[sl], ref_o) and torch.allclose(lse2[sl], ref_l)
    assert torch.equal(out2[:, :, 2:], out[:, :, 2:])


# ------------------------------------------------------------------ ring == full attention, every rank
@pytest.mark.parametrize("world", [1, 2, 3, 4, 8])
@pytest.mark.parametrize("causal", [True, False])
def test_every_rank_matches_full_attention(world, causal):
    B, H, Sc, D = 1, 2, 6, 4
    S = world * Sc
    q, k, v, do = (rnd(B, H, S, D, seed=60 + i) for i in range(4))
    scale = 1 / math.sqrt(D)
    full_o, full_lse = ring.full_attention_closed_form(q, k, v, scale, causal)
    ks, vs = k.chunk(world, 2), v.chunk(world, 2)
    for r in range(world):
        o_r, lse_r = ring.rank_forward(q[:, :, r * Sc:(r + 1) * Sc], ks, vs, r, scale, causal)
        assert torch.allclose(o_r, full_o[:, :, r * Sc:(r + 1) * Sc], atol=1e-12)
        assert torch.allclose(lse_r, full_lse[:, :, r * Sc:(r + 1) * Sc], atol=1e-12)
    o, lse = ring.all_ranks_forward(q, k, v, world, scale, causal)
    assert torch.allclose(o, full_o, atol=1e-12)

    qg, kg, vg = (t.clone().requires_grad_() for t in (q, k, v))
    ref_o, _ = ring.full_attention_closed_form(qg, kg, vg, scale, causal)
    gq, gk, gv = torch.autograd.grad(ref_o, (qg, kg, vg), do)
    dq, dk, dv = ring.all_ranks_backward(do, q, k, v, o, lse, world, scale, causal)
    for a, b in ((dq, gq), (dk, gk), (dv, gv)):
        assert torch.allclose(a, b, atol=1e-11)


def test_offset_causal_closed_form_equals_rank_ring():
    """One launch over K[0:(r+1)Sc] with the diagonal shifted by r*Sc is the rank's merged ring."""
    W, Sc, D = 4, 5, 4
    q, k, v = (rnd(1, 1, W * Sc, D, seed=70 + i) for i in range(3))
    for r in range(W):
        q_r = q[:, :, r * Sc:(r + 1) * Sc]
        o_r, lse_r = ring.rank_forward(q_r, k.chunk(W, 2), v.chunk(W, 2), r, 0.5, True)
        o2, lse2 = ring.full_attention_closed_form(q_r, k[:, :, :(r + 1) * Sc], v[:, :, :(r + 1) * Sc], 0.5, True,
                                                   q_offset=r * Sc)
        assert torch.allclose(o_r, o2, atol=1e-12) and torch.allclose(lse_r, lse2, atol=1e-12)
