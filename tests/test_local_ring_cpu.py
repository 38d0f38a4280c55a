"""Host logic of the virtual-rank ring (RingAttentionFunc, LocalRing, ContextCommunicate) on the CPU.

The kernel wrappers the ring calls are replaced by fp32 torch stand-ins (block maths written out below), so that
what is under test is the schedule, the mailbox and the accumulation of dK / dV across ranks -- checked against
full-sequence attention differentiated by autograd, which knows nothing of chunks or rings.  The GPU tests run the
same scenarios on the HIP kernels.
"""
import math

import pytest
import torch

from oracle import ring as OR


def _expand(q, k, v):
    rep = q.size(1) // k.size(1)
    return q.float(), k.float().repeat_interleave(rep, 1), v.float().repeat_interleave(rep, 1), rep


def _fold(g, rep):
    B, H, S, D = g.shape
    return g.view(B, H // rep, rep, S, D).sum(2)


def fake_attn_fwd(q, k, v, sm_scale, causal, q_offset=0, out=None, lse=None, merge=False, out_dtype=torch.bfloat16,
                  bshd_out=False):
    assert q_offset == 0
    qf, kf, vf, _ = _expand(q, k, v)
    bo, bl = OR.block_forward(qf, kf, vf, sm_scale, causal)
    if merge:
        o, l = OR.merge(out, lse.unsqueeze(-1), bo, bl)
        out.copy_(o)
        lse.copy_(l.squeeze(-1))
    elif out is None:
        out, lse = bo.to(out_dtype), bl
    else:
        out.copy_(bo)
        lse.copy_(bl)
    return out, lse


def fake_attn_bwd_preprocess(dout, out, dq_acc=None, delta=None):
    return (dout.float() * out.float()).sum(-1)


def fake_attn_bwd(dout, q, k, v, lse, delta, sm_scale, causal, q_offset=0, dq=None, dk=None, dv=None,
                  dq_accumulate=False, dkv_accumulate=False, dq_dtype=torch.float32, dkv_dtype=torch.float32,
                  dq_like=None, want_dq=True, want_dkv=True, side_stream=None, out=None, dkv_like=None):
    qf, kf, vf, rep = _expand(q, k, v)
    do = dout.float()
    if delta is None:
        delta = (do * out.float()).sum(-1)
    s = qf @ kf.transpose(-1, -2) * sm_scale
    if causal:
        s = s.masked_fill(OR.causal_mask(q.size(2)), float("-inf"))
    p = torch.exp(s - lse.unsqueeze(-1))
    b_dv = _fold(p.transpose(-1, -2) @ do, rep)
    ds = p * (do @ vf.transpose(-1, -2) - delta.unsqueeze(-1))
    b_dq = ds @ kf * sm_scale
    b_dk = _fold(ds.transpose(-1, -2) @ qf * sm_scale, rep)

    def put(buf, val, acc, dtype):
        if buf is None:
            return val.to(dtype)
        if acc:
            buf.add_(val)
        else:
            buf.copy_(val)
        return buf

    dq = put(dq, b_dq, dq_accumulate, dq_dtype) if want_dq else None
    dk = put(dk, b_dk, dkv_accumulate, dkv_dtype) if want_dkv else None
    dv = put(dv, b_dv, dkv_accumulate, dkv_dtype) if want_dkv else None
    return dq, dk, dv


def fake_convert_f32(src, dtype, like=None, bshd=False, strides=None):
    return src.to(dtype)


def _full_scores(q, k_all, sm_scale, causal, q_offset):
    s = q @ k_all.transpose(-1, -2) * sm_scale
    if causal:
        qi = torch.arange(q.size(2)).unsqueeze(1) + q_offset
        kj = torch.arange(k_all.size(2)).unsqueeze(0)
        s = s.masked_fill(kj > qi, float("-inf"))
    return s


def fake_attn_fwd_chunks(q, ks, vs, sm_scale, causal, q_offset=0, out=None, lse=None, merge=False, out_dtype=torch.bfloat16,
                         bshd_out=False, rope=None, q_pos_offset=0, want_q_rot=False, checked=False):
    """All listed chunks in one go: softmax over their concatenation, query i at position q_offset + i."""
    assert rope is None and not merge
    qf, kf, vf, _ = _expand(q, torch.cat(ks, 2), torch.cat(vs, 2))
    s = _full_scores(qf, kf, sm_scale, causal, q_offset)
    return (torch.softmax(s, -1) @ vf).to(out_dtype), torch.logsumexp(s, -1), None


def fake_attn_bwd_chunks(dout, q, ks, vs, lse, sm_scale, causal, q_offset=0, dq=None, dks=None, dvs=None, dq_accumulate=False,
                         dkv_accumulate=None, out=None, delta=None, rope=None, q_pos_offset=0, k_pos_offset=0,
                         dk_finals=None, dv_finals=None, checked=False):
    assert rope is None
    Sc = ks[0].size(2)
    qf, kf, vf, rep = _expand(q, torch.cat(ks, 2), torch.cat(vs, 2))
    do = dout.float()
    if delta is None:
        delta = (do * out.float()).sum(-1)
    p = torch.exp(_full_scores(qf, kf, sm_scale, causal, q_offset) - lse.unsqueeze(-1))
    ds = p * (do @ vf.transpose(-1, -2) - delta.unsqueeze(-1))
    b_dv = _fold(p.transpose(-1, -2) @ do, rep)
    b_dk = _fold(ds.transpose(-1, -2) @ qf * sm_scale, rep)
    if dq is not None:
        b_dq = ds @ kf * sm_scale
        dq.add_(b_dq) if dq_accumulate else dq.copy_(b_dq)
    for c in range(len(ks)):
        sl = slice(c * Sc, (c + 1) * Sc)
        if dk_finals is not None and dk_finals[c] is not None:
            # the block that completes the chunk's sums: total = sums so far (if any) + this block, cast once
            add = dkv_accumulate is not None and dkv_accumulate[c]
            dk_finals[c].copy_(b_dk[:, :, sl] + (dks[c] if add else 0))
            dv_finals[c].copy_(b_dv[:, :, sl] + (dvs[c] if add else 0))
            continue
        if dks is None or dks[c] is None:
            continue
        if dkv_accumulate is not None and dkv_accumulate[c]:
            dks[c].add_(b_dk[:, :, sl])
            dvs[c].add_(b_dv[:, :, sl])
        else:
            dks[c].copy_(b_dk[:, :, sl])
            dvs[c].copy_(b_dv[:, :, sl])
    return delta


@pytest.fixture(params=["one_launch_per_rank", "one_launch_per_ring_step"])
def ring(monkeypatch, request):
    """Both shapes of the ring: all steps of a rank in one call over the chunk list (the default when the chunks fit
    one launch; the stand-in says they do) and the reference's one call per ring step with hops between."""
    import picotron_amd.process_group_manager as pgm
    from picotron_amd import ops
    from picotron_amd.context_parallel import context_parallel as cp
    monkeypatch.setattr(ops, "attn_fwd", fake_attn_fwd)
    monkeypatch.setattr(ops, "attn_bwd", fake_attn_bwd)
    monkeypatch.setattr(ops, "attn_bwd_preprocess", fake_attn_bwd_preprocess)
    monkeypatch.setattr(ops, "convert_f32", fake_convert_f32)
    monkeypatch.setattr(ops, "attn_fwd_chunks", fake_attn_fwd_chunks)
    monkeypatch.setattr(ops, "attn_bwd_chunks", fake_attn_bwd_chunks)
    monkeypatch.setattr(ops, "chunks_fit_one_launch", lambda ks, vs: request.param == "one_launch_per_rank")
    monkeypatch.setattr(ops, "FINAL_TOTAL_DTYPES", (torch.bfloat16, torch.float32))   # the stand-in handles fp32 as well
    yield pgm, cp
    pgm.setup_process_group_manager(1, 1, 1, 1)


def _inputs(W, seed, B=1, H=4, Hkv=2, Sc=16, D=8):
    g = torch.Generator().manual_seed(seed)
    S = W * Sc
    q, k, v, do = (torch.randn(B, h, S, D, generator=g) for h in (H, Hkv, Hkv, H))
    return q, k, v, do


def _want(q, k, v, do, causal):
    qf, kf, vf = (t.clone().requires_grad_() for t in (q, k, v))
    rep = q.size(1) // k.size(1)
    o, _ = OR.full_attention_closed_form(qf, kf.repeat_interleave(rep, 1), vf.repeat_interleave(rep, 1),
                                         1 / math.sqrt(q.size(-1)), causal)
    return (o.detach(),) + torch.autograd.grad(o, (qf, kf, vf), do)


def _play(mgr, cp, q, k, v, causal, W, order=None, stage=False):
    Sc = q.size(2) // W
    ks = [k[:, :, r * Sc:(r + 1) * Sc] for r in range(W)]
    vs = [v[:, :, r * Sc:(r + 1) * Sc] for r in range(W)]
    if stage:
        for r in range(W):
            mgr.cp_ring.stage_kv(r, ks[r], vs[r])
    outs = {}
    for r in (order or range(W)):
        mgr.set_cp_rank(r)
        outs[r] = cp.ring_attention(q[:, :, r * Sc:(r + 1) * Sc], ks[r], vs[r], 1 / math.sqrt(q.size(-1)), causal)
    return [outs[r] for r in range(W)]


def close(a, b, tol=1e-5):
    return ((a.double() - b.double()).norm() / b.double().norm()).item() <= tol


def test_two_passes_on_one_manager_both_match(ring):
    """A second forward + backward on the same manager (next micro-batch / optimiser step) must not see anything of
    the first: no stale K / V, no gradient left in an accumulator."""
    pgm, cp = ring
    W = 4
    mgr = pgm.setup_process_group_manager(1, W, 1, 1)
    for seed in (1, 2, 3):
        q, k, v, do = _inputs(W, seed)
        qd, kd, vd = (t.clone().requires_grad_() for t in (q, k, v))
        out = torch.cat(_play(mgr, cp, qd, kd, vd, True, W), dim=2)
        (out * do).sum().backward()
        w_o, w_q, w_k, w_v = _want(q, k, v, do, True)
        assert close(out, w_o) and close(qd.grad, w_q) and close(kd.grad, w_k) and close(vd.grad, w_v), seed
    assert all(c.grads.dk is None for c in mgr.cp_ring.chunks.values())     # accumulators were handed back and freed


@pytest.mark.parametrize("W", [2, 4])
def test_non_causal_ring_forward_and_backward(ring, W):
    """Without a mask every rank reads every chunk (``context_parallel.py:36,78``): stage all chunks, play the ranks
    in any order."""
    pgm, cp = ring
    mgr = pgm.setup_process_group_manager(1, W, 1, 1)
    q, k, v, do = _inputs(W, 7)
    for order in (list(range(W)), list(reversed(range(W)))):
        qd, kd, vd = (t.clone().requires_grad_() for t in (q, k, v))
        out = torch.cat(_play(mgr, cp, qd, kd, vd, False, W, order=order, stage=True), dim=2)
        (out * do).sum().backward()
        w_o, w_q, w_k, w_v = _want(q, k, v, do, False)
        assert close(out, w_o) and close(qd.grad, w_q) and close(kd.grad, w_k) and close(vd.grad, w_v)


def test_last_reader_hands_back_the_totals_itself(ring, monkeypatch):
    """One launch per rank: the rank whose block completes a chunk's dK / dV (every rank that read the chunk has added
    its block) writes the rounded totals in the same call, so a whole backward needs no cast pass at all; when the
    ranks' losses are differentiated one at a time no block is ever the last of its pass, and the chunks' own nodes
    cast the sums they hold."""
    pgm, cp = ring
    from picotron_amd import ops
    if not ops.chunks_fit_one_launch(None, None):
        pytest.skip("the per-step ring keeps the reference's shape: fp32 sums, cast at the end")
    casts = {"n": 0}
    real = ops.convert_f32
    monkeypatch.setattr(ops, "convert_f32", lambda *a, **k: (casts.__setitem__("n", casts["n"] + 1), real(*a, **k))[1])
    W = 4
    mgr = pgm.setup_process_group_manager(1, W, 1, 1)
    q, k, v, do = _inputs(W, 21)
    Sc = q.size(2) // W
    w_o, w_q, w_k, w_v = _want(q, k, v, do, True)
    qd, kd, vd = (t.clone().requires_grad_() for t in (q, k, v))
    out = torch.cat(_play(mgr, cp, qd, kd, vd, True, W), dim=2)
    (out * do).sum().backward()
    assert casts["n"] == 0
    assert close(qd.grad, w_q) and close(kd.grad, w_k) and close(vd.grad, w_v)
    qd, kd, vd = (t.clone().requires_grad_() for t in (q, k, v))
    outs = _play(mgr, cp, qd, kd, vd, True, W)
    for r in (2, 0, 3, 1):
        (outs[r] * do[:, :, r * Sc:(r + 1) * Sc]).sum().backward()
    assert casts["n"] > 0
    assert close(qd.grad, w_q) and close(kd.grad, w_k) and close(vd.grad, w_v)


def test_missing_chunk_raises_instead_of_delivering_zeros(ring):
    pgm, cp = ring
    mgr = pgm.setup_process_group_manager(1, 2, 1, 1)
    q, k, v, _ = _inputs(2, 5)
    with pytest.raises(RuntimeError, match="has not been published"):
        _play(mgr, cp, q, k, v, False, 2)                   # non-causal, nothing staged: rank 0 needs rank 1's chunk
    mgr.cp_ring.reset()
    with pytest.raises(RuntimeError, match="has not been published"):
        _play(mgr, cp, q, k, v, True, 2, order=[1, 0])      # causal, descending: rank 1 needs rank 0's chunk


def test_stale_chunk_of_an_earlier_pass_is_never_delivered(ring):
    """Pass 1 plays both ranks; pass 2 plays rank 1 only after rank 0 published new K / V -- and if rank 0 has not
    played yet in pass 2, rank 1 must be refused rather than fed pass 1's chunk."""
    pgm, cp = ring
    mgr = pgm.setup_process_group_manager(1, 2, 1, 1)
    q, k, v, _ = _inputs(2, 5)
    _play(mgr, cp, q, k, v, True, 2)
    q2, k2, v2, _ = _inputs(2, 6)
    # rank 1 starts pass 2: its publish drops pass 1's chunks, so rank 0's old chunk cannot be read
    with pytest.raises(RuntimeError, match="has not been published"):
        _play(mgr, cp, q2, k2, v2, True, 2, order=[1])


def test_backward_one_rank_at_a_time_in_any_order(ring):
    """Each rank's loss differentiated by its own backward call: the chunks' nodes run once per call and hand back
    that call's share, so the leaves end with the same sums."""
    pgm, cp = ring
    W = 4
    mgr = pgm.setup_process_group_manager(1, W, 1, 1)
    q, k, v, do = _inputs(W, 9)
    Sc = q.size(2) // W
    w_o, w_q, w_k, w_v = _want(q, k, v, do, True)
    for order in ([0, 1, 2, 3], [3, 2, 1, 0], [2, 0, 3, 1]):
        qd, kd, vd = (t.clone().requires_grad_() for t in (q, k, v))
        outs = _play(mgr, cp, qd, kd, vd, True, W)
        for r in order:
            (outs[r] * do[:, :, r * Sc:(r + 1) * Sc]).sum().backward()
        assert close(qd.grad, w_q) and close(kd.grad, w_k) and close(vd.grad, w_v), order


def test_forward_then_backward_rank_by_rank(ring):
    """rank 0 forward + backward, then rank 1 forward + backward, ...: a later rank's backward still reaches the
    earlier ranks' chunks."""
    pgm, cp = ring
    W = 3
    mgr = pgm.setup_process_group_manager(1, W, 1, 1)
    q, k, v, do = _inputs(W, 11)
    Sc = q.size(2) // W
    qd, kd, vd = (t.clone().requires_grad_() for t in (q, k, v))
    scale = 1 / math.sqrt(q.size(-1))
    for r in range(W):
        mgr.set_cp_rank(r)
        sl = slice(r * Sc, (r + 1) * Sc)
        o = cp.ring_attention(qd[:, :, sl], kd[:, :, sl], vd[:, :, sl], scale, True)
        (o * do[:, :, sl]).sum().backward()
    _, w_q, w_k, w_v = _want(q, k, v, do, True)
    assert close(qd.grad, w_q) and close(kd.grad, w_k) and close(vd.grad, w_v)


def test_no_grad_forward_and_frozen_kv(ring):
    pgm, cp = ring
    W = 2
    mgr = pgm.setup_process_group_manager(1, W, 1, 1)
    q, k, v, do = _inputs(W, 13)
    w_o, w_q, _, _ = _want(q, k, v, do, True)
    with torch.no_grad():
        out = torch.cat(_play(mgr, cp, q, k, v, True, W), dim=2)
    assert close(out, w_o)
    qd = q.clone().requires_grad_()
    out = torch.cat(_play(mgr, cp, qd, k, v, True, W), dim=2)      # K / V do not require gradients
    (out * do).sum().backward()
    assert close(qd.grad, w_q)


def test_context_communicate_protocol(ring):
    """The K / V hop itself: at ring step s rank r receives the chunk of rank (r - s - 1) mod W."""
    pgm, cp = ring
    from picotron_amd.context_parallel.cp_communications import ContextCommunicate
    W = 4
    mgr = pgm.setup_process_group_manager(1, W, 1, 1)
    for r in range(W):
        mgr.cp_ring.publish_kv(0, r, torch.full((2,), 10.0 + r), torch.full((2,), 20.0 + r))
    c = ContextCommunicate("comm", rank=2, slot=0)
    assert (c.rank, c.world_size, c.send_rank, c.recv_rank) == (2, 4, 3, 1)
    with pytest.raises(RuntimeError, match="Wait called before commit"):
        c.wait()
    for s in range(W - 1):
        gk = c.send_recv(torch.zeros(2))
        gv = c.send_recv(torch.zeros(2))
        c.commit()
        if s == 0:
            with pytest.raises(RuntimeError, match="Commit called twice"):
                c.commit()
        c.wait()
        src = (2 - s - 1) % W
        assert torch.equal(gk, torch.full((2,), 10.0 + src)) and torch.equal(gv, torch.full((2,), 20.0 + src))
    # a chunk that is absent: refused when needed, NaN when the caller says it will not read it
    mgr.cp_ring.reset()
    c = ContextCommunicate("comm", rank=0, slot=0)
    got = c.send_recv(torch.zeros(2))
    c.commit()
    with pytest.raises(RuntimeError, match="has not been published"):
        c.wait()
    c.wait(needed=False)
    assert torch.isnan(got).all()
