"""Ring attention on one MI355X: the API of ``picotron/context_parallel/context_parallel.py`` over HIP kernels.

Every function keeps the reference's name, arguments and return values:

* ``ring_attention_forward``  (:112-128) -> one launch of the MFMA forward kernel (no score matrix in HBM)
* ``ring_attention_backward`` (:130-155) -> delta pre-pass + one launch of the MFMA backward kernel
* ``update_out_and_lse``      (:157-187) -> the lse-merge kernel
* ``RingAttentionFunc``       (:17-110)  -> same ring schedule and fp32 accumulation; the per-step
  block + merge pair is ONE launch (the forward kernel continues its online softmax from the running
  out / lse), and dK/dV blocks are added into the travelling fp32 accumulators inside the kernel
* ``update_rope_for_context_parallel`` (:189-195) -> unchanged integer slicing

The cp ranks are virtual (one process plays them in turn); hops go through
``cp_communications.ContextCommunicate``'s in-process mailbox.  Causal attention: play the ranks in ascending
order.  Attention without a mask reads every rank's chunk, so all chunks are handed over first
(``cp_ring.stage_kv``); a model of several layers cannot be played rank after rank in that case (rank 0's
second layer would need rank 1's first), a single ring_attention call can.  Differences from the reference that a
caller can observe: lse is always fp32 (the reference keeps it in q.dtype), and block results of the
backward are fp32.
"""
from __future__ import annotations

import os
from typing import Any, Optional, Tuple

import torch

import picotron_amd.process_group_manager as pgm
from picotron_amd import ops
from picotron_amd.context_parallel.cp_communications import ContextCommunicate


def apply_context_parallel(model):
    os.environ["CONTEXT_PARALLEL"] = "1" if pgm.process_group_manager.cp_world_size > 1 else "0"
    return model


def ring_attention(q, k, v, sm_scale, is_causal, rope=None):
    """``ring_attention(q, k, v, sm_scale, is_causal)`` of ``context_parallel.py:14-15``.  With ``rope=(cos, sin)`` --
    tables indexed by ABSOLUTE position -- q and k arrive un-rotated and the call computes the ring attention of
    RoPE(q), RoPE(k) at the rank's positions (rank * Sc + row): q is rotated inside the attention forward, k by one
    launch before its chunk is published, and dq / dk come back un-rotated from the backward kernels' epilogues."""
    return RingAttentionFunc.apply(q, k, v, sm_scale, is_causal, rope=rope)


def ring_schedule(world: int, rank: int, is_causal: bool):
    """[(step, rank whose chunk is held, block runs?, block masked?)]: the loop of ``context_parallel.py:30-45``."""
    return [(s, (rank - s) % world, (not is_causal) or s <= rank, bool(is_causal) and s == 0) for s in range(world)]


def _per_step() -> bool:
    """PICO_RING_PER_STEP=1 runs the ring the way the reference does, one block launch per ring step with a hop between
    the steps, also where all chunks are at hand (default: one launch per rank and direction over the chunk list)."""
    return os.getenv("PICO_RING_PER_STEP", "0") == "1"


class _PublishKV(torch.autograd.Function):
    """Identity on a rank's (k, v) chunk that marks where the ring's dK / dV come back.  Every rank that reads the
    chunk takes the outputs of this node as autograd inputs, so the engine runs this node's backward only after all
    of them have run theirs -- in any order of ranks, and with whichever subset of the ranks' losses is being
    differentiated.  Their blocks were summed in fp32 in `box` (the reference's travelling accumulators,
    ``context_parallel.py:85-106``); here the total is rounded once to the chunk's dtype (:110).

    With `rope` = (cos, sin, first position) the node also rotates k (what the peers read is the rotated chunk); the
    sums in `box` are then gradients of the UN-rotated k already (the backward kernels rotate every block back before
    they add it), so nothing else happens on the way back."""

    @staticmethod
    def forward(ctx, k, v, box, rope=None):
        ctx.box = box
        ctx.rope = rope
        ctx.set_materialize_grads(False)
        # layout only, no saved tensors: the node may run in several backward calls (one rank's loss at a time)
        ctx.layout = tuple((t.dtype, t.stride() if ops._dense(t) and t.stride(-1) == 1 else None) for t in (k, v))
        box.layout = ctx.layout
        if rope is not None:
            cos, sin, pos0 = rope
            return ops.rope(k, cos, sin, pos_offset=pos0), v.view_as(v)
        return k.view_as(k), v.view_as(v)

    @staticmethod
    def backward(ctx, gk, gv):
        box = ctx.box
        dk = dv = None
        box.arrived = 0
        if box.final_dk is not None:
            # the last reader's kernel wrote the rounded totals itself
            dk, dv = box.final_dk, box.final_dv
            box.final_dk = box.final_dv = box.dk = box.dv = None
        elif box.dk is not None:
            (k_dtype, k_strides), (v_dtype, v_strides) = ctx.layout
            dk = ops.convert_f32(box.dk, k_dtype, strides=k_strides)
            dv = ops.convert_f32(box.dv, v_dtype, strides=v_strides)
            box.dk = box.dv = None      # the next backward through this chunk starts a fresh sum
        if gk is not None:
            if ctx.rope is not None:    # a gradient that reached the rotated chunk some other way
                cos, sin, pos0 = ctx.rope
                gk = ops.rope(gk, cos, sin, pos_offset=pos0, inverse=True)
            dk = gk if dk is None else dk + gk
        if gv is not None:
            dv = gv if dv is None else dv + gv
        return dk, dv, None, None


def publish_chunk(ring, slot, rank, k, v, rope=None):
    """Puts rank `rank`'s chunk into the mailbox (once per pass) and returns it."""
    chunk = ring.publish_kv(slot, rank, k, v)
    if chunk.k is chunk.src_k:
        if torch.is_grad_enabled() and (k.requires_grad or v.requires_grad):
            chunk.k, chunk.v = _PublishKV.apply(k, v, chunk.grads, rope)
        elif rope is not None:
            chunk.k = ops.rope(k, rope[0], rope[1], pos_offset=rope[2])
    return chunk


class RingAttentionFunc(torch.autograd.Function):
    """``RingAttentionFunc.apply(q, k, v, sm_scale, is_causal)`` as in ``context_parallel.py:17-110``.

    With virtual ranks the chunks of the other ranks are tensors of this process, so they enter the autograd node as
    extra inputs (``apply`` looks them up in the mailbox); the node adds its dK / dV blocks to each chunk's fp32
    accumulator and the chunks' own nodes (``_PublishKV``) return the sums.

    All chunks a rank will read are at hand when its turn comes, so by default the loop over the ring steps
    (:30-45, :63-106) runs INSIDE one launch per direction: the kernels take the list of chunk tensors as it is (no
    concatenation, no hop copies), carry the online softmax across the chunks, write the output in q's dtype and add
    each chunk's dK / dV block to that chunk's accumulator.  Chunks that do not fit one launch (see
    ``ops.chunks_fit_one_launch``), or ``PICO_RING_PER_STEP=1``, take the reference's shape: one launch per ring step
    with the hop between steps."""

    @classmethod
    def apply(cls, q, k, v, sm_scale, is_causal, rope=None):
        mgr = pgm.process_group_manager
        world, rank = mgr.cp_world_size, mgr.cp_rank
        Sc = q.size(2)
        table = None if rope is None else (rope[0], rope[1], rank * Sc)
        if world == 1:
            return super().apply(q, k, v, sm_scale, is_causal, None, table)
        ring = mgr.cp_ring
        slot = ring.take_slot()
        own = publish_chunk(ring, slot, rank, k, v, table)
        chunks = {rank: own}
        for _, held, runs, _ in ring_schedule(world, rank, is_causal):
            if runs and held != rank:
                chunks[held] = ring.fetch(slot, held, rank)
        peers = [c for c in sorted(chunks) if c != rank]
        flat = [t for c in peers for t in (chunks[c].k, chunks[c].v)]
        if torch.is_grad_enabled():
            for c in chunks.values():
                if c.k.requires_grad or c.v.requires_grad:
                    c.grads.readers += 1
        return super().apply(q, own.k, own.v, sm_scale, is_causal, (slot, rank, world, chunks, peers), table, *flat)

    @staticmethod
    def forward(ctx, q, k, v, sm_scale, is_causal, plan=None, rope=None, *peer_kv):
        B, H, Sq, D = q.shape
        ctx.sm_scale, ctx.is_causal, ctx.plan, ctx.rope, ctx.one_launch = sm_scale, is_causal, plan, rope, None
        if plan is None:
            # one chunk: write the final dtype directly, in [B,S,H,D] memory so the caller's reshape is a view
            if rope is not None:
                cos, sin, pos0 = rope
                k = ops.rope(k, cos, sin, pos_offset=pos0)
                out, lse, q = ops.attn_fwd_rope(q, k, v, cos, sin, sm_scale, is_causal, 0, pos0, out_dtype=q.dtype)
            else:
                out, lse = ops.attn_fwd(q, k, v, sm_scale, is_causal, 0, out_dtype=q.dtype, bshd_out=True)
            ctx.save_for_backward(q, k, v, out, lse)
            return out
        slot, rank, world, chunks, _ = plan
        cs = (rope[0], rope[1]) if rope is not None else None
        q_pos = rope[2] if rope is not None else 0
        schedule = ring_schedule(world, rank, is_causal)
        # the chunks this rank reads, in the order of their positions (the ring delivers them in descending order)
        order = sorted(held for _, held, runs, _ in schedule if runs)
        ks = [k if c == rank else chunks[c].k.detach() for c in order]
        vs = [v if c == rank else chunks[c].v.detach() for c in order]
        contiguous_positions = order == list(range(order[0], order[0] + len(order))) and (not is_causal or order[-1] == rank)
        if not _per_step() and contiguous_positions and ops.chunks_fit_one_launch(ks, vs):
            q_off = (rank - order[0]) * Sq if is_causal else 0
            out, lse, q_rot = ops.attn_fwd_chunks(q, ks, vs, sm_scale, is_causal, q_off, out_dtype=q.dtype, bshd_out=True,
                                                  rope=cs, q_pos_offset=q_pos, want_q_rot=rope is not None, checked=True)
            ctx.one_launch = (order, q_off)
            ctx.save_for_backward(q_rot if rope is not None else q, out, lse)
            return out
        comm = ContextCommunicate("comm", rank=rank, slot=slot, chunks=chunks)
        out = lse = q_rot = None
        next_k = next_v = None
        for step, _, runs, masked in schedule:
            if step + 1 != world:
                next_k = comm.send_recv(k)
                next_v = comm.send_recv(v)
                comm.commit()
            if runs:
                # block forward fused with update_out_and_lse (:37-40)
                first = out is None
                if first:
                    out = torch.empty(B, H, Sq, D, dtype=torch.float32, device=q.device)
                    lse = torch.empty(B, H, Sq, dtype=torch.float32, device=q.device)
                if rope is not None and first:
                    # q is rotated in the first block's prologue; the later blocks read the rotated copy it leaves
                    _, _, q_rot = ops.attn_fwd_rope(q, k, v, cs[0], cs[1], sm_scale, masked, 0, q_pos, out=out, lse=lse)
                else:
                    ops.attn_fwd(q_rot if rope is not None else q, k, v, sm_scale, masked, 0, out=out, lse=lse, merge=not first)
            if step + 1 != world:
                comm.wait(needed=schedule[step + 1][2])
                k, v = next_k, next_v
        out = ops.convert_f32(out, q.dtype, bshd=True)  # out.to(q.dtype) (:47), laid out [B,S,H,D]
        ctx.save_for_backward(q_rot if rope is not None else q, out, lse)
        return out

    @staticmethod
    def backward(ctx, dout, *args):
        sm_scale, is_causal, plan, rope = ctx.sm_scale, ctx.is_causal, ctx.plan, ctx.rope
        cs = (rope[0], rope[1]) if rope is not None else None
        q_pos = rope[2] if rope is not None else 0
        if plan is None:
            q, k, v, out, softmax_lse = ctx.saved_tensors
            # delta = sum_d dout * out is computed inside the call (by the dQ kernel's prologue)
            if rope is not None:
                dq = torch.empty_strided(q.shape, q.stride(), dtype=q.dtype, device=q.device)
                dk = torch.empty_strided(k.shape, k.stride(), dtype=k.dtype, device=k.device)
                dv = torch.empty_strided(k.shape, k.stride(), dtype=k.dtype, device=k.device)
                ops.attn_bwd_rope(dout, q, k, v, out, softmax_lse, cs[0], cs[1], sm_scale, is_causal, dq, dk, dv, 0, q_pos, q_pos)
                return dq, dk, dv, None, None, None, None
            dq, dk, dv = ops.attn_bwd(dout, q, k, v, softmax_lse, None, sm_scale, is_causal, 0, dq_dtype=q.dtype,
                                      dq_like=q, dkv_dtype=k.dtype, out=out,
                                      dkv_like=k if k.stride() == v.stride() else None)
            return dq, dk, dv, None, None, None, None

        q, out, softmax_lse = ctx.saved_tensors      # (q is the rotated copy when rope is given)
        slot, rank, world, chunks, peers = plan
        # which chunks want gradients: inputs 1, 2 are this rank's own (k, v), the peers follow `plan`
        wants = {rank: ctx.needs_input_grad[1] or ctx.needs_input_grad[2]}
        for i, c in enumerate(peers):
            wants[c] = ctx.needs_input_grad[7 + 2 * i] or ctx.needs_input_grad[8 + 2 * i]
        nothing = (None,) * (7 + 2 * len(peers))

        def boxes(c):
            """(dk, dv, add?) of chunk c's travelling accumulators; the first block to reach them writes."""
            box = chunks[c].grads
            fresh = box.dk is None
            if fresh:
                shape = chunks[c].k.shape
                box.dk = torch.empty(shape, dtype=torch.float32, device=q.device)
                box.dv = torch.empty(shape, dtype=torch.float32, device=q.device)
            return box.dk, box.dv, not fresh

        def finals(c):
            """bf16 buffers for chunk c's totals if this rank's block is the last one they wait for (every rank that
            read the chunk has added its block), in the chunk's own layout; else None."""
            box = chunks[c].grads
            box.arrived += 1
            (k_dtype, k_strides), (v_dtype, v_strides) = box.layout if box.layout is not None else ((None, None), (None, None))
            if box.arrived != box.readers or k_dtype not in ops.FINAL_TOTAL_DTYPES or v_dtype != k_dtype:
                return None
            shape = chunks[c].k.shape
            if k_strides is not None and k_strides == v_strides:
                box.final_dk = torch.empty_strided(shape, k_strides, dtype=k_dtype, device=q.device)
                box.final_dv = torch.empty_strided(shape, k_strides, dtype=k_dtype, device=q.device)
            else:   # chunks that are views with gaps (or k and v laid out differently): contiguous gradients
                box.final_dk = torch.empty(shape, dtype=k_dtype, device=q.device)
                box.final_dv = torch.empty(shape, dtype=k_dtype, device=q.device)
            return box.final_dk, box.final_dv

        if ctx.one_launch is not None:
            order, q_off = ctx.one_launch
            ks = [chunks[c].k.detach() for c in order]
            vs = [chunks[c].v.detach() for c in order]
            fin = {c: finals(c) if wants[c] else None for c in order}
            # a chunk whose totals leave from this launch needs fp32 sums only if earlier blocks left some
            got = [(None, None, False) if not wants[c] else
                   ((chunks[c].grads.dk, chunks[c].grads.dv, chunks[c].grads.dk is not None) if fin[c] is not None else boxes(c))
                   for c in order]
            dq = None
            if ctx.needs_input_grad[0]:
                dq = (torch.empty_strided(q.shape, q.stride(), dtype=q.dtype, device=q.device)
                      if ops._dense(q) and q.stride(-1) == 1 else torch.empty(q.shape, dtype=q.dtype, device=q.device))
            ops.attn_bwd_chunks(dout, q, ks, vs, softmax_lse, sm_scale, is_causal, q_off, dq, [g[0] for g in got],
                                [g[1] for g in got], dkv_accumulate=[g[2] for g in got], out=out, rope=cs,
                                q_pos_offset=q_pos, k_pos_offset=q_pos - q_off if is_causal else 0,
                                dk_finals=[fin[c][0] if fin[c] is not None else None for c in order],
                                dv_finals=[fin[c][1] if fin[c] is not None else None for c in order],
                                checked=True)   # (the forward asked chunks_fit_one_launch about these same tensors)
            return (dq,) + nothing[1:]

        delta = ops.attn_bwd_preprocess(dout, out)
        kv_comm = ContextCommunicate("kv_comm", rank=rank, slot=slot, chunks=chunks)
        k, v = chunks[rank].k.detach(), chunks[rank].v.detach()
        dq = None
        next_k = next_v = None
        schedule = ring_schedule(world, rank, is_causal)
        Sc = q.size(2)
        for step, held, runs, masked in schedule:
            if step + 1 != world:
                next_k = kv_comm.send_recv(k)
                next_v = kv_comm.send_recv(v)
                kv_comm.commit()
            if runs and (wants[held] or ctx.needs_input_grad[0]):
                # dq += block_dq (:85-93) and the chunk's travelling dk / dv += block_dk / block_dv, all inside the
                # kernels; the first block to reach an accumulator writes it instead of adding
                dk_c, dv_c, add = boxes(held) if wants[held] else (None, None, False)
                first = dq is None
                if first:
                    dq = torch.empty(q.shape, dtype=torch.float32, device=q.device)
                ops.attn_bwd_chunks(dout, q, [k], [v], softmax_lse, sm_scale, masked, 0, dq if ctx.needs_input_grad[0] else None,
                                    [dk_c], [dv_c], dq_accumulate=not first, dkv_accumulate=[add], delta=delta, rope=cs,
                                    q_pos_offset=q_pos, k_pos_offset=q_pos + (held - rank) * Sc)
            if step + 1 != world:
                kv_comm.wait(needed=schedule[step + 1][2])
                k, v = next_k, next_v
        dq = ops.convert_f32(dq, q.dtype, like=q) if ctx.needs_input_grad[0] and dq is not None else None
        return (dq,) + nothing[1:]


def ring_attention_forward(q, k, v, sm_scale, is_causal):
    """One attention block; returns (O [B,H,Sq,D] in q.dtype, lse [B,H,Sq] fp32)."""
    return ops.attn_fwd(q, k, v, sm_scale, is_causal, 0, out_dtype=q.dtype)


def ring_attention_backward(dO, Q, K, V, O, softmax_lse, sm_scale, is_causal):
    """Gradients of one block given the final (merged) O and lse; returns fp32 (dQ, dK, dV)."""
    delta = ops.attn_bwd_preprocess(dO, O)
    lse = softmax_lse if softmax_lse.dtype == torch.float32 else softmax_lse.float()
    return ops.attn_bwd(dO, Q, K, V, lse, delta, sm_scale, is_causal, 0)


def update_out_and_lse(
    out: Optional[torch.Tensor],
    lse: Optional[torch.Tensor],
    block_out: torch.Tensor,
    block_lse: torch.Tensor,
    slice_: Optional[Any] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Merges a block into the running (out fp32 [B,H,S,D], lse [B,H,S,1]); the first call adopts the block."""
    if out is None:
        if slice_ is not None:
            raise RuntimeError("first update_out_and_lse should not pass slice_ args")
        return block_out.to(torch.float32), block_lse.unsqueeze(dim=-1).to(torch.float32)
    if slice_ is not None:
        o_s, l_s = out[slice_].contiguous(), lse[slice_].squeeze(-1).contiguous()
        ops.lse_merge_(o_s, l_s, block_out, block_lse.to(torch.float32))
        out[slice_], lse[slice_] = o_s, l_s.unsqueeze(-1)
        return out, lse
    out = out if out.is_contiguous() else out.contiguous()
    l_flat = lse.squeeze(-1)
    l_flat = l_flat if l_flat.is_contiguous() else l_flat.contiguous()
    ops.lse_merge_(out, l_flat, block_out, block_lse.to(torch.float32))
    return out, l_flat.unsqueeze(-1)


def update_rope_for_context_parallel(cos, sin):
    """Rows of the [S, D] tables that belong to the current cp rank: [rank * S/W, (rank + 1) * S/W).

    The returned slices remember the whole table they were cut from (attribute ``whole_table`` = (table, first row)):
    kernels that rotate at absolute positions -- RoPE inside the ring, where a rank also un-rotates the gradients of
    other ranks' keys -- are given the whole table and an offset instead of the slice."""
    mgr = pgm.process_group_manager
    total = cos.size(0)
    assert total % mgr.cp_world_size == 0, (
        f"Input sequence length ({total}) must be divisible by cp_world_size ({mgr.cp_world_size})")
    per_rank = total // mgr.cp_world_size
    lo = mgr.cp_rank * per_rank
    out = []
    for table in (cos, sin):
        piece = table[lo:lo + per_rank]
        piece.whole_table = (table, lo)
        out.append(piece)
    return out[0], out[1]
