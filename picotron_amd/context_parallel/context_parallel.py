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


def ring_attention(q, k, v, sm_scale, is_causal):
    return RingAttentionFunc.apply(q, k, v, sm_scale, is_causal)


def ring_schedule(world: int, rank: int, is_causal: bool):
    """[(step, rank whose chunk is held, block runs?, block masked?)]: the loop of ``context_parallel.py:30-45``."""
    return [(s, (rank - s) % world, (not is_causal) or s <= rank, bool(is_causal) and s == 0) for s in range(world)]


class _PublishKV(torch.autograd.Function):
    """Identity on a rank's (k, v) chunk that marks where the ring's dK / dV come back.  Every rank that reads the
    chunk takes the outputs of this node as autograd inputs, so the engine runs this node's backward only after all
    of them have run theirs -- in any order of ranks, and with whichever subset of the ranks' losses is being
    differentiated.  Their blocks were summed in fp32 in `box` (the reference's travelling accumulators,
    ``context_parallel.py:85-106``); here the total is rounded once to the chunk's dtype (:110)."""

    @staticmethod
    def forward(ctx, k, v, box):
        ctx.box = box
        ctx.set_materialize_grads(False)
        # layout only, no saved tensors: the node may run in several backward calls (one rank's loss at a time)
        ctx.layout = tuple((t.dtype, t.stride() if ops._dense(t) and t.stride(-1) == 1 else None) for t in (k, v))
        return k.view_as(k), v.view_as(v)

    @staticmethod
    def backward(ctx, gk, gv):
        box = ctx.box
        dk = dv = None
        if box.dk is not None:
            (k_dtype, k_strides), (v_dtype, v_strides) = ctx.layout
            dk = ops.convert_f32(box.dk, k_dtype, strides=k_strides)
            dv = ops.convert_f32(box.dv, v_dtype, strides=v_strides)
            box.dk = box.dv = None      # the next backward through this chunk starts a fresh sum
        if gk is not None:
            dk = gk if dk is None else dk + gk
        if gv is not None:
            dv = gv if dv is None else dv + gv
        return dk, dv, None


def publish_chunk(ring, slot, rank, k, v):
    """Puts rank `rank`'s chunk into the mailbox (once per pass) and returns it."""
    chunk = ring.publish_kv(slot, rank, k, v)
    if chunk.k is chunk.src_k and torch.is_grad_enabled() and (k.requires_grad or v.requires_grad):
        chunk.k, chunk.v = _PublishKV.apply(k, v, chunk.grads)
    return chunk


class RingAttentionFunc(torch.autograd.Function):
    """``RingAttentionFunc.apply(q, k, v, sm_scale, is_causal)`` as in ``context_parallel.py:17-110``.

    With virtual ranks the chunks of the other ranks are tensors of this process, so they enter the autograd node as
    extra inputs (``apply`` looks them up in the mailbox); the node adds its dK / dV blocks to each chunk's fp32
    accumulator and the chunks' own nodes (``_PublishKV``) return the sums."""

    @classmethod
    def apply(cls, q, k, v, sm_scale, is_causal):
        mgr = pgm.process_group_manager
        world, rank = mgr.cp_world_size, mgr.cp_rank
        if world == 1:
            return super().apply(q, k, v, sm_scale, is_causal)
        ring = mgr.cp_ring
        slot = ring.take_slot()
        own = publish_chunk(ring, slot, rank, k, v)
        chunks = {rank: own}
        for _, held, runs, _ in ring_schedule(world, rank, is_causal):
            if runs and held != rank:
                chunks[held] = ring.fetch(slot, held, rank)
        peers = [c for c in sorted(chunks) if c != rank]
        flat = [t for c in peers for t in (chunks[c].k, chunks[c].v)]
        return super().apply(q, own.k, own.v, sm_scale, is_causal, (slot, rank, world, chunks, peers), *flat)

    @staticmethod
    def forward(ctx, q, k, v, sm_scale, is_causal, plan=None, *peer_kv):
        B, H, Sq, D = q.shape
        ctx.sm_scale, ctx.is_causal, ctx.plan = sm_scale, is_causal, plan
        if plan is None:
            # one chunk: write the final dtype directly, in [B,S,H,D] memory so the caller's reshape is a view
            out, lse = ops.attn_fwd(q, k, v, sm_scale, is_causal, 0, out_dtype=q.dtype, bshd_out=True)
            ctx.save_for_backward(q, k, v, out, lse)
            return out
        slot, rank, world, chunks, _ = plan
        comm = ContextCommunicate("comm", rank=rank, slot=slot, chunks=chunks)
        out = lse = None
        next_k = next_v = None
        schedule = ring_schedule(world, rank, is_causal)
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
                ops.attn_fwd(q, k, v, sm_scale, masked, 0, out=out, lse=lse, merge=not first)
            if step + 1 != world:
                comm.wait(needed=schedule[step + 1][2])
                k, v = next_k, next_v
        out = ops.convert_f32(out, q.dtype, bshd=True)  # out.to(q.dtype) (:47), laid out [B,S,H,D]
        ctx.save_for_backward(q, out, lse)
        return out

    @staticmethod
    def backward(ctx, dout, *args):
        sm_scale, is_causal, plan = ctx.sm_scale, ctx.is_causal, ctx.plan
        if plan is None:
            q, k, v, out, softmax_lse = ctx.saved_tensors
            # delta = sum_d dout * out is computed inside the call (by the dQ kernel's prologue)
            dq, dk, dv = ops.attn_bwd(dout, q, k, v, softmax_lse, None, sm_scale, is_causal, 0, dq_dtype=q.dtype,
                                      dq_like=q, dkv_dtype=k.dtype, out=out,
                                      dkv_like=k if k.stride() == v.stride() else None)
            return dq, dk, dv, None, None, None

        q, out, softmax_lse = ctx.saved_tensors
        slot, rank, world, chunks, peers = plan
        delta = ops.attn_bwd_preprocess(dout, out)
        # which chunks want gradients: inputs 1, 2 are this rank's own (k, v), the peers follow `plan`
        wants = {rank: ctx.needs_input_grad[1] or ctx.needs_input_grad[2]}
        for i, c in enumerate(peers):
            wants[c] = ctx.needs_input_grad[6 + 2 * i] or ctx.needs_input_grad[7 + 2 * i]
        kv_comm = ContextCommunicate("kv_comm", rank=rank, slot=slot, chunks=chunks)
        k, v = chunks[rank].k.detach(), chunks[rank].v.detach()
        dq = None
        next_k = next_v = None
        schedule = ring_schedule(world, rank, is_causal)
        for step, held, runs, masked in schedule:
            if step + 1 != world:
                next_k = kv_comm.send_recv(k)
                next_v = kv_comm.send_recv(v)
                kv_comm.commit()
            if runs:
                # dq += block_dq (:85-93) and the chunk's travelling dk / dv += block_dk / block_dv, all inside the
                # kernels; the first block to reach an accumulator writes it instead of adding
                box = chunks[held].grads
                fresh = box.dk is None
                if wants[held] and fresh:
                    box.dk = torch.empty(k.shape, dtype=torch.float32, device=k.device)
                    box.dv = torch.empty(k.shape, dtype=torch.float32, device=k.device)
                first = dq is None
                if first:
                    dq = torch.empty(q.shape, dtype=torch.float32, device=q.device)
                ops.attn_bwd(dout, q, k, v, softmax_lse, delta, sm_scale, masked, 0, dq,
                             box.dk if wants[held] else None, box.dv if wants[held] else None,
                             dq_accumulate=not first, dkv_accumulate=not fresh, want_dq=ctx.needs_input_grad[0],
                             want_dkv=wants[held])
            if step + 1 != world:
                kv_comm.wait(needed=schedule[step + 1][2])
                k, v = next_k, next_v
        dq = ops.convert_f32(dq, q.dtype, like=q) if ctx.needs_input_grad[0] else None
        return (dq, None, None, None, None, None) + (None,) * (2 * len(peers))


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
    """Rows of the [S, D] tables that belong to the current cp rank: [rank * S/W, (rank + 1) * S/W)."""
    mgr = pgm.process_group_manager
    total = cos.size(0)
    assert total % mgr.cp_world_size == 0, (
        f"Input sequence length ({total}) must be divisible by cp_world_size ({mgr.cp_world_size})")
    per_rank = total // mgr.cp_world_size
    lo = mgr.cp_rank * per_rank
    return cos[lo:lo + per_rank], sin[lo:lo + per_rank]
