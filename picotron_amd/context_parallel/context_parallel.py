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
``cp_communications.ContextCommunicate``'s in-process mailbox.  Differences from the reference that a
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


class RingAttentionFunc(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, sm_scale, is_causal):
        mgr = pgm.process_group_manager
        comm = ContextCommunicate("comm")
        world, rank = comm.world_size, comm.rank
        slot = mgr.cp_ring.take_slot()
        comm.bind_slot(slot)
        k_og, v_og = k, v  # never written to, so no clone is needed to keep them for the backward
        if world > 1:
            mgr.cp_ring.publish_kv(slot, rank, k_og, v_og)

        B, H, Sq, D = q.shape
        if world == 1:
            # one chunk: write the final dtype directly, in [B,S,H,D] memory so the caller's reshape is a view
            out, lse = ops.attn_fwd(q, k, v, sm_scale, is_causal, 0, out_dtype=q.dtype, bshd_out=True)
        else:
            out = lse = None
            next_k = next_v = None
            for step in range(world):
                if step + 1 != world:
                    next_k = comm.send_recv(k)
                    next_v = comm.send_recv(v)
                    comm.commit()
                if not is_causal or step <= rank:
                    # block forward fused with update_out_and_lse (:37-40)
                    first = out is None
                    if first:
                        out = torch.empty(B, H, Sq, D, dtype=torch.float32, device=q.device)
                        lse = torch.empty(B, H, Sq, dtype=torch.float32, device=q.device)
                    ops.attn_fwd(q, k, v, sm_scale, is_causal and step == 0, 0, out=out, lse=lse, merge=not first)
                if step + 1 != world:
                    comm.wait()
                    k, v = next_k, next_v
            out = ops.convert_f32(out, q.dtype, bshd=True)  # out.to(q.dtype) (:47), laid out [B,S,H,D]
        ctx.save_for_backward(q, k_og, v_og, out, lse)
        ctx.sm_scale = sm_scale
        ctx.is_causal = is_causal
        ctx.cp_rank, ctx.cp_world, ctx.slot = rank, world, slot
        return out

    @staticmethod
    def backward(ctx, dout, *args):
        q, k, v, out, softmax_lse = ctx.saved_tensors
        sm_scale, is_causal = ctx.sm_scale, ctx.is_causal
        world, rank, slot = ctx.cp_world, ctx.cp_rank, ctx.slot
        B, H, Sq, D = q.shape

        delta = ops.attn_bwd_preprocess(dout, out)

        if world == 1:
            dq, dk, dv = ops.attn_bwd(dout, q, k, v, softmax_lse, delta, sm_scale, is_causal, 0, dq_dtype=q.dtype,
                                      dq_like=q, dkv_dtype=k.dtype)
            return dq, dk, dv, None, None

        if not is_causal:
            raise NotImplementedError(
                "non-causal ring backward on virtual ranks: a rank's dK/dV needs every other rank's block, which a "
                "one-rank-at-a-time replay cannot deliver; use ring_attention_backward per block instead")
        kv_comm = ContextCommunicate("kv_comm", rank=rank, slot=slot)
        d_kv_comm = ContextCommunicate("d_kv_comm", rank=rank, slot=slot)
        dq = dk = dv = None
        next_dk = next_dv = None
        next_k = next_v = None
        for step in range(world):
            if step + 1 != world:
                next_k = kv_comm.send_recv(k)
                next_v = kv_comm.send_recv(v)
                kv_comm.commit()
            if step <= rank or not is_causal:
                bwd_causal = is_causal and step == 0
                if dk is None:
                    # first block: fresh fp32 accumulators (:85-88)
                    dq, dk, dv = ops.attn_bwd(dout, q, k, v, softmax_lse, delta, sm_scale, bwd_causal, 0)
                else:
                    # dq += block_dq ; dk = block_dk + next_dk (:90-93), the adds happen inside the kernels
                    d_kv_comm.wait()
                    dk, dv = next_dk, next_dv
                    ops.attn_bwd(dout, q, k, v, softmax_lse, delta, sm_scale, bwd_causal, 0, dq, dk, dv,
                                 dq_accumulate=True, dkv_accumulate=True)
            elif step != 0:
                d_kv_comm.wait()
                dk, dv = next_dk, next_dv
            if step + 1 != world:
                kv_comm.wait()
                k, v = next_k, next_v
            next_dk = d_kv_comm.send_recv(dk)
            next_dv = d_kv_comm.send_recv(dv)
            d_kv_comm.commit()
        d_kv_comm.wait()

        have = pgm.process_group_manager.cp_ring.deposited.get((slot, rank), set())
        missing = [r for r in range(rank, world) if r not in have]
        if missing:
            raise RuntimeError(
                f"local ring backward of cp rank {rank}: ranks {missing} have not added their dK/dV blocks yet; "
                "backpropagate the ranks together (sum their losses) or from the last rank to the first")
        return dq, next_dk, next_dv, None, None


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
