"""Oracle (test infrastructure): blockwise ring attention, restated on the CPU.

Follows the algorithm of the reference file
``picotron/context_parallel/context_parallel.py``:

* ``block_forward``   <- ``ring_attention_forward``   (:112-128)
* ``block_backward``  <- ``ring_attention_backward``  (:130-155)
* ``merge``           <- ``update_out_and_lse``       (:157-187)
* ``schedule``, ``rank_forward``, ``rank_backward``, ``all_ranks_*``
                      <- ``RingAttentionFunc.forward/backward`` (:19-110) with the P2P
                         hops replaced by indexing a list of chunks
* ``rope_slice``      <- ``update_rope_for_context_parallel`` (:189-195)
* ``position_ids``    <- ``MicroBatchDataLoader.collate_batch`` (``picotron/data.py:105-109``)

All maths runs in the dtype of the inputs (use fp32/fp64 for checking).  Tensors are
[B, H, S, D] as in the reference.
"""
from __future__ import annotations

from typing import Any, List, Optional, Sequence, Tuple

import torch


# --------------------------------------------------------------------------- integer work
def causal_mask(seqlen: int) -> torch.Tensor:
    """mask[i, j] = (j > i): True where a query must NOT see the key (:116)."""
    i = torch.arange(seqlen).unsqueeze(1)
    j = torch.arange(seqlen).unsqueeze(0)
    return j > i


def schedule(world_size: int, rank: int, is_causal: bool) -> List[Tuple[int, int, bool, bool]]:
    """Ring steps of ``rank``: (step, kv_chunk_held, executed, block_is_causal).

    At step s the rank holds the K/V chunk that started on rank (rank - s) mod W
    (every hop moves a chunk to rank+1, ``process_group_manager.py:43-44``); the block is
    computed iff ``not causal or s <= rank`` (:36, :78) and masked only at s == 0 (:38, :79).
    """
    steps = []
    for s in range(world_size):
        held = (rank - s) % world_size
        run = (not is_causal) or (s <= rank)
        steps.append((s, held, run, bool(is_causal and s == 0)))
    return steps


def rope_slice(cos: torch.Tensor, sin: torch.Tensor, rank: int, world_size: int):
    """Rows [rank*S/W, (rank+1)*S/W) of the [S, D] tables (:189-195)."""
    seq_len = cos.size(0)
    assert seq_len % world_size == 0, (
        f"Input sequence length ({seq_len}) must be divisible by cp_world_size ({world_size})")
    per = seq_len // world_size
    lo = rank * per
    return cos[lo:lo + per], sin[lo:lo + per]


def position_ids(rank: int, seq_length: int, world_size: int, batch_size: int) -> torch.Tensor:
    """Absolute positions of a rank's tokens (``data.py:105-109``)."""
    per = seq_length // world_size
    lo = rank * per
    return torch.arange(lo, lo + per, dtype=torch.long).unsqueeze(0).expand(batch_size, -1).contiguous()


# --------------------------------------------------------------------------- one block
def block_forward(q, k, v, sm_scale: float, is_causal: bool):
    """One attention block with a materialised score matrix (:112-128).

    Returns (O [B,H,Sq,D], lse [B,H,Sq]) with lse = log(sum exp(s - max)) + max.
    """
    scores = torch.matmul(q, k.transpose(-2, -1)) * sm_scale
    if is_causal:
        sq = q.size(2)
        scores = scores.masked_fill(causal_mask(sq).to(scores.device), float("-inf"))
    row_max = scores.amax(dim=-1, keepdim=True)
    e = torch.exp(scores - row_max)
    denom = e.sum(dim=-1, keepdim=True)
    lse = (torch.log(denom) + row_max).squeeze(-1)
    out = torch.matmul(e / denom, v)
    return out, lse


def block_backward(d_out, q, k, v, out, lse, sm_scale: float, is_causal: bool):
    """Gradients of one block given the FINAL (merged) out and lse (:130-155)."""
    scores = torch.matmul(q, k.transpose(-2, -1)) * sm_scale
    masked = None
    if is_causal:
        masked = causal_mask(q.size(2)).to(scores.device)
        scores = scores.masked_fill(masked, float("-inf"))
    p = torch.exp(scores - lse.unsqueeze(-1))
    d_v = torch.matmul(p.transpose(-2, -1), d_out)
    d_p = torch.matmul(d_out, v.transpose(-2, -1))
    delta = (d_out * out).sum(dim=-1, keepdim=True)
    d_s = p * (d_p - delta)
    if masked is not None:
        d_s = d_s.masked_fill(masked, 0)
    d_q = torch.matmul(d_s, k) * sm_scale
    d_k = torch.matmul(d_s.transpose(-2, -1), q) * sm_scale
    return d_q, d_k, d_v


def merge(out: Optional[torch.Tensor], lse: Optional[torch.Tensor], block_out: torch.Tensor,
          block_lse: torch.Tensor, slice_: Optional[Any] = None):
    """Online-softmax merge of a new block into the running (out, lse) (:157-187).

    out is fp32 [B,H,Sq,D], lse is [B,H,Sq,1]; the first call adopts the block.
    """
    block_out = block_out.to(torch.float32) if block_out.dtype not in (torch.float32, torch.float64) else block_out
    block_lse = block_lse.unsqueeze(-1)
    if out is None:
        if slice_ is not None:
            raise RuntimeError("first update_out_and_lse should not pass slice_ args")
        return block_out, block_lse

    def upd(o, l):
        o = o - torch.sigmoid(block_lse - l) * (o - block_out)
        l = l - torch.nn.functional.logsigmoid(l - block_lse)
        return o, l

    if slice_ is not None:
        out[slice_], lse[slice_] = upd(out[slice_], lse[slice_])
    else:
        out, lse = upd(out, lse)
    return out, lse


# --------------------------------------------------------------------------- one rank's ring
def rank_forward(q_r, k_chunks: Sequence[torch.Tensor], v_chunks: Sequence[torch.Tensor], rank: int,
                 sm_scale: float, is_causal: bool):
    """What rank ``rank`` computes in ``RingAttentionFunc.forward`` (:19-51).

    ``k_chunks[c]`` is the chunk that starts on rank c.  Returns (out in q dtype, lse [B,H,Sq]).
    """
    world = len(k_chunks)
    out = lse = None
    for _, held, run, blk_causal in schedule(world, rank, is_causal):
        if run:
            b_out, b_lse = block_forward(q_r, k_chunks[held], v_chunks[held], sm_scale, blk_causal)
            out, lse = merge(out, lse, b_out, b_lse)
    return out.to(q_r.dtype), lse.squeeze(-1)


def rank_backward(d_out_r, q_r, k_chunks, v_chunks, out_r, lse_r, rank: int, sm_scale: float, is_causal: bool):
    """Rank ``rank``'s share of ``RingAttentionFunc.backward`` (:53-110).

    Returns dq (fp32) and {chunk: (dk_contrib, dv_contrib)} -- the amounts this rank adds to
    the travelling dK/dV accumulators of each chunk it touches (:85-93).
    """
    world = len(k_chunks)
    dq = None
    contrib = {}
    for _, held, run, blk_causal in schedule(world, rank, is_causal):
        if not run:
            continue
        b_dq, b_dk, b_dv = block_backward(d_out_r, q_r, k_chunks[held], v_chunks[held], out_r, lse_r,
                                          sm_scale, blk_causal)
        acc_t = torch.float64 if b_dq.dtype == torch.float64 else torch.float32
        dq = b_dq.to(acc_t) if dq is None else dq + b_dq
        contrib[held] = (b_dk.to(acc_t), b_dv.to(acc_t))
    return dq, contrib


def all_ranks_forward(q, k, v, world_size: int, sm_scale: float, is_causal: bool):
    """Every rank of the ring, one after another; returns full-sequence (out, lse)."""
    qs, ks, vs = (t.chunk(world_size, dim=2) for t in (q, k, v))
    outs, lses = [], []
    for r in range(world_size):
        o, l = rank_forward(qs[r], ks, vs, r, sm_scale, is_causal)
        outs.append(o)
        lses.append(l)
    return torch.cat(outs, dim=2), torch.cat(lses, dim=2)


def all_ranks_backward(d_out, q, k, v, out, lse, world_size: int, sm_scale: float, is_causal: bool):
    """Every rank's backward; dK/dV contributions are summed per chunk as the ring would (:90-93)."""
    qs, ks, vs, dos, os_, ls = (t.chunk(world_size, dim=2) for t in (q, k, v, d_out, out, lse))
    dqs = []
    dk_acc = [None] * world_size
    dv_acc = [None] * world_size
    for r in range(world_size):
        dq, contrib = rank_backward(dos[r], qs[r], ks, vs, os_[r], ls[r], r, sm_scale, is_causal)
        dqs.append(dq)
        for c, (dk_c, dv_c) in contrib.items():
            dk_acc[c] = dk_c if dk_acc[c] is None else dk_acc[c] + dk_c
            dv_acc[c] = dv_c if dv_acc[c] is None else dv_acc[c] + dv_c
    return torch.cat(dqs, dim=2), torch.cat(dk_acc, dim=2), torch.cat(dv_acc, dim=2)


# --------------------------------------------------------------------------- closed forms used to pin the above
def full_attention_closed_form(q, k, v, sm_scale: float, is_causal: bool, q_offset: int = 0):
    """softmax(QK^T*s + mask) V and logsumexp, with query i sitting at absolute position q_offset+i."""
    s = torch.matmul(q, k.transpose(-2, -1)) * sm_scale
    if is_causal:
        qi = torch.arange(q.size(2)).unsqueeze(1) + q_offset
        kj = torch.arange(k.size(2)).unsqueeze(0)
        s = s.masked_fill(kj > qi, float("-inf"))
    return torch.matmul(torch.softmax(s, dim=-1), v), torch.logsumexp(s, dim=-1)
