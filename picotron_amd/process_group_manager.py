"""Single-process stand-in for ``picotron/process_group_manager.py``.

picotron builds a 4-D grid of torch.distributed ranks (dp x pp x cp x tp, ``process_group_manager.py:13``)
and the model / context-parallel code reads ``pgm.process_group_manager.{tp_world_size, cp_rank,
cp_world_size, cp_send_rank, cp_recv_rank, ...}`` from a module global (``:65-67``).  This build runs
on ONE GPU: tp = pp = dp = 1, and the cp "ranks" are virtual -- the same process plays rank
0, 1, ... in turn, and the ring hops are served from an in-process mailbox (``LocalRing``).  The
attribute names are the reference's so that code written against it reads the same.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch


class GradBox:
    """fp32 dK / dV accumulators of one published chunk: what travels round the ring in the reference
    (``context_parallel.py:85-106``).  Every rank's backward adds its block here; the chunk's own autograd node
    hands the total back once all of them have run."""

    __slots__ = ("dk", "dv", "readers", "arrived", "final_dk", "final_dv", "layout")

    def __init__(self):
        self.dk: Optional[torch.Tensor] = None
        self.dv: Optional[torch.Tensor] = None
        self.readers = 0        # ranks whose forward read the chunk and will add a block in their backward
        self.arrived = 0        # ... and how many of them have done so since the sums were last handed back
        # the block that completes the sums is written rounded, in the chunk's own dtype and layout, by the kernel
        # that computes it (one pass less than fp32 sums + a cast); `layout` = ((k dtype, strides), (v dtype, strides))
        self.final_dk: Optional[torch.Tensor] = None
        self.final_dv: Optional[torch.Tensor] = None
        self.layout = None


class RingChunk:
    """The K / V chunk one virtual rank holds at ring step 0 of one ring_attention call."""

    __slots__ = ("slot", "rank", "src_k", "src_v", "k", "v", "grads")

    def __init__(self, slot: int, rank: int, src_k: torch.Tensor, src_v: torch.Tensor):
        self.slot, self.rank = slot, rank
        self.src_k, self.src_v = src_k, src_v      # what the caller passed (to recognise a chunk staged ahead)
        self.k, self.v = src_k, src_v              # what peers read; replaced by autograd-tracked aliases on publish
        self.grads = GradBox()


def _same_tensor(a: torch.Tensor, b: torch.Tensor) -> bool:
    return a is b or (a.data_ptr() == b.data_ptr() and a.shape == b.shape and a.stride() == b.stride()
                      and a.dtype == b.dtype and a._version == b._version)


class LocalRing:
    """Mailbox that stands in for the cp ring's P2P hops (``cp_communications.py:22-41``).

    The chunk a rank holds at ring step 0 is published under (slot, rank); what rank r receives at step s is
    the chunk published by rank (r - s - 1) mod W for the same slot (every hop moves a chunk one rank up,
    ``process_group_manager.py:43-44``).  A slot is one call site of ring_attention within a rank's pass
    (layer i of the model), numbered by call order.

    A pass is one play of the ranks.  Publishing a (slot, rank) that the mailbox already holds means a new pass
    has begun (the next micro-batch or optimiser step): everything from the old pass is dropped first, so a
    chunk of an earlier pass can never be delivered.  Asking for a chunk that is not there raises.

    Under a causal mask rank r reads chunks 0..r, so playing the ranks in ascending order needs nothing else.
    Without a mask every rank reads every chunk; ``stage_kv`` lets the caller hand over all ranks' K / V
    before the first rank is played.
    """

    def __init__(self, world_size: int):
        self.world_size = world_size
        self.chunks: Dict[Tuple[int, int], RingChunk] = {}
        self._next_slot = 0

    def reset(self) -> None:
        """Forget every published chunk.  The mailbox keeps the last pass's K / V alive until the next pass begins
        (a later rank, or a rank's forward that follows another rank's backward, may still read them); call this to
        free them earlier.  A loop that feeds the SAME k / v tensor objects to every pass (a benchmark, a step that is
        recorded into a HIP graph after warm-up passes) must call it at the start of each pass: unchanged tensors are
        otherwise taken for chunks staged ahead of the play, and the pass would reuse the previous pass's autograd
        nodes (harmless in eager runs, but a recorded graph would miss their work)."""
        self.chunks.clear()
        self._next_slot = 0

    def begin_rank(self) -> None:
        """A new virtual rank starts its pass: its ring_attention calls are numbered from slot 0 again."""
        self._next_slot = 0

    def take_slot(self) -> int:
        s = self._next_slot
        self._next_slot += 1
        return s

    def publish_kv(self, slot: int, rank: int, k: torch.Tensor, v: torch.Tensor) -> RingChunk:
        key = (slot, rank)
        held = self.chunks.get(key)
        if held is not None:
            if _same_tensor(held.src_k, k) and _same_tensor(held.src_v, v):
                return held                      # staged ahead of the play by stage_kv
            self.chunks.clear()                  # a new pass: nothing of the old one may be delivered
        chunk = RingChunk(slot, rank, k, v)
        self.chunks[key] = chunk
        return chunk

    def stage_kv(self, rank: int, k: torch.Tensor, v: torch.Tensor, slot: int = 0) -> RingChunk:
        """Hand over rank `rank`'s chunk before that rank is played (needed when attention is not causal: every
        rank reads every chunk).  ring_attention recognises the same tensors when the rank's turn comes."""
        from picotron_amd.context_parallel.context_parallel import publish_chunk
        return publish_chunk(self, slot, rank, k, v)

    def fetch(self, slot: int, rank: int, reader: int) -> RingChunk:
        chunk = self.chunks.get((slot, rank))
        if chunk is None or chunk.k is None:
            raise RuntimeError(
                f"local cp ring: rank {reader} needs the K/V chunk of rank {rank} (ring_attention call {slot} of the "
                f"pass), which has not been published in this pass; play the ranks in ascending order (causal) or "
                f"hand all chunks over first with cp_ring.stage_kv(rank, k, v)")
        return chunk


class ProcessGroupManager:
    def __init__(self, tp_size: int, cp_size: int, pp_size: int, dp_size: int, cp_rank: int = 0):
        world = tp_size * cp_size * pp_size * dp_size
        assert tp_size == 1 and pp_size == 1 and dp_size == 1, (
            f"World size ({world}) != TP ({tp_size}) * CP ({cp_size}) * PP ({pp_size}) * DP ({dp_size}): "
            "this build runs one GPU, only cp_size may exceed 1 (virtual ranks)")
        assert cp_size >= 1 and 0 <= cp_rank < cp_size
        self.global_rank = 0
        self.world_size = cp_size
        self.local_rank = 0
        self.tp_rank = self.pp_rank = self.dp_rank = 0
        self.tp_world_size = self.pp_world_size = self.dp_world_size = 1
        self.tp_group = self.pp_group = self.dp_group = self.cp_group = self.cp_dp_group = None
        self.cp_world_size = cp_size
        self.cp_dp_world_size = cp_size
        self.cp_first_rank, self.cp_last_rank = 0, cp_size - 1
        self.pp_is_first_stage = self.pp_is_last_stage = True
        self.cp_ring = LocalRing(cp_size)
        self.set_cp_rank(cp_rank)

    def set_cp_rank(self, cp_rank: int) -> None:
        """Switch the virtual cp rank this process plays (ring neighbours as in the reference, :43-44)."""
        assert 0 <= cp_rank < self.cp_world_size
        self.cp_rank = cp_rank
        self.cp_send_rank = (cp_rank + 1) % self.cp_world_size
        self.cp_recv_rank = (cp_rank - 1) % self.cp_world_size
        self.cp_ring.begin_rank()

    def __str__(self):
        return f"TP(1)-CP({self.cp_world_size})-PP(1)-DP(1)-Rank({self.cp_rank})"


process_group_manager: Optional[ProcessGroupManager] = None


def setup_process_group_manager(tp_size: int, cp_size: int, pp_size: int, dp_size: int, cp_rank: int = 0):
    global process_group_manager
    process_group_manager = ProcessGroupManager(tp_size, cp_size, pp_size, dp_size, cp_rank)
    return process_group_manager
