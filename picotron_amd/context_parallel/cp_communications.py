"""Local provider with the API of ``picotron/context_parallel/cp_communications.py``.

Same class name, methods, attributes and error behaviour (``Commit called twice`` :39, ``Wait called
before commit`` :44), but the peer is the in-process ``LocalRing`` mailbox instead of
``dist.batch_isend_irecv`` -- there is one GPU and no collective.

What a communicator carries is the K / V ring of ``context_parallel.py:21,60``: every ``send_recv`` of a ring
step posts one tensor (K first, then V); ``wait`` completes the step by copying the peer's chunk into the
receive buffers, which is the hop.  At ring step s rank r receives the chunk published by rank
(r - s - 1) mod W.  ``msg`` is a label for the log lines, as in the reference.

The reference's third ring (``d_kv_comm``, :61) moves the fp32 dK / dV accumulators from rank to rank.  Virtual
ranks share one address space, so the accumulators do not travel: they live with the published chunk
(``process_group_manager.GradBox``), every rank's backward adds its block there inside the kernel, and the chunk's
autograd node returns the total after the last rank has added its part.
"""
from __future__ import annotations

import os
from typing import List, Optional

import torch

import picotron_amd.process_group_manager as pgm

STEP, VERBOSE = 0, os.environ.get("VERBOSE", "0") == "1"


class ContextCommunicate:
    def __init__(self, msg: str = "", rank: Optional[int] = None, slot: Optional[int] = None, chunks=None):
        """`rank` / `slot` default to the rank being played and must be bound before the first wait(); `chunks`
        ({rank: RingChunk}) serves the hops from chunks the caller already holds instead of the mailbox (a backward
        pass reads the chunks its forward saw, whatever has been published since)."""
        mgr = pgm.process_group_manager
        self.msg = msg
        self.world_size = mgr.cp_world_size
        self.rank = mgr.cp_rank if rank is None else rank
        self.send_rank = (self.rank + 1) % self.world_size
        self.recv_rank = (self.rank - 1) % self.world_size
        self._ring = mgr.cp_ring
        self._slot = slot
        self._chunks = chunks
        self._step = 0               # ring steps completed so far
        self._pending: List[tuple] = []   # (sent tensor, receive buffer) of the open step
        self._active = None
        if VERBOSE:
            print(f"RingComm ({msg}) | initialized | RANK:{self.rank} | WORLD_SIZE:{self.world_size} | "
                  f"SEND_RANK:{self.send_rank} | RECV_RANK:{self.recv_rank}", flush=True)

    def bind_slot(self, slot: int) -> None:
        self._slot = slot

    def send_recv(self, tensor_to_send, recv_tensor=None):
        # (the receive buffer needs no clearing: wait() overwrites all of it, with the peer's chunk or with NaN)
        result = torch.empty_like(tensor_to_send) if recv_tensor is None else recv_tensor
        self._pending.append((tensor_to_send, result))
        return result

    def commit(self):
        if self._active is not None:
            raise RuntimeError("Commit called twice")
        self._active = list(self._pending)
        if VERBOSE:
            print(f"RingComm | commit | STEP:{STEP} | RANK:{self.rank} | NUM_OPS:{len(self._pending)}", flush=True)

    def wait(self, needed: bool = True):
        """Completes the open ring step.  `needed=False` says the arriving chunk will not be read (a causal ring
        receives chunks of later ranks that it never uses): a chunk that is not in the mailbox is then skipped and
        the receive buffers are filled with NaN, where `needed=True` raises."""
        if self._active is None:
            raise RuntimeError("Wait called before commit")
        W, r, s = self.world_size, self.rank, self._step
        if self._slot is None and self._chunks is None:
            raise RuntimeError("ContextCommunicate: no ring slot bound (use ring_attention / RingAttentionFunc)")
        if len(self._active) > 2:
            raise RuntimeError("ContextCommunicate: a ring step carries K and V (at most two tensors)")
        src_rank = (r - s - 1) % W
        held = self._chunks.get(src_rank) if self._chunks is not None else self._ring.chunks.get((self._slot, src_rank))
        if held is None or held.k is None:
            if needed:
                if self._chunks is not None:
                    raise RuntimeError(f"local cp ring: rank {r} was not given the K/V chunk of rank {src_rank}")
                self._ring.fetch(self._slot, src_rank, r)      # raises, naming the chunk
            for _, buf in self._active:
                buf.fill_(float("nan"))
        else:
            for (_, buf), src in zip(self._active, (held.k, held.v)):
                buf.copy_(src.detach())                        # the hop: the peer's chunk arrives in the receive buffer
        self._step += 1
        self._active = None
        self._pending = []
        if VERBOSE:
            print(f"RingComm | wait | STEP:{STEP} | RANK:{self.rank} | ACTION:all_operations_completed", flush=True)
