"""Local provider with the API of ``picotron/context_parallel/cp_communications.py``.

Same class name, methods, attributes and error behaviour (``Commit called twice`` :39, ``Wait called
before commit`` :44), but the peer is the in-process ``LocalRing`` mailbox instead of
``dist.batch_isend_irecv`` -- there is one GPU and no collective.  The communicator is told by its
``msg`` which protocol it carries, exactly the three the reference opens (``context_parallel.py:21,60,61``):

* ``"comm"`` / ``"kv_comm"``: K then V per ring step; step s delivers the chunk of rank (r-s-1) mod W.
* ``"d_kv_comm"``: dK then dV per ring step; delivers the travelling fp32 accumulators.
"""
from __future__ import annotations

import os
from typing import List, Optional

import torch

import picotron_amd.process_group_manager as pgm

STEP, VERBOSE = 0, os.environ.get("VERBOSE", "0") == "1"


class ContextCommunicate:
    def __init__(self, msg: str = "", rank: Optional[int] = None, slot: Optional[int] = None):
        mgr = pgm.process_group_manager
        self.msg = msg
        self.world_size = mgr.cp_world_size
        self.rank = mgr.cp_rank if rank is None else rank
        self.send_rank = (self.rank + 1) % self.world_size
        self.recv_rank = (self.rank - 1) % self.world_size
        self._ring = mgr.cp_ring
        self._slot = slot
        self._step = 0               # ring steps committed so far
        self._pending: List[tuple] = []   # (sent tensor, receive buffer) of the open step
        self._active = None
        if VERBOSE:
            print(f"RingComm ({msg}) | initialized | RANK:{self.rank} | WORLD_SIZE:{self.world_size} | "
                  f"SEND_RANK:{self.send_rank} | RECV_RANK:{self.recv_rank}", flush=True)

    # -- protocol helpers -------------------------------------------------------------
    def bind_slot(self, slot: int) -> None:
        self._slot = slot

    def _is_grad_channel(self) -> bool:
        return self.msg == "d_kv_comm"

    def send_recv(self, tensor_to_send, recv_tensor=None):
        result = torch.zeros_like(tensor_to_send) if recv_tensor is None else recv_tensor
        self._pending.append((tensor_to_send, result))
        return result

    def commit(self):
        if self._active is not None:
            raise RuntimeError("Commit called twice")
        self._active = list(self._pending)
        if VERBOSE:
            print(f"RingComm | commit | STEP:{STEP} | RANK:{self.rank} | NUM_OPS:{len(self._pending)}", flush=True)

    def wait(self):
        if self._active is None:
            raise RuntimeError("Wait called before commit")
        W, r, s = self.world_size, self.rank, self._step
        if self._slot is None:
            raise RuntimeError("ContextCommunicate: no ring slot bound (use ring_attention / RingAttentionFunc)")
        if self._is_grad_channel():
            # what leaves is the accumulator of chunk (r - s) mod W; what arrives is that of chunk (r - s - 1) mod W
            out_chunk, in_chunk = (r - s) % W, (r - s - 1) % W
            sent = [t for t, _ in self._active]
            key = (self._slot, out_chunk)
            if s == 0 and key in self._ring.acc:
                # a fresh accumulator meets contributions already left by ranks replayed earlier
                for have, new in zip(self._ring.acc[key], sent):
                    have.add_(new)
            else:
                self._ring.acc[key] = [t if t.dtype == torch.float32 else t.float() for t in sent]
            self._ring.deposited.setdefault(key, set()).add(r)
            have = self._ring.acc.get((self._slot, in_chunk))
            for i, (_, buf) in enumerate(self._active):
                if have is not None:
                    buf.copy_(have[i])      # the hop: running total of the chunk arrives in the receive buffer
                else:
                    buf.zero_()
        else:
            in_chunk = (r - s - 1) % W
            have = self._ring.kv.get((self._slot, in_chunk))
            if have is not None:
                for (_, buf), src in zip(self._active, have):
                    buf.copy_(src)          # the hop: the peer's chunk arrives in the receive buffer
            # else: chunk of a rank that has not been replayed yet; under a causal mask it is never used
        self._step += 1
        self._active = None
        self._pending = []
        if VERBOSE:
            print(f"RingComm | wait | STEP:{STEP} | RANK:{self.rank} | ACTION:all_operations_completed", flush=True)
