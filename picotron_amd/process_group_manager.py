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


class LocalRing:
    """Mailbox that stands in for the cp ring's P2P hops (``cp_communications.py:22-41``).

    K/V: the chunk a rank holds at ring step 0 is published under (slot, rank); what rank r
    receives at step s is the chunk published by rank (r - s - 1) mod W for the same slot
    (every hop moves a chunk one rank up, ``process_group_manager.py:43-44``).  A slot is one call
    site of ring_attention within a rank's pass (layer i of the model), numbered by call order.

    dK/dV: ``acc[(slot, c)]`` is the travelling fp32 accumulator of chunk c.  A rank receives the
    running total and sends back total + its own block, so replaying ranks one after another leaves
    the same sums the real ring produces (``context_parallel.py:85-106``).
    """

    def __init__(self, world_size: int):
        self.world_size = world_size
        self.kv: Dict[Tuple[int, int], Tuple[torch.Tensor, torch.Tensor]] = {}
        self.acc: Dict[Tuple[int, int], list] = {}
        self.deposited: Dict[Tuple[int, int], set] = {}
        self._next_slot = 0

    def reset(self) -> None:
        """Forget every published chunk and accumulator (call between optimiser steps)."""
        self.kv.clear()
        self.acc.clear()
        self.deposited.clear()
        self._next_slot = 0

    def begin_rank(self) -> None:
        """A new virtual rank starts its pass: its ring_attention calls are numbered from slot 0 again."""
        self._next_slot = 0

    def take_slot(self) -> int:
        s = self._next_slot
        self._next_slot += 1
        return s

    def publish_kv(self, slot: int, rank: int, k: torch.Tensor, v: torch.Tensor) -> None:
        self.kv[(slot, rank)] = (k, v)


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
