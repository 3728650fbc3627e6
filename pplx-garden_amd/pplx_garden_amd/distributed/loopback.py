"""The expert-parallel group when every rank lives on one GPU.

The reference builds an operator on `ParallelGroup` objects backed by
torch.distributed, one process per GPU
(python/pplx_garden/distributed/process_group.py:102-285).  Here the group is
a plain in-process object: `LoopbackWorld(world_size)` stands for the whole
group and `world.group(rank)` is what one logical rank passes as
`global_group`.  All operators built on groups of one world share one native
context, so their buffers and routing tables sit in the same HBM.

A collective is complete when every rank has made the call.  In one process
the ranks call one after the other, so the world collects the arguments of a
collective call and the call of the LAST rank launches the work for all of
them; results are defined once every rank of the world has called.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional, Tuple

import torch


@dataclass(frozen=True)
class LoopbackGroup:
    """What a logical rank knows about its group: the counterpart of the
    reference's `ParallelGroup` (`rank`, `size`) for one process."""

    world: "LoopbackWorld"
    rank: int

    @property
    def size(self) -> int:
        return self.world.size

    @property
    def node_size(self) -> int:
        return self.world.node_size

    def barrier(self) -> None:
        """All logical ranks share the caller's thread: nothing to wait for."""


@dataclass(frozen=True)
class LoopbackSubGroup:
    """A slice of the world, e.g. the ranks that hold the same tokens (`dp_group`) or the ranks of
    one node (`node_group`): only `size` and the caller's `rank` inside it matter to the operator."""

    size: int
    rank: int


class LoopbackWorld:
    def __init__(self, world_size: int, node_size: Optional[int] = None,
                 device: Optional[torch.device] = None, context_flags: int = 0) -> None:
        if world_size < 1:
            raise ValueError("world_size must be at least 1")
        node_size = world_size if node_size is None else node_size
        if node_size < 1 or world_size % node_size != 0:
            raise ValueError(f"node_size {node_size} does not divide world_size {world_size}")
        self.size = world_size
        self.node_size = node_size
        self.device = device
        self.context_flags = context_flags   # A2A_FLAG_* bits for the contexts created in this world
        self._contexts: Dict[Tuple, Any] = {}
        self._users: Dict[Tuple, int] = {}
        self._pending: Dict[Tuple[Tuple, str], Dict[int, Any]] = {}

    def group(self, rank: int) -> LoopbackGroup:
        if not 0 <= rank < self.size:
            raise ValueError(f"rank {rank} out of range [0, {self.size})")
        return LoopbackGroup(self, rank)

    def dp_group(self, rank: int, dp_size: int) -> LoopbackSubGroup:
        """The group of `dp_size` consecutive ranks that share `rank`'s tokens."""
        if dp_size < 1 or self.node_size % dp_size != 0:
            raise ValueError(f"dp_size {dp_size} does not divide node_size {self.node_size}")
        return LoopbackSubGroup(size=dp_size, rank=rank % dp_size)

    @property
    def groups(self) -> List[LoopbackGroup]:
        return [self.group(r) for r in range(self.size)]

    # -- shared native context ---------------------------------------------

    def acquire_context(self, key: Tuple, factory: Callable[[], Any]) -> Any:
        """The context for configuration `key`, created by the first operator."""
        if key not in self._contexts:
            self._contexts[key] = factory()
            self._users[key] = 0
        self._users[key] += 1
        return self._contexts[key]

    def release_context(self, key: Tuple) -> None:
        if key not in self._contexts:
            return
        self._users[key] -= 1
        if self._users[key] <= 0:
            ctx = self._contexts.pop(key)
            self._users.pop(key)
            for pending_key in [k for k in self._pending if k[0] == key]:
                self._pending.pop(pending_key)
            ctx.destroy()

    # -- collectives --------------------------------------------------------

    def post(self, key: Tuple, kind: str, rank: int, payload: Any) -> Optional[List[Any]]:
        """Record `rank`'s arguments for collective `kind`.  Returns the
        arguments of all ranks, in rank order, once the last rank has posted."""
        slot = self._pending.setdefault((key, kind), {})
        if rank in slot:
            missing = sorted(set(range(self.size)) - set(slot))
            raise RuntimeError(
                f"rank {rank} called {kind}() twice before ranks {missing} called it: in loopback "
                "a collective runs when every logical rank has made the call")
        slot[rank] = payload
        if len(slot) < self.size:
            return None
        del self._pending[(key, kind)]
        return [slot[r] for r in range(self.size)]

    def pending(self, key: Tuple, kind: str) -> List[int]:
        return sorted(self._pending.get((key, kind), {}))
