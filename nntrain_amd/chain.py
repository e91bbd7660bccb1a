"""A chain of dependent fused mat-vecs enqueued as one unit of work (nnhip_chain_*).

The reference issues the projections of a token one kernel after the other (ForwardTokenDevice,
NNtrain.Core/Modules/Qwen35QuantizedModel.cs:451-513); a chain keeps the same steps, in the same order and with the same
buffers, but hands them to the library together, which runs consecutive steps of one storage type as a single launch
whose workgroups pass from step to step on their own.
"""
from __future__ import annotations

import ctypes
from ctypes import c_int, c_void_p

from .lane import HipExecutionLane
from .native import FusedMatvecDesc, check


class HipMatvecChain:
    """Steps are FusedMatvecDesc structures (HipQuantizedMatrix.fused_descriptor); the buffers they name must stay
    alive, and keep their contents' meaning, for as long as the chain is launched."""

    def __init__(self, lane: HipExecutionLane, steps: list[FusedMatvecDesc]):
        if not steps:
            raise ValueError("A chain needs at least one step.")
        self._lane = lane
        array = (FusedMatvecDesc * len(steps))(*steps)
        handle = c_void_p()
        check(lane._lib.nnhip_chain_create(lane._handle, array, len(steps), ctypes.byref(handle)), "chain_create")
        self._handle = handle
        self.steps = len(steps)

    @property
    def launches(self) -> int:
        """Kernel launches one launch() of the chain enqueues."""
        n = c_int()
        check(self._lane._lib.nnhip_chain_launches(self._lane._handle, self._handle, ctypes.byref(n)), "chain_launches")
        return n.value

    def launch(self) -> None:
        with self._lane.kernel("chain"):
            check(self._lane._lib.nnhip_chain_launch(self._lane._handle, self._handle), "chain_launch")

    def gave_up(self) -> bool:
        """Blocks until the lane has drained; True when a workgroup's bounded wait for a step ran out since the last call."""
        flag = c_int()
        check(self._lane._lib.nnhip_chain_status(self._lane._handle, self._handle, ctypes.byref(flag)), "chain_status")
        return bool(flag.value)

    def dispose(self) -> None:
        if self._handle is not None and not self._lane.disposed:
            check(self._lane._lib.nnhip_chain_destroy(self._lane._handle, self._handle), "chain_destroy")
        self._handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.dispose()


__all__ = ["HipMatvecChain"]
