"""The "sum" and "gather d" output rules when every rank's shard lives on ONE HIP device.

The reference rendezvouses W rank threads and moves data between devices
(src/tensor_parallel/communications.py:21-171, cross_device_ops.py:30-50). Here the W partials are already
on the same GPU: the threads still rendezvous (an op object is called as `op(x, rank)` from W threads, as
in the reference, communications.py:16-18), but the work is one kernel launch: a W-way elementwise sum
(`tpamd_reduce_partials`) or a concatenation done by the region mover. No inter-GPU collective exists.

All ranks enqueue on the device's current stream, so the kernels that produced the partials are ordered
before the reduction by the stream itself; the host-side barrier only makes sure they were enqueued.
"""
from __future__ import annotations

import threading
from typing import Any, Callable, List, Optional

import torch

from . import _native
from .shard_modules import _guard
from .slicing import concat_dim

RENDEZVOUS_TIMEOUT_S = 600.0

# Rank threads that share ONE device take turns on the host: a rank holds the "turn" lock while it runs module
# code and gives it up only while it waits in a rendezvous. All ranks enqueue onto the same device anyway, so
# nothing is lost, and host-side lazy initialisation inside torch (attention backends, BLAS handles) is never
# entered by two rank threads at once. The lock of the running forward is published per thread here.
_turn = threading.local()


def set_turn_lock(lock: Optional[threading.Lock]) -> None:
    _turn.lock = lock


def _rendezvous(barrier: threading.Barrier, timeout: float) -> None:
    lock = getattr(_turn, "lock", None)
    if lock is None:
        barrier.wait(timeout)
        return
    lock.release()
    try:
        barrier.wait(timeout)
    finally:
        lock.acquire()


class CollectiveOpetationBase:
    def __call__(self, x: torch.Tensor, rank: int):
        raise NotImplementedError()


class CollectiveOperation(CollectiveOpetationBase):
    """All ranks hand in a value; rank 0 runs `func(*values)`, which returns one result per rank
    (reference: communications.py:21-52). An exception raised by `func` is re-raised on every rank."""

    def __init__(self, world_size: int, func: Callable[..., List[Any]], timeout: float = RENDEZVOUS_TIMEOUT_S):
        self.world_size = world_size
        self.func = func
        self.timeout = timeout
        self._barrier = threading.Barrier(world_size)
        self._inputs: List[Any] = [None] * world_size
        self._outputs: List[Any] = [None] * world_size
        self._error: Optional[BaseException] = None

    def __call__(self, x: Any, rank: int):
        try:
            self._inputs[rank] = x
            _rendezvous(self._barrier, self.timeout)
            if rank == 0:
                try:
                    result = self.func(*self._inputs)
                    for i in range(self.world_size):
                        self._outputs[i] = result[i]
                    self._error = None
                except BaseException as e:  # fan the failure out to every rank
                    self._error = e
            _rendezvous(self._barrier, self.timeout)
            if self._error is not None:
                raise self._error
            return self._outputs[rank]
        finally:
            self._inputs[rank] = None
            # the third rendezvous keeps a fast rank from starting the next call while a slow one still reads
            try:
                _rendezvous(self._barrier, self.timeout)
            except threading.BrokenBarrierError:
                pass
            self._outputs[rank] = None


class DeviceAllReduce(CollectiveOperation):
    """out = p_0 + p_1 + ... + p_{W-1}, delivered to every rank. `accum` picks the arithmetic
    (`_native.ACCUM_STEPWISE`: the running sum is rounded to the tensor dtype after each add, which is what
    the reference's `sum([...])` of same-dtype tensors does, cross_device_ops.py:49, taken in rank order)."""

    def __init__(self, world_size: int, accum: int = _native.ACCUM_STEPWISE, timeout: float = RENDEZVOUS_TIMEOUT_S):
        super().__init__(world_size, self._reduce, timeout)
        self.accum = accum

    def _reduce(self, *parts: torch.Tensor):
        out = _native.reduce_partials([p.detach() for p in parts], accum=self.accum)
        # each rank continues with a tensor of its own: later in-place ops on one rank must not leak
        return [_guard(o, *parts) for o in [out] + [out.clone() for _ in range(self.world_size - 1)]]


class DeviceAllGather(CollectiveOperation):
    """Concatenate every rank's tensor on `dim` (column-parallel outputs back to full width)."""

    def __init__(self, world_size: int, dim: int = -1, timeout: float = RENDEZVOUS_TIMEOUT_S):
        super().__init__(world_size, self._gather, timeout)
        self.dim = dim

    def _gather(self, *parts: torch.Tensor):
        for p in parts:
            _native.require_device(p, "gather")
        out = concat_dim([p.detach() for p in parts], self.dim)
        return [_guard(o, *parts) for o in [out] + [out.clone() for _ in range(self.world_size - 1)]]
