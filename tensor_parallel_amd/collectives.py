"""The "sum" and "gather d" output rules when every rank's shard lives on ONE HIP device.

The reference rendezvouses W rank threads and moves data between devices
(src/tensor_parallel/communications.py:21-171, cross_device_ops.py:30-50). Here the W partials are already
on the same GPU: the ranks still rendezvous (an op object is called as `op(x, rank)` by each of the W ranks, as
in the reference, communications.py:16-18), but the work is one kernel launch: a W-way elementwise sum
(`tpamd_reduce_partials`) or a concatenation done by the region mover. No inter-GPU collective exists.

All ranks enqueue on the device's current stream, so the kernels that produced the partials are ordered
before the reduction by the stream itself; the host-side barrier only makes sure they were enqueued.
"""
from __future__ import annotations

import contextvars
import os
import threading
from typing import Any, Callable, List, Optional

import torch

from . import _native
from .shard_modules import _guard
from .slicing import concat_dim

RENDEZVOUS_TIMEOUT_S = 600.0

# Ranks that share ONE device take turns on the host: a rank holds the turn while it runs module code and gives it up
# only while it waits in a collective. All ranks enqueue onto the same device anyway, so nothing is lost, and host-side
# lazy initialisation inside torch (attention backends, BLAS handles) is never entered by two ranks at once. The ranks
# are greenlets of the calling thread where the greenlet package is there (a switch costs about a microsecond), else
# threads (a hand-over through a condition variable costs tens of microseconds, twice per collective). The turn of the
# running forward is published per rank here: context variables are per thread and per greenlet.
_turn: contextvars.ContextVar = contextvars.ContextVar("tpamd_turn", default=None)


class Turn:
    """What the rank threads of one forward on one device share: the lock that says whose turn it is, a condition on that
    lock on which ranks wait inside a collective, and a flag that a rank has failed (its peers stop waiting)."""

    __slots__ = ("lock", "cond", "failed")

    def __init__(self):
        self.lock = threading.Lock()
        self.cond = threading.Condition(self.lock)
        self.failed = False

    def wait(self, timeout: float) -> bool:
        """Gives the turn away until a peer wakes this rank; False after `timeout` seconds without that."""
        return self.cond.wait(timeout)

    def wake(self) -> None:
        """A round of a collective is complete: its waiting ranks may go on when they get the turn."""
        self.cond.notify_all()

    def fail(self) -> None:
        """Called by a failing rank while it holds the lock: wakes every waiting peer."""
        self.failed = True
        self.cond.notify_all()


class GreenTurn:
    """The same for ranks that are greenlets of one thread: the turn is whichever greenlet runs. A rank that waits
    switches to `hub`, the greenlet that started the ranks and hands the turn round (tensor_parallel.parallel_apply_simple);
    `events` counts completed rounds and finished ranks, which is how the hub sees that the ranks still get anywhere."""

    __slots__ = ("hub", "events", "failed")

    def __init__(self, hub):
        self.hub = hub
        self.events = 0
        self.failed = False

    def wait(self, timeout: float) -> bool:
        self.hub.switch()
        return True

    def wake(self) -> None:
        self.events += 1

    def fail(self) -> None:
        self.failed = True


def set_turn_lock(turn) -> None:
    _turn.set(turn)


def current_turn():
    return _turn.get()


# ---- the sum folded into the last Linear of a row-parallel module -------------------------------------------------
# A module whose output rule is "sum" usually ends in its row-parallel Linear (attention output projection, MLP down
# projection). The rank that reaches that Linear while the partials of the other ranks are already waiting in the op
# can add them in the GEMM's epilogue (`tpamd_linear_add`) instead of leaving a separate M x N pass to the reduction
# kernel. A wrapper with such a rule publishes a SumContext for its rank while its module runs; shard Linears
# consult it (shard_modules.linear_in_context); the op learns from it what the value it is handed already contains.
FUSE_SUM = os.environ.get("TPAMD_FUSE_SUM", "1") != "0"
_contexts: contextvars.ContextVar = contextvars.ContextVar("tpamd_sum_contexts", default=None)


class SumContext:
    """One call of a wrapped module whose output 0 goes to `op`, on one rank."""

    __slots__ = ("op", "rank", "owner", "last_linear", "last_out", "calls", "fused_out", "fused_mask")

    def __init__(self, op: "DeviceAllReduce", rank: int, owner: Any):
        self.op, self.rank, self.owner = op, rank, owner
        self.last_linear = self.last_out = self.fused_out = None
        self.calls: dict = {}
        self.fused_mask = 0

    def settle(self, value: Any) -> None:
        """Called by the wrapper with the value its module returned for the summed output, before the rules run. If a
        Linear folded the waiting partials in, that value must be the Linear's output itself. Otherwise this call
        teaches the Linear that produced exactly this value (and ran once) that it feeds the sum: next time it may fold."""
        if self.fused_out is not None:
            if value is not self.fused_out:
                raise RuntimeError(
                    "tensor_parallel_amd: a row-parallel Linear added the other ranks' partial sums in its epilogue, but its "
                    "module then returned a different tensor; set TPAMD_FUSE_SUM=0 to keep the sum in its own kernel")
        elif self.last_linear is not None:
            feeds = value is self.last_out and self.calls.get(id(self.last_linear)) == 1
            self.last_linear.__dict__["_tp_feeds_sum"] = self.owner if feeds else None


def push_sum_context(ctx: Optional[SumContext]) -> None:
    stack = _contexts.get()
    if stack is None:
        stack = []
        _contexts.set(stack)
    stack.append(ctx)


def pop_sum_context() -> None:
    _contexts.get().pop()


def current_sum_context() -> Optional[SumContext]:
    stack = _contexts.get()
    return stack[-1] if stack else None


def _rendezvous(barrier: threading.Barrier, timeout: float) -> None:
    barrier.wait(timeout)


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
        self._arrived = 0  # turn-taking ranks: how many have handed in their value this round
        self._round = 0

    def _call_in_turns(self, x: Any, rank: int, turn):
        """The same exchange for ranks that take turns on one device (the caller holds the turn): a rank
        hands in its value and waits on the turn, which gives it away; the rank that arrives last
        runs `func` and wakes the others. One wake-up per waiting rank and collective instead of three barrier rounds.
        The results of a round stay in place until the next round of this op completes, which needs every rank to have
        come back, so nobody can miss its result."""
        self._inputs[rank] = x
        self._arrived += 1
        if self._arrived == self.world_size:
            try:
                result = self.func(*self._inputs)
                self._outputs = [result[i] for i in range(self.world_size)]
                self._error = None
            except BaseException as e:  # fan the failure out to every rank
                self._outputs = [None] * self.world_size
                self._error = e
            self._inputs = [None] * self.world_size
            self._arrived = 0
            self._round += 1
            turn.wake()
        else:
            started = self._round
            while self._round == started:
                if turn.failed:
                    self._inputs[rank] = None
                    self._arrived -= 1
                    raise threading.BrokenBarrierError
                if not turn.wait(self.timeout):
                    self._inputs[rank] = None
                    self._arrived -= 1
                    raise threading.BrokenBarrierError
        if self._error is not None:
            raise self._error
        return self._outputs[rank]

    def __call__(self, x: Any, rank: int):
        turn = current_turn()
        if turn is not None:
            return self._call_in_turns(x, rank, turn)
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
    the reference's `sum([...])` of same-dtype tensors does, cross_device_ops.py:49, taken in rank order).

    A value handed in may already hold the sum over several ranks (see SumContext): rank r's Linear added what
    `addend_for(r)` gave it. `_masks[r]` records which ranks value r covers; the reduction then adds only what is
    still missing, in rank order, and launches nothing when one value covers every rank."""

    def __init__(self, world_size: int, accum: int = _native.ACCUM_STEPWISE, timeout: float = RENDEZVOUS_TIMEOUT_S):
        super().__init__(world_size, self._reduce, timeout)
        self.accum = accum
        self._masks: List[int] = [0] * world_size

    @property
    def fusable(self) -> bool:
        return FUSE_SUM and self.accum == _native.ACCUM_STEPWISE and self.world_size > 1

    def addend_for(self, rank: int):
        """(tensor, ranks it covers as a bit mask) that rank `rank`'s last Linear may add to its own partial so that
        the result is a step of the rank-ordered sum, or None. Two ranks: whatever the other rank has handed in (a sum
        of two is the same in either order). More ranks: the running sum over ranks 0 .. rank-1, once rank-1 has
        handed it in. Only for ranks that take turns on one device (the waiting value is then complete and
        visible)."""
        if not self.fusable or current_turn() is None:
            return None
        if self.world_size == 2:
            other = 1 - rank
            if self._inputs[other] is not None and self._masks[other] == 1 << other:
                return self._inputs[other], 1 << other
            return None
        below = (1 << rank) - 1
        if rank > 0 and self._inputs[rank - 1] is not None and self._masks[rank - 1] == below:
            return self._inputs[rank - 1], below
        return None

    def __call__(self, x: Any, rank: int):
        mask = 1 << rank
        ctx = current_sum_context()
        if ctx is not None and ctx.op is self and ctx.fused_out is not None and x is ctx.fused_out:
            mask |= ctx.fused_mask  # this value already holds what the rank's Linear was given by addend_for()
        self._masks[rank] = mask
        try:
            return super().__call__(x, rank)
        finally:
            self._masks[rank] = 0

    def _reduce(self, *parts: torch.Tensor):
        masks = list(self._masks)
        widest = max(range(self.world_size), key=lambda r: bin(masks[r]).count("1"))
        todo = [parts[widest]] + [parts[r] for r in range(self.world_size) if not masks[widest] >> r & 1]
        # the widest value is a running sum from rank 0 on (or covers both of two ranks); what it lacks are higher ranks
        out = todo[0].detach() if len(todo) == 1 else _native.reduce_partials([p.detach() for p in todo], accum=self.accum)
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
        # each rank continues with a tensor of its own, all written by the same launch where their jobs fit one
        outs = concat_dim([p.detach() for p in parts], self.dim, copies=self.world_size)
        return [_guard(o, *parts) for o in (outs if self.world_size > 1 else [outs])]
