"""State actions: how one parameter or buffer becomes a rank's shard, and how shards recombine.

Same protocol and constructor signatures as the reference (src/tensor_parallel/state_actions.py:10-119):
`action(tensor, rank)` gives the shard, `action.undo(tensors)` the full tensor. Here the splitting
actions do not build torch views: they compile to a `SliceSpec` (index ranges on one axis), which the HIP
region mover executes, alone or batched over a whole state dict (`BatchSlicer`). Results are fresh
contiguous tensors on the HIP device. Meta tensors pass through as shapes.
"""
from __future__ import annotations

from abc import ABC, abstractmethod
from typing import Callable, Optional, Sequence

import torch
from torch import Tensor

from . import _native
from .slicing import SliceSpec, apply_spec, concat_specs, normalize_dim, tensor_split_range


class StateAction(ABC):
    @abstractmethod
    def __call__(self, tensor: Tensor, rank: int) -> Tensor:
        ...

    @abstractmethod
    def undo(self, tensors: Sequence[Tensor]) -> Tensor:
        ...


class LegacyStateAction(StateAction):
    """A user callable (and optional inverse) used as a state rule: runs as given, on whatever it is given."""

    def __init__(
        self,
        action: Callable[[Tensor, int], Tensor],
        reverse_action: Optional[Callable[[Sequence[Tensor]], Tensor]] = None,
    ):
        self.action = action
        self.reverse_action = reverse_action

    def __call__(self, tensor: Tensor, rank: int) -> Tensor:
        return self.action(tensor, rank)

    def undo(self, tensors: Sequence[Tensor]) -> Tensor:
        if self.reverse_action is None:
            raise Exception(f"No reverse action provided for {self.action}. Can't undo.")
        return self.reverse_action(tensors)


class SegmentedAction(StateAction):
    """Base of the actions that keep index ranges of one axis. Subclasses define `spec`."""

    world_size: int

    def spec(self, shape: Sequence[int], rank: int) -> SliceSpec:
        raise NotImplementedError

    def __call__(self, tensor: Tensor, rank: int) -> Tensor:
        return apply_spec(tensor, self.spec(tuple(tensor.shape), rank))

    def full_shape(self, shard_shapes: Sequence[Sequence[int]]) -> tuple:
        dim = self._dim_for(len(shard_shapes[0]))
        shape = list(shard_shapes[0])
        shape[dim] = sum(s[dim] for s in shard_shapes)
        return tuple(shape)

    def _dim_for(self, ndim: int) -> int:
        raise NotImplementedError

    def undo(self, tensors: Sequence[Tensor]) -> Tensor:
        """Full tensor from all ranks' shards, in rank order. Unlike the reference, which concatenates on the
        host (state_actions.py:50-51), the result stays on the HIP device."""
        if len(tensors) != self.world_size:
            raise ValueError(f"undo needs {self.world_size} shards, got {len(tensors)}")
        full = self.full_shape([tuple(t.shape) for t in tensors])
        specs = [self.spec(full, r) for r in range(self.world_size)]
        return concat_specs(list(tensors), specs)


class Split(SegmentedAction):
    """XXXXXXXXXXXXXXX -> (world_size = 3) -> [XXXXX, XXXXX, XXXXX]; uneven lengths as torch.tensor_split
    (reference: state_actions.py:39-51)."""

    def __init__(self, world_size: int, dim: int):
        super().__init__()
        self.world_size = world_size
        self.dim = dim

    def _dim_for(self, ndim: int) -> int:
        return normalize_dim(self.dim, ndim)

    def spec(self, shape: Sequence[int], rank: int) -> SliceSpec:
        dim = self._dim_for(len(shape))
        return SliceSpec(tuple(shape), dim, (tensor_split_range(shape[dim], self.world_size, rank),))


class Scale(StateAction):
    """Every rank keeps tensor / world_size, so that a later sum over ranks restores it
    (reference: state_actions.py:54-63)."""

    def __init__(self, world_size: int):
        super().__init__()
        self.world_size = world_size

    def __call__(self, tensor: Tensor, rank: int) -> Tensor:
        if tensor.device.type == "meta":
            return torch.empty_like(tensor)
        if tensor.device.type == "cpu":
            _native.lib()  # no host implementation: fail before touching the device if the library is absent
            tensor = tensor.to(torch.device("cuda", torch.cuda.current_device()))
        return _native.scale(tensor, self.world_size)

    def undo(self, tensors: Sequence[Tensor]) -> Tensor:
        first = tensors[0]
        if first.device.type == "meta":
            return torch.empty_like(first)
        return _native.scale(first, self.world_size, multiply=True)


class SplitInChunks(Split):
    """AAABBBCCCDDDEEE -> (world_size = 3, chunk_size = 3) -> [AAABBB, CCCDDD, EEE]: split that keeps
    chunks (attention heads) whole (reference: state_actions.py:66-90)."""

    def __init__(self, world_size: int, dim: int, chunk_size: int, optional: bool = False):
        super().__init__(world_size, dim)
        self.chunk_size = chunk_size
        self.optional = optional

    def __call__(self, tensor: Optional[Tensor], rank: int) -> Optional[Tensor]:
        if tensor is None and self.optional:
            return None
        return super().__call__(tensor, rank)

    def spec(self, shape: Sequence[int], rank: int) -> SliceSpec:
        dim = self._dim_for(len(shape))
        assert shape[dim] % self.chunk_size == 0, tuple(shape)
        start, length = tensor_split_range(shape[dim] // self.chunk_size, self.world_size, rank)
        return SliceSpec(tuple(shape), dim, ((start * self.chunk_size, length * self.chunk_size),))


class SplitInGroupedChunks(Split):
    """AABBCCDDEE AABBCCDDEE AABBCCDDEE -> (world_size = 3, num_groups = 3, chunk_size = 2) ->
    [AABB AABB AABB, CCDD CCDD CCDD, EE EE EE]: the axis is `num_groups` equal groups laid end to end (a fused
    QKV weight); every group is split in whole chunks and a rank keeps its piece of every group
    (reference: state_actions.py:93-119). `dim` must not be negative."""

    def __init__(self, world_size: int, dim: int, num_groups: int, chunk_size: int) -> None:
        super().__init__(world_size, dim)
        if dim < 0:
            raise ValueError("SplitInGroupedChunks needs a non-negative dim")
        self.num_groups = num_groups
        self.chunk_size = chunk_size

    def spec(self, shape: Sequence[int], rank: int) -> SliceSpec:
        dim = self.dim
        n = shape[dim]
        group = n // self.num_groups
        if group * self.num_groups != n or group % self.chunk_size != 0:
            raise RuntimeError(
                f"shape {tuple(shape)} is invalid for {self.num_groups} groups of chunks of {self.chunk_size} on dim {dim}"
            )
        start, length = tensor_split_range(group // self.chunk_size, self.world_size, rank)
        segs = tuple((g * group + start * self.chunk_size, length * self.chunk_size) for g in range(self.num_groups))
        return SliceSpec(tuple(shape), dim, segs)
