"""Oracle for the slicing actions. Works on numpy arrays of any dtype (bf16 travels as uint16: slicing is
pure element movement). Each function restates the reference's own steps - reshape, split, flatten - rather
than the closed-form index ranges the product uses, so that the two can disagree."""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np


def tensor_split(a: np.ndarray, world_size: int, dim: int) -> List[np.ndarray]:
    """torch.tensor_split(a, world_size, dim) with an integer section count: the first n % W sections get
    one extra element. numpy's array_split follows the same rule."""
    return np.array_split(a, world_size, axis=dim)


def split(a: np.ndarray, world_size: int, dim: int, rank: int) -> np.ndarray:
    """Split.__call__ (state_actions.py:47-48)."""
    return np.ascontiguousarray(tensor_split(a, world_size, dim)[rank])


def split_undo(parts: Sequence[np.ndarray], dim: int) -> np.ndarray:
    """Split.undo / SplitInChunks.undo: concatenation on dim (state_actions.py:50-51, 89-90)."""
    return np.concatenate(list(parts), axis=dim)


def split_in_chunks(a: Optional[np.ndarray], world_size: int, dim: int, chunk_size: int, rank: int, optional: bool = False):
    """SplitInChunks.__call__ (state_actions.py:76-87): view the axis as (n/chunk, chunk), split the chunk
    axis, flatten the two axes back."""
    if a is None and optional:
        return None
    assert a.shape[dim] % chunk_size == 0, a.shape
    if dim < 0:
        dim = (a.ndim + dim) % a.ndim
    shape = list(a.shape)
    shape[dim] //= chunk_size
    shape.insert(dim + 1, chunk_size)
    part = tensor_split(a.reshape(shape), world_size, dim)[rank]
    out_shape = list(part.shape)
    out_shape[dim : dim + 2] = [part.shape[dim] * part.shape[dim + 1]]
    return np.ascontiguousarray(part).reshape(out_shape)


def split_in_grouped_chunks(a: np.ndarray, world_size: int, dim: int, num_groups: int, chunk_size: int, rank: int) -> np.ndarray:
    """SplitInGroupedChunks.__call__ (state_actions.py:101-109): view the axis as (groups, chunks, chunk),
    split the chunks axis, flatten the three axes back."""
    shape = list(a.shape)
    shape[dim] //= num_groups
    shape.insert(dim, num_groups)
    shape[dim + 1] //= chunk_size
    shape.insert(dim + 2, chunk_size)
    part = tensor_split(a.reshape(shape), world_size, dim + 1)[rank]
    out_shape = list(part.shape)
    out_shape[dim : dim + 3] = [part.shape[dim] * part.shape[dim + 1] * part.shape[dim + 2]]
    return np.ascontiguousarray(part).reshape(out_shape)


def split_in_grouped_chunks_undo(parts: Sequence[np.ndarray], dim: int, num_groups: int) -> np.ndarray:
    """SplitInGroupedChunks.undo (state_actions.py:111-119): regroup every shard as (groups, rest),
    concatenate on the rest axis, flatten."""
    grouped = []
    for p in parts:
        shape = list(p.shape)
        shape[dim] //= num_groups
        shape.insert(dim, num_groups)
        grouped.append(p.reshape(shape))
    cat = np.concatenate(grouped, axis=dim + 1)
    out_shape = list(cat.shape)
    out_shape[dim : dim + 2] = [cat.shape[dim] * cat.shape[dim + 1]]
    return cat.reshape(out_shape)


def in_axis_fastest(shard: np.ndarray) -> np.ndarray:
    """Memory image of a 2-D shard stored with its first axis fastest: the row-major array of its transpose. A weight
    that the model code keeps as [in, out] (transformers' Conv1D, sliced by slicing_configs.py:192-201) read this way
    is the [out, in] matrix of the equivalent torch.nn.Linear. Pinned by numpy's own transpose."""
    assert shard.ndim == 2, shard.shape
    return np.ascontiguousarray(shard.T)


def scale(a: np.ndarray, world_size: int) -> np.ndarray:
    """Scale.__call__ for float32 input (state_actions.py:59-60)."""
    return (a / np.float32(world_size)).astype(a.dtype)


def split_num_heads(num_heads: int, rank: int, world_size: int) -> int:
    """aux_actions.py:34-36: length of the rank's piece of a length-num_heads axis, but never 0."""
    owned = tensor_split(np.empty(num_heads, dtype=np.uint8), world_size, 0)[rank].size
    return owned if owned != 0 else 1


def split_inner_dim(inner_dim: int, rank: int, num_heads: int, world_size: int) -> int:
    """aux_actions.py:39-40."""
    return split_num_heads(num_heads, rank, world_size) * (inner_dim // num_heads)
