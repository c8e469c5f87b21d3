"""Head-aligned shape arithmetic used by the model rule tables.

Follows the reference's helpers (src/tensor_parallel/aux_actions.py:18-40): attention weights are split on
whole heads, and the integer attributes of an attention module (head counts, inner widths) shrink to what
one rank owns. The KV-cache plumbing of the reference (aux_actions.py:7-15) is not part of this package.
"""
from __future__ import annotations

from typing import Optional

import torch

from .slicing import SliceSpec, apply_spec, normalize_dim, tensor_split_range


def split_heads(
    tensor: Optional[torch.Tensor], *, dim: int, head_dim: int, rank: int, world_size: int, optional: bool = False
) -> Optional[torch.Tensor]:
    """Rank's part of `tensor` along `dim`, cut on multiples of `head_dim` (aux_actions.py:18-31). A rank that
    would own no head gets a zero tensor shaped like the input without the head axis, as the reference builds."""
    if tensor is None and optional:
        return None
    assert tensor.shape[dim] % head_dim == 0, tensor.shape
    d = normalize_dim(dim, tensor.dim())
    start, length = tensor_split_range(tensor.shape[d] // head_dim, world_size, rank)
    if length == 0:
        shape = list(tensor.shape)
        shape[d] = head_dim
        return torch.zeros(shape, dtype=torch.get_default_dtype())
    return apply_spec(tensor, SliceSpec(tuple(tensor.shape), d, ((start * head_dim, length * head_dim),)))


def split_num_heads(num_heads: int, *, rank: int, world_size: int) -> int:
    """Heads owned by `rank`; never 0, a rank without heads reports 1 (aux_actions.py:34-36)."""
    owned = tensor_split_range(num_heads, world_size, rank)[1]
    return owned if owned != 0 else 1


def split_inner_dim(inner_dim: int, *, rank: int, num_heads: int, world_size: int) -> int:
    """Width owned by `rank` of an axis made of `num_heads` equal heads (aux_actions.py:39-40)."""
    return split_num_heads(num_heads=num_heads, rank=rank, world_size=world_size) * (inner_dim // num_heads)


def alibi_spec(shape, *, rank: int, num_heads: int, world_size: int) -> SliceSpec:
    """Rows of an alibi tensor [batch * num_heads, ...] that belong to `rank`'s heads: the same head range out of
    every batch entry, in batch order (aux_actions.py:43-47)."""
    shape = tuple(shape)
    assert shape[0] % num_heads == 0, shape
    start, length = tensor_split_range(num_heads, world_size, rank)
    segments = tuple((b * num_heads + start, length) for b in range(shape[0] // num_heads))
    return SliceSpec(shape, 0, segments)


def split_alibi(alibi: torch.Tensor, *, rank: int, num_heads: int, world_size: int) -> torch.Tensor:
    """Rank's heads of an alibi tensor of shape [batch_size * num_heads, ...] (aux_actions.py:43-47)."""
    return apply_spec(alibi, alibi_spec(alibi.shape, rank=rank, num_heads=num_heads, world_size=world_size))
