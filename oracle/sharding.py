"""Oracle for the ZeRO-3 side-car: how the parameters a rule table leaves replicated are laid out as one flat
shard per rank, and how the shards recombine (reference: src/tensor_parallel/sharding.py). numpy on raw element
arrays; each function restates the reference's own steps (flatten, tensor_split, concatenate, split_with_sizes)
rather than the offsets the product computes.

TEST INFRASTRUCTURE ONLY, like the rest of this package.

Pinned by (tests/test_oracle_sharding.py): combine(make(x)) == x on ragged sizes; every rank's flat shard has the
same length; the parameter counts of the reference's own test (tests/test_basic.py:110-135: for
Embedding(1337, 64) + LayerNorm(64) + Linear(64, 128) + Linear(128, 10) under the default rules, the sharded model
holds exactly the original count at W = 1, 2 and 4 more at W = 3); torch.tensor_split lengths on every (n, W).
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

import numpy as np


def extract_param_shards(params: Sequence[np.ndarray], rank: int, world_size: int) -> List[np.ndarray]:
    """_extract_param_shards (sharding.py:96-108): rank's section of every flattened parameter."""
    return [np.array_split(p.reshape(-1), world_size)[rank] for p in params]


def make_flat_shards(params_by_rank: Sequence[Sequence[np.ndarray]], world_size: int) -> Tuple[List[np.ndarray], List[List[int]]]:
    """_make_flat_shards (sharding.py:137-157). `params_by_rank[r]` are rank r's copies of the replicated parameters,
    all in the same order. Returns the equally long flat shards and, per rank, the section sizes followed by the
    amount of zero padding."""
    extracted = [extract_param_shards(params_by_rank[r], r, world_size) for r in range(len(params_by_rank))]
    sizes = [[int(s.size) for s in shards] for shards in extracted]
    longest = max(sum(s) for s in sizes)
    sizes_with_pad = [s + [longest - sum(s)] for s in sizes]
    flat = [np.concatenate(list(shards) + [np.zeros(pad[-1], dtype=shards[0].dtype)]) for shards, pad in zip(extracted, sizes_with_pad)]
    return flat, sizes_with_pad


def combine_shards(flat_shards: Sequence[np.ndarray], sizes_with_pad: Sequence[Sequence[int]], shapes: Sequence[Sequence[int]]) -> List[np.ndarray]:
    """_combine_shards (sharding.py:169-180): cut every flat shard at its section sizes, join the sections of one
    parameter in rank order, give it its shape back."""
    sections = [np.split(flat, np.cumsum(sizes)[:-1]) for flat, sizes in zip(flat_shards, sizes_with_pad)]
    return [np.concatenate([sections[r][i] for r in range(len(flat_shards))]).reshape(shape) for i, shape in enumerate(shapes)]
