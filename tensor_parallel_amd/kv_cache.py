"""Rank-local attention caches.

Every rank's attention works on its own heads, so its keys and values are its own too. The reference moves tuples
of per-device tensors between ranks for this (`PerDeviceTensors`, `select_kv_for_rank`, `gather_kv`:
src/tensor_parallel/aux_actions.py:7-15, per_device_tensors.py). Current transformers hands the model ONE cache
object that attention layers write into; here that object is given a sibling per extra rank (made when the cache is
first seen, while it is still empty), rank r's modules are handed sibling r, and batch-level operations on the
caller's object (beam reordering, cropping, batch selection, reset) are repeated on the siblings. Rank 0 writes
into the caller's own object, so what the caller reads from it (the number of cached positions) stays true.
"""
from __future__ import annotations

import copy
import functools
from typing import Any, List

import torch

_BATCH_LEVEL = ("reorder_cache", "crop", "batch_repeat_interleave", "batch_select_indices", "reset")


def is_kv_cache(obj: Any) -> bool:
    """A transformers-style cache object: written by attention layers through `update`, asked for its length."""
    return (not isinstance(obj, (torch.Tensor, tuple, list, dict)) and callable(getattr(obj, "update", None))
            and callable(getattr(obj, "get_seq_length", None)))


def rank_caches(cache: Any, world_size: int) -> List[Any]:
    """The per-rank caches behind `cache`: the object itself for rank 0 and one sibling for each other rank."""
    siblings = cache.__dict__.get("_tp_rank_siblings")
    if siblings is not None:
        if len(siblings) + 1 != world_size:
            raise ValueError(f"this cache was split for {len(siblings) + 1} ranks, not {world_size}")
        return [cache] + siblings
    if cache.get_seq_length() != 0:
        raise NotImplementedError(
            "a cache that already holds keys and values for all heads cannot be handed to rank shards; start from an empty cache"
        )
    siblings = [copy.deepcopy(cache) for _ in range(world_size - 1)]
    for name in _BATCH_LEVEL:
        original = getattr(cache, name, None)
        if original is None:
            continue

        def both(*args, _original=original, _name=name, **kwargs):
            result = _original(*args, **kwargs)
            for sibling in siblings:
                getattr(sibling, _name)(*args, **kwargs)
            return result

        setattr(cache, name, functools.wraps(original)(both))
    cache.__dict__["_tp_rank_siblings"] = siblings
    return [cache] + siblings
