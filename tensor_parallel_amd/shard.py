"""Shard builder: one rank's copy of a module, with sliced state, wrapped submodules and fixed attributes
(reference: src/tensor_parallel/shard.py:16-187)."""
from __future__ import annotations

import logging
from copy import deepcopy
from itertools import chain
from typing import Collection, Dict, Optional, Tuple

import torch
from torch import nn

from . import _native
from .config import Config, MappedActions, ModuleRules, get_parameter_name_mapping
from .shard_modules import install_shard_kernels, is_conv1d
from .slicing import BatchSlicer
from .state_actions import SegmentedAction
from .wrapper import TensorParallelWrapper

logger = logging.getLogger(__file__)


def _placeholder(x: torch.Tensor, device: torch.device):
    target = x.device if x.device.type == "meta" else device
    empty = torch.empty(0, dtype=x.dtype, device=target, requires_grad=x.requires_grad)
    return nn.Parameter(empty, x.requires_grad) if isinstance(x, nn.Parameter) else empty


def make_shard(
    module: nn.Module,
    device: torch.device,
    config: Config,
    *,
    rank: int,
    world_size: int,
    batch: Optional[BatchSlicer] = None,
) -> Tuple[nn.Module, Collection[str]]:
    """Rank `rank`'s shard of `module` on `device`, and the (sharded-model) names of the tensors that were split.

    The module tree is copied without its tensors (every parameter and buffer is replaced by an empty
    placeholder through deepcopy's memo, which also keeps tied weights tied), then `process_state_` fills the
    copy with sliced data (shard.py:34-56). With `batch`, the slicing kernels are only queued: the caller
    launches them, once, for all ranks.
    """
    assert len(list(module.children())) != 0, "Please ensure module is a container (e.g. Sequential), not a single layer"
    device = torch.device(device)
    source = dict(chain(module.named_parameters(), module.named_buffers()))
    if device.type != "cuda" and any(t.device.type != "meta" for t in source.values()):
        raise _native.NativeLibraryError(
            f"shards must live on a HIP device, got {device}: tensor_parallel_amd has no host implementation"
        )
    memo = {id(t): _placeholder(t, device) for t in source.values()}
    shard = deepcopy(module, memo=memo)
    del module, memo

    own_batch = batch is None
    if own_batch:
        batch = BatchSlicer(device if device.type == "cuda" else None)
    modified = process_state_(shard, source, config, rank=rank, world_size=world_size, batch=batch)
    if own_batch:
        batch.run()
        batch.close()
    del source

    wrapped: Dict[nn.Module, nn.Module] = {}
    with torch.no_grad():
        for name, sub in shard.named_modules():
            if sub in wrapped:
                continue
            new = _maybe_wrap_submodule(config, name, sub, rank=rank, world_size=world_size)
            if new is not sub:
                wrapped[sub] = new
    for parent in list(shard.modules()):
        for child_name, child in list(parent.named_children()):
            if child in wrapped and not isinstance(parent, TensorParallelWrapper):
                setattr(parent, child_name, wrapped[child])

    fix_general_attributes(shard)
    install_shard_kernels(shard)
    shard = wrapped.get(shard, shard)
    return shard, set(get_parameter_name_mapping(modified, config).values())


def _maybe_wrap_submodule(config: Config, name: str, module: nn.Module, *, rank: int, world_size: int) -> nn.Module:
    """Apply attr rules in place; wrap the module if it has input or output rules (shard.py:99-113)."""
    attr_actions = find_matching_actions("attr", name, config.attr_rules)
    input_actions = find_matching_actions("input", name, config.input_rules)
    output_actions = find_matching_actions("output", name, config.output_rules)
    if attr_actions:
        process_attrs_(module, attr_actions, rank=rank, world_size=world_size)
    if input_actions or output_actions:
        return TensorParallelWrapper(module, input_actions, output_actions, rank=rank, world_size=world_size)
    return module


def find_matching_actions(action_type: str, name: str, rules: ModuleRules) -> MappedActions:
    """Union of the rules of every pattern that matches `name`; two different actions for one key raise
    (shard.py:116-129). Digit-string keys address positions."""
    found: MappedActions = {}
    for pattern, actions in rules.items():
        if pattern.search(name) is None:
            continue
        for key, action in actions.items():
            if isinstance(key, str) and key.strip().isdigit():
                key = int(key)
            if key in found and found[key] != action:
                raise ValueError(f"Found conflicting {action_type} rule for module {name}, key {key}: {found[key]} vs {action}")
            found[key] = action
    return found


@torch.no_grad()
def process_state_(
    sharded_module: nn.Module,
    source_tensors: Dict[str, torch.Tensor],
    config: Config,
    *,
    rank: int,
    world_size: int,
    batch: Optional[BatchSlicer] = None,
) -> Collection[str]:
    """Fill the shard's parameters and buffers: the first state rule whose pattern matches a name decides its
    action, unmatched tensors are copied whole (shard.py:132-166). Splitting actions go to `batch`."""
    modified = set()
    unused = set(config.state_rules.keys())
    own_batch = batch is None
    if own_batch:
        batch = BatchSlicer()
    # [in, out] weights that the shard's kernels want with the `in` axis fastest: sliced and transposed in one pass
    in_out_weights = {f"{prefix}.weight" if prefix else "weight" for prefix, sub in sharded_module.named_modules() if is_conv1d(sub)}
    for name, state in chain(sharded_module.named_parameters(), sharded_module.named_buffers()):
        src = source_tensors[name]
        for pattern, action in config.state_rules.items():
            if pattern.search(name) is not None:
                if isinstance(action, SegmentedAction) and src is not None:
                    new = batch.add(src, action.spec(tuple(src.shape), rank), k_major=name in in_out_weights)
                else:
                    new = action(src, rank=rank)
                    new = new.clone() if new.device == state.device else new
                modified.add(name)
                unused.discard(pattern)
                break
        else:
            new = src.clone()
        # the shard owns its storage and sits on the shard's device
        state.data = new.detach().to(state.device).requires_grad_(state.requires_grad)
    if own_batch:
        batch.run()
        batch.close()
    if unused:
        logger.warning(f"The following patterns in state_rules were unused: {[str(p) for p in unused]}")
    return modified


def process_attrs_(module: nn.Module, actions: MappedActions, rank: int, world_size: int):
    """Rewrite module attributes in place, once (shard.py:169-174)."""
    assert not getattr(module, "__tensor_parallel_process_attrs", False), "process_attrs was called more than once"
    for attr, action in actions.items():
        if not hasattr(module, attr):
            # rule tables name the attributes of the model code they were written for; other versions of
            # that code may compute the value from tensor shapes instead
            logger.debug(f"attr rule for {attr!r} skipped: {type(module).__name__} has no such attribute")
            continue
        setattr(module, attr, action(getattr(module, attr), rank=rank))
    module.__tensor_parallel_process_attrs = True


@torch.no_grad()
def fix_general_attributes(sharded_module: nn.Module):
    """Make well-known attributes agree with the sliced weights: Linear in/out features (shard.py:177-187)."""
    for module in sharded_module.modules():
        if isinstance(module, nn.Linear):
            module.out_features, module.in_features = module.weight.shape
