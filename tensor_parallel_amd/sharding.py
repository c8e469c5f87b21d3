"""ZeRO-3 side-car: parameters that the rule table leaves replicated are kept as one flat shard per rank and put
back together before a forward (reference: src/tensor_parallel/sharding.py:17-180).

Layout, as in the reference: the replicated parameters are taken in a fixed order, each one flattened and cut
like `torch.tensor_split(flat, world_size)`; rank r's flat shard is its sections laid end to end, zero-padded to
the longest rank's length. Building the shards and recombining them are both one launch of the region mover over
a table of contiguous byte runs. All ranks live on one HIP device here, so recombination writes ONE buffer that
every rank's modules view (256-byte aligned per parameter), where the reference hands every device its own
gathered copy. The buffer is refreshed in place when a flat shard's version counter changes. Recombination is
not differentiable: the flat shards do not require grad.
"""
from __future__ import annotations

import logging
from typing import Collection, Dict, List, Optional, Sequence, Tuple

import torch
from torch import nn

from . import _native
from .slicing import tensor_split_range

logger = logging.getLogger(__file__)

GATHER_ALIGN_BYTES = 256


def flat_layout(numels: Sequence[int], world_size: int) -> Tuple[List[List[Tuple[int, int]]], List[int], int]:
    """For every rank the (start, length) section of every flattened parameter, the zero padding that brings the
    rank's flat shard to the common length, and that length (sharding.py:137-150)."""
    sections = [[tensor_split_range(n, world_size, rank) for n in numels] for rank in range(world_size)]
    totals = [sum(length for _, length in per_rank) for per_rank in sections]
    flat_len = max(totals) if totals else 0
    return sections, [flat_len - t for t in totals], flat_len


def _identity(p: torch.Tensor):
    return (p.data_ptr(), p.storage_offset(), tuple(p.stride()), tuple(p.shape))


def find_all_occurences(model: nn.Module, param_names: Sequence[str]) -> Tuple[List[Tuple[nn.Module, str]], ...]:
    """Every (submodule, attribute) under which each named parameter is reachable, tied copies included
    (sharding.py:111-134)."""
    wanted = set(param_names)
    name_of: Dict[tuple, str] = {}
    for module_name, sub in model.named_modules():
        for pname, p in sub.named_parameters(recurse=False):
            full = f"{module_name}.{pname}" if module_name else pname
            if full in wanted:
                name_of[_identity(p)] = full
    found: Dict[str, List[Tuple[nn.Module, str]]] = {name: [] for name in param_names}
    for module_name, sub in model.named_modules():
        for pname, p in sub.named_parameters(recurse=False):
            full = f"{module_name}.{pname}" if module_name else pname
            full = name_of.get(_identity(p), full)
            if full in found:
                found[full].append((sub, pname))
    for name in param_names:
        assert found[name], f"could not find param {name} in model"
    return tuple(found[name] for name in param_names)


class Sharded(nn.Module):
    def __init__(self, module, world_size: Optional[int] = None, replicated_param_names: Optional[Collection[str]] = None):
        """Partition the named parameters (default: all that tensor parallelism did not touch) of a TensorParallel
        module between its ranks, so that every value is stored once."""
        super().__init__()
        self.preserve_shards_when_saving: bool = True
        module_shards = module.module_shards
        if len(module_shards) == 1:
            return
        if replicated_param_names is None:
            if any(p.device.type == "meta" for p in module.parameters()):
                raise RuntimeError(
                    "Trying to shard a model containing 'meta' parameters. Please set `sharded=False` during model creation and call `.apply_sharding()` only after dispatch"
                )
            modified = module.modified_parameters_names
            replicated_param_names = [n for n, _ in module_shards[0].named_parameters() if n not in modified]
        names = tuple(replicated_param_names)
        # one flat buffer holds one dtype: the dtype that most of the named elements have is sharded, parameters of any
        # other dtype (fp32 norms beside 16-bit weights) stay replicated on every rank
        by_name0 = dict(module_shards[0].named_parameters())
        volume = {}
        for n in names:
            if n in by_name0:
                volume[by_name0[n].dtype] = volume.get(by_name0[n].dtype, 0) + by_name0[n].numel()
        if len(volume) > 1:
            main = max(volume, key=volume.get)
            left = [n for n in names if n in by_name0 and by_name0[n].dtype != main]
            logger.warning(f"{len(left)} parameters are not {main} and stay replicated on every rank: {left[:3]}{'...' if len(left) > 3 else ''}")
            names = tuple(n for n in names if n not in left)
        self.sharded_param_names = names
        if not names:
            logger.warning("Did not find any parameters to shard")
            return
        self.world_size = world_size = world_size if world_size is not None else len(module_shards)
        if world_size != len(module_shards):
            raise ValueError(f"world_size {world_size} does not match the {len(module_shards)} module shards")

        per_rank = []
        for shard in module_shards:
            by_name = dict(shard.named_parameters())
            missing = [n for n in names if n not in by_name]
            if missing:
                raise KeyError(f"parameters {missing[:3]} are not in the module shards")
            per_rank.append([by_name[n] for n in names])
        first = per_rank[0][0]
        for params in per_rank:
            for n, p in zip(names, params):
                if p.dtype != first.dtype or p.device != first.device or p.device.type != "cuda":
                    raise ValueError(
                        f"sharded parameters must share one dtype on one HIP device; {n} is {p.dtype} on {p.device}, "
                        f"{names[0]} is {first.dtype} on {first.device}"
                    )
        self._sharded_param_shapes = [tuple(p.shape) for p in per_rank[0]]
        numels = [p.numel() for p in per_rank[0]]
        self._sections, pads, flat_len = flat_layout(numels, world_size)
        self._shard_sizes_with_pad = [[length for _, length in sec] + [pad] for sec, pad in zip(self._sections, pads)]
        itemsize = first.element_size()

        # build the flat shards: rank r's sections are read from rank r's own copy of each parameter
        flats, jobs, keep = [], [], []
        for rank, (params, sections, pad) in enumerate(zip(per_rank, self._sections, pads)):
            flat = torch.empty(flat_len, dtype=first.dtype, device=first.device)
            if pad:
                flat[flat_len - pad:].zero_()
            at = 0
            for p, (start, length) in zip(params, sections):
                if length:
                    src = p.detach().contiguous()
                    keep.append(src)
                    nbytes = length * itemsize
                    jobs.append((src.data_ptr() + start * itemsize, flat.data_ptr() + at * itemsize, 1, nbytes, nbytes, nbytes))
                at += length
            flats.append(flat)
        _native.run_copy_jobs(jobs, first.device)
        torch.cuda.current_stream(first.device).synchronize()  # the originals are dropped below
        del keep
        self.flat_shards = nn.ParameterList([nn.Parameter(f, requires_grad=False) for f in flats])

        # all places the parameters are used from, per rank; the originals go away
        self.param_occurences_by_rank = [find_all_occurences(shard, names) for shard in module_shards]
        for occurences_of_rank in self.param_occurences_by_rank:
            for occurences in occurences_of_rank:
                for submodule, pname in occurences:
                    submodule._parameters.pop(pname, None)
                    setattr(submodule, pname, None)

        # one buffer for the recombined parameters, every parameter on a 256-byte boundary
        step = GATHER_ALIGN_BYTES // itemsize
        self._bases, at = [], 0
        for n in numels:
            self._bases.append(at)
            at += -(-n // step) * step
        self._gathered_numel = at
        self._gathered: Optional[torch.Tensor] = None
        self._plan: Optional[_native.CopyPlan] = None
        self._plan_key = None
        self._last_versions = None

    def _ensure_plan(self) -> None:
        flats = list(self.flat_shards)
        key = tuple(f.data_ptr() for f in flats) + (flats[0].dtype, flats[0].device)
        if self._plan is not None and key == self._plan_key:
            return
        first = flats[0]
        itemsize = first.element_size()
        self._gathered = torch.empty(self._gathered_numel, dtype=first.dtype, device=first.device)
        jobs = []
        for rank, (flat, sections) in enumerate(zip(flats, self._sections)):
            at = 0
            for base, (start, length) in zip(self._bases, sections):
                if length:
                    nbytes = length * itemsize
                    jobs.append((flat.data_ptr() + at * itemsize, self._gathered.data_ptr() + (base + start) * itemsize, 1, nbytes, nbytes, nbytes))
                at += length
        if self._plan is not None:
            torch.cuda.current_stream(self._plan.device).synchronize()
            self._plan.close()
        self._plan = _native.CopyPlan(jobs, first.device)
        self._plan_key = key
        self._last_versions = None
        views = [self._gathered[base: base + torch.Size(shape).numel()].view(shape) for base, shape in zip(self._bases, self._sharded_param_shapes)]
        for occurences_of_rank in self.param_occurences_by_rank:
            assert len(views) == len(occurences_of_rank)
            for view, occurences in zip(views, occurences_of_rank):
                for submodule, pname in occurences:
                    setattr(submodule, pname, view)

    def synchronize_weights(self, all_cuda: bool = True):
        """Recombine the flat shards into the parameters the rank modules use; a no-op while no flat shard has been
        written since the last call (sharding.py:69-84)."""
        if not hasattr(self, "flat_shards"):
            return
        self._ensure_plan()
        versions = tuple(f._version for f in self.flat_shards)
        if versions == self._last_versions:
            logger.debug("Using previously gathered parameters")
            return
        logger.debug("Gathering sharded parameters")
        self._plan.run()
        self._last_versions = versions

    def state_dict(self, *args, **kwargs):
        if self.preserve_shards_when_saving:
            return super().state_dict(*args, **kwargs)
        return kwargs["destination"]
