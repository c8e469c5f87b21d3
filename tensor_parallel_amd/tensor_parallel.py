"""`TensorParallel`: a module split into W rank shards that all live on one HIP device
(reference: src/tensor_parallel/tensor_parallel.py:26-315).

Construction slices the whole state for all ranks with one launch of the region mover. A forward runs the
W shards side by side on the host, as the reference does with W threads (tensor_parallel.py:237-287): here as W
greenlets of the calling thread, or W threads where the greenlet package is missing; they meet in the
"sum" / "gather" ops, which are single-device kernels here. `sharded=True` keeps the parameters the rule table
leaves replicated as flat per-rank shards (`sharding.Sharded`) and recombines them on the device before a forward.
"""
from __future__ import annotations

import contextlib
import functools
import logging
import os
import threading
from operator import attrgetter
from typing import Any, Collection, Optional, Sequence, Union

import torch
from torch import nn

from .autoconfig import get_default_config
from .collectives import GreenTurn, Turn, set_turn_lock
from .config import Config, add_lora_rules
from .int8 import ShardLinearW8
from .kv_cache import is_kv_cache, rank_caches
from .shard import make_shard
from .sharding import Sharded
from .slicing import BatchSlicer, concat_specs
from .state_actions import SegmentedAction
from .utils import nested_flatten, nested_pack

logger = logging.getLogger(__file__)


# keyword names under which transformers modules take the legacy tuple-of-tensors key/value cache
LEGACY_CACHE_KWARGS = ("past_key_values", "past_key_value", "layer_past")


def _holds_tensors(value) -> bool:
    """True for a (nested) tuple or list with a tensor somewhere inside."""
    if isinstance(value, (tuple, list)):
        return any(isinstance(v, torch.Tensor) or _holds_tensors(v) for v in value)
    return False


def canonicalize_device(device: Union[torch.device, str, int]) -> torch.device:
    device = torch.device(device)
    if device.type == "cuda" and device.index is None:
        device = torch.device("cuda", 0)
    return device


def check_device_ids(device_ids: Optional[Sequence[Union[torch.device, str]]]) -> Sequence[torch.device]:
    if device_ids is None:
        device_ids = list(range(torch.cuda.device_count())) if torch.cuda.is_available() else []
        device_ids = [torch.device("cuda", i) for i in device_ids]
    return tuple(canonicalize_device(d) for d in device_ids)


class TensorParallel(nn.Module):
    """Public attributes, as in the reference (tensor_parallel.py:27-108): `module_shards`, `devices`, `device_ids`,
    `output_device_index`, `all_cuda`, `tensor_parallel_config`, `modified_parameters_names`, `param_fractions`,
    `sharding_manager`, `need_delayed_init`, `preserve_shards_when_saving`, `_sanity_check_params`."""

    def __init__(
        self,
        module: nn.Module,
        device_ids: Optional[Sequence[torch.device]] = None,
        output_device: Optional[torch.device] = None,
        output_device_index: Optional[int] = None,
        tensor_parallel_config: Optional[Config] = None,
        delay_init: bool = False,
        distributed: bool = True,
        sharded: bool = True,
        sharded_param_names: Optional[Collection[str]] = None,
    ):
        super().__init__()
        self.devices = check_device_ids(device_ids)
        self.output_device_index = self._pick_output_rank(output_device, output_device_index)
        self.device_ids = [d.index if d.type == "cuda" else None for d in self.devices]
        self.all_cuda = all(d.type == "cuda" for d in self.devices)
        self.need_delayed_init = bool(delay_init)
        self.sharding_manager = None
        self.module_shards = nn.ModuleList()

        if len(self.devices) < 2:  # nothing to split: the module itself is the only shard
            self.module_shards.append(module)
            if self.devices and not delay_init:
                module.to(self.devices[0])
            return

        params_before = sum(p.numel() for p in module.parameters())
        if tensor_parallel_config is None:
            logger.info("No slicing config given: every Linear and Embedding gets the generic rules")
            tensor_parallel_config = get_default_config(module, self.devices)
        self.tensor_parallel_config = add_lora_rules(module, tensor_parallel_config)
        self._slice_into_shards(module, self.tensor_parallel_config.create_collective_ops(self.devices, distributed))
        self._report_replication(params_before)

        # An empty parameter per rank that sits where the rank's shard belongs: `model.cuda()` / `model.to(...)` on
        # the whole wrapper moves it, which forward() then notices. A model built on the meta device keeps them on
        # meta until its weights are loaded.
        on_meta = all(t.device.type == "meta" for t in module.state_dict().values())
        markers = [torch.empty(0, device="meta" if on_meta else d) for d in self.devices]
        self._sanity_check_params = nn.ParameterList([nn.Parameter(m, requires_grad=False) for m in markers])
        self.preserve_shards_when_saving: bool = True
        if sharded:
            self.apply_sharding(sharded_param_names)
        if delay_init:
            # The slicing engine works on the device, so the shards were cut there; they wait in host memory until
            # the first forward puts them back (the reference builds them on the host, tensor_parallel.py:80-81).
            # Flat ZeRO-3 shards belong to the sharding manager and stay where they are.
            for shard in self.module_shards:
                shard.to("cpu")

    def _pick_output_rank(self, output_device, output_device_index) -> int:
        if output_device is not None and output_device_index is not None:
            raise AssertionError("output_device and output_device_index name the same thing: give one of them")
        if output_device is None:
            return 0 if output_device_index is None else output_device_index
        wanted = canonicalize_device(output_device)
        if wanted not in self.devices:
            raise AssertionError(f"output_device {wanted} is not one of device_ids {list(self.devices)}")
        return self.devices.index(wanted)

    def _slice_into_shards(self, module: nn.Module, config_with_ops: Config) -> None:
        """Queues every rank's slicing in one BatchSlicer per device and launches each once."""
        world_size = len(self.devices)
        slicers = {d: BatchSlicer(d if d.type == "cuda" else None) for d in dict.fromkeys(self.devices)}
        self.modified_parameters_names = set()
        for rank, device in enumerate(self.devices):
            shard, touched = make_shard(module, device, config_with_ops, rank=rank, world_size=world_size, batch=slicers[device])
            self.module_shards.append(shard)
            self.modified_parameters_names |= set(touched)
        self.sliced_bytes = sum(slicer.run() for slicer in slicers.values())
        for device, slicer in slicers.items():
            if device.type == "cuda" and slicer.plan is not None:
                torch.cuda.synchronize(device)  # host sources uploaded for the launch are released by close()
            slicer.close()

    def _report_replication(self, params_before: int) -> None:
        """Parameters the rules leave whole exist once per rank; say how much memory that costs."""
        per_shard = [sum(p.numel() for p in shard.parameters()) for shard in self.module_shards]
        if sum(per_shard) < params_before:
            raise AssertionError(f"slicing lost parameters: {params_before} before, {per_shard} in the shards")
        self.param_fractions = tuple(n / params_before for n in per_shard) if params_before else ()
        extra = (sum(self.param_fractions) - 1) / len(self.devices)
        logger.log(
            logging.WARNING if extra >= 0.1 else logging.DEBUG,
            "%d parameters became shards of %s parameters: %.3f%% of the model is held again on every device",
            params_before, per_shard, extra * 100,
        )

    def apply_sharding(self, replicated_param_names: Optional[Collection[str]] = None):
        if self.sharding_manager is not None:
            raise Exception("sharding was applied a second time; construct with `sharded=False` to apply it yourself later")
        self.sharding_manager = Sharded(self, len(self.devices), replicated_param_names)

    def prepare_args_kwargs_for_forward(self, *args, **kwargs):
        """One copy of (args, kwargs) per rank; every tensor is moved to that rank's device (tensor_parallel.py:121-137).
        An attention cache object becomes that rank's own cache (see kv_cache)."""
        if len(self.devices) > 1:
            for name in LEGACY_CACHE_KWARGS:
                if _holds_tensors(kwargs.get(name)):
                    raise NotImplementedError(
                        f"`{name}` is a tuple/list of key and value tensors. Every rank attends over its own heads, so such "
                        "a cache cannot be handed to all ranks; pass a transformers Cache object (for example DynamicCache), "
                        "which gets one sibling per rank, or none."
                    )
        structure = (args, kwargs)
        flat = list(nested_flatten(structure))
        caches = {i: rank_caches(x, len(self.devices)) for i, x in enumerate(flat) if is_kv_cache(x)}
        per_rank = []
        for rank, device in enumerate(self.devices):
            leaves = [
                x.to(device, non_blocking=True) if isinstance(x, torch.Tensor) else (caches[i][rank] if i in caches else x)
                for i, x in enumerate(flat)
            ]
            per_rank.append(nested_pack(leaves, structure))
        return zip(*per_rank)

    def forward(self, *args, **kwargs):
        if self.need_delayed_init:  # shards parked on the host by delay_init=True (tensor_parallel.py:140-143)
            for shard, device in zip(self.module_shards, self.devices):
                shard.to(device)
            self.need_delayed_init = False
        if self.sharding_manager is not None:
            self.sharding_manager.synchronize_weights(self.all_cuda)
        if len(self.module_shards) <= 1:
            return [self.module_shards[0](*args, **kwargs)][self.output_device_index]
        if not all(p.device == d for p, d in zip(self._sanity_check_params, self.devices) if p.device.type != "meta"):
            raise ValueError(
                "the shards are no longer on their devices: the whole TensorParallel module was moved "
                "(`.cuda()` / `.to(device)`), which puts every rank on one device. Build it again instead."
            )
        inputs, kwargs_tup = self.prepare_args_kwargs_for_forward(*args, **kwargs)
        return parallel_apply_simple(self.module_shards, inputs, kwargs_tup, self.devices)[self.output_device_index]

    def set_preserve_shards_when_saving(self, value: bool):
        self.preserve_shards_when_saving = value
        if self.sharding_manager is not None:
            self.sharding_manager.preserve_shards_when_saving = value

    def state_dict(self, *args, **kwargs):
        """Sharded names by default; inside `save_tensor_parallel` the original model's names and full tensors,
        rebuilt with each rule's `undo` (tensor_parallel.py:168-221)."""
        state_dict = super().state_dict(*args, **kwargs)
        if self.preserve_shards_when_saving or len(self.module_shards) <= 1:
            return state_dict
        world_size = len(self.module_shards)
        if any(isinstance(m, ShardLinearW8) for m in self.module_shards[0].modules()):
            raise RuntimeError("tensor_parallel_amd: full weights cannot be rebuilt from int8 Linears (int8.quantize_linears_); "
                               "save the shards as they are (outside save_tensor_parallel)")
        for name in [n for n in state_dict if "_sanity_check_params." in n]:
            del state_dict[name]
        for name in [n for n in state_dict if "tp_wrapped_module." in n]:
            state_dict[name.replace("tp_wrapped_module.", "")] = state_dict.pop(name)
        marker = "module_shards."
        first = next((n for n in state_dict if marker in n), None)
        if first is None:  # nothing is tensor parallel
            return self.process_sharded_state_dict(state_dict, kwargs.get("prefix", ""))
        shards_prefix = first[: first.find(marker) + len(marker)]
        module_prefix = shards_prefix[: -len(marker)]
        rank0 = shards_prefix + "0."
        for key in [n for n in state_dict if n.startswith(rank0)]:
            unsharded = key[len(rank0):]
            pieces = [state_dict.pop(f"{shards_prefix}{r}.{unsharded}") for r in range(world_size)]
            for pattern, action in self.tensor_parallel_config.state_rules.items():
                if pattern.search(unsharded) is not None:
                    state_dict[module_prefix + unsharded] = action.undo(pieces)
                    break
            else:
                state_dict[module_prefix + unsharded] = pieces[0]
        return self.process_sharded_state_dict(state_dict, kwargs.get("prefix", ""))

    def process_sharded_state_dict(self, destination, prefix):
        """The ZeRO-3 parameters, recombined, under their names in the original model (tensor_parallel.py:223-234)."""
        manager = self.sharding_manager
        if manager is not None and hasattr(manager, "flat_shards"):
            manager.synchronize_weights(self.all_cuda)
            for name in manager.sharded_param_names:
                value = attrgetter(name)(self.module_shards[0])
                destination[prefix + name.replace("tp_wrapped_module.", "")] = value
        return destination


try:
    import greenlet as _greenlet
except ImportError:  # the ranks of a shared device are threads then
    _greenlet = None
RANK_GREENLETS = _greenlet is not None and os.environ.get("TPAMD_RANK_GREENLETS", "1") != "0"


def _apply_in_greenlets(modules: Sequence[nn.Module], inputs, kwargs_tup, device: torch.device):
    """The ranks of one device as greenlets of the calling thread. They run on the caller's stream, device and grad mode
    because they are the caller's thread. A rank runs until it has to wait in a collective, which switches back here;
    the ranks get the turn in rotation until all have returned. When a whole rotation passes in which no collective
    completed and no rank finished, the live ranks wait for one that will not come (it has returned or failed): they
    are told to give up."""
    hub = _greenlet.getcurrent()
    turn = GreenTurn(hub)
    results: dict = {}

    def body(i, module, args, kwargs):
        set_turn_lock(turn)  # a greenlet starts with an empty context of its own
        try:
            if not isinstance(args, (list, tuple)):
                args = (args,)
            results[i] = (True, module(*args, **kwargs))
        except BaseException as e:  # noqa: BLE001 - handed to the caller below
            results[i] = (False, e)
            turn.fail()  # its peers must not wait for it

    ranks = [_greenlet.greenlet(functools.partial(body, i, m, a, k), parent=hub)
             for i, (m, a, k) in enumerate(zip(modules, inputs, kwargs_tup))]
    alive = list(range(len(ranks)))
    with torch.cuda.device(device) if device.type == "cuda" else contextlib.nullcontext():
        position = idle = 0
        while alive:
            r = alive[position % len(alive)]
            before = turn.events
            ranks[r].switch()
            if ranks[r].dead:
                alive.remove(r)
                turn.events += 1
            else:
                position += 1
            idle = 0 if turn.events != before else idle + 1
            if idle > len(alive):
                turn.fail()
    failures = [results[i] for i in range(len(ranks)) if not results[i][0]]
    if failures:
        real = [e for ok, e in failures if not isinstance(e, threading.BrokenBarrierError)]
        raise (real[0] if real else failures[0][1])
    return [results[i][1] for i in range(len(ranks))]


def parallel_apply_simple(modules: Sequence[nn.Module], inputs, kwargs_tup, devices: Sequence[torch.device]):
    """Run shard i on (inputs[i], kwargs_tup[i]), all shards side by side (greenlets of this thread when they share a
    device and the greenlet package is there, else a thread each); re-raise the first failure (tensor_parallel.py:237-287)."""
    assert len(modules) == len(inputs)
    kwargs_tup = kwargs_tup if kwargs_tup is not None else ({},) * len(modules)
    assert len(modules) == len(kwargs_tup)
    results: dict = {}
    lock = threading.Lock()
    grad_enabled = torch.is_grad_enabled()
    # ranks that share one device take turns on the host (see collectives.set_turn_lock)
    shared = len(modules) > 1 and all(d.type == "cuda" and d == devices[0] for d in devices)
    if shared and RANK_GREENLETS:
        return _apply_in_greenlets(modules, inputs, kwargs_tup, devices[0])
    turn = Turn() if shared else None
    # a thread starts on its device's default stream: the rank threads work on the stream the caller is on instead, so that
    # what the caller enqueued before the forward is ordered before it and what it enqueues afterwards behind it
    streams = [torch.cuda.current_stream(d) if d.type == "cuda" else None for d in devices]

    def worker(i, module, args, kwargs, device):
        torch.set_grad_enabled(grad_enabled)
        if turn is not None:
            turn.lock.acquire()
            set_turn_lock(turn)
        try:
            if streams[i] is not None:
                with torch.cuda.stream(streams[i]):
                    _run(i, module, args, kwargs, device)
            else:
                _run(i, module, args, kwargs, device)
        finally:
            if turn is not None:
                set_turn_lock(None)
                turn.lock.release()

    def _run(i, module, args, kwargs, device):
        try:
            if device.type == "cuda":
                torch.cuda.set_device(device)
            if not isinstance(args, (list, tuple)):
                args = (args,)
            out = module(*args, **kwargs)
            with lock:
                results[i] = (True, out)
        except BaseException as e:
            with lock:
                results[i] = (False, e)
            # a rank that fails must not leave its peers waiting in a collective
            if turn is not None:
                turn.fail()
            for m in module.modules():
                for rules in (getattr(m, "input_actions", {}), getattr(m, "output_actions", {})):
                    for op in rules.values():
                        barrier = getattr(op, "_barrier", None)
                        if barrier is not None:
                            barrier.abort()

    threads = [
        threading.Thread(target=worker, args=(i, m, a, k, d))
        for i, (m, a, k, d) in enumerate(zip(modules, inputs, kwargs_tup, devices))
    ]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    # barriers aborted by a failing rank are usable again for the next forward
    failures = [r for r in results.values() if not r[0]]
    if failures:
        for module in modules:
            for m in module.modules():
                for rules in (getattr(m, "input_actions", {}), getattr(m, "output_actions", {})):
                    for op in rules.values():
                        barrier = getattr(op, "_barrier", None)
                        if barrier is not None:
                            barrier.reset()
        real = [e for ok, e in failures if not isinstance(e, threading.BrokenBarrierError)]
        raise (real[0] if real else failures[0][1])
    return [results[i][1] for i in range(len(modules))]
