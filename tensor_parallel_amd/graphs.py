"""One forward of a module recorded as a HIP graph and replayed.

The reference has no counterpart: its forwards are Python all the way (src/tensor_parallel/tensor_parallel.py:139-161), and
a small model spends most of a forward in the host code between kernel launches. All rank shards of a `TensorParallel`
on one HIP device run on one stream of one thread (the ranks are greenlets of the caller), so a whole forward, the
"sum" / "gather" ops included, can be captured by `torch.cuda.graph` like the forward of a plain module:

    graphed = tp.graphs.capture(model, input_ids=ids, use_cache=False)
    out = graphed(input_ids=other_ids)        # same shapes; new values are copied into the captured inputs

What a capture fixes: every shape, every argument that is not a tensor, and every host-side decision the forward took.
A key/value cache that grows from call to call therefore stays outside; a decode step on one of transformers' static
caches (preallocated, its number of cached positions kept on the device) can be captured once the attention modules
read that count on the device, which `tp.attention.fuse_rotary_(model, assume_no_padding=True)` makes them do:

    cache = StaticCache(config=model.config, max_cache_len=4096)
    model(input_ids=prompt, past_key_values=cache, use_cache=True)                  # the prefill, eager
    step = tp.graphs.capture(model, input_ids=token, past_key_values=cache, use_cache=True)
    logits = step(input_ids=next_token, past_key_values=cache, use_cache=True).logits   # every further token: one replay

The forwards that a capture runs beforehand (to let first uses happen outside it) advance such a cache like any other
forward: the counts of static caches among the arguments, and the tensors named in `restore`, are put back to what
they were before `capture` returns; what those forwards wrote behind the count is overwritten by the steps that follow.
The tensors inside the returned value are the graph's own output buffers: the next replay overwrites them. The recorded
kernels also keep using the scratch buffer that the library gave the capture stream: replays of graphs, and eager work on
a stream that torch hands out again later, are the caller's to order, as the kernels of any two launches that share
memory are.
"""
from __future__ import annotations

import importlib
from typing import Any, List, Sequence, Tuple

import torch
from torch import nn

from . import _native


def _walk(value: Any, leaves: List[Tuple[str, Any]], path: str) -> None:
    if isinstance(value, (tuple, list)):
        for i, item in enumerate(value):
            _walk(item, leaves, f"{path}[{i}]")
    elif isinstance(value, dict):
        for key in value:
            _walk(value[key], leaves, f"{path}[{key!r}]")
    else:
        leaves.append((path, value))


def _rebuild(value: Any, replace) -> Any:
    if isinstance(value, tuple):
        return tuple(_rebuild(v, replace) for v in value)
    if isinstance(value, list):
        return [_rebuild(v, replace) for v in value]
    if isinstance(value, dict):
        return {k: _rebuild(v, replace) for k, v in value.items()}
    return replace(value)


def _caches_with_counts(leaves) -> list:
    """Cache objects among the arguments whose layers keep a count of cached positions on the device, with the per-rank
    siblings that `tp.TensorParallel` gave them."""
    found = []
    for _, value in leaves:
        layers = getattr(value, "layers", None)
        if isinstance(layers, list) and any(hasattr(layer, "cumulative_length") for layer in layers):
            found.append(value)
    return found


def _count_tensors(cache) -> list:
    out = []
    for one in [cache] + list(cache.__dict__.get("_tp_rank_siblings") or []):
        out.append([getattr(layer, "cumulative_length", None) for layer in one.layers])
    return out


class GraphedForward:
    """`module(*args, **kwargs)` captured once; calls replay it on new values of the same tensors."""

    def __init__(self, module: nn.Module, *args, warmup: int = 2, restore: Sequence[torch.Tensor] = (), **kwargs):
        # (the package attribute `tensor_parallel` is the factory function, not the module)
        tp_module = importlib.import_module(__package__ + ".tensor_parallel")

        self.module = module
        devices = {t.device for _, t in self._leaves(args, kwargs) if isinstance(t, torch.Tensor)}
        devices |= {p.device for p in module.parameters()}
        if len(devices) != 1 or next(iter(devices)).type != "cuda":
            raise ValueError(f"graphs.capture: the module and its tensor arguments must live on one HIP device, found {sorted(map(str, devices))}")
        self.device = next(iter(devices))
        shards = getattr(module, "module_shards", None)
        if shards is None:
            shards = getattr(getattr(module, "wrapped_model", None), "module_shards", None)
        if shards is not None and len(shards) > 1 and not tp_module.RANK_GREENLETS:
            raise RuntimeError("graphs.capture: the rank shards run as threads (no greenlet package, or TPAMD_RANK_GREENLETS=0); "
                               "only ranks that run as greenlets of the calling thread share the stream that is captured")
        _native.lib()  # a missing library is reported here, not from inside a capture
        # the captured inputs: clones that the replays read
        self._static_args, self._static_kwargs = _rebuild((args, kwargs), lambda v: v.clone() if isinstance(v, torch.Tensor) else v)
        self._static_leaves = self._leaves(self._static_args, self._static_kwargs)
        # state that the forwards below advance and that is put back afterwards
        caches = _caches_with_counts(self._static_leaves)
        counts_before = [[None if c is None else c.clone() for c in _count_tensors(cache)[0]] for cache in caches]
        kept = [(t, t.clone()) for t in restore]
        with torch.cuda.device(self.device):
            stream = torch.cuda.Stream()
            stream.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(stream), torch.no_grad():
                # first uses (scratch buffers of this stream, lazily built tables) happen outside the capture
                for _ in range(max(1, warmup)):
                    module(*self._static_args, **self._static_kwargs)
            torch.cuda.current_stream().wait_stream(stream)
            torch.cuda.synchronize(self.device)
            self.graph = torch.cuda.CUDAGraph()
            with torch.no_grad(), torch.cuda.graph(self.graph, stream=stream):
                self.output = module(*self._static_args, **self._static_kwargs)
            with torch.no_grad():
                for cache, before in zip(caches, counts_before):
                    for per_rank in _count_tensors(cache):  # the rank siblings exist by now; every rank's layer i holds the same count
                        for count, was in zip(per_rank, before):
                            if isinstance(count, torch.Tensor):
                                count.fill_(0) if was is None else count.copy_(was)
                for tensor, was in kept:
                    tensor.copy_(was)
        self._stream = stream  # its scratch buffer in the library belongs to the graph from now on

    @staticmethod
    def _leaves(args, kwargs) -> List[Tuple[str, Any]]:
        leaves: List[Tuple[str, Any]] = []
        _walk(args, leaves, "args")
        _walk(kwargs, leaves, "kwargs")
        return leaves

    def __call__(self, *args, **kwargs):
        leaves = self._leaves(args, kwargs)
        if [p for p, _ in leaves] != [p for p, _ in self._static_leaves]:
            raise ValueError("graphs: the call's arguments differ in structure from the captured ones")
        for (path, new), (_, static) in zip(leaves, self._static_leaves):
            if isinstance(static, torch.Tensor):
                if not isinstance(new, torch.Tensor) or new.shape != static.shape or new.dtype != static.dtype:
                    got = f"{tuple(new.shape)} {new.dtype}" if isinstance(new, torch.Tensor) else type(new).__name__
                    raise ValueError(f"graphs: {path} was captured as {tuple(static.shape)} {static.dtype}, got {got}")
                static.copy_(new)
            elif isinstance(new, torch.Tensor) or new != static:
                raise ValueError(f"graphs: {path} was captured as {static!r} and cannot change between replays, got {new!r}")
        self.graph.replay()
        return self.output

    def replay(self):
        """Replay on whatever the captured inputs hold now (`static_inputs` to fill them in place)."""
        self.graph.replay()
        return self.output

    @property
    def static_inputs(self):
        return self._static_args, self._static_kwargs


def capture(module: nn.Module, *args, warmup: int = 2, restore: Sequence[torch.Tensor] = (), **kwargs) -> GraphedForward:
    """Record `module(*args, **kwargs)` (inference, no gradients) as a HIP graph; the result is called with new values of
    the same tensors and returns the forward's value. `restore`: tensors that a forward changes in place and that are to
    hold their present values again when this returns."""
    return GraphedForward(module, *args, warmup=warmup, restore=restore, **kwargs)
