"""Nested-structure helpers for replicating forward arguments over shards (reference: src/tensor_parallel/utils.py:44-128)."""
from __future__ import annotations

from itertools import chain
from typing import Dict, Iterator, List, Optional

from torch import nn


def nested_flatten(t) -> Iterator:
    """Leaves of nested lists/tuples/dicts, depth first; dict values in sorted-key order."""
    if isinstance(t, (list, tuple)):
        for item in t:
            yield from nested_flatten(item)
    elif isinstance(t, dict):
        for key in sorted(t):
            yield from nested_flatten(t[key])
    else:
        yield t


def _is_namedtuple(x) -> bool:
    cls = type(x)
    return (
        len(cls.__bases__) == 1
        and cls.__bases__[0] is tuple
        and isinstance(getattr(cls, "_fields", None), tuple)
        and all(isinstance(f, str) for f in cls._fields)
    )


def _pack(leaves: Iterator, like):
    if _is_namedtuple(like):
        return type(like)(*[_pack(leaves, item) for item in like])
    if isinstance(like, (list, tuple)):
        return type(like)(_pack(leaves, item) for item in like)
    if isinstance(like, dict):
        packed = {key: _pack(leaves, like[key]) for key in sorted(like)}
        try:
            return type(like)(packed) if type(like) is not dict else packed
        except Exception:
            return packed
    return next(leaves)


def nested_pack(flat, structure):
    """Inverse of nested_flatten: fill `structure`'s shape with the items of `flat`."""
    return _pack(iter(flat), structure)


def nested_map(fn, structure):
    return nested_pack((fn(x) for x in nested_flatten(structure)), structure)


def find_tied_weight_aliases(module: nn.Module, destination: Optional[Dict[int, List[str]]] = None, prefix: str = "") -> Dict[int, List[str]]:
    """id(tensor) -> every qualified name under which `module` holds that parameter or buffer."""
    if destination is None:
        destination = {}
    for name, tensor in chain(module._parameters.items(), module._buffers.items()):
        if tensor is not None:
            destination.setdefault(id(tensor), []).append(prefix + name)
    for name, child in module._modules.items():
        if child is not None:
            find_tied_weight_aliases(child, destination, prefix + name + ".")
    return destination


def verify_peft_version() -> None:
    """LoRA layers are only understood in the layout of peft >= 0.3.0 (imports.py:4-7)."""
    import sys

    try:
        from importlib.metadata import version

        found = version("peft")
    except Exception:
        found = getattr(sys.modules.get("peft"), "__version__", None)
    if found is None:
        raise ImportError("tensor_parallel only works with peft>=0.3.0")
    if tuple(int(x) for x in found.split(".")[:2] if x.isdigit()) < (0, 3):
        raise ImportError("tensor_parallel only works with peft>=0.3.0")


def check_lora(module: nn.Module) -> bool:
    """True for peft's LoRA-augmented Linear: a class named `Linear` defined in `peft.tuners.lora` (utils.py:131-144)."""
    if type(module).__module__ != "peft.tuners.lora":
        return False
    verify_peft_version()
    return type(module).__name__ == "Linear"
