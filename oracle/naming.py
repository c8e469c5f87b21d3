"""Oracle for parameter renaming and state-dict conversion, in plain Python over the oracle's slicing."""
from __future__ import annotations

import re
from typing import Callable, Dict, Iterable, List, Mapping, Sequence, Tuple

import numpy as np

WRAPPED = "tp_wrapped_module."


def get_parameter_name_mapping(names: Iterable[str], module_patterns: Sequence[str]) -> Dict[str, str]:
    """config.py:157-191. `module_patterns` are the regex strings of the input rules followed by those of the
    output rules. A trailing '$' is dropped; '\\.' is appended unless the pattern ends with '.'; duplicates
    collapse; for every pattern that matches a name, 'tp_wrapped_module.' goes in at the end of the match,
    rightmost position first."""
    stripped = [p[:-1] if p.endswith("$") else p for p in module_patterns]
    unique = {p if p.endswith(".") else p + r"\." for p in stripped}
    names = list(names)
    cuts: Dict[str, List[int]] = {n: [] for n in names}
    for p in unique:
        rx = re.compile(p)
        for n in names:
            m = rx.search(n)
            if m is not None:
                cuts[n].append(m.span()[1])
    out = {}
    for n in names:
        new = n
        for pos in sorted(cuts[n])[::-1]:
            new = new[:pos] + WRAPPED + new[pos:]
        out[n] = new
    return out


# A state rule for the oracle: (regex string, function(array, rank) -> array)
StateRule = Tuple[str, Callable[[np.ndarray, int], np.ndarray]]


def convert_state_dict(
    state: Mapping[str, np.ndarray],
    state_rules: Sequence[StateRule],
    module_patterns: Sequence[str],
    world_size: int,
    for_pretrained: bool = False,
) -> Dict[str, object]:
    """dispatch.py:75-131: for every rank, slice by the first matching rule (unmatched tensors pass through
    as the same object), rename, prefix with 'module_shards.{rank}.', add '_sanity_check_params.{rank}'."""
    compiled = [(re.compile(p), f) for p, f in state_rules]
    out: Dict[str, object] = {}
    for rank in range(world_size):
        shard: Dict[str, object] = {}
        for name, value in state.items():
            for rx, fn in compiled:
                if rx.search(name) is not None:
                    shard[name] = fn(value, rank)
                    break
            else:
                shard[name] = value
        mapping = get_parameter_name_mapping(shard.keys(), module_patterns)
        shard = {mapping[n]: v for n, v in shard.items()}
        for n, v in shard.items():
            out[f"module_shards.{rank}.{n}"] = v
        out[f"_sanity_check_params.{rank}"] = np.empty(0, dtype=np.float32)
    if for_pretrained:
        out = {"wrapped_model." + n: v for n, v in out.items()}
    return out
