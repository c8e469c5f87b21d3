"""Slicing rules of a tensor-parallel model (reference: src/tensor_parallel/config.py:37-191).

`Config` keeps four regex-keyed rule sets:
  state_rules   parameter/buffer name -> StateAction       (first match in dict order wins)
  input_rules   module name -> {argument: action}          (all matches merge; a clash is an error)
  output_rules  module name -> {output index: action}
  attr_rules    module name -> {attribute: callable}
Action values for inputs/outputs are a StateAction, a callable `(x, rank=...)`, or one of the strings
"split d", "scale", "sum", "gather d".
"""
from __future__ import annotations

import dataclasses
import logging
import re
from itertools import chain
from typing import Any, Callable, Dict, Iterable, Mapping, Sequence, Union

import torch
from torch import nn

from .collectives import DeviceAllGather, DeviceAllReduce
from .state_actions import LegacyStateAction, StateAction

logger = logging.getLogger(__file__)

Arg = Union[int, str]
Action = Callable[[Any, int], Any]
MappedActions = Dict[Arg, Action]
StateRules = Dict[re.Pattern, StateAction]
ModuleRules = Dict[re.Pattern, MappedActions]


def convert_legacy_state_action(state_action: Any) -> StateAction:
    """Accept the pre-StateAction rule forms: a bare callable, or a (split, undo) pair (config.py:68-83)."""
    if isinstance(state_action, StateAction):
        return state_action
    if callable(state_action):
        logger.warning("Using callables in state_rules is deprecated. Please use StateAction instead.")
        return LegacyStateAction(state_action)
    if isinstance(state_action, tuple) and len(state_action) == 2 and all(callable(f) for f in state_action):
        logger.warning("Using tuples of callables in state_rules is deprecated. Please use StateAction instead.")
        return LegacyStateAction(*state_action)
    raise Exception(f"Can't convert {state_action} of type {type(state_action)} to StateAction")


def _compiled(rules: Mapping) -> dict:
    return {re.compile(pattern): value for pattern, value in rules.items()}


@dataclasses.dataclass
class Config:
    state_rules: Dict[str, StateAction]
    input_rules: Dict[str, MappedActions]
    output_rules: Dict[str, MappedActions]
    attr_rules: Dict[str, MappedActions]

    def __init__(self, state_rules, input_rules, output_rules, attr_rules):
        self.state_rules = _compiled({p: convert_legacy_state_action(a) for p, a in state_rules.items()})
        self.input_rules = _compiled(input_rules)
        self.output_rules = _compiled(output_rules)
        self.attr_rules = _compiled(attr_rules)

    def create_collective_ops(self, devices: Sequence[torch.device], distributed: bool = True) -> "Config":
        """Copy of the config whose "sum"/"gather d" strings are replaced by op objects shared by all ranks
        (config.py:55-65). Call once, before the shards are made."""
        return dataclasses.replace(
            self,
            input_rules=create_collective_ops(self.input_rules, devices, distributed),
            output_rules=create_collective_ops(self.output_rules, devices, distributed),
        )


def create_collective_ops(rules: dict, devices: Sequence[torch.device], distributed: bool = True) -> dict:
    """One op object per distinct rule string (config.py:86-125). Only the single-device ops exist here."""
    world_size = len(devices)
    ops: Dict[str, Any] = {}
    for actions in rules.values():
        for rule in actions.values():
            if not isinstance(rule, str) or rule in ops:
                continue
            kind, *opts = rule.split()
            if kind == "sum":
                ops[rule] = DeviceAllReduce(world_size)
            elif kind == "gather":
                ops[rule] = DeviceAllGather(world_size, int(opts[0]) if opts else -1)
    return {pattern: {key: ops.get(rule, rule) if isinstance(rule, str) else rule for key, rule in actions.items()}
            for pattern, actions in rules.items()}


def add_lora_rules(model: nn.Module, config: Config) -> Config:
    """Extend `config`, in place, for the low-rank branches of peft LoRA Linears (config.py:128-154).

    A LoRA Linear adds lora_B(lora_A(x)) to its base Linear. If the base weight is split on its output axis, lora_B's
    weight takes the same split and lora_A stays whole. If it is split on its input axis, every rank sees only its
    part of x: lora_A's input is gathered back to the full x and its output divided by the world size, so that the
    sum over ranks that follows the base layer counts the low-rank branch once."""
    from .state_actions import Split
    from .utils import check_lora

    state_rules, input_rules, output_rules = {}, {}, {}
    for name, module in model.named_modules():
        if not check_lora(module):
            continue
        for pattern, action in config.state_rules.items():
            if pattern.search(name + ".weight") is None:
                continue
            if not isinstance(action, Split):
                raise Exception(
                    f"Can't apply action {action} since it uses LoRA. The only actions with LoRA support are Split and it's variations."
                )
            if action.dim == 0:
                state_rules[re.compile(rf"^{re.escape(name)}\.lora_B")] = action
            elif action.dim == 1:
                branch = re.compile(rf"^{re.escape(name)}\.lora_A\..+")
                input_rules[branch] = {0: "gather -1"}
                output_rules[branch] = {0: "scale"}
            else:
                raise Exception(f"Expected dim in [0, 1]. Don't know what to do with LoRA linear split along dim {action.dim}")
    config.state_rules.update(state_rules)
    config.input_rules.update(input_rules)
    config.output_rules.update(output_rules)
    return config


def get_parameter_name_mapping(names: Iterable[str], tensor_parallel_config: Config) -> Mapping[str, str]:
    """Original parameter name -> name inside the sharded model (config.py:157-191).

    Every module that has an input or output rule gets wrapped, and the wrapper holds the module as
    `tp_wrapped_module`; so "tp_wrapped_module." is inserted after each place where a module pattern
    (trailing "$" dropped, "\\." appended unless it already ends with ".") matches the name."""
    names = list(names)
    seen = set()
    for regex in chain(tensor_parallel_config.input_rules, tensor_parallel_config.output_rules):
        pattern = regex.pattern
        if pattern.endswith("$"):
            pattern = pattern[:-1]
        if not pattern.endswith("."):
            pattern += r"\."
        seen.add(pattern)
    compiled = [re.compile(p) for p in seen]

    mapping = {}
    for name in names:
        cuts = sorted(m.end() for m in (p.search(name) for p in compiled) if m is not None)
        new_name = name
        for pos in reversed(cuts):
            new_name = new_name[:pos] + "tp_wrapped_module." + new_name[pos:]
        mapping[name] = new_name
    return mapping
