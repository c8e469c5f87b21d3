"""`import tensor_parallel as tp` for code written against BlackSamorez/tensor_parallel
(reference: src/tensor_parallel/__init__.py:6-13): the same top-level names and the same submodule paths
(`tensor_parallel.slicing_configs`, `tensor_parallel.state_actions`, ...), all served by `tensor_parallel_amd`.
Nothing is implemented here."""
import importlib
import sys

import tensor_parallel_amd as _impl
from tensor_parallel_amd import *  # noqa: F401,F403
from tensor_parallel_amd import __all__ as _names

# submodules the reference has and user code imports from; pretrained_model pulls in transformers, so it is aliased
# on first use instead
_SUBMODULES = ("autoconfig", "aux_actions", "config", "dispatch", "factory", "legacy", "shard", "sharding", "slicing_configs",
               "state_actions", "tensor_parallel", "utils", "wrapper")
for _name in _SUBMODULES:
    _module = importlib.import_module(f"tensor_parallel_amd.{_name}")
    sys.modules[f"{__name__}.{_name}"] = _module
    if _name not in _names:  # `tensor_parallel.tensor_parallel` is the factory function, as in the reference
        globals()[_name] = _module

__all__ = list(_names) + ["TensorParallelPreTrainedModel"]


def __getattr__(name):
    if name in ("TensorParallelPreTrainedModel", "pretrained_model"):
        module = importlib.import_module("tensor_parallel_amd.pretrained_model")
        sys.modules[f"{__name__}.pretrained_model"] = module
        return module if name == "pretrained_model" else module.TensorParallelPreTrainedModel
    return getattr(_impl, name)
