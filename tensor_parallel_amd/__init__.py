"""MI355X-native per-rank hot path of tensor parallelism: state-dict slicing, rank-shard Linears and the
single-device partial-sum reduction, behind the Python surface of BlackSamorez/tensor_parallel
(reference: src/tensor_parallel/__init__.py:6-13).

    import tensor_parallel_amd as tp
    model = tp.tensor_parallel(model, ["cuda:0", "cuda:0"])      # two rank shards on one GPU
    shards = tp.convert_state_dict(state_dict, config, world_size=2)
"""
from . import _native, attention, graphs, int8, kv_cache, state_actions
from .config import Config
from .dispatch import convert_state_dict, infer_sharded_device_map, save_tensor_parallel
from .factory import tensor_parallel
from .legacy import Sharded
from .state_actions import Scale, Split, SplitInChunks, SplitInGroupedChunks, StateAction
from .tensor_parallel import TensorParallel

__all__ = [
    "Config",
    "Scale",
    "Sharded",
    "Split",
    "SplitInChunks",
    "SplitInGroupedChunks",
    "StateAction",
    "TensorParallel",
    "convert_state_dict",
    "infer_sharded_device_map",
    "save_tensor_parallel",
    "tensor_parallel",
]


def __getattr__(name):
    # the Hugging Face wrapper imports transformers, which is slow: load it on first use
    if name == "TensorParallelPreTrainedModel":
        from .pretrained_model import TensorParallelPreTrainedModel

        return TensorParallelPreTrainedModel
    raise AttributeError(name)
