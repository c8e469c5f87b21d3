"""State-dict conversion and saving helpers (reference: src/tensor_parallel/dispatch.py:13-131)."""
from __future__ import annotations

from contextlib import contextmanager
from typing import Dict, Optional

import torch

from .config import Config, get_parameter_name_mapping
from .slicing import BatchSlicer
from .state_actions import SegmentedAction
from .utils import find_tied_weight_aliases


@contextmanager
def save_tensor_parallel(model):
    """Inside the block, `model.state_dict()` gives the original model's names and full tensors (dispatch.py:13-32)."""
    model.set_preserve_shards_when_saving(False)
    try:
        yield
    finally:
        model.set_preserve_shards_when_saving(True)


def infer_sharded_data_device_id(name: str) -> int:
    """Rank index encoded in a sharded parameter name (dispatch.py:35-48)."""
    for marker in ("_sanity_check_params.", "module_shards.", "flat_shards."):
        at = name.find(marker)
        if at != -1:
            digits = name[at + len(marker):].split(".", 1)[0]
            return int(digits)
    raise KeyError(f"Can't decide where to put {name}. Are you sure you passed a tensor_parallel parameter was passed?")


def infer_sharded_device_map(tp_model) -> dict:
    """Parameter/buffer name (every alias of tied tensors) -> device of the rank that owns it (dispatch.py:51-72)."""
    owner = {}
    for name, tensor in list(tp_model.named_parameters()) + list(tp_model.named_buffers()):
        owner[id(tensor)] = tp_model.devices[infer_sharded_data_device_id(name)]
    return {alias: owner[i] for i, aliases in find_tied_weight_aliases(tp_model).items() for alias in aliases}


def convert_state_dict(
    input_state_dict: Dict[str, torch.Tensor],
    tensor_parallel_config: Config,
    world_size: int,
    for_pretrained: bool = False,
    device: Optional[torch.device] = None,
) -> Dict[str, torch.Tensor]:
    """State dict of the base model -> state dict of the tensor-parallel model (dispatch.py:75-131).

    Per rank: the first matching state rule slices each tensor, names get `tp_wrapped_module.` where a module
    is wrapped and the `module_shards.{rank}.` prefix, and an empty `_sanity_check_params.{rank}` is added.
    Tensors no rule matches are passed through as the same object for every rank, as in the reference
    (dispatch.py:110). All splitting of all ranks runs as ONE launch of the region mover; sliced tensors are
    fresh, contiguous and on the HIP device (`device`, or the device of the inputs, or the current one).
    Tied weights are not handled, as in the reference.
    """
    batch = BatchSlicer(device)
    names = list(input_state_dict.keys())
    renamed = get_parameter_name_mapping(names, tensor_parallel_config)
    output: Dict[str, torch.Tensor] = {}
    for rank in range(world_size):
        for name in names:
            state = input_state_dict[name]
            for pattern, action in tensor_parallel_config.state_rules.items():
                if pattern.search(name) is not None:
                    if isinstance(action, SegmentedAction) and state is not None:
                        new = batch.add(state, action.spec(tuple(state.shape), rank))
                    else:
                        new = action(state, rank=rank)
                    break
            else:
                new = state
            output[f"module_shards.{rank}.{renamed[name]}"] = new
        output[f"_sanity_check_params.{rank}"] = torch.empty(0, device="cpu")
    batch.run()
    if batch.device is not None and batch.plan is not None:
        torch.cuda.synchronize(batch.device)  # uploaded sources are dropped with the batch
    batch.close()
    if for_pretrained:
        output = {"wrapped_model." + name: tensor for name, tensor in output.items()}
    return output
