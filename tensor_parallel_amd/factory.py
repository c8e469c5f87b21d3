"""`tensor_parallel(module, device_ids, ...)`: the one-call entry point (reference: src/tensor_parallel/factory.py:17-79)."""
from __future__ import annotations

import logging
from typing import Collection, Optional, Sequence, Union

import torch
from torch import nn

from .config import Config
from .tensor_parallel import TensorParallel

logger = logging.getLogger(__file__)


def tensor_parallel(
    module: nn.Module,
    device_ids: Optional[Sequence[Union[torch.device, str]]] = None,
    tensor_parallel_config: Optional[Config] = None,
    distributed: Optional[bool] = None,
    sharded: Optional[bool] = None,
    sharded_param_names: Optional[Collection[str]] = None,
    **kwargs,
) -> nn.Module:
    """Wrap `module` with tensor parallelism over `device_ids` and return the equivalent module.

    `device_ids` may name the same HIP device several times: that many rank shards then share the device, and
    the "sum"/"gather" rules run as single-device kernels. As in the reference, the default `sharded=None`
    means no ZeRO-3 (factory.py:22,66,76). `distributed=True` (one process per rank under torchrun) is not
    available: there is no inter-GPU collective in this package.
    """
    if distributed:
        raise NotImplementedError("distributed=True needs inter-GPU collectives, which tensor_parallel_amd does not have")
    try:
        from transformers import PreTrainedModel
    except ImportError:  # pragma: no cover
        PreTrainedModel = ()
    common = dict(device_ids=device_ids, tensor_parallel_config=tensor_parallel_config, distributed=False,
                  sharded=sharded, sharded_param_names=sharded_param_names, **kwargs)
    if PreTrainedModel and isinstance(module, PreTrainedModel):
        from .pretrained_model import TensorParallelPreTrainedModel

        return TensorParallelPreTrainedModel(module, **common)
    return TensorParallel(module, **common)
