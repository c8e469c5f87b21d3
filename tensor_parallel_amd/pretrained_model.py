"""Thin Hugging Face wrapper: picks the model family's rule table and delegates forward
(reference: src/tensor_parallel/pretrained_model.py:21-76). Generation helpers, cache reordering and the
encoder wrapper of the reference are not carried."""
from __future__ import annotations

import logging
from typing import Optional, Sequence

import torch
from transformers import PretrainedConfig, PreTrainedModel

from .config import Config
from .slicing_configs import PREDEFINED_CONFIGS
from .tensor_parallel import TensorParallel, check_device_ids

logger = logging.getLogger(__file__)


def find_predefined_tensor_parallel_config(model_config: PretrainedConfig, device_ids: Optional[Sequence[torch.device]]) -> Optional[Config]:
    device_ids = check_device_ids(device_ids)
    getter = PREDEFINED_CONFIGS.get(model_config.model_type)
    if getter is None:
        logger.warning("Using automatic config: tensor parallel config not provided and no custom config registered for the model")
        return None
    return getter(model_config, device_ids)


class TensorParallelPreTrainedModel(PreTrainedModel):
    is_parallelizable = model_parallel = True
    # the wrapper only delegates to the wrapped model, whatever attention implementation that one runs
    _supports_sdpa = _supports_flash_attn = _supports_flex_attn = _supports_attention_backend = True

    def __init__(
        self,
        module: PreTrainedModel,
        device_ids: Optional[Sequence[torch.device]] = None,
        output_device: Optional[torch.device] = None,
        output_device_index: Optional[int] = None,
        tensor_parallel_config: Optional[Config] = None,
        **kwargs,
    ):
        super().__init__(module.config)
        if tensor_parallel_config is None:
            tensor_parallel_config = find_predefined_tensor_parallel_config(module.config, device_ids)
        self.wrapped_model = TensorParallel(module, device_ids, output_device, output_device_index, tensor_parallel_config, **kwargs)

    @property
    def devices(self):
        return self.wrapped_model.devices

    @property
    def tensor_parallel_config(self):
        return self.wrapped_model.tensor_parallel_config

    def set_preserve_shards_when_saving(self, value: bool):
        self.wrapped_model.set_preserve_shards_when_saving(value)

    def apply_sharding(self, *args, **kwargs):
        self.wrapped_model.apply_sharding(*args, **kwargs)

    def forward(self, *args, **kwargs):
        return self.wrapped_model(*args, **kwargs)

    def state_dict(self, *args, **kwargs):
        state_dict = super().state_dict(*args, **kwargs)
        if self.wrapped_model.preserve_shards_when_saving:
            return state_dict
        return {(k[len("wrapped_model."):] if k.startswith("wrapped_model.") else k): v for k, v in state_dict.items()}
