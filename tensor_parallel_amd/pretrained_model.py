"""Hugging Face wrapper: picks the model family's rule table, delegates forward, and lets `generate` drive the
rank shards (reference: src/tensor_parallel/pretrained_model.py:21-165). The attention cache is rank-local
(see kv_cache): there is no cache reordering hook here, the cache objects reorder themselves."""
from __future__ import annotations

import importlib
import logging
from typing import Optional, Sequence

import torch
from transformers import GenerationMixin, PretrainedConfig, PreTrainedModel

from . import attention, graphs
from .config import Config
from .slicing_configs import PREDEFINED_CONFIGS
from .tensor_parallel import TensorParallel, check_device_ids, parallel_apply_simple

logger = logging.getLogger(__file__)


def find_predefined_tensor_parallel_config(model_config: PretrainedConfig, device_ids: Optional[Sequence[torch.device]]) -> Optional[Config]:
    device_ids = check_device_ids(device_ids)
    getter = PREDEFINED_CONFIGS.get(model_config.model_type)
    if getter is None:
        logger.warning("Using automatic config: tensor parallel config not provided and no custom config registered for the model")
        return None
    return getter(model_config, device_ids)


class _EncoderWrapper(torch.nn.Module):
    """The encoders of all rank shards, run side by side like the whole model (pretrained_model.py:108-165)."""

    def __init__(self, tp_model: "TensorParallelPreTrainedModel"):
        super().__init__()
        self.__dict__["tp_model"] = tp_model  # not a submodule: the model owns the shards
        shards = tp_model.wrapped_model.module_shards
        self.__dict__["encoder_shards"] = [shard.get_encoder() for shard in shards]
        self.main_input_name = getattr(self.encoder_shards[0], "main_input_name", "input_ids")

    def forward(self, *args, **kwargs):
        wrapped = self.tp_model.wrapped_model
        if wrapped.sharding_manager is not None:
            wrapped.sharding_manager.synchronize_weights(wrapped.all_cuda)
        inputs, kwargs_tup = wrapped.prepare_args_kwargs_for_forward(*args, **kwargs)
        return parallel_apply_simple(self.encoder_shards, inputs, kwargs_tup, wrapped.devices)[wrapped.output_device_index]


class TensorParallelPreTrainedModel(PreTrainedModel, GenerationMixin):
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
        if hasattr(module, "_hf_hook"):
            from accelerate.hooks import remove_hook_from_module

            remove_hook_from_module(module, recurse=True)
        self.main_input_name = module.main_input_name
        generation_config = getattr(module, "generation_config", None)
        self.wrapped_model = TensorParallel(module, device_ids, output_device, output_device_index, tensor_parallel_config, **kwargs)
        if generation_config is not None:
            self.generation_config = generation_config
        self._encoder_wrapper: Optional[_EncoderWrapper] = None

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

    # ---- what `generate` asks the model itself: answered by the first rank shard, which is the model class
    def _validate_model_class(self):
        return self.wrapped_model.module_shards[0]._validate_model_class()

    def _validate_model_kwargs(self, model_kwargs):
        return self.wrapped_model.module_shards[0]._validate_model_kwargs(model_kwargs)

    def _prepare_model_inputs(self, *args, **kwargs):
        return self.wrapped_model.module_shards[0]._prepare_model_inputs(*args, **kwargs)

    def prepare_inputs_for_generation(self, *args, **kwargs):
        return self.wrapped_model.module_shards[0].prepare_inputs_for_generation(*args, **kwargs)

    def _supports_default_dynamic_cache(self) -> bool:
        return self.wrapped_model.module_shards[0]._supports_default_dynamic_cache()

    def _valid_auto_compile_criteria(self, model_kwargs, generation_config) -> bool:
        # `generate` wraps the forward in torch.compile when it is given a static cache. The rank shards call a C ABI
        # through ctypes and take turns as greenlets, which a tracing compiler cannot follow. What takes its place: the
        # decode step recorded as one HIP graph (get_compiled_call below), where a step can be recorded at all, i.e. where
        # every attention module reads the count of cached positions on the device
        # (`tp.attention.fuse_rotary_(model, assume_no_padding=True)`); the forward as it is otherwise.
        if generation_config.disable_compile:
            return False
        cache = model_kwargs.get("past_key_values")
        layers = getattr(cache, "layers", None)
        if not isinstance(layers, list) or not layers or not all(hasattr(layer, "cumulative_length") for layer in layers):
            return False
        return self._decode_step_can_be_recorded()

    def _decode_step_can_be_recorded(self) -> bool:
        tp_module = importlib.import_module(__package__ + ".tensor_parallel")
        shards = self.wrapped_model.module_shards
        if len(shards) > 1 and not tp_module.RANK_GREENLETS:
            return False
        if any(device.type != "cuda" for device in self.wrapped_model.devices) or len(set(self.wrapped_model.devices)) != 1:
            return False
        return all(attention.decode_step_is_static(shard) for shard in shards)

    def get_compiled_call(self, compile_config=None):
        """What `generate` calls for every decode step once `_valid_auto_compile_criteria` has said yes: the step recorded
        as one HIP graph by `tp.graphs.capture` at its first call and replayed afterwards. The padding mask is left out
        of the recorded arguments (it grows by a column per step, and the fused attention was promised that there is no
        padding). One graph is kept: a step on another cache object, or with other shapes, records a new one; the graph
        holds its cache alive until then. `generate(..., disable_compile=True)` keeps the forward as it is."""
        return self._recorded_decode_step

    def _recorded_decode_step(self, **model_inputs):
        tokens = model_inputs.get("input_ids")
        if tokens is None or tokens.dim() != 2 or tokens.shape[1] != 1:
            return self(**model_inputs)  # a chunk of a prefill: its attention asks the cache's count on the host
        model_inputs.pop("attention_mask", None)
        model_inputs = {k: v for k, v in model_inputs.items() if v is not None}
        graphed = self.__dict__.get("_tp_decode_graph")
        if graphed is not None:
            try:
                return graphed(**model_inputs)
            except ValueError:  # another cache object, batch size or set of arguments: record again
                self.__dict__["_tp_decode_graph"] = graphed = None
        graphed = graphs.capture(self, **model_inputs)
        self.__dict__["_tp_decode_graph"] = graphed
        return graphed(**model_inputs)

    def get_encoder(self, *args, **kwargs):
        shards = self.wrapped_model.module_shards
        assert len(shards), "Can't get encoder since no module shards present"
        if len(shards) == 1:
            return shards[0].get_encoder(*args, **kwargs)
        if self._encoder_wrapper is None:
            self.__dict__["_encoder_wrapper"] = _EncoderWrapper(self)
        return self._encoder_wrapper

    def state_dict(self, *args, **kwargs):
        state_dict = super().state_dict(*args, **kwargs)
        if self.wrapped_model.preserve_shards_when_saving:
            return state_dict
        return {(k[len("wrapped_model."):] if k.startswith("wrapped_model.") else k): v for k, v in state_dict.items()}
