"""Generic rules for a model without a hand-written table: every Linear is column-parallel, every
embedding is split on its hidden axis, and a Linear tied to an embedding consumes a split input and sums
(reference: src/tensor_parallel/autoconfig.py:12-39). The reference's convolution rules (autoconfig.py:40-78) are not
carried: convolution layers get no rule, so every rank keeps them whole and computes them in full."""
from __future__ import annotations

import logging
from typing import Sequence

import torch
from torch import nn
from torch.nn.modules import conv

from .config import Config
from .state_actions import Scale, Split

logger = logging.getLogger(__file__)


def get_default_config(module: nn.Module, device_ids: Sequence[torch.device]) -> Config:
    world_size = len(device_ids)
    embedding_weights = {m.weight for m in module.modules() if isinstance(m, (nn.Embedding, nn.EmbeddingBag))}
    state_rules, input_rules, output_rules = {}, {}, {}
    for name, sub in module.named_modules():
        if isinstance(sub, (nn.Embedding, nn.EmbeddingBag)):
            assert sub.max_norm is None or sub.norm_type < 2
            state_rules[f"^{name}.weight$"] = Split(world_size=world_size, dim=1)
            if hasattr(sub, "bias"):
                state_rules[f"^{name}.bias$"] = Split(world_size=world_size, dim=0)
            output_rules[f"^{name}$"] = {0: "gather -1"}
        elif isinstance(sub, nn.Linear) and "lora_A" not in name and "lora_B" not in name:
            assert sub.weight.shape == (sub.out_features, sub.in_features)
            assert sub.bias is None or sub.bias.shape == (sub.out_features,)
            if sub.weight not in embedding_weights:
                state_rules[f"^{name}.(weight|bias)$"] = Split(world_size=world_size, dim=0)
                output_rules[f"^{name}$"] = {0: "gather -1"}
            else:
                # the tied weight is already split on the hidden axis (dim 1) by the embedding's rule:
                # feed this Linear the matching slice of its input and sum the partial products
                input_rules[f"^{name}$"] = {0: Split(world_size=world_size, dim=-1)}
                output_rules[f"^{name}$"] = {0: "sum"}
                if sub.bias is not None:
                    state_rules[f"^{name}.bias$"] = Scale(world_size=world_size)
        elif isinstance(sub, conv._ConvNd):
            logger.warning(f"{name}: convolution layers have no automatic tensor-parallel rules here; every rank keeps this "
                           "layer whole (pass a Config with rules for it to split it)")
    return Config(state_rules, input_rules, output_rules, {})
