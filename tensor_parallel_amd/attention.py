"""Rank-local attention core as an attention implementation of the wrapped transformers modules.

The reference leaves attention to the wrapped module: every rank runs the model's own attention on the heads the
attr rules left it (src/tensor_parallel/wrapper.py:69-72, src/tensor_parallel/slicing_configs.py:382-389). Here
the same call site can be served by the HIP kernel behind `tpamd_attention`: `register()` adds an implementation
named "tpamd" to transformers' attention registry, and a model picks it with
`attn_implementation="tpamd"` (or `model.config._attn_implementation = "tpamd"`) before it is wrapped.

The kernel covers causal self-attention of decoder models without padding (prefill, and decode on a cache:
the queries are the last positions of the keys) and unmasked attention. A call with an explicit mask, dropout or a
head_dim other than 64 / 128 raises: there is no second implementation to fall back to.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _native

IMPLEMENTATION_NAME = "tpamd"


def attention_forward(module: torch.nn.Module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                      attention_mask: Optional[torch.Tensor], dropout: float = 0.0, scaling: Optional[float] = None,
                      is_causal: Optional[bool] = None, **kwargs) -> Tuple[torch.Tensor, None]:
    """Signature of transformers' attention functions: query [B, Hq, Sq, D], key / value [B, Hkv, Skv, D];
    returns ([B, Sq, Hq, D], None)."""
    if attention_mask is not None:
        raise NotImplementedError(
            "tensor_parallel_amd attention: an explicit attention mask was passed (padding or a non-causal pattern); "
            "the kernel implements causal and unmasked attention only"
        )
    if dropout and module.training:
        raise NotImplementedError("tensor_parallel_amd attention: dropout is not implemented (inference kernels)")
    if kwargs.get("output_attentions"):
        raise NotImplementedError("tensor_parallel_amd attention: attention weights are never materialised")
    causal = is_causal if is_causal is not None else getattr(module, "is_causal", True)
    # one new position on a cache sees every key: the aligned-to-the-end causal rule says the same
    out = _native.attention(query, key, value, scale=scaling, causal=bool(causal))
    return out, None


def register() -> str:
    """Adds "tpamd" to transformers' attention (and mask) registries; returns the name."""
    from transformers import AttentionInterface, AttentionMaskInterface
    from transformers.masking_utils import sdpa_mask

    AttentionInterface.register(IMPLEMENTATION_NAME, attention_forward)
    # mask construction as for sdpa: a purely causal mask is skipped (None reaches attention_forward)
    AttentionMaskInterface.register(IMPLEMENTATION_NAME, sdpa_mask)
    return IMPLEMENTATION_NAME
