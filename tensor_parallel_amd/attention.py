"""Rank-local attention core as an attention implementation of the wrapped transformers modules.

The reference leaves attention to the wrapped module: every rank runs the model's own attention on the heads the
attr rules left it (src/tensor_parallel/wrapper.py:69-72, src/tensor_parallel/slicing_configs.py:382-389). Here
the same call site can be served by the HIP kernel behind `tpamd_attention`: `register()` adds an implementation
named "tpamd" to transformers' attention registry, and a model picks it with
`attn_implementation="tpamd"` (or `model.config._attn_implementation = "tpamd"`) before it is wrapped.

The kernel covers causal self-attention of decoder models without padding (prefill, and decode on a cache:
the queries are the last positions of the keys) and unmasked attention. A call with an explicit mask, dropout or a
head_dim other than 64 / 128 raises: there is no second implementation to fall back to.

`fuse_rotary_(model)` goes one step further for attention modules of the Llama pattern (q_proj / k_proj / v_proj / o_proj,
rotary position embeddings handed in as `position_embeddings`, a transformers cache object): their forward then runs the
rotary embedding, the hand-over to the cache and the attention core on the library's kernels too (`tpamd_rope_append` +
`tpamd_attention` at prefill, `tpamd_attention_decode_rope` for one new position), writing into buffers with room to grow
that the cache layer's `keys` / `values` are views of. A call those kernels do not cover takes the module's own forward.
"""
from __future__ import annotations

import inspect
import types
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


# ---- rotary embedding + cache append + attention core for attention modules of the Llama pattern ------------------------
_MIN_CAPACITY = 256


def _cache_layer(cache, layer_idx: int):
    """The plain growing layer `layer_idx` of a transformers cache (made on demand as `Cache.update` would), or None when the
    cache is of another kind (static, sliding window, quantised, offloaded): those keep the module's own forward."""
    from transformers.cache_utils import DynamicLayer

    layers = getattr(cache, "layers", None)
    if layers is None or getattr(cache, "offloading", False):
        return None
    if len(layers) <= layer_idx:
        if getattr(cache, "layer_class_to_replicate", None) is not DynamicLayer:
            return None
        while len(layers) <= layer_idx:
            layers.append(DynamicLayer())
    layer = layers[layer_idx]
    return layer if type(layer) is DynamicLayer else None


def _static_layer(cache, layer_idx: int):
    """Layer `layer_idx` of a transformers static cache (preallocated keys / values, the number of cached positions kept on
    the device as `cumulative_length`), or None."""
    from transformers.cache_utils import StaticLayer

    layers = getattr(cache, "layers", None)
    if layers is None or getattr(cache, "offloading", False) or len(layers) <= layer_idx:
        return None
    layer = layers[layer_idx]
    return layer if type(layer) is StaticLayer else None


def _buffers_with_room(layer, B: int, Hkv: int, D: int, need: int, like: torch.Tensor):
    """(k, v) buffers [B, Hkv, capacity >= need, D] that hold the layer's cached positions: the ones its keys / values are
    views of when they still are and have room, else new ones (twice the need) with the cached positions copied over."""
    have = layer.get_seq_length()
    bufs = layer.__dict__.get("_tp_buffers")
    if bufs is not None and have > 0:
        kb, vb = bufs
        same = (layer.keys.data_ptr() == kb.data_ptr() and layer.values.data_ptr() == vb.data_ptr()
                and layer.keys.shape == (B, Hkv, have, D) and layer.keys.stride() == kb.stride() and layer.values.stride() == vb.stride())
        if not same:
            bufs = None
    if bufs is None or bufs[0].shape[:2] != (B, Hkv) or bufs[0].shape[2] < need or bufs[0].dtype != like.dtype or bufs[0].device != like.device:
        cap = max(2 * need, _MIN_CAPACITY)
        kb = torch.empty((B, Hkv, cap, D), dtype=like.dtype, device=like.device)
        vb = torch.empty_like(kb)
        if have > 0:
            kb[:, :, :have].copy_(layer.keys)
            vb[:, :, :have].copy_(layer.values)
        bufs = layer.__dict__["_tp_buffers"] = (kb, vb)
    return bufs


def _share_qkv_storage(module: torch.nn.Module) -> bool:
    """Lay the weights of q_proj / k_proj / v_proj out as one [Nq + Nk + Nv, K] matrix (each Linear's weight becomes a view
    of its rows), so that the fused forward makes one projection call instead of three. Only for plain shard Linears with
    16-bit weights on one HIP device and all or none with a bias."""
    from .shard_modules import ShardLinear, _has_hooks

    parts = [module._modules.get(n) for n in ("q_proj", "k_proj", "v_proj")]
    if not all(type(p) is ShardLinear and not _has_hooks(p) for p in parts):
        return False
    ws = [p.weight for p in parts]
    first = ws[0]
    if first.device.type != "cuda" or first.dtype not in (torch.bfloat16, torch.float16):
        return False
    if any(w.dtype != first.dtype or w.device != first.device or w.dim() != 2 or w.shape[1] != first.shape[1] for w in ws):
        return False
    biases = [p.bias for p in parts]
    if any(b is None for b in biases) != all(b is None for b in biases):
        return False
    with torch.no_grad():
        fused_w = torch.cat([w.detach() for w in ws], 0)
        fused_b = None if biases[0] is None else torch.cat([b.detach() for b in biases], 0)
        row = 0
        for p, w, b in zip(parts, ws, biases):
            n = w.shape[0]
            p.weight = torch.nn.Parameter(fused_w[row:row + n], requires_grad=w.requires_grad)
            if b is not None:
                p.bias = torch.nn.Parameter(fused_b[row:row + n], requires_grad=b.requires_grad)
            row += n
    module.__dict__["_tp_qkv"] = (fused_w, fused_b)
    return True


def _project_qkv(self, hidden_states: torch.Tensor, D: int):
    """q, k, v as [B, S, heads, D]: one call on the shared weight matrix when the three Linears still are views of it."""
    from .shard_modules import ShardLinear, _guard

    B, S, _ = hidden_states.shape
    shared = self.__dict__.get("_tp_qkv")
    if shared is not None:
        w, b = shared
        q_proj, k_proj, v_proj = self.q_proj, self.k_proj, self.v_proj
        intact = type(q_proj) is ShardLinear and type(k_proj) is ShardLinear and type(v_proj) is ShardLinear
        if intact:
            nk = k_proj.weight.shape[0]
            nq = w.shape[0] - 2 * nk
            row_bytes = w.stride(0) * w.element_size()
            intact = (q_proj.weight.data_ptr() == w.data_ptr() and q_proj.weight.shape[0] == nq and v_proj.weight.shape[0] == nk
                      and k_proj.weight.data_ptr() == w.data_ptr() + nq * row_bytes
                      and v_proj.weight.data_ptr() == w.data_ptr() + (nq + nk) * row_bytes)
        if intact and hidden_states.dtype == w.dtype:
            qkv = _guard(_native.linear(hidden_states.detach(), w, b), hidden_states, q_proj.weight)
            return (qkv[..., :nq].view(B, S, -1, D), qkv[..., nq:nq + nk].view(B, S, -1, D), qkv[..., nq + nk:].view(B, S, -1, D))
        if not intact:  # a projection was replaced (quantised, re-assigned): three calls from now on
            del self.__dict__["_tp_qkv"]
    return (self.q_proj(hidden_states).view(B, S, -1, D), self.k_proj(hidden_states).view(B, S, -1, D),
            self.v_proj(hidden_states).view(B, S, -1, D))


def _attend_on_cache(q, k, v, cos, sin, layer, static, scale, layer_idx: int) -> torch.Tensor:
    """Rotary embedding of the new q / k rows, their hand-over to the cache and the attention core, for the new positions
    q / k / v [B, S, heads, D] (views of the projection output): on the growing layer `layer`, or on the static layer
    `static`. Returns [B, S, Hq, D] (5-dimensional grouped queries come back flat)."""
    B, S, D = q.shape[0], q.shape[1], q.shape[-1]
    Hkv = k.shape[2]
    Hq = q.shape[2] if q.dim() == 4 else q.shape[2] * q.shape[3]
    cos, sin = cos.to(k.dtype), sin.to(k.dtype)
    if static is not None:
        # Preallocated keys / values and a count that lives on the device: a decode step reads the count inside the kernels
        # (no host value depends on the step, so the forward can be replayed as a HIP graph); a prefill reads it back.
        if not static.is_initialized:
            static.lazy_initialization(k.transpose(1, 2), v.transpose(1, 2))
        kb, vb = static.keys, static.values
        if S > 1 and kb.shape[1] != Hkv and kb.shape[0] == B and kb.shape[3] == D and int(static.cumulative_length) == 0:
            # laid out ahead of its first use (transformers does that for a prefill in chunks), with the whole model's
            # key/value heads: an empty layer is laid out again for the heads of this rank
            static.lazy_initialization(k.transpose(1, 2), v.transpose(1, 2))
            kb, vb = static.keys, static.values
        if kb.shape[0] != B or kb.shape[1] != Hkv or kb.shape[3] != D or kb.dtype != k.dtype:
            raise ValueError(f"the static cache of layer {layer_idx} holds {tuple(kb.shape)} {kb.dtype}, this call needs "
                             f"[{B}, {Hkv}, positions, {D}] {k.dtype}")
        count = static.cumulative_length
        if S == 1:
            out = _native.attention_decode_rope(q, k, v, cos, sin, kb, vb, count.reshape(1), scale=scale)
        else:
            pos0 = int(count)
            if pos0 + S > kb.shape[2]:
                raise ValueError(f"{pos0} cached + {S} new positions do not fit the static cache of {kb.shape[2]}")
            q_rot = _native.rope_append(q, k, v, cos, sin, kb, vb, pos0)
            out = _native.attention(q_rot, kb[:, :, :pos0 + S], vb[:, :, :pos0 + S], scale=scale, causal=True)
        count.add_(S)
        return out.reshape(B, S, Hq, D)
    pos0 = layer.get_seq_length()
    kb, vb = _buffers_with_room(layer, B, Hkv, D, pos0 + S, k)
    if S == 1:
        out = _native.attention_decode_rope(q, k, v, cos, sin, kb, vb, pos0, scale=scale)
    else:
        q_rot = _native.rope_append(q, k, v, cos, sin, kb, vb, pos0)
        out = _native.attention(q_rot, kb[:, :, :pos0 + S], vb[:, :, :pos0 + S], scale=scale, causal=True)
    if not layer.is_initialized:
        layer.dtype, layer.device = k.dtype, k.device
        layer.is_initialized = True
    layer.keys, layer.values = kb[:, :, :pos0 + S], vb[:, :, :pos0 + S]
    return out.reshape(B, S, Hq, D)


def _fused_rotary_forward(self, hidden_states: torch.Tensor, position_embeddings=None, attention_mask=None, past_key_values=None,
                          **kwargs):
    own = type(self).forward
    D = getattr(self, "head_dim", None)
    layer = static = None
    no_padding = self.__dict__.get("_tp_no_padding", False)  # the caller's word: masks are the causal pattern and nothing else
    usable = (position_embeddings is not None and past_key_values is not None and not self.training
              and hidden_states.dim() == 3 and hidden_states.device.type == "cuda"
              and hidden_states.dtype in (torch.bfloat16, torch.float16) and D in (64, 128)
              and not kwargs.get("output_attentions") and getattr(self, "is_causal", True))
    if usable and (attention_mask is None or no_padding):
        layer = _cache_layer(past_key_values, self.layer_idx)
        if layer is None and no_padding:  # a static cache always comes with a materialised mask
            static = _static_layer(past_key_values, self.layer_idx)
    if layer is None and static is None:
        return own(self, hidden_states, position_embeddings=position_embeddings, attention_mask=attention_mask,
                   past_key_values=past_key_values, **kwargs)
    B, S, _ = hidden_states.shape
    q, k, v = _project_qkv(self, hidden_states, D)
    cos, sin = position_embeddings
    out = _attend_on_cache(q, k, v, cos, sin, layer, static, getattr(self, "scaling", None), self.layer_idx)
    return self.o_proj(out.reshape(B, S, -1)), None


def _fused_falcon_forward(self, hidden_states: torch.Tensor, alibi=None, attention_mask=None, position_ids=None, layer_past=None,
                          use_cache: bool = False, output_attentions: bool = False, position_embeddings=None, **kwargs):
    """FalconAttention with rotary embeddings and grouped heads (the new decoder architecture). transformers always
    hands this module a materialised mask; it is ignored here, which is what `fuse_rotary_(..., assume_no_padding=True)`
    was told is right (the mask is then the causal pattern the kernels apply themselves)."""
    D = self.head_dim
    layer = static = None
    usable = (alibi is None and position_embeddings is not None and layer_past is not None and not self.training and not output_attentions
              and self.new_decoder_architecture and hidden_states.dim() == 3 and hidden_states.device.type == "cuda"
              and hidden_states.dtype in (torch.bfloat16, torch.float16) and D in (64, 128))
    if usable:
        layer = _cache_layer(layer_past, self.layer_idx)
        if layer is None:
            static = _static_layer(layer_past, self.layer_idx)
    if layer is None and static is None:
        return type(self).forward(self, hidden_states, alibi, attention_mask, position_ids=position_ids, layer_past=layer_past,
                                  use_cache=use_cache, output_attentions=output_attentions, position_embeddings=position_embeddings, **kwargs)
    B, S, _ = hidden_states.shape
    fused_qkv = self.query_key_value(hidden_states)
    # [.., kv head, its query heads + key + value, D]
    per = self.num_heads // self.num_kv_heads
    qkv = fused_qkv.view(B, S, self.num_kv_heads, per + 2, D)
    q, k, v = qkv[:, :, :, :per], qkv[:, :, :, per], qkv[:, :, :, per + 1]
    cos, sin = position_embeddings
    out = _attend_on_cache(q, k, v, cos, sin, layer, static, self.inv_norm_factor, self.layer_idx)
    return self.dense(out.reshape(B, S, self.num_heads * D)), None


FUSABLE_ATTENTION_CLASSES = ("LlamaAttention",)


def _is_llama_pattern(module: torch.nn.Module, class_names) -> bool:
    """An attention module whose own forward is exactly: q / k / v projections, rotary embedding of q and k from
    `position_embeddings`, cache update, attention, output projection (no norms on q / k, no sliding window, no softcap)."""
    if type(module).__name__ not in class_names:
        return False
    children = set(module._modules)
    if children != {"q_proj", "k_proj", "v_proj", "o_proj"}:
        return False
    if not hasattr(module, "layer_idx") or not hasattr(module, "head_dim") or getattr(module, "sliding_window", None) is not None:
        return False
    try:
        params = inspect.signature(type(module).forward).parameters
    except (TypeError, ValueError):
        return False
    return "position_embeddings" in params and "past_key_values" in params and "attention_mask" in params


def _is_rotary_falcon(module: torch.nn.Module) -> bool:
    """transformers' FalconAttention with rotary embeddings and grouped heads (the 40B layout)."""
    if type(module).__name__ != "FalconAttention" or set(module._modules) != {"query_key_value", "dense", "attention_dropout"}:
        return False
    config = getattr(module, "config", None)
    return getattr(config, "alibi", True) is False and module.new_decoder_architecture and getattr(module, "layer_idx", None) is not None


def decode_step_is_static(model: torch.nn.Module) -> bool:
    """True when every attention module under `model` has the fused forward in the form that reads a static cache's
    count of cached positions on the device (`fuse_rotary_(model, assume_no_padding=True)`): a decode step then takes no
    host decision that depends on the step, which is what recording it as a HIP graph needs."""
    fused = 0
    for module in model.modules():
        func = getattr(module.__dict__.get("forward"), "__func__", None)
        if func is _fused_falcon_forward:
            fused += 1
        elif func is _fused_rotary_forward:
            if not module.__dict__.get("_tp_no_padding", False):
                return False
            fused += 1
    layers = getattr(getattr(model, "config", None), "num_hidden_layers", None)
    return fused > 0 and (layers is None or fused >= layers)


def fuse_rotary_(model: torch.nn.Module, class_names=FUSABLE_ATTENTION_CLASSES, assume_no_padding: bool = False,
                 share_qkv: bool = True) -> int:
    """Give every attention module under `model` (before or after `tp.tensor_parallel`) whose class is named in
    `class_names` and whose structure is the Llama pattern the forward described in the module docstring. Returns how many
    modules took it. Name further classes only when their forward is the same sequence of operations.

    `assume_no_padding=True` is the caller's word that the batches carry no padding, so that a mask handed to an attention
    module is the causal pattern and can be ignored. With it the Llama-pattern modules also take transformers' static
    caches (which always come with a materialised mask): preallocated keys and values whose number of cached positions
    lives on the device, read there by the decode kernels, so that a decode step makes no host decision that depends
    on the step and `tp.graphs.capture` can record it once and replay it for every new token. It also takes transformers' FalconAttention (rotary, grouped heads: the 40B layout): that model
    hands its attention modules a materialised mask on every call, which cannot be told from a padding mask without
    reading it back, so the caller vouches that the batches carry no padding and the mask is ignored. Such a module then
    caches its key/value heads once, not once per query head as its own forward does: every call of a fused model must
    be one the fused forward takes (16-bit tensors on the device, a growing cache, inference).

    `share_qkv=True` (Llama pattern, rank shards already on the device): the weights of q_proj / k_proj / v_proj move into
    one matrix that each of them keeps a view of (names, shapes and values in `state_dict` stay what they were), and the
    fused forward multiplies by it once instead of three times: two launches and two host calls fewer per module and
    decode step. A projection that is replaced later (quantised, say) ends the sharing for its module."""
    count = 0
    for module in model.modules():
        if "forward" in module.__dict__:
            # already fused (a second call may still bring the caller's word about padding, or find the projections on the
            # device now), or somebody else's forward
            if getattr(module.__dict__["forward"], "__func__", None) is _fused_rotary_forward:
                if assume_no_padding:
                    module.__dict__["_tp_no_padding"] = True
                if share_qkv and "_tp_qkv" not in module.__dict__:
                    _share_qkv_storage(module)
            continue
        if _is_llama_pattern(module, class_names):
            module.forward = types.MethodType(_fused_rotary_forward, module)
            if assume_no_padding:
                module.__dict__["_tp_no_padding"] = True
            if share_qkv:
                _share_qkv_storage(module)
            count += 1
        elif assume_no_padding and _is_rotary_falcon(module):
            module.forward = types.MethodType(_fused_falcon_forward, module)
            count += 1
    return count
