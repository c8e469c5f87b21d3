"""Hand-written rule tables for model families (reference: src/tensor_parallel/slicing_configs.py).

Carried here: Llama (slicing_configs.py:345-406), Falcon / RefinedWeb (:409-462) and GPT-2 (:32-72 in spirit,
rules at :180-240). The state rules - which tensor is split how - are those of the reference. The KV-cache
rules of the reference (`select_kv_for_rank`, `gather_kv`) are not carried: shards are run without a cache.
Attribute rules name the attributes of the model classes the reference was written against; attributes
a given transformers version no longer has are skipped when the shard is built.
"""
from __future__ import annotations

from functools import partial
from typing import Callable, Dict, Sequence

import torch

from .aux_actions import split_inner_dim, split_num_heads
from .config import Config
from .state_actions import Scale, Split, SplitInChunks, SplitInGroupedChunks

ConfigGetter = Callable[[object, Sequence[torch.device]], Config]


def get_llama_config(model_config, devices: Sequence[torch.device]) -> Config:
    assert model_config.model_type == "llama", f"Trying to pass {model_config.model_type} as llama config"
    world_size = len(devices)
    head_dim = model_config.hidden_size // model_config.num_attention_heads
    num_kv = getattr(model_config, "num_key_value_heads", None)
    grouped = num_kv is not None
    if not grouped:
        num_kv = model_config.num_attention_heads
    q_per_kv = model_config.num_attention_heads // num_kv

    def q_heads(n, rank):
        return q_per_kv * split_num_heads(n // q_per_kv, rank=rank, world_size=world_size)

    attn_attrs = {
        "hidden_size": partial(split_inner_dim, num_heads=num_kv, world_size=world_size),
        "num_heads": q_heads,
    }
    if grouped:
        attn_attrs["num_key_value_heads"] = partial(split_num_heads, world_size=world_size)

    return Config(
        state_rules={
            # attention: q/k/v column-parallel on whole KV groups, o row-parallel on the same groups
            r".*self_attn\.q_proj\.weight$": SplitInChunks(world_size=world_size, dim=0, chunk_size=q_per_kv * head_dim),
            r".*self_attn\.k_proj\.weight$": SplitInChunks(world_size=world_size, dim=0, chunk_size=head_dim),
            r".*self_attn\.v_proj\.weight$": SplitInChunks(world_size=world_size, dim=0, chunk_size=head_dim),
            r".*self_attn\.o_proj\.weight$": SplitInChunks(world_size=world_size, dim=1, chunk_size=q_per_kv * head_dim),
            # MLP: gate/up column-parallel, down row-parallel
            r".*mlp\.gate_proj\.weight$": Split(world_size=world_size, dim=0),
            r".*mlp\.down_proj\.weight$": Split(world_size=world_size, dim=1),
            r".*mlp\.up_proj\.weight$": Split(world_size=world_size, dim=0),
            # embeddings on the hidden axis, head on the vocabulary axis
            r".*embed_tokens.weight$": Split(world_size=world_size, dim=1),
            r".*lm_head\.weight$": Split(world_size=world_size, dim=0),
        },
        input_rules={},
        output_rules={
            r".*self_attn$": {0: "sum"},
            r".*mlp$": {0: "sum"},
            r".*embed_tokens$": {0: "gather -1"},
            r".*lm_head$": {0: "gather -1"},
        },
        attr_rules={r".*self_attn$": attn_attrs},
    )


def get_refined_web_config(model_config, devices: Sequence[torch.device]) -> Config:
    """Falcon with grouped KV heads: the fused query_key_value weight is laid out as num_kv groups of
    (q_per_kv query heads, one key head, one value head), so splitting on whole groups of
    (q_per_kv + 2) * head_dim rows keeps every rank's q, k and v together (slicing_configs.py:430-435)."""
    assert model_config.model_type in ("RefinedWeb", "falcon"), f"Trying to pass {model_config.model_type} as RefinedWeb config"
    assert not getattr(model_config, "bias", False) and not getattr(model_config, "alibi", False), (
        "Running Falcon with biases or alibi is not supported"
    )
    world_size = len(devices)
    num_heads = model_config.num_attention_heads
    num_kv = getattr(model_config, "n_head_kv", None) or getattr(model_config, "num_kv_heads", None)
    head_dim = model_config.hidden_size // num_heads
    q_per_kv = num_heads // num_kv

    def q_heads(n, rank):
        return q_per_kv * split_num_heads(n // q_per_kv, rank=rank, world_size=world_size)

    return Config(
        state_rules={
            r".*self_attention\.query_key_value\.weight$": SplitInChunks(world_size=world_size, dim=0, chunk_size=(2 + q_per_kv) * head_dim),
            r".*self_attention\.dense\.weight$": SplitInChunks(world_size=world_size, dim=1, chunk_size=q_per_kv * head_dim),
            r".*mlp\.dense_h_to_4h\.weight$": Split(world_size=world_size, dim=0),
            r".*mlp\.dense_4h_to_h\.weight$": Split(world_size=world_size, dim=1),
            r".*word_embeddings\.weight$": Split(world_size=world_size, dim=1),
            # the head is tied to the embeddings, hence split on its input axis
            r".*lm_head\.weight$": Split(world_size=world_size, dim=1),
        },
        input_rules={r".*lm_head$": {0: "split -1"}},
        output_rules={
            r".*self_attention$": {0: "sum"},
            r".*\.mlp$": {0: "sum"},
            r".*word_embeddings$": {0: "gather -1"},
            r".*lm_head$": {0: "sum"},
        },
        attr_rules={
            r".*self_attention$": {
                "num_kv": partial(split_num_heads, world_size=world_size),
                "num_kv_heads": partial(split_num_heads, world_size=world_size),
                "num_heads": q_heads,
            }
        },
    )


def get_gpt2_config(model_config, devices: Sequence[torch.device]) -> Config:
    """GPT-2 stores Conv1D weights as [in, out]; c_attn fuses q, k, v as three groups on the output axis,
    which is the grouped-chunk split (slicing_configs.py:192-193)."""
    world_size = len(devices)
    num_heads = model_config.num_attention_heads
    head_dim = model_config.hidden_size // num_heads
    return Config(
        state_rules={
            r".*c_attn\.weight$": SplitInGroupedChunks(world_size=world_size, dim=1, num_groups=3, chunk_size=head_dim),
            r".*c_attn\.bias$": SplitInGroupedChunks(world_size=world_size, dim=0, num_groups=3, chunk_size=head_dim),
            r".*q_attn\.weight$": SplitInChunks(world_size=world_size, dim=1, chunk_size=head_dim),
            r".*q_attn\.bias$": SplitInChunks(world_size=world_size, dim=0, chunk_size=head_dim),
            r".*attn\.c_proj\.weight$": SplitInChunks(world_size=world_size, dim=0, chunk_size=head_dim),
            r".*attn\.c_proj\.bias$": Scale(world_size=world_size),
            r".*c_fc\.weight$": Split(world_size=world_size, dim=1),
            r".*c_fc\.bias$": Split(world_size=world_size, dim=0),
            r".*mlp\.c_proj\.weight$": Split(world_size=world_size, dim=0),
            r".*mlp\.c_proj\.bias$": Scale(world_size=world_size),
            r".*wte\.weight$": Split(world_size=world_size, dim=1),
            r".*wpe\.weight$": Split(world_size=world_size, dim=1),
            r".*lm_head\.weight$": Split(world_size=world_size, dim=1),
        },
        input_rules={r".*lm_head$": {0: "split -1"}},
        output_rules={
            r".*[0-9]\.attn$": {0: "sum"},
            r".*mlp$": {0: "sum"},
            r".*wte$": {0: "gather -1"},
            r".*wpe$": {0: "gather -1"},
            r".*lm_head$": {0: "sum"},
        },
        attr_rules={
            r".*attn\.c_attn$": {"nf": partial(split_inner_dim, num_heads=num_heads, world_size=world_size)},
            r".*attn\.q_attn$": {"nf": partial(split_inner_dim, num_heads=num_heads, world_size=world_size)},
            r".*mlp\.c_fc$": {"nf": partial(split_num_heads, world_size=world_size)},
            r".*[0-9]\.attn$": {
                "embed_dim": partial(split_inner_dim, num_heads=num_heads, world_size=world_size),
                "num_heads": partial(split_num_heads, world_size=world_size),
                "split_size": partial(split_inner_dim, num_heads=num_heads, world_size=world_size),
            },
        },
    )


PREDEFINED_CONFIGS: Dict[str, ConfigGetter] = {
    "gpt2": get_gpt2_config,
    "llama": get_llama_config,
    "RefinedWeb": get_refined_web_config,
    "falcon": get_refined_web_config,
}
