"""Hand-written rule tables for model families (reference: src/tensor_parallel/slicing_configs.py).

Carried here: BLOOM (slicing_configs.py:32-72), T5 (:75-137), BERT (:140-177), GPT-2 (:180-238), GPT-NeoX (:241-282),
CodeGen (:285-342), Llama (:345-406) and Falcon / RefinedWeb (:409-462). The state rules - which tensor is split
how - are those of the reference. The KV-cache rules of the reference (`select_kv_for_rank`, `gather_kv`) have no
counterpart in the tables: every rank is handed its own cache object (see kv_cache), so an attention module's cache
stays rank-local without a rule.
Attribute rules name the attributes of the model classes the reference was written against; attributes
a given transformers version no longer has are skipped when the shard is built.
"""
from __future__ import annotations

from functools import partial
from typing import Callable, Dict, Sequence

import torch

from .aux_actions import split_alibi, split_inner_dim, split_num_heads
from .config import Config
from .slicing import SliceSpec, tensor_split_range
from .state_actions import Scale, SegmentedAction, Split, SplitInChunks, SplitInGroupedChunks

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


def get_bloom_config(model_config, devices: Sequence[torch.device]) -> Config:
    """BLOOM fuses q, k, v per head: the fused weight's rows are heads of (q, k, v) * head_dim, so whole chunks of
    3 * head_dim rows go to a rank. The alibi bias arrives as [batch * heads, 1, keys] and is cut to the rank's
    heads on the way in (slicing_configs.py:32-72)."""
    world_size = len(devices)
    num_heads = model_config.n_head
    head_dim = model_config.hidden_size // num_heads
    return Config(
        state_rules={
            r".*self_attention\.query_key_value\.(weight|bias)$": SplitInChunks(world_size=world_size, dim=0, chunk_size=3 * head_dim),
            r".*self_attention\.dense\.weight$": SplitInChunks(world_size=world_size, dim=1, chunk_size=head_dim),
            r".*self_attention\.dense\.bias$": Scale(world_size=world_size),
            r".*mlp\.dense_h_to_4h\.(weight|bias)$": Split(world_size=world_size, dim=0),
            r".*mlp\.dense_4h_to_h\.weight$": Split(world_size=world_size, dim=1),
            r".*mlp\.dense_4h_to_h\.bias$": Scale(world_size=world_size),
            r".*word_embeddings\.weight$": Split(world_size=world_size, dim=1),
            # the head is tied to the embeddings, hence split on its input axis
            r".*lm_head\.weight$": Split(world_size=world_size, dim=1),
        },
        input_rules={
            r".*self_attention$": {"alibi": partial(split_alibi, num_heads=num_heads, world_size=world_size)},
            r".*lm_head$": {0: "split -1"},
        },
        output_rules={
            r".*self_attention\.dense$": {0: "sum"},
            r".*mlp\.dense_4h_to_h$": {0: "sum"},
            r".*word_embeddings$": {0: "gather -1"},
            r".*lm_head$": {0: "sum"},
        },
        attr_rules={r".*self_attention$": {"num_heads": partial(split_num_heads, world_size=world_size)}},
    )


def get_t5_config(model_config, devices: Sequence[torch.device]) -> Config:
    """T5: separate q, k, v of num_heads * d_kv rows each; the relative position bias is an embedding with one
    column per head (slicing_configs.py:75-137)."""
    world_size = len(devices)
    num_heads = model_config.num_heads
    head_dim = model_config.d_kv
    heads = partial(split_num_heads, world_size=world_size)
    state_rules = {
        rf".*SelfAttention\.{proj}\.(weight|bias)$": SplitInChunks(world_size=world_size, dim=0, chunk_size=head_dim)
        for proj in ("q", "k", "v")
    }
    state_rules.update({
        r".*relative_attention_bias\.weight$": Split(world_size=world_size, dim=1),
        r".*SelfAttention\.o\.weight$": SplitInChunks(world_size=world_size, dim=1, chunk_size=head_dim),
        # plain and gated feed-forward: wi / wi_0 / wi_1 column-parallel, wo row-parallel
        r".*DenseReluDense\.wi\.weight$": Split(world_size=world_size, dim=0),
        r".*DenseReluDense\.wi_0\.weight$": Split(world_size=world_size, dim=0),
        r".*DenseReluDense\.wi_1\.weight$": Split(world_size=world_size, dim=0),
        r".*DenseReluDense\.wo\.weight$": Split(world_size=world_size, dim=1),
        # embeddings on the hidden axis; the head is tied to them
        r".*embed_tokens\.weight$": Split(world_size=world_size, dim=1),
        r".*shared\.weight$": Split(world_size=world_size, dim=1),
        r".*lm_head\.weight$": Split(world_size=world_size, dim=1),
    })
    return Config(
        state_rules=state_rules,
        input_rules={r".*lm_head$": {0: "split -1"}},
        output_rules={
            r".*SelfAttention$": {0: "sum"},
            r".*DenseReluDense$": {0: "sum"},
            r".*shared$": {0: "gather -1"},
            r".*embed_tokens$": {0: "gather -1"},
            r".*lm_head$": {0: "sum"},
        },
        attr_rules={
            r".*SelfAttention$": {
                "n_heads": heads,
                "inner_dim": partial(split_inner_dim, num_heads=num_heads, world_size=world_size),
            },
            r".*relative_attention_bias$": {"embedding_dim": heads},
        },
    )


def get_bert_config(model_config, devices: Sequence[torch.device]) -> Config:
    """BERT (slicing_configs.py:140-177). The key and value patterns are unanchored in the reference and are kept so."""
    world_size = len(devices)
    num_heads = model_config.num_attention_heads
    head_dim = int(model_config.hidden_size / num_heads)
    by_head = SplitInChunks(world_size=world_size, dim=0, chunk_size=head_dim)
    return Config(
        state_rules={
            r".*self\.query\.(weight|bias)$": by_head,
            r"self\.key\.(weight|bias)": by_head,
            r"self\.value\.(weight|bias)": by_head,
            r".*attention\.output\.dense\.weight$": SplitInChunks(world_size=world_size, dim=1, chunk_size=head_dim),
            r".*attention\.output\.dense\.bias$": Scale(world_size=world_size),
            r".*intermediate\.dense\.(weight|bias)$": Split(world_size=world_size, dim=0),
            r".*[0-9]\.output\.dense\.weight$": Split(world_size=world_size, dim=1),
            r".*[0-9]\.output\.dense\.bias$": Scale(world_size=world_size),
            r".*word_embeddings\.weight$": Split(world_size=world_size, dim=1),
            r".*position_embeddings\.weight$": Split(world_size=world_size, dim=1),
            r".*token_type_embeddings\.weight$": Split(world_size=world_size, dim=1),
        },
        input_rules={},
        output_rules={
            r".*attention\.output\.dense$": {0: "sum"},
            r".*[0-9]\.output\.dense$": {0: "sum"},
            r".*word_embeddings$": {0: "gather -1"},
            r".*position_embeddings$": {0: "gather -1"},
            r".*token_type_embeddings$": {0: "gather -1"},
        },
        attr_rules={
            r".*attention\.self$": {
                "num_attention_heads": partial(split_num_heads, world_size=world_size),
                "all_head_size": partial(split_inner_dim, num_heads=num_heads, world_size=world_size),
            },
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


def get_gpt_neox_config(model_config, devices: Sequence[torch.device]) -> Config:
    """GPT-NeoX: fused per-head (q, k, v) rows like BLOOM, an untied output embedding split on the vocabulary
    (slicing_configs.py:241-282)."""
    world_size = len(devices)
    num_heads = model_config.num_attention_heads
    head_dim = model_config.hidden_size // num_heads
    return Config(
        state_rules={
            r".*attention\.query_key_value\.(weight|bias)$": SplitInChunks(world_size=world_size, dim=0, chunk_size=3 * head_dim),
            r".*attention\.dense\.weight$": SplitInChunks(world_size=world_size, dim=1, chunk_size=head_dim),
            r".*attention\.dense\.bias$": Scale(world_size=world_size),
            r".*mlp\.dense_h_to_4h\.(weight|bias)$": Split(world_size=world_size, dim=0),
            r".*mlp\.dense_4h_to_h\.weight$": Split(world_size=world_size, dim=1),
            r".*mlp\.dense_4h_to_h\.bias$": Scale(world_size=world_size),
            r".*embed_in\.weight$": Split(world_size=world_size, dim=1),
            r".*embed_out\.(weight|bias)$": Split(world_size=world_size, dim=0),
        },
        input_rules={},
        output_rules={
            r".*attention$": {0: "sum"},
            r".*mlp$": {0: "sum"},
            r".*embed_in$": {0: "gather -1"},
            r".*embed_out$": {0: "gather -1"},
        },
        attr_rules={
            r".*attention$": {
                "num_attention_heads": partial(split_num_heads, world_size=world_size),
                "hidden_size": partial(split_inner_dim, num_heads=num_heads, world_size=world_size),
            }
        },
    )


class SplitCodegenQKV(SegmentedAction):
    """CodeGen's fused qkv_proj weight [3 * hidden, hidden] is laid out for 4 model-parallel blocks: its rows read
    as (block, {q, v, k}, head within block, head_dim). A rank takes whole groups of 4 consecutive heads in
    (block, head) order and lays them out again as 4 blocks of its own, so the module's own un-fusing still works
    on the shard (slicing_configs.py:294-308, which does this with two reshape/permute round trips). `undo` scatters
    the shards back to the rows they came from, a true inverse (the reference inherits a plain concatenation)."""

    BLOCKS = 4

    def __init__(self, world_size: int, head_dim: int):
        super().__init__()
        self.world_size = world_size
        self.head_dim = head_dim

    def _dim_for(self, ndim: int) -> int:
        return 0

    def spec(self, shape: Sequence[int], rank: int) -> SliceSpec:
        rows, hd, blocks = shape[0], self.head_dim, self.BLOCKS
        assert rows % (3 * blocks * hd) == 0, tuple(shape)
        per_block = rows // (3 * blocks * hd)  # heads of one block; also the number of 4-head groups
        start, length = tensor_split_range(per_block, self.world_size, rank)
        if length == 0:
            raise ValueError(f"rank {rank} of {self.world_size} would own no CodeGen head group ({per_block} groups)")
        segments = []
        for out_block in range(blocks):
            for part in range(3):
                for i in range(length):
                    head = blocks * start + out_block * length + i  # position in (block, head) order
                    src = ((head // per_block * 3 + part) * per_block + head % per_block) * hd
                    if segments and segments[-1][0] + segments[-1][1] == src:
                        segments[-1] = (segments[-1][0], segments[-1][1] + hd)
                    else:
                        segments.append((src, hd))
        return SliceSpec(tuple(shape), 0, tuple(segments))



def get_codegen_config(model_config, devices: Sequence[torch.device]) -> Config:
    """CodeGen (slicing_configs.py:285-342): heads move in groups of 4, the block count its fused qkv is laid out for."""
    world_size = len(devices)
    num_heads = model_config.num_attention_heads
    head_dim = model_config.hidden_size // num_heads

    def head_groups(n, rank):
        return 4 * split_num_heads(n // 4, rank=rank, world_size=world_size)

    return Config(
        state_rules={
            r".*attn\.qkv_proj\.weight$": SplitCodegenQKV(world_size=world_size, head_dim=head_dim),
            r".*attn\.out_proj\.weight$": SplitInChunks(world_size=world_size, dim=1, chunk_size=4 * head_dim),
            r".*mlp\.fc_in\.(weight|bias)$": Split(world_size=world_size, dim=0),
            r".*mlp\.fc_out\.weight$": Split(world_size=world_size, dim=1),
            r".*mlp\.fc_out\.bias$": Scale(world_size=world_size),
            r".*wte\.weight$": Split(world_size=world_size, dim=1),
            r".*lm_head\.(weight|bias)$": Split(world_size=world_size, dim=0),
        },
        input_rules={},
        output_rules={
            r".*attn$": {0: "sum"},
            r".*mlp$": {0: "sum"},
            r".*wte$": {0: "gather -1"},
            r".*lm_head$": {0: "gather -1"},
        },
        attr_rules={
            r".*attn$": {
                "embed_dim": partial(split_inner_dim, num_heads=num_heads // 4, world_size=world_size),
                "num_attention_heads": head_groups,
            }
        },
    )


PREDEFINED_CONFIGS: Dict[str, ConfigGetter] = {
    "bloom": get_bloom_config,
    "t5": get_t5_config,
    "bert": get_bert_config,
    "gpt2": get_gpt2_config,
    "gpt_neox": get_gpt_neox_config,
    "codegen": get_codegen_config,
    "llama": get_llama_config,
    "RefinedWeb": get_refined_web_config,
    "falcon": get_refined_web_config,
}
