"""The predefined rule tables against vectors written by the reference's own tables.

`tests/golden/rule_tables.json` was produced by `tests/golden/make_rule_tables.py`, which ran the reference's
PREDEFINED_CONFIGS (src/tensor_parallel/slicing_configs.py:32-462) on integer-filled parameters and recorded every
rank's shard shape and two order-sensitive checksums, the module rules' patterns and string actions, and the
attribute rules' results. Here the package's tables produce slice specs for the same shapes; the specs are applied
with numpy (no device needed) and must reproduce the recorded shards. KV-cache rules are not carried by the
package: the reference's entries that exist only for the cache are listed in CACHE_ONLY and skipped.
"""
import json
import re
from pathlib import Path
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from tensor_parallel_amd.aux_actions import alibi_spec
from tensor_parallel_amd.slicing_configs import PREDEFINED_CONFIGS
from tensor_parallel_amd.state_actions import Scale, SegmentedAction

GOLDEN = json.loads((Path(__file__).parent / "golden" / "rule_tables.json").read_text())
MOD = (1 << 61) - 1
H, HEADS, HD = 96, 12, 8
MODEL_CONFIGS = {
    "bloom": SimpleNamespace(model_type="bloom", n_head=HEADS, hidden_size=H),
    "t5": SimpleNamespace(model_type="t5", num_heads=HEADS, d_kv=HD),
    "bert": SimpleNamespace(model_type="bert", num_attention_heads=HEADS, hidden_size=H),
    "gpt2": SimpleNamespace(model_type="gpt2", num_attention_heads=HEADS, hidden_size=H),
    "gpt_neox": SimpleNamespace(model_type="gpt_neox", num_attention_heads=HEADS, hidden_size=H),
    "codegen": SimpleNamespace(model_type="codegen", num_attention_heads=HEADS, hidden_size=H),
    "llama": SimpleNamespace(model_type="llama", num_attention_heads=HEADS, num_key_value_heads=4, hidden_size=H),
    "RefinedWeb": SimpleNamespace(model_type="RefinedWeb", num_attention_heads=HEADS, n_head=HEADS, n_head_kv=4, hidden_size=H,
                                  bias=False, alibi=False),
}
ATTR_SAMPLES = {"num_heads": HEADS, "n_heads": HEADS, "num_attention_heads": HEADS, "inner_dim": H, "hidden_size": H, "embed_dim": H,
                "all_head_size": H, "split_size": H, "nf": 3 * H, "embedding_dim": HEADS,
                "num_key_value_heads": 4, "num_kv": 4}
# arguments / outputs whose reference rules only move the attention cache between ranks
CACHE_ONLY = {"layer_past", "past_key_value", "1", "2"}
# attributes the package also rewrites because the in-library Falcon of current transformers renamed them
EXTRA_ATTRS = {"num_kv_heads"}
CASES = [(f, w) for f in MODEL_CONFIGS for w in (2, 3)]


def fill(shape):
    return (np.arange(int(np.prod(shape)), dtype=np.int64) * 7 + 3).reshape(shape)


def checksums(a):
    flat = a.reshape(-1).astype(np.int64)
    weights = np.arange(1, flat.size + 1, dtype=np.int64)
    return [int(flat.sum() % MOD), int(((flat % 1000003) * (weights % 1000033)).sum() % MOD)]


def take(a, spec):
    return np.concatenate([np.take(a, np.arange(s, s + n), axis=spec.dim) for s, n in spec.segments], axis=spec.dim)


def config_for(family, world):
    return PREDEFINED_CONFIGS[family](MODEL_CONFIGS[family], [torch.device("cpu")] * world)


def state_action(cfg, name):
    return next((a for p, a in cfg.state_rules.items() if (p if hasattr(p, "search") else re.compile(p)).search(name)), None)


@pytest.mark.parametrize("family,world", CASES)
def test_state_rules_give_the_reference_shards(family, world):
    cfg = config_for(family, world)
    for name, want in GOLDEN[family][str(world)]["params"].items():
        action = state_action(cfg, name)
        if want["rule"] is None:
            assert action is None, name
        elif want["rule"] == "scale":
            assert isinstance(action, Scale) and action.world_size == world, name
        else:
            assert isinstance(action, SegmentedAction), name
            full = fill(want["shape"])
            for rank, shard in enumerate(want["shards"]):
                spec = action.spec(tuple(want["shape"]), rank)
                got = take(full, spec)
                assert list(got.shape) == shard["shape"] == list(spec.out_shape), (name, rank)
                assert checksums(got) == shard["sums"], (name, rank)


@pytest.mark.parametrize("family,world", CASES)
def test_shards_partition_every_split_parameter(family, world):
    """Size-independent property: over all ranks every element of a split parameter is taken exactly once."""
    cfg = config_for(family, world)
    for name, want in GOLDEN[family][str(world)]["params"].items():
        action = state_action(cfg, name)
        if not isinstance(action, SegmentedAction):
            continue
        shape = tuple(want["shape"])
        taken = np.concatenate([take(fill(shape), action.spec(shape, r)).reshape(-1) for r in range(world)])
        assert np.array_equal(np.sort(taken), fill(shape).reshape(-1)), name


@pytest.mark.parametrize("family,world", CASES)
def test_module_rules_match_the_reference(family, world):
    cfg = config_for(family, world)
    want = GOLDEN[family][str(world)]
    for kind, rules in (("input_rules", cfg.input_rules), ("output_rules", cfg.output_rules)):
        mine = {(p.pattern if hasattr(p, "pattern") else p): {str(k): (v if isinstance(v, str) else "<callable>") for k, v in a.items()}
                for p, a in rules.items()}
        ref = {p: {k: v for k, v in a.items() if k not in CACHE_ONLY} for p, a in want[kind].items()}
        ref = {p: a for p, a in ref.items() if a}
        assert mine == ref, kind


@pytest.mark.parametrize("family,world", CASES)
def test_attr_rules_match_the_reference(family, world):
    cfg = config_for(family, world)
    want = GOLDEN[family][str(world)]["attr_rules"]
    mine = {(p.pattern if hasattr(p, "pattern") else p): a for p, a in cfg.attr_rules.items()}
    assert set(mine) == set(want)
    for pattern, attrs in want.items():
        assert set(mine[pattern]) - set(attrs) <= EXTRA_ATTRS and set(attrs) <= set(mine[pattern]), pattern
        for attr, per_rank in attrs.items():
            assert [mine[pattern][attr](ATTR_SAMPLES[attr], rank=r) for r in range(world)] == per_rank, (pattern, attr)


@pytest.mark.parametrize("world", [2, 3])
def test_alibi_rows_match_the_reference(world):
    full = fill((2 * HEADS, 1, 5))
    for rank, (s0, s1, *shape) in enumerate(GOLDEN["bloom_alibi"][str(world)]):
        got = take(full, alibi_spec(full.shape, rank=rank, num_heads=HEADS, world_size=world))
        assert list(got.shape) == shape and checksums(got) == [s0, s1]


def test_codegen_qkv_split_against_the_permutation_written_out():
    """Independent of the fixture: the shard must equal what un-fusing, taking whole 4-head groups in (block, head)
    order and re-fusing gives, written with numpy reshapes (a different formulation from the action's index runs)."""
    heads, hd, hidden = 24, 4, 10
    w = fill((3 * heads * hd, hidden))
    for world in (1, 2, 3, 4):
        cfg = PREDEFINED_CONFIGS["codegen"](SimpleNamespace(model_type="codegen", num_attention_heads=heads, hidden_size=heads * hd),
                                            [torch.device("cpu")] * world)
        action = state_action(cfg, "h.0.attn.qkv_proj.weight")
        per_block = heads // 4
        by_head = w.reshape(4, 3, per_block, hd, hidden).transpose(0, 2, 1, 3, 4).reshape(heads, 3, hd, hidden)
        bounds = np.array_split(np.arange(per_block), world)
        for rank in range(world):
            mine_heads = by_head[4 * bounds[rank][0]: 4 * (bounds[rank][-1] + 1)]
            n = len(bounds[rank])
            want = mine_heads.reshape(4, n, 3, hd, hidden).transpose(0, 2, 1, 3, 4).reshape(-1, hidden)
            assert np.array_equal(take(w, action.spec(w.shape, rank)), want), (world, rank)
