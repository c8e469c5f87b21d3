"""Pins oracle/naming.py against hand-derived names and the golden vectors written by the reference's own
code (tests/golden/make_golden.py -> tests/golden/naming.json)."""
import json
from pathlib import Path

import numpy as np
import pytest

from oracle import naming as onm
from oracle import slicing as osl

GOLDEN = json.loads((Path(__file__).parent / "golden" / "naming.json").read_text())


def test_hand_derived_llama_names():
    patterns = [r".*self_attn$", r".*self_attn$", r".*mlp$", r".*embed_tokens$", r".*lm_head$"]
    names = [
        "model.layers.0.self_attn.q_proj.weight",
        "model.layers.0.mlp.gate_proj.weight",
        "model.embed_tokens.weight",
        "lm_head.weight",
        "model.norm.weight",
    ]
    got = onm.get_parameter_name_mapping(names, patterns)
    assert got == {
        names[0]: "model.layers.0.self_attn.tp_wrapped_module.q_proj.weight",
        names[1]: "model.layers.0.mlp.tp_wrapped_module.gate_proj.weight",
        names[2]: "model.embed_tokens.tp_wrapped_module.weight",
        names[3]: "lm_head.tp_wrapped_module.weight",
        names[4]: "model.norm.weight",
    }


@pytest.mark.parametrize("case", GOLDEN["name_mapping"], ids=lambda c: c["label"])
def test_name_mapping_golden(case):
    assert onm.get_parameter_name_mapping(case["names"], case["module_patterns"]) == case["mapping"]


def _llama_rules(world):
    hd, q_per_kv = 8, 2
    return [
        (r".*self_attn\.q_proj\.weight$", lambda a, r: osl.split_in_chunks(a, world, 0, q_per_kv * hd, r)),
        (r".*self_attn\.k_proj\.weight$", lambda a, r: osl.split_in_chunks(a, world, 0, hd, r)),
        (r".*self_attn\.v_proj\.weight$", lambda a, r: osl.split_in_chunks(a, world, 0, hd, r)),
        (r".*self_attn\.o_proj\.weight$", lambda a, r: osl.split_in_chunks(a, world, 1, q_per_kv * hd, r)),
        (r".*mlp\.gate_proj\.weight$", lambda a, r: osl.split(a, world, 0, r)),
        (r".*mlp\.down_proj\.weight$", lambda a, r: osl.split(a, world, 1, r)),
        (r".*mlp\.up_proj\.weight$", lambda a, r: osl.split(a, world, 0, r)),
        (r".*embed_tokens.weight$", lambda a, r: osl.split(a, world, 1, r)),
        (r".*lm_head\.weight$", lambda a, r: osl.split(a, world, 0, r)),
    ]


@pytest.mark.parametrize("case", GOLDEN["convert_state_dict"], ids=lambda c: f"W{c['world_size']}-pre{int(c['for_pretrained'])}")
def test_convert_state_dict_golden(case):
    world = case["world_size"]
    state = {k: np.zeros(shape, dtype=np.uint8) for k, shape in case["input"].items()}
    patterns = [r".*self_attn$", r".*self_attn$", r".*mlp$", r".*embed_tokens$", r".*lm_head$"]
    out = onm.convert_state_dict(state, _llama_rules(world), patterns, world, for_pretrained=case["for_pretrained"])
    assert list(out.keys()) == list(case["output"].keys()) or set(out.keys()) == set(case["output"].keys())
    for k, shape in case["output"].items():
        assert list(out[k].shape) == shape, k


def test_first_match_and_passthrough():
    state = {"a.weight": np.arange(12).reshape(6, 2), "a.bias": np.arange(6), "norm.weight": np.arange(4)}
    rules = [
        (r"a\.(weight|bias)$", lambda a, r: osl.split(a, 2, 0, r)),
        (r"a\.weight$", lambda a, r: osl.split(a, 2, 1, r)),  # shadowed by the first rule
    ]
    out = onm.convert_state_dict(state, rules, [], 2)
    assert out["module_shards.1.a.weight"].shape == (3, 2) and out["module_shards.1.a.weight"][0, 0] == 6
    assert out["module_shards.0.a.bias"].tolist() == [0, 1, 2]
    assert out["module_shards.0.norm.weight"] is state["norm.weight"] is out["module_shards.1.norm.weight"]
    assert out["_sanity_check_params.1"].size == 0
