"""Writes tests/golden/naming.json by running the REFERENCE's own name-mapping and state-dict conversion code.

Run by hand, in the development container only (needs /root/reference): `python tests/golden/make_golden.py`.
Covers the two functions whose behaviour is string/regex handling that no closed form pins:
`get_parameter_name_mapping` (src/tensor_parallel/config.py:157-191) and the key layout of
`convert_state_dict` (src/tensor_parallel/dispatch.py:75-131). Tensors are meta tensors: only names and
shapes are recorded. The fixture is data; nothing of the reference's source is stored.
"""
import json
import sys
from pathlib import Path
from types import SimpleNamespace

sys.path.insert(0, "/root/reference/src")

import torch  # noqa: E402
from tensor_parallel.config import Config, get_parameter_name_mapping  # noqa: E402
from tensor_parallel.dispatch import convert_state_dict  # noqa: E402
from tensor_parallel.slicing_configs import get_llama_config, get_refined_web_config  # noqa: E402

OUT = Path(__file__).resolve().parent / "naming.json"


def llama_names(layers=2):
    names = ["model.embed_tokens.weight", "model.norm.weight", "lm_head.weight"]
    for i in range(layers):
        p = f"model.layers.{i}."
        names += [p + s for s in (
            "self_attn.q_proj.weight", "self_attn.k_proj.weight", "self_attn.v_proj.weight", "self_attn.o_proj.weight",
            "mlp.gate_proj.weight", "mlp.up_proj.weight", "mlp.down_proj.weight",
            "input_layernorm.weight", "post_attention_layernorm.weight")]
    return names


def falcon_names(layers=2):
    names = ["transformer.word_embeddings.weight", "transformer.ln_f.weight", "transformer.ln_f.bias", "lm_head.weight"]
    for i in range(layers):
        p = f"transformer.h.{i}."
        names += [p + s for s in (
            "self_attention.query_key_value.weight", "self_attention.dense.weight", "mlp.dense_h_to_4h.weight",
            "mlp.dense_4h_to_h.weight", "ln_attn.weight", "ln_attn.bias", "ln_mlp.weight", "ln_mlp.bias")]
    return names


def main():
    cases = []
    devices = [torch.device("cpu")] * 2
    llama_cfg = get_llama_config(SimpleNamespace(model_type="llama", hidden_size=64, num_attention_heads=8, num_key_value_heads=4), devices)
    falcon_cfg = get_refined_web_config(
        SimpleNamespace(model_type="RefinedWeb", hidden_size=64, n_head=8, n_head_kv=2, num_attention_heads=8, bias=False, alibi=False), devices)

    def record(label, cfg, names):
        patterns = [p.pattern for p in cfg.input_rules] + [p.pattern for p in cfg.output_rules]
        cases.append({"label": label, "module_patterns": patterns, "names": names,
                      "mapping": dict(get_parameter_name_mapping(names, cfg))})

    record("llama", llama_cfg, llama_names())
    record("falcon", falcon_cfg, falcon_names())
    adversarial = Config(
        state_rules={},
        input_rules={r"^a\.b$": {0: "split -1"}, r"block\.": {0: "scale"}, r"c": {0: "scale"}},
        output_rules={r"^a\.b$": {0: "sum"}, r"a\.b": {0: "sum"}, r".*mlp$": {0: "sum"}, r"x.y$": {0: "sum"}},
        attr_rules={},
    )
    record("adversarial", adversarial, [
        "a.b.weight", "a.b", "a.bc.weight", "block.0.mlp.fc.weight", "block.0.mlp.mlp.weight", "c.d.c.e", "xzy.w", "x.y.z",
        "prefix.a.b.bias", "mlp", "mlp.", "deep.mlp.a.b.c.weight",
    ])

    # convert_state_dict: names and shapes, llama rules, W = 2 and 3
    conv = []
    for world in (2, 3):
        devs = [torch.device("cpu")] * world
        cfg = get_llama_config(SimpleNamespace(model_type="llama", hidden_size=64, num_attention_heads=8, num_key_value_heads=4), devs)
        state = {}
        for n in llama_names(1):
            if "embed_tokens" in n or "lm_head" in n:
                shape = (100, 64)
            elif "norm" in n:
                shape = (64,)
            elif "q_proj" in n or "o_proj" in n:
                shape = (64, 64)
            elif "k_proj" in n or "v_proj" in n:
                shape = (32, 64)
            elif "down_proj" in n:
                shape = (64, 172)
            else:
                shape = (172, 64)
            state[n] = torch.empty(shape, device="meta")
        for pre in (False, True):
            out = convert_state_dict(state, cfg, world, for_pretrained=pre)
            conv.append({"world_size": world, "for_pretrained": pre,
                         "input": {k: list(v.shape) for k, v in state.items()},
                         "output": {k: list(v.shape) for k, v in out.items()}})
    OUT.write_text(json.dumps({"name_mapping": cases, "convert_state_dict": conv}, indent=1, sort_keys=True))
    print("wrote", OUT, len(cases), len(conv))


if __name__ == "__main__":
    main()
