"""Writes tests/golden/rule_tables.json by running the REFERENCE's predefined slicing configs
(src/tensor_parallel/slicing_configs.py:32-462) on synthetic parameters.

Run by hand, in the development container only (needs /root/reference): `python tests/golden/make_rule_tables.py`.
For every model family and world size it records, per parameter and rank, the shard's shape and two checksums of
its contents (parameters are filled with distinct integers, so the checksums identify WHICH elements a rank got
and in which order), the patterns and string values of the module rules, and what the attribute rules return on
sample values. The fixture is data; nothing of the reference's source is stored.
"""
import json
import sys
from pathlib import Path
from types import SimpleNamespace

sys.path.insert(0, "/root/reference/src")

import torch  # noqa: E402
from tensor_parallel.slicing_configs import PREDEFINED_CONFIGS  # noqa: E402
from tensor_parallel.state_actions import Scale  # noqa: E402

OUT = Path(__file__).resolve().parent / "rule_tables.json"
MOD = (1 << 61) - 1


def fill(shape):
    n = 1
    for s in shape:
        n *= s
    return (torch.arange(n, dtype=torch.int64) * 7 + 3).reshape(shape)


def checksums(t):
    flat = t.reshape(-1).to(torch.int64)
    weights = torch.arange(1, flat.numel() + 1, dtype=torch.int64)
    return [int(flat.sum().item() % MOD), int(((flat % 1000003) * (weights % 1000033)).sum().item() % MOD)]


# model type -> (config namespace, [(parameter name, shape)], sample attribute values)
H, HEADS, HD, FF, V = 96, 12, 8, 384, 50
FAMILIES = {
    "bloom": (SimpleNamespace(model_type="bloom", n_head=HEADS, hidden_size=H), [
        ("transformer.h.0.self_attention.query_key_value.weight", (3 * H, H)), ("transformer.h.0.self_attention.query_key_value.bias", (3 * H,)),
        ("transformer.h.0.self_attention.dense.weight", (H, H)), ("transformer.h.0.self_attention.dense.bias", (H,)),
        ("transformer.h.0.mlp.dense_h_to_4h.weight", (FF, H)), ("transformer.h.0.mlp.dense_h_to_4h.bias", (FF,)),
        ("transformer.h.0.mlp.dense_4h_to_h.weight", (H, FF)), ("transformer.h.0.mlp.dense_4h_to_h.bias", (H,)),
        ("transformer.word_embeddings.weight", (V, H)), ("lm_head.weight", (V, H)), ("transformer.ln_f.weight", (H,))]),
    "t5": (SimpleNamespace(model_type="t5", num_heads=HEADS, d_kv=HD), [
        ("encoder.block.0.layer.0.SelfAttention.q.weight", (H, H)), ("encoder.block.0.layer.0.SelfAttention.k.weight", (H, H)),
        ("encoder.block.0.layer.0.SelfAttention.v.weight", (H, H)), ("encoder.block.0.layer.0.SelfAttention.o.weight", (H, H)),
        ("encoder.block.0.layer.0.SelfAttention.relative_attention_bias.weight", (32, HEADS)),
        ("encoder.block.0.layer.1.DenseReluDense.wi.weight", (FF, H)), ("decoder.block.0.layer.2.DenseReluDense.wi_0.weight", (FF, H)),
        ("decoder.block.0.layer.2.DenseReluDense.wi_1.weight", (FF, H)), ("encoder.block.0.layer.1.DenseReluDense.wo.weight", (H, FF)),
        ("shared.weight", (V, H)), ("encoder.embed_tokens.weight", (V, H)), ("lm_head.weight", (V, H)), ("encoder.final_layer_norm.weight", (H,))]),
    "bert": (SimpleNamespace(model_type="bert", num_attention_heads=HEADS, hidden_size=H), [
        ("bert.encoder.layer.0.attention.self.query.weight", (H, H)), ("bert.encoder.layer.0.attention.self.query.bias", (H,)),
        ("bert.encoder.layer.0.attention.self.key.weight", (H, H)), ("bert.encoder.layer.0.attention.self.key.bias", (H,)),
        ("bert.encoder.layer.0.attention.self.value.weight", (H, H)), ("bert.encoder.layer.0.attention.self.value.bias", (H,)),
        ("bert.encoder.layer.0.attention.output.dense.weight", (H, H)), ("bert.encoder.layer.0.attention.output.dense.bias", (H,)),
        ("bert.encoder.layer.0.intermediate.dense.weight", (FF, H)), ("bert.encoder.layer.0.intermediate.dense.bias", (FF,)),
        ("bert.encoder.layer.0.output.dense.weight", (H, FF)), ("bert.encoder.layer.0.output.dense.bias", (H,)),
        ("bert.embeddings.word_embeddings.weight", (V, H)), ("bert.embeddings.position_embeddings.weight", (64, H)),
        ("bert.embeddings.token_type_embeddings.weight", (2, H)), ("bert.embeddings.LayerNorm.weight", (H,))]),
    "gpt2": (SimpleNamespace(model_type="gpt2", num_attention_heads=HEADS, hidden_size=H), [
        ("transformer.h.0.attn.c_attn.weight", (H, 3 * H)), ("transformer.h.0.attn.c_attn.bias", (3 * H,)),
        ("transformer.h.0.attn.c_proj.weight", (H, H)), ("transformer.h.0.attn.c_proj.bias", (H,)),
        ("transformer.h.0.mlp.c_fc.weight", (H, FF)), ("transformer.h.0.mlp.c_fc.bias", (FF,)),
        ("transformer.h.0.mlp.c_proj.weight", (FF, H)), ("transformer.h.0.mlp.c_proj.bias", (H,)),
        ("transformer.wte.weight", (V, H)), ("transformer.wpe.weight", (64, H)), ("lm_head.weight", (V, H))]),
    "gpt_neox": (SimpleNamespace(model_type="gpt_neox", num_attention_heads=HEADS, hidden_size=H), [
        ("gpt_neox.layers.0.attention.query_key_value.weight", (3 * H, H)), ("gpt_neox.layers.0.attention.query_key_value.bias", (3 * H,)),
        ("gpt_neox.layers.0.attention.dense.weight", (H, H)), ("gpt_neox.layers.0.attention.dense.bias", (H,)),
        ("gpt_neox.layers.0.mlp.dense_h_to_4h.weight", (FF, H)), ("gpt_neox.layers.0.mlp.dense_h_to_4h.bias", (FF,)),
        ("gpt_neox.layers.0.mlp.dense_4h_to_h.weight", (H, FF)), ("gpt_neox.layers.0.mlp.dense_4h_to_h.bias", (H,)),
        ("gpt_neox.embed_in.weight", (V, H)), ("embed_out.weight", (V, H)), ("gpt_neox.final_layer_norm.weight", (H,))]),
    "codegen": (SimpleNamespace(model_type="codegen", num_attention_heads=HEADS, hidden_size=H), [
        ("transformer.h.0.attn.qkv_proj.weight", (3 * H, H)), ("transformer.h.0.attn.out_proj.weight", (H, H)),
        ("transformer.h.0.mlp.fc_in.weight", (FF, H)), ("transformer.h.0.mlp.fc_in.bias", (FF,)),
        ("transformer.h.0.mlp.fc_out.weight", (H, FF)), ("transformer.h.0.mlp.fc_out.bias", (H,)),
        ("transformer.wte.weight", (V, H)), ("lm_head.weight", (V, H)), ("lm_head.bias", (V,))]),
    "llama": (SimpleNamespace(model_type="llama", num_attention_heads=HEADS, num_key_value_heads=4, hidden_size=H), [
        ("model.layers.0.self_attn.q_proj.weight", (H, H)), ("model.layers.0.self_attn.k_proj.weight", (4 * HD, H)),
        ("model.layers.0.self_attn.v_proj.weight", (4 * HD, H)), ("model.layers.0.self_attn.o_proj.weight", (H, H)),
        ("model.layers.0.mlp.gate_proj.weight", (FF, H)), ("model.layers.0.mlp.up_proj.weight", (FF, H)),
        ("model.layers.0.mlp.down_proj.weight", (H, FF)), ("model.embed_tokens.weight", (V, H)), ("lm_head.weight", (V, H)),
        ("model.norm.weight", (H,))]),
    "RefinedWeb": (SimpleNamespace(model_type="RefinedWeb", num_attention_heads=HEADS, n_head=HEADS, n_head_kv=4, hidden_size=H,
                                   bias=False, alibi=False), [
        ("transformer.h.0.self_attention.query_key_value.weight", ((HEADS + 8) * HD, H)), ("transformer.h.0.self_attention.dense.weight", (H, H)),
        ("transformer.h.0.mlp.dense_h_to_4h.weight", (FF, H)), ("transformer.h.0.mlp.dense_4h_to_h.weight", (H, FF)),
        ("transformer.word_embeddings.weight", (V, H)), ("lm_head.weight", (V, H)), ("transformer.ln_f.weight", (H,))]),
}
ATTR_SAMPLES = {"num_heads": HEADS, "n_heads": HEADS, "num_attention_heads": HEADS, "inner_dim": H, "hidden_size": H, "embed_dim": H,
                "all_head_size": H, "split_size": H, "nf": 3 * H, "embedding_dim": HEADS,
                "num_key_value_heads": 4, "num_kv": 4}


def main():
    out = {}
    for family, (cfg_ns, params) in FAMILIES.items():
        out[family] = {}
        for world in (2, 3):
            cfg = PREDEFINED_CONFIGS[family](cfg_ns, [torch.device("cpu")] * world)
            entry = {"params": {}, "input_rules": {}, "output_rules": {}, "attr_rules": {}}
            for name, shape in params:
                action = next((a for p, a in cfg.state_rules.items() if p.search(name)), None)
                if action is None:
                    entry["params"][name] = {"shape": list(shape), "rule": None}
                    continue
                if isinstance(action, Scale):
                    entry["params"][name] = {"shape": list(shape), "rule": "scale"}
                    continue
                t = fill(shape)
                shards = [action(t, rank=r) for r in range(world)]
                entry["params"][name] = {"shape": list(shape), "rule": "split",
                                         "shards": [{"shape": list(s.shape), "sums": checksums(s)} for s in shards]}
            for kind, rules in (("input_rules", cfg.input_rules), ("output_rules", cfg.output_rules)):
                for pattern, actions in rules.items():
                    entry[kind][pattern.pattern] = {str(k): (v if isinstance(v, str) else "<callable>") for k, v in actions.items()}
            for pattern, actions in cfg.attr_rules.items():
                entry["attr_rules"][pattern.pattern] = {
                    attr: [fn(ATTR_SAMPLES[attr], rank=r) for r in range(world)] for attr, fn in actions.items()}
            out[family][str(world)] = entry
    # bloom's alibi input rule: [batch * heads, 1, keys] split over heads
    from tensor_parallel.aux_actions import split_alibi
    alibi = fill((2 * HEADS, 1, 5))
    out["bloom_alibi"] = {str(w): [checksums(split_alibi(alibi, rank=r, num_heads=HEADS, world_size=w)) + list(split_alibi(alibi, rank=r, num_heads=HEADS, world_size=w).shape)
                                   for r in range(w)] for w in (2, 3)}
    OUT.write_text(json.dumps(out, indent=1, sort_keys=True) + "\n")
    print("wrote", OUT, OUT.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
