"""The predefined rule tables on the device: shards cut by the HIP region mover against the vectors the reference's
tables wrote (bit-exact), and tiny random models of every family run as two rank shards against the unsplit model."""
import json
from copy import deepcopy
from pathlib import Path
from types import SimpleNamespace

import pytest
import torch

import tensor_parallel_amd as tp
from tensor_parallel_amd.aux_actions import split_alibi
from tensor_parallel_amd.slicing_configs import PREDEFINED_CONFIGS
from tensor_parallel_amd.state_actions import SegmentedAction

from test_rule_tables import CASES, GOLDEN, HEADS, MOD, MODEL_CONFIGS, state_action

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def fill(shape):
    n = 1
    for s in shape:
        n *= s
    return (torch.arange(n, dtype=torch.int64) * 7 + 3).reshape(shape)


def checksums(t):
    flat = t.reshape(-1).to(torch.int64).cpu()
    weights = torch.arange(1, flat.numel() + 1, dtype=torch.int64)
    return [int(flat.sum().item() % MOD), int(((flat % 1000003) * (weights % 1000033)).sum().item() % MOD)]


@pytest.mark.parametrize("family,world", CASES)
def test_device_shards_match_the_reference_vectors(family, world):
    cfg = PREDEFINED_CONFIGS[family](MODEL_CONFIGS[family], [DEV] * world)
    for name, want in GOLDEN[family][str(world)]["params"].items():
        action = state_action(cfg, name)
        if not isinstance(action, SegmentedAction):
            continue
        full = fill(want["shape"]).to(DEV)
        shards = [action(full, rank) for rank in range(world)]
        for rank, (got, ref) in enumerate(zip(shards, want["shards"])):
            assert got.is_cuda and got.is_contiguous() and list(got.shape) == ref["shape"], (name, rank)
            assert checksums(got) == ref["sums"], (name, rank)
        assert torch.equal(action.undo(shards), full), name  # un-sharding restores every element to its place


@pytest.mark.parametrize("world", [2, 3])
def test_device_alibi_split(world):
    full = fill((2 * HEADS, 1, 5)).to(DEV)
    for rank, (s0, s1, *shape) in enumerate(GOLDEN["bloom_alibi"][str(world)]):
        got = split_alibi(full, rank=rank, num_heads=HEADS, world_size=world)
        assert list(got.shape) == shape and checksums(got) == [s0, s1]


def _tiny(family):
    import transformers as tf

    if family == "bloom":
        return tf.BloomForCausalLM(tf.BloomConfig(hidden_size=64, n_head=4, n_layer=2, vocab_size=128)), "causal"
    if family == "gpt_neox":
        return tf.GPTNeoXForCausalLM(tf.GPTNeoXConfig(hidden_size=64, num_attention_heads=4, num_hidden_layers=2, intermediate_size=256,
                                                        vocab_size=128, max_position_embeddings=64)), "causal"
    if family == "gpt2":
        return tf.GPT2LMHeadModel(tf.GPT2Config(n_embd=64, n_head=4, n_layer=2, vocab_size=128, n_positions=64)), "causal"
    if family == "codegen":
        return tf.CodeGenForCausalLM(tf.CodeGenConfig(n_embd=64, n_head=8, n_layer=2, rotary_dim=8, vocab_size=128, n_positions=64,
                                                        n_ctx=64)), "causal"
    if family == "bert":
        return tf.BertModel(tf.BertConfig(hidden_size=64, num_attention_heads=4, num_hidden_layers=2, intermediate_size=128, vocab_size=128,
                                           max_position_embeddings=64)), "encoder"
    if family == "t5":
        return tf.T5ForConditionalGeneration(tf.T5Config(d_model=64, d_kv=16, num_heads=4, d_ff=128, num_layers=2, vocab_size=128,
                                                           decoder_start_token_id=0)), "seq2seq"
    raise KeyError(family)


@pytest.mark.parametrize("family", ["bloom", "gpt_neox", "gpt2", "codegen", "bert", "t5"])
def test_tiny_model_as_two_rank_shards(family):
    """fp32, N(0, 0.05) weights from seed 0, batch 2 x 12 tokens, W = 2 on one device: the outputs of the sharded model
    against the unsplit one (rtol 1e-5 on fp32 Linears, as for the rank-shard Linear itself)."""
    torch.manual_seed(0)
    model, kind = _tiny(family)
    model = model.eval()
    with torch.no_grad():
        for p in model.parameters():
            p.normal_(0.0, 0.05)
    ids = torch.randint(0, 128, (2, 12), generator=torch.Generator().manual_seed(1))
    kwargs = {"input_ids": ids}
    if kind == "seq2seq":
        kwargs["decoder_input_ids"] = torch.randint(0, 128, (2, 7), generator=torch.Generator().manual_seed(2))
    if kind != "encoder":
        kwargs["use_cache"] = False

    def first(out):
        return out.logits if hasattr(out, "logits") else out.last_hidden_state

    with torch.no_grad():
        ref = first(model(**kwargs))
    model_tp = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    total = sum(p.numel() for p in model.parameters())
    for shard in model_tp.wrapped_model.module_shards:  # the table matched: a rank holds about half of the weights
        assert sum(p.numel() for p in shard.parameters()) < 0.8 * total
    with torch.no_grad():
        out = first(model_tp(**{k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in kwargs.items()}))
    assert out.shape == ref.shape
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-5, atol=1e-4 * ref.abs().max().item())
