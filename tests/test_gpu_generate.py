"""`generate` on a model run as rank shards: every rank keeps the keys and values of its own heads in its own cache,
and the tokens must be those of the unsplit model (the reference's usage example: `model.generate(...)` on the
object `tensor_parallel` returns; its cache plumbing is src/tensor_parallel/aux_actions.py:7-15). fp32, greedy and
beam search, random tiny models of four families."""
from copy import deepcopy

import pytest
import torch

import tensor_parallel_amd as tp

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def tiny(family):
    import transformers as tf

    torch.manual_seed(0)
    common = dict(vocab_size=96, bos_token_id=1, eos_token_id=None, pad_token_id=0)
    if family == "llama":
        model = tf.LlamaForCausalLM(tf.LlamaConfig(hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
                                                   num_key_value_heads=2, max_position_embeddings=64, **common))
    elif family == "gpt2":
        model = tf.GPT2LMHeadModel(tf.GPT2Config(n_embd=64, n_head=4, n_layer=2, n_positions=64, **common))
    elif family == "bloom":
        model = tf.BloomForCausalLM(tf.BloomConfig(hidden_size=64, n_head=4, n_layer=2, **common))
    elif family == "t5":
        model = tf.T5ForConditionalGeneration(tf.T5Config(d_model=64, d_kv=16, num_heads=4, d_ff=128, num_layers=2, decoder_start_token_id=0,
                                                          **common))
    else:
        raise KeyError(family)
    model = model.eval()
    with torch.no_grad():
        for p in model.parameters():
            p.normal_(0.0, 0.2)  # far from flat logits: the argmax does not hinge on rounding
    return model


@pytest.mark.parametrize("family", ["llama", "gpt2", "bloom", "t5"])
@pytest.mark.parametrize("beams", [1, 3])
def test_generate_matches_the_unsplit_model(family, beams):
    model = tiny(family)
    ids = torch.randint(2, 96, (2, 6), generator=torch.Generator().manual_seed(1))
    kwargs = dict(max_new_tokens=8, do_sample=False, num_beams=beams, attention_mask=torch.ones_like(ids))
    with torch.no_grad():
        want = model.generate(ids, **kwargs)
    model_tp = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    with torch.no_grad():
        got = model_tp.generate(ids.to(DEV), **{k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in kwargs.items()})
    assert got.shape == want.shape and torch.equal(got.cpu(), want)


def test_each_rank_caches_its_own_heads():
    from transformers import DynamicCache

    model = tiny("llama")
    model_tp = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    ids = torch.randint(2, 96, (1, 5), generator=torch.Generator().manual_seed(1)).to(DEV)
    cache = DynamicCache(config=model.config)
    with torch.no_grad():
        ref = model(ids.cpu(), use_cache=True)
        out = model_tp(ids, past_key_values=cache, use_cache=True)
    assert out.past_key_values is cache and cache.get_seq_length() == 5
    mine, sibling = tp.kv_cache.rank_caches(cache, 2)
    assert mine is cache and sibling is not cache and sibling.get_seq_length() == 5
    k0, k1 = mine.layers[0].keys, sibling.layers[0].keys  # one of the two KV heads each
    assert k0.shape == k1.shape == (1, 1, 5, 16)
    torch.testing.assert_close(torch.cat([k0, k1], dim=1).cpu(), ref.past_key_values.layers[0].keys, rtol=1e-5, atol=1e-5)
    with torch.no_grad():  # one more token on top of the caches
        step = model_tp(ids[:, -1:], past_key_values=cache, use_cache=True)
        ref_step = model(ids[:, -1:].cpu(), past_key_values=ref.past_key_values, use_cache=True)
    assert cache.get_seq_length() == sibling.get_seq_length() == 6
    torch.testing.assert_close(step.logits.cpu(), ref_step.logits, rtol=1e-4, atol=1e-4)
    cache.crop(3)  # batch-level operations reach the siblings
    assert cache.get_seq_length() == sibling.get_seq_length() == 3
    with pytest.raises(ValueError, match="ranks"):
        tp.kv_cache.rank_caches(cache, 3)


def test_a_cache_filled_by_an_unsplit_model_is_refused():
    model = tiny("llama")
    ids = torch.randint(2, 96, (1, 5), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        full = model(ids, use_cache=True).past_key_values
    model_tp = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    with pytest.raises(NotImplementedError, match="empty cache"), torch.no_grad():
        model_tp(ids[:, -1:].to(DEV), past_key_values=full, use_cache=True)
