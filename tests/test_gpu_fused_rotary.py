"""`tp.attention.fuse_rotary_`: the attention modules of a Llama run rotary embedding, cache append and attention core on the
library's kernels, inside `tp.tensor_parallel` on two ranks, against the same model with the module's own forward (torch
rotary embedding and cache update, the library's attention core): logits of the prefill and of decode steps, the cache
contents bit for bit, `generate`."""
from copy import deepcopy

import pytest
import torch

import tensor_parallel_amd as tp

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)
RTOL = 2e-2


def tiny_llama(dtype):
    from transformers import LlamaConfig, LlamaForCausalLM

    name = tp.attention.register()
    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=300, hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, max_position_embeddings=2048, attn_implementation="eager", bos_token_id=1, eos_token_id=None,
                      pad_token_id=0)
    model = LlamaForCausalLM(cfg).to(dtype).eval()
    model.config._attn_implementation = name
    return model


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_rotary_attention_inside_tensor_parallel(dtype):
    from transformers import DynamicCache

    model = tiny_llama(dtype)
    plain = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    fused = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    assert tp.attention.fuse_rotary_(fused) == 2 * 2  # ranks x layers
    assert tp.attention.fuse_rotary_(fused) == 0      # once
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(2, 300, (2, 300), generator=g).to(DEV)  # more positions than the buffers' first capacity holds
    steps = [torch.randint(2, 300, (2, 1), generator=g).to(DEV) for _ in range(6)]
    caches = [DynamicCache(), DynamicCache()]
    with torch.no_grad():
        outs = [m(input_ids=ids, past_key_values=c, use_cache=True).logits.float() for m, c in zip((plain, fused), caches)]
        scale = outs[0].std().item()
        torch.testing.assert_close(outs[1], outs[0], rtol=RTOL, atol=RTOL * scale)
        for i, tok in enumerate(steps):
            if i == 3:  # beam search reorders the batch: the layer's tensors are new ones then, and are taken over again
                for c in caches:
                    c.reorder_cache(torch.tensor([1, 0], device=DEV))
            a, b = (m(input_ids=tok, past_key_values=c, use_cache=True).logits.float() for m, c in zip((plain, fused), caches))
            torch.testing.assert_close(b, a, rtol=RTOL, atol=RTOL * scale, msg=lambda m: f"decode step {i}: {m}")
    for cache in caches:
        assert cache.get_seq_length() == 306
    # rank 0 writes into the caller's cache object: first layer's keys (rotated by the kernel / by torch) and values.
    # The first layer sees the same inputs in both models, so its cache rows must be the same bits.
    k_plain, v_plain = caches[0].layers[0].keys, caches[0].layers[0].values
    k_fused, v_fused = caches[1].layers[0].keys, caches[1].layers[0].values
    assert k_fused.shape == k_plain.shape == (2, 1, 306, 64)  # this rank's one key/value head
    assert torch.equal(k_fused.view(torch.int16), k_plain.view(torch.int16))
    assert torch.equal(v_fused.view(torch.int16), v_plain.view(torch.int16))


def test_generate_with_fused_rotary_attention():
    model = tiny_llama(torch.float16)
    with torch.no_grad():
        for p in model.parameters():
            p.normal_(0.0, 0.05)
    plain = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    fused = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    tp.attention.fuse_rotary_(fused)
    ids = torch.randint(2, 300, (3, 7), generator=torch.Generator().manual_seed(3)).to(DEV)
    kwargs = dict(max_new_tokens=12, do_sample=False, attention_mask=torch.ones_like(ids), output_scores=True, return_dict_in_generate=True)
    with torch.no_grad():
        a = plain.generate(ids, **kwargs)
        b = fused.generate(ids, **kwargs)
    assert a.sequences.shape == b.sequences.shape == (3, 19)
    # greedy tokens can part ways where two logits are a rounding apart: compare the scores until they do
    for step, (sa, sb) in enumerate(zip(a.scores, b.scores)):
        same_so_far = torch.equal(a.sequences[:, :7 + step], b.sequences[:, :7 + step])
        if not same_so_far:
            break
        torch.testing.assert_close(sb.float(), sa.float(), rtol=RTOL, atol=3 * RTOL * sa.float().std().item())
    assert step >= 3


def test_modules_outside_the_pattern_keep_their_forward():
    from transformers import GPT2Config, GPT2LMHeadModel

    model = GPT2LMHeadModel(GPT2Config(n_embd=64, n_head=4, n_layer=1, n_positions=32, vocab_size=50))
    assert tp.attention.fuse_rotary_(model) == 0
    llama = tiny_llama(torch.float32)  # float32: the fused forward hands such calls to the module's own forward
    assert tp.attention.fuse_rotary_(llama) == 2
    llama = llama.to(DEV)
    llama.config._attn_implementation = "eager"
    ids = torch.randint(2, 300, (1, 9), generator=torch.Generator().manual_seed(4)).to(DEV)
    with torch.no_grad():
        out = llama(input_ids=ids, use_cache=True)
    assert out.logits.shape == (1, 9, 300) and out.past_key_values.get_seq_length() == 9


def test_fused_rotary_falcon_inside_tensor_parallel():
    """transformers' Falcon with rotary embeddings in the 40B layout (grouped heads in a fused query_key_value) on two
    ranks: its own forward (torch rotary embedding, cache update and attention on every query head's copy of the keys)
    against the fused one, which keeps each rank's key/value heads once."""
    from transformers import DynamicCache, FalconConfig, FalconForCausalLM

    torch.manual_seed(0)
    cfg = FalconConfig(vocab_size=300, hidden_size=512, num_hidden_layers=2, num_attention_heads=8, num_kv_heads=4,
                       new_decoder_architecture=True, multi_query=True, parallel_attn=True, alibi=False, bias=False,
                       max_position_embeddings=1024, bos_token_id=1, eos_token_id=None, pad_token_id=0)
    model = FalconForCausalLM(cfg).to(torch.bfloat16).eval()
    plain = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    fused = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    assert tp.attention.fuse_rotary_(fused) == 0  # Falcon only on the caller's word that there is no padding
    assert tp.attention.fuse_rotary_(fused, assume_no_padding=True) == 2 * 2
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(2, 300, (2, 70), generator=g).to(DEV)
    steps = [torch.randint(2, 300, (2, 1), generator=g).to(DEV) for _ in range(4)]
    caches = [DynamicCache(), DynamicCache()]
    with torch.no_grad():
        outs = [m(input_ids=ids, past_key_values=c, use_cache=True).logits.float() for m, c in zip((plain, fused), caches)]
        scale = outs[0].std().item()
        torch.testing.assert_close(outs[1], outs[0], rtol=RTOL, atol=RTOL * scale)
        for i, tok in enumerate(steps):
            a, b = (m(input_ids=tok, past_key_values=c, use_cache=True).logits.float() for m, c in zip((plain, fused), caches))
            torch.testing.assert_close(b, a, rtol=RTOL, atol=RTOL * scale, msg=lambda m: f"decode step {i}: {m}")
    assert caches[1].get_seq_length() == 74
    # the fused forward keeps this rank's key/value heads once (2 of the 4 groups), the module's own one copy per query head
    assert caches[1].layers[0].keys.shape == (2, 2, 74, 64) and caches[0].layers[0].keys.shape == (2, 4, 74, 64)
    # the same model on a static cache, the decode step replayed as one HIP graph
    from transformers import StaticCache

    static = StaticCache(config=cfg, max_cache_len=96)
    growing = DynamicCache()
    with torch.no_grad():
        want = plain(input_ids=ids, past_key_values=growing, use_cache=True).logits.float()
        got = fused(input_ids=ids, past_key_values=static, use_cache=True).logits.float()
        torch.testing.assert_close(got, want, rtol=RTOL, atol=RTOL * scale)
        step = tp.graphs.capture(fused, input_ids=steps[0], past_key_values=static, use_cache=True)
        for i, tok in enumerate(steps):
            got = step(input_ids=tok, past_key_values=static, use_cache=True).logits.float().clone()
            want = plain(input_ids=tok, past_key_values=growing, use_cache=True).logits.float()
            torch.testing.assert_close(got, want, rtol=RTOL, atol=RTOL * scale, msg=lambda m: f"replayed step {i}: {m}")
    assert int(static.get_seq_length()) == 74 and static.layers[0].keys.shape == (2, 2, 96, 64)
    # ... and through generate, which records the step by itself on a static cache (greedy tokens of a random model can
    # flip between two orders of summation, so the first tokens are compared, and the recorded run with the eager one)
    short = ids[:, :20]
    eager = fused.generate(short, max_new_tokens=6, do_sample=False, cache_implementation="static", disable_compile=True)
    got = fused.generate(short, max_new_tokens=6, do_sample=False, cache_implementation="static")
    assert "_tp_decode_graph" in fused.__dict__ and torch.equal(got, eager)
    assert torch.equal(got[:, :21], plain.generate(short, max_new_tokens=1, do_sample=False))


def test_static_cache_decode_eager_and_as_one_graph():
    """A transformers static cache behind the fused attention forward: the count of cached positions stays on the device
    (the decode kernels read it there), so one captured decode step is replayed for every new token. Against the same model
    with the module's own forward on a growing cache, step by step."""
    from transformers import DynamicCache, StaticCache

    model = tiny_llama(torch.bfloat16)
    plain = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    fused = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    assert tp.attention.fuse_rotary_(fused) == 2 * 2
    assert tp.attention.fuse_rotary_(fused, assume_no_padding=True) == 0  # nothing new to fuse, but the word about padding is taken
    g = torch.Generator().manual_seed(3)
    ids = torch.randint(2, 300, (2, 37), generator=g).to(DEV)
    steps = [torch.randint(2, 300, (2, 1), generator=g).to(DEV) for _ in range(40)]  # past a tile of 64 keys
    growing, static = DynamicCache(), StaticCache(config=model.config, max_cache_len=128)
    with torch.no_grad():
        want = plain(input_ids=ids, past_key_values=growing, use_cache=True).logits.float()
        got = fused(input_ids=ids, past_key_values=static, use_cache=True).logits.float()
        scale = want.std().item()
        torch.testing.assert_close(got, want, rtol=RTOL, atol=RTOL * scale)
        for tok in steps[:2]:  # eager decode steps
            want = plain(input_ids=tok, past_key_values=growing, use_cache=True).logits.float()
            got = fused(input_ids=tok, past_key_values=static, use_cache=True).logits.float()
            torch.testing.assert_close(got, want, rtol=RTOL, atol=RTOL * scale)
        assert int(static.get_seq_length()) == 39
        step = tp.graphs.capture(fused, input_ids=steps[2], past_key_values=static, use_cache=True)
        # the forwards that a capture runs first advanced every rank's counts; they are back where they were
        for cache in [static] + static.__dict__["_tp_rank_siblings"]:
            assert [int(layer.cumulative_length) for layer in cache.layers] == [39, 39]
        for i, tok in enumerate(steps[2:]):
            got = step(input_ids=tok, past_key_values=static, use_cache=True).logits.float().clone()
            torch.cuda.synchronize()
            want = plain(input_ids=tok, past_key_values=growing, use_cache=True).logits.float()  # eager work between the replays
            torch.testing.assert_close(got, want, rtol=RTOL, atol=RTOL * scale, msg=lambda m: f"replayed step {i}: {m}")
        assert int(static.get_seq_length()) == growing.get_seq_length() == 37 + 40
    # the first layer sees the same inputs in both models: its cached keys (rotated by the kernel / by torch) are the same bits
    k_static = static.layers[0].keys[:, :, :77]
    assert torch.equal(k_static.view(torch.int16), growing.layers[0].keys.view(torch.int16))


def test_generate_on_a_static_cache():
    """`generate(cache_implementation="static")`: transformers would hand the forward to torch.compile for such a cache. The
    wrapper records the decode step as one HIP graph instead, when every attention module reads the cache's count on the
    device, and declines otherwise; either way the tokens are those of the growing cache."""
    model = tiny_llama(torch.bfloat16)
    plain = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    fused = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    tp.attention.fuse_rotary_(fused, assume_no_padding=True)
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(2, 300, (2, 12), generator=g).to(DEV)
    want = plain.generate(ids, max_new_tokens=8, do_sample=False)
    eager = fused.generate(ids, max_new_tokens=8, do_sample=False, cache_implementation="static", disable_compile=True)
    assert torch.equal(eager, want) and "_tp_decode_graph" not in fused.__dict__
    got = fused.generate(ids, max_new_tokens=8, do_sample=False, cache_implementation="static")
    assert torch.equal(got, want)
    # transformers builds a new cache for every such call, and a step on another cache is recorded anew; a cache of the
    # caller's that is reset between calls keeps its recording
    from transformers import StaticCache

    cache = StaticCache(config=model.config, max_cache_len=32)
    assert torch.equal(fused.generate(ids, max_new_tokens=8, do_sample=False, past_key_values=cache), want)
    first = fused.__dict__["_tp_decode_graph"]
    cache.reset()
    other = torch.randint(2, 300, (2, 12), generator=g).to(DEV)
    assert torch.equal(fused.generate(other, max_new_tokens=8, do_sample=False, past_key_values=cache), plain.generate(other, max_new_tokens=8, do_sample=False))
    assert fused.__dict__["_tp_decode_graph"] is first
    # another batch size: a new cache, a new recording
    ids3 = torch.randint(2, 300, (3, 9), generator=g).to(DEV)
    want3 = plain.generate(ids3, max_new_tokens=6, do_sample=False)
    assert torch.equal(fused.generate(ids3, max_new_tokens=6, do_sample=False, cache_implementation="static"), want3)
    assert fused.__dict__["_tp_decode_graph"] is not first
    # a prefill in chunks goes through the same hook: its chunks run as they are, the decode steps are replayed
    long_ids = torch.randint(2, 300, (2, 24), generator=g).to(DEV)
    chunked = fused.generate(long_ids, max_new_tokens=6, do_sample=False, cache_implementation="static", prefill_chunk_size=8)
    assert torch.equal(chunked, plain.generate(long_ids, max_new_tokens=6, do_sample=False))
    # modules that were fused without the caller's word about padding take no static cache step as a graph
    halfway = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    tp.attention.fuse_rotary_(halfway)
    assert not halfway._decode_step_can_be_recorded() and not plain._decode_step_can_be_recorded()
    assert fused._decode_step_can_be_recorded()


def test_shared_qkv_storage_keeps_the_state_and_survives_a_replaced_projection():
    from transformers import DynamicCache

    model = tiny_llama(torch.bfloat16)
    separate = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    shared = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    before = {k: v.clone() for k, v in shared.state_dict().items()}
    assert tp.attention.fuse_rotary_(separate, share_qkv=False) == 4
    assert tp.attention.fuse_rotary_(shared) == 4
    attn = shared.wrapped_model.module_shards[1].model.layers[0].self_attn.tp_wrapped_module
    w, b = attn.__dict__["_tp_qkv"]
    assert b is None and w.shape == (2 * 64 + 64 + 64, 256)  # this rank's 2 query heads and 1 key/value head
    assert attn.k_proj.weight.data_ptr() == w.data_ptr() + 128 * 256 * 2
    after = shared.state_dict()
    assert after.keys() == before.keys() and all(torch.equal(after[k], before[k]) for k in before)  # un-sharded: the model's own weights
    g = torch.Generator().manual_seed(4)
    ids = torch.randint(2, 300, (2, 20), generator=g).to(DEV)
    tok = torch.randint(2, 300, (2, 1), generator=g).to(DEV)
    caches = [DynamicCache(), DynamicCache()]
    with torch.no_grad():
        for inp in (ids, tok, tok):
            a, b2 = (m(input_ids=inp, past_key_values=c, use_cache=True).logits.float() for m, c in zip((separate, shared), caches))
            torch.testing.assert_close(b2, a, rtol=RTOL, atol=RTOL * a.std().item())
        # a projection replaced afterwards: the module goes back to three calls
        assert tp.int8.quantize_linears_(shared, skip=lambda name, m: not name.endswith("layers.0.self_attn.tp_wrapped_module.k_proj")) == 2
        want = separate(input_ids=tok, past_key_values=caches[0], use_cache=True).logits.float()
        got = shared(input_ids=tok, past_key_values=caches[1], use_cache=True).logits.float()
        assert "_tp_qkv" not in attn.__dict__
        torch.testing.assert_close(got, want, rtol=5e-2, atol=5e-2 * want.std().item())  # one int8 projection in


def test_fusing_before_wrapping_then_sharing_the_projections_afterwards():
    """`fuse_rotary_` on the plain model (its Linears are still torch's, on the host), `tp.tensor_parallel`, then a second call:
    the rank shards' projections now live on the device and move into one matrix."""
    from transformers import DynamicCache

    model = tiny_llama(torch.bfloat16)
    reference = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    early = deepcopy(model)
    assert tp.attention.fuse_rotary_(early) == 2
    early = tp.tensor_parallel(early, [DEV, DEV])
    attn = early.wrapped_model.module_shards[0].model.layers[1].self_attn.tp_wrapped_module
    assert "_tp_qkv" not in attn.__dict__
    assert tp.attention.fuse_rotary_(early) == 0 and "_tp_qkv" in attn.__dict__
    ids = torch.randint(2, 300, (2, 16), generator=torch.Generator().manual_seed(6)).to(DEV)
    with torch.no_grad():
        want = reference(input_ids=ids, past_key_values=DynamicCache(), use_cache=True).logits.float()
        got = early(input_ids=ids, past_key_values=DynamicCache(), use_cache=True).logits.float()
    torch.testing.assert_close(got, want, rtol=RTOL, atol=RTOL * want.std().item())
