"""`tp.graphs.capture`: one forward of a `tp.tensor_parallel` model (two rank shards on one GPU, their "sum" and "gather"
ops included) recorded as a HIP graph. Every replay is checked against the eager forward on the same inputs, with eager
work and synchronisations between the replays."""
import importlib
from copy import deepcopy

import pytest
import torch
from torch import nn

import tensor_parallel_amd as tp

pytestmark = pytest.mark.gpu
tp_module = importlib.import_module("tensor_parallel_amd.tensor_parallel")
DEV = torch.device("cuda", 0)


def tiny_opt():
    from transformers import OPTConfig, OPTForCausalLM

    torch.manual_seed(0)
    cfg = OPTConfig(vocab_size=512, hidden_size=128, ffn_dim=256, num_hidden_layers=2, num_attention_heads=4,
                    max_position_embeddings=128, word_embed_proj_dim=128)
    return OPTForCausalLM(cfg).eval()


def test_opt_fp32_forward_replays_match_eager():
    model = tp.tensor_parallel(tiny_opt(), [DEV, DEV])
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(0, 512, (2, 48), generator=g).to(DEV)
    graphed = tp.graphs.capture(model, input_ids=ids, use_cache=False)
    for trial in range(4):
        new = torch.randint(0, 512, (2, 48), generator=g).to(DEV)
        got = graphed(input_ids=new, use_cache=False).logits.clone()
        torch.cuda.synchronize()
        with torch.no_grad():
            want = model(input_ids=new, use_cache=False).logits  # eager work between the replays
        # fp32 tolerance of the path; the eager and the captured forward may take different torch attention kernels
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5, msg=lambda m: f"replay {trial}: {m}")
    # the value returned is the graph's own buffer: a replay on other inputs overwrites it
    first = graphed(input_ids=ids, use_cache=False).logits
    kept = first.clone()
    second = graphed(input_ids=new, use_cache=False).logits
    assert second.data_ptr() == first.data_ptr()
    assert not torch.equal(kept, second)


def test_llama_bf16_forward_replays_match_eager():
    from transformers import LlamaConfig, LlamaForCausalLM

    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=300, hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, max_position_embeddings=256)
    model = tp.tensor_parallel(LlamaForCausalLM(cfg).to(torch.bfloat16).eval(), [DEV, DEV])
    g = torch.Generator().manual_seed(2)
    ids = torch.randint(0, 300, (3, 40), generator=g).to(DEV)
    graphed = tp.graphs.capture(model, input_ids=ids, use_cache=False)
    for trial in range(3):
        new = torch.randint(0, 300, (3, 40), generator=g).to(DEV)
        got = graphed(input_ids=new, use_cache=False).logits.float().clone()
        with torch.no_grad():
            want = model(input_ids=new, use_cache=False).logits.float()
        # transformers hands torch's attention an explicit mask while a stream is being captured and none otherwise: two
        # different torch kernels, each with its own bf16 rounding, so the floor is twice the usual one
        torch.testing.assert_close(got, want, rtol=2e-2, atol=4e-2 * want.std().item(), msg=lambda m: f"replay {trial}: {m}")


def test_plain_module_positional_arguments_and_in_place_inputs():
    torch.manual_seed(0)
    block = nn.Sequential(nn.Linear(256, 512), nn.GELU(), nn.Linear(512, 256)).to(torch.bfloat16)
    model = tp.tensor_parallel(deepcopy(block), [DEV, DEV])
    x = torch.randn(24, 256, device=DEV).to(torch.bfloat16)
    graphed = tp.graphs.capture(model, x)
    y = torch.randn(24, 256, device=DEV).to(torch.bfloat16)
    with torch.no_grad():
        want = model(y)
    assert torch.equal(graphed(y), want)  # the same kernels on the same inputs
    (static_x,), _ = graphed.static_inputs
    static_x.copy_(x)
    with torch.no_grad():
        assert torch.equal(graphed.replay(), model(x))


def test_what_a_capture_fixes_is_checked():
    model = tp.tensor_parallel(tiny_opt(), [DEV, DEV])
    ids = torch.zeros(2, 16, dtype=torch.int64, device=DEV)
    graphed = tp.graphs.capture(model, input_ids=ids, use_cache=False)
    with pytest.raises(ValueError, match="captured as"):
        graphed(input_ids=ids[:, :8], use_cache=False)
    with pytest.raises(ValueError, match="cannot change"):
        graphed(input_ids=ids, use_cache=True)
    with pytest.raises(ValueError, match="structure"):
        graphed(input_ids=ids)
    with pytest.raises(ValueError, match="one HIP device"):
        tp.graphs.capture(model, input_ids=ids.cpu(), use_cache=False)


def test_ranks_that_run_as_threads_are_refused(monkeypatch):
    model = tp.tensor_parallel(tiny_opt(), [DEV, DEV])
    ids = torch.zeros(2, 16, dtype=torch.int64, device=DEV)
    monkeypatch.setattr(tp_module, "RANK_GREENLETS", False)
    with pytest.raises(RuntimeError, match="greenlets"):
        tp.graphs.capture(model, input_ids=ids, use_cache=False)


def test_int8_shard_linears_inside_a_captured_decode_step():
    """Rank shards with int8 weight-only Linears (their K-split kernels keep partial sums in the stream's scratch buffer) on
    a static cache: the captured decode step against the same model run eagerly, token by token."""
    from copy import deepcopy as dc

    from transformers import LlamaConfig, LlamaForCausalLM, StaticCache

    name = tp.attention.register()
    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=300, hidden_size=1024, intermediate_size=2048, num_hidden_layers=2, num_attention_heads=8,
                      num_key_value_heads=4, max_position_embeddings=256, attn_implementation="eager")
    model = LlamaForCausalLM(cfg).to(torch.bfloat16).eval()
    model.config._attn_implementation = name
    models = []
    for _ in range(2):
        m = tp.tensor_parallel(dc(model), [DEV, DEV])
        tp.attention.fuse_rotary_(m, assume_no_padding=True)
        assert tp.int8.quantize_linears_(m, skip=lambda n, mod: "lm_head" in n) == 2 * 2 * 7
        models.append(m)
    eager, graphed_model = models
    g = torch.Generator().manual_seed(5)
    prompt = torch.randint(2, 300, (4, 9), generator=g).to(DEV)
    toks = [torch.randint(2, 300, (4, 1), generator=g).to(DEV) for _ in range(6)]
    caches = [StaticCache(config=cfg, max_cache_len=64), StaticCache(config=cfg, max_cache_len=64)]
    with torch.no_grad():
        for m, c in zip(models, caches):
            m(input_ids=prompt, past_key_values=c, use_cache=True)
        step = tp.graphs.capture(graphed_model, input_ids=toks[0], past_key_values=caches[1], use_cache=True)
        for i, tok in enumerate(toks):
            want = eager(input_ids=tok, past_key_values=caches[0], use_cache=True).logits.float()
            got = step(input_ids=tok, past_key_values=caches[1], use_cache=True).logits.float()
            # the same kernels on the same inputs; only torch's attention-mask handling differs under capture, and the
            # fused attention ignores the mask
            torch.testing.assert_close(got, want, rtol=2e-2, atol=2e-2 * want.std().item(), msg=lambda m: f"step {i}: {m}")
