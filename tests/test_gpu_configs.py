"""BASELINE configurations 3 and 4 at their real shapes, through the drop-in API."""
import math
from types import SimpleNamespace

import pytest
import torch
import torch.nn.functional as F

import tensor_parallel_amd as tp
from conftest import to_bits
from oracle import slicing as osl
from tensor_parallel_amd import _native
from tensor_parallel_amd.config import get_parameter_name_mapping
from tensor_parallel_amd.slicing_configs import get_llama_config, get_refined_web_config

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def llama_7b_state():
    """A Llama-2-7B-shaped bf16 state dict generated on the device (291 tensors, 13.48 GB)."""
    g = torch.Generator(device=DEV).manual_seed(0)

    def t(*shape):
        return torch.empty(shape, device=DEV, dtype=torch.bfloat16).normal_(0, 0.02, generator=g)

    state = {"model.embed_tokens.weight": t(32000, 4096)}
    for i in range(32):
        p = f"model.layers.{i}."
        for n in ("q_proj", "k_proj", "v_proj", "o_proj"):
            state[p + f"self_attn.{n}.weight"] = t(4096, 4096)
        state[p + "mlp.gate_proj.weight"] = t(11008, 4096)
        state[p + "mlp.up_proj.weight"] = t(11008, 4096)
        state[p + "mlp.down_proj.weight"] = t(4096, 11008)
        state[p + "input_layernorm.weight"] = t(4096)
        state[p + "post_attention_layernorm.weight"] = t(4096)
    state["model.norm.weight"] = t(4096)
    state["lm_head.weight"] = t(32000, 4096)
    return state


@pytest.mark.parametrize("world", [2, 4, 8])
def test_convert_llama2_7b_state_dict(world):
    """Configuration 3: every shard of the whole dict in one launch. Checked on ALL tensors by size-independent
    properties (shapes, integer checksums adding up, split -> undo identity) and bit for bit against
    `torch.tensor_split` on the device (what the reference's Split computes, state_actions.py:47-48; with 32 heads
    and W in {2, 4, 8} the head-aligned splits of q/k/v/o are the same ranges), and bit for bit against the oracle on
    rows sampled from four tensors."""
    state = llama_7b_state()
    assert len(state) == 291
    cfg = get_llama_config(SimpleNamespace(model_type="llama", hidden_size=4096, num_attention_heads=32, num_key_value_heads=32), [DEV] * world)
    out = tp.convert_state_dict(state, cfg, world)
    assert len(out) == 291 * world + world
    names = get_parameter_name_mapping(state.keys(), cfg)

    def checksum(t):
        return int(t.view(torch.int16).to(torch.int64).sum())

    for name, full in state.items():
        shards = [out[f"module_shards.{r}.{names[name]}"] for r in range(world)]
        if full.dim() == 1:  # norms: replicated, same object for every rank
            assert all(s is full for s in shards)
            continue
        assert sum(s.numel() for s in shards) == full.numel()
        assert sum(checksum(s) for s in shards) == checksum(full), name
        action = next(a for p, a in cfg.state_rules.items() if p.search(name))
        for r, piece in enumerate(torch.tensor_split(full, world, dim=action.dim)):
            assert shards[r].is_contiguous() and torch.equal(shards[r], piece), (name, r)
        assert torch.equal(action.undo(shards), full), name
    for name in ("model.layers.0.self_attn.o_proj.weight", "model.layers.31.mlp.down_proj.weight", "model.embed_tokens.weight", "lm_head.weight"):
        full = state[name]
        action = next(a for p, a in cfg.state_rules.items() if p.search(name))
        shards = [out[f"module_shards.{r}.{names[name]}"] for r in range(world)]
        assert torch.equal(action.undo(shards), full), name
        rows = torch.tensor([0, 1, full.shape[0] // 2, full.shape[0] - 1], device=DEV)
        bits = to_bits(full[rows])
        for r in (0, world - 1):
            if getattr(action, "dim", 0) % 2 == 1:  # split on the inner axis: the sampled rows are split the same way
                want = osl.split(bits, world, 1, r) if not hasattr(action, "chunk_size") else osl.split_in_chunks(bits, world, 1, action.chunk_size, r)
                assert (to_bits(shards[r][rows]) == want).all(), (name, r)
    down = out[f"module_shards.{world - 1}.{names['model.layers.5.mlp.down_proj.weight']}"]
    assert down.shape == (4096, 11008 // world) and down.is_contiguous()


def test_falcon_40b_attention_block_shard():
    """Configuration 4: Falcon-40B-shape attention block, rank 0 of W=2. The fused query_key_value weight
    [9216, 8192] is split on whole KV groups of (16 + 2) * 64 rows, dense [8192, 8192] on the matching input
    columns; the two shard Linears are checked at decode (M = 8) and prefill (M = 1024) sizes, and the two ranks'
    dense partials recombine to the unsplit projection."""
    g = torch.Generator(device=DEV).manual_seed(0)
    d, heads, kv, hd = 8192, 128, 8, 64
    wqkv = torch.empty((kv * (heads // kv + 2) * hd, d), device=DEV, dtype=torch.bfloat16).normal_(0, 0.02, generator=g)
    wdense = torch.empty((d, d), device=DEV, dtype=torch.bfloat16).normal_(0, 0.02, generator=g)
    cfg = get_refined_web_config(SimpleNamespace(model_type="RefinedWeb", hidden_size=d, n_head=heads, n_head_kv=kv, num_attention_heads=heads,
                                                 bias=False, alibi=False), [DEV, DEV])
    state = {"transformer.h.0.self_attention.query_key_value.weight": wqkv, "transformer.h.0.self_attention.dense.weight": wdense}
    out = tp.convert_state_dict(state, cfg, 2)
    pre = "transformer.h.0.self_attention.tp_wrapped_module."
    qkv = [out[f"module_shards.{r}.{pre}query_key_value.weight"] for r in range(2)]
    dense = [out[f"module_shards.{r}.{pre}dense.weight"] for r in range(2)]
    assert qkv[0].shape == (4608, 8192) and dense[0].shape == (8192, 4096)
    # rank 0 owns KV groups 0..3: rows [0, 4608); within a group 16 query heads, then the key head, then the value head
    assert torch.equal(qkv[0], wqkv[:4608]) and torch.equal(qkv[1], wqkv[4608:])
    assert torch.equal(dense[0], wdense[:, :4096]) and torch.equal(dense[1], wdense[:, 4096:])
    attn = cfg.attr_rules[next(iter(cfg.attr_rules))]
    assert attn["num_kv"](kv, rank=0) == 4 and attn["num_heads"](heads, rank=0) == 64

    for M in (8, 1024):
        x = torch.randn(M, d, generator=g, device=DEV).to(torch.bfloat16)
        y = _native.linear(x, qkv[0])
        want = F.linear(x.float().cpu(), qkv[0].float().cpu())
        torch.testing.assert_close(y.float().cpu(), want, rtol=2e-2, atol=2e-2 * 0.02 * math.sqrt(d))
        # the attention core sits between the two Linears; feed the dense shards a stand-in of the right shape
        ctx = torch.randn(M, d, generator=g, device=DEV).to(torch.bfloat16)
        parts = [_native.linear(torch.tensor_split(ctx, 2, dim=1)[r], dense[r]) for r in range(2)]
        full = F.linear(ctx.float().cpu(), wdense.float().cpu())
        torch.testing.assert_close(_native.reduce_partials(parts).float().cpu(), full, rtol=2e-2, atol=2e-2 * 0.02 * math.sqrt(d))
