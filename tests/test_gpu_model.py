"""Whole-module parity through the drop-in API: rank shards on one GPU recombine to the unsplit module."""
from copy import deepcopy
from types import SimpleNamespace

import pytest
import torch
from torch import nn

import tensor_parallel_amd as tp
from tensor_parallel_amd.shard_modules import ShardLinear
from tensor_parallel_amd.slicing_configs import get_llama_config

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def toy():
    return nn.Sequential(nn.Embedding(1337, 64), nn.LayerNorm(64), nn.Linear(64, 128), nn.ReLU(), nn.Linear(128, 12))


@pytest.mark.parametrize("world", [1, 2, 3, 4])
def test_embeds_and_linear_forward_parity(world):
    # forward half of tests/test_basic.py:32-56 of the reference, fp32, atol 1e-6 / rtol 1e-5
    torch.manual_seed(0)
    model = toy()
    inputs = torch.randint(1, 1000, size=(1, 10))
    with torch.no_grad():
        ref = model(inputs)
    model_tp = tp.TensorParallel(deepcopy(model), [DEV] * world, sharded=False)
    with torch.no_grad():
        out = model_tp(inputs.to(DEV))
    torch.testing.assert_close(out.cpu(), ref, atol=1e-6, rtol=1e-5)
    if world > 1:
        assert all(isinstance(m, ShardLinear) for m in model_tp.modules() if isinstance(m, nn.Linear))
        for m in model_tp.modules():
            if isinstance(m, nn.Linear):
                assert m.weight.shape == (m.out_features, m.in_features)
        # un-shard: original names and bit-identical tensors (tests/test_saving.py:43-62 of the reference)
        with tp.save_tensor_parallel(model_tp):
            sd = model_tp.state_dict()
        assert set(sd) == set(model.state_dict())
        for k, v in model.state_dict().items():
            assert torch.equal(sd[k].cpu(), v), k


def test_forward_runs_on_the_callers_stream():
    """The rank threads enqueue on the stream the caller is on: an input produced on a side stream just before the forward
    (behind a long chain of kernels) is complete when the shards read it, and the result is ready for what the caller
    enqueues next on that stream."""
    torch.manual_seed(0)
    model = nn.Sequential(nn.Linear(512, 1024), nn.ReLU(), nn.Linear(1024, 256)).to(torch.bfloat16)
    model_tp = tp.TensorParallel(deepcopy(model), [DEV] * 2, sharded=False)
    a = torch.randn(2048, 2048, device=DEV, dtype=torch.bfloat16) * 0.02
    seed = torch.randn(2048, 512, device=DEV, dtype=torch.bfloat16)
    with torch.no_grad():
        want_x = seed
        for _ in range(30):
            want_x = (a @ want_x.repeat(1, 4))[:, :512] * 0.5
        want = model_tp(want_x).clone()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            x = seed
            for _ in range(30):  # tens of microseconds each: still running when the forward is enqueued
                x = (a @ x.repeat(1, 4))[:, :512] * 0.5
            out = model_tp(x)
            doubled = out * 2
        side.synchronize()
    assert torch.equal(out, want)
    assert torch.equal(doubled, want * 2)


def test_backward_is_refused():
    model_tp = tp.TensorParallel(toy(), [DEV] * 2, sharded=False)
    out = model_tp(torch.randint(1, 1000, size=(1, 10), device=DEV))
    with pytest.raises(NotImplementedError):
        out.norm().backward()


def test_worker_failure_is_raised_not_hung():
    class Boom(nn.Module):
        def forward(self, x):
            raise RuntimeError("shard failed")

    model = nn.Sequential(nn.Linear(8, 8), Boom())
    model_tp = tp.TensorParallel(model, [DEV] * 2, sharded=False)
    with pytest.raises(RuntimeError, match="shard failed"):
        model_tp(torch.randn(2, 8, device=DEV))
    with pytest.raises(ValueError):
        model_tp.to("cpu")(torch.randn(2, 8))


def test_one_failing_rank_frees_its_peers_and_the_next_forward_works():
    """Only one rank fails, between two collectives, while its peer may already wait in the next one: the forward raises
    the rank's error (not a timeout), and the collective ops are usable again afterwards."""
    class Flaky(nn.Module):
        calls, armed = 0, False

        def forward(self, x):
            Flaky.calls += 1
            if Flaky.armed and Flaky.calls % 2 == 0:
                raise RuntimeError("one rank failed")
            return x

    torch.manual_seed(0)
    model = nn.Sequential(nn.Linear(16, 32), Flaky(), nn.Linear(32, 8))
    model_tp = tp.TensorParallel(deepcopy(model), [DEV] * 2, sharded=False)
    x = torch.randn(5, 16)
    with torch.no_grad():
        want = model(x)
        torch.testing.assert_close(model_tp(x.to(DEV)).cpu(), want, rtol=1e-5, atol=1e-5)
        Flaky.armed = True
        with pytest.raises(RuntimeError, match="one rank failed"):
            model_tp(x.to(DEV))
        Flaky.armed = False
        for _ in range(2):
            torch.testing.assert_close(model_tp(x.to(DEV)).cpu(), want, rtol=1e-5, atol=1e-5)


class LlamaMLP(nn.Module):
    def __init__(self, d, f):
        super().__init__()
        self.gate_proj, self.up_proj, self.down_proj = nn.Linear(d, f, bias=False), nn.Linear(d, f, bias=False), nn.Linear(f, d, bias=False)
        self.act_fn = nn.SiLU()

    def forward(self, x):
        return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))


class Block(nn.Module):
    def __init__(self, d, f):
        super().__init__()
        self.mlp = LlamaMLP(d, f)

    def forward(self, x):
        return self.mlp(x)


@pytest.mark.parametrize("world", [2, 4])
@pytest.mark.parametrize("tokens", [3, 200])
def test_llama_mlp_block_with_llama_rules(world, tokens):
    torch.manual_seed(0)
    d, f = 256, 688
    block = Block(d, f)
    for p in block.parameters():
        nn.init.normal_(p, std=0.05)
    block = block.to(torch.bfloat16)
    x = torch.randn(2, tokens, d).to(torch.bfloat16)
    with torch.no_grad():
        ref = block.float()(x.float())
    block = block.to(torch.bfloat16)
    cfg = get_llama_config(SimpleNamespace(model_type="llama", hidden_size=d, num_attention_heads=4, num_key_value_heads=4), [DEV] * world)
    model_tp = tp.TensorParallel(block, [DEV] * world, tensor_parallel_config=cfg, sharded=False)
    shard_mlp = model_tp.module_shards[0].mlp.tp_wrapped_module
    assert shard_mlp.gate_proj.weight.shape == (f // world, d) and shard_mlp.down_proj.weight.shape == (d, f // world)
    with torch.no_grad():
        out = model_tp(x.to(DEV))
    torch.testing.assert_close(out.float().cpu(), ref, rtol=2e-2, atol=2e-2 * ref.std().item())


@pytest.mark.parametrize("tokens", [6, 7])
def test_llama_mlp_block_at_decode_batch_sizes_of_real_width(tokens):
    """A Llama-7B-wide MLP (d = 4096, ffn 11008) at W = 2 with 12 and 14 tokens per forward: the sizes at which the
    library serves the shards' gate/up pair and down projection with its x-resident weight-streaming kernel by
    default. The two shards' partial sums recombine to the unsplit module."""
    torch.manual_seed(0)
    d, f, world = 4096, 11008, 2
    block = Block(d, f).to(torch.bfloat16)
    for p in block.parameters():
        nn.init.normal_(p, std=0.02)
    x = torch.randn(2, tokens, d).to(torch.bfloat16)
    cfg = get_llama_config(SimpleNamespace(model_type="llama", hidden_size=d, num_attention_heads=32, num_key_value_heads=32), [DEV] * world)
    model_tp = tp.TensorParallel(deepcopy(block), [DEV] * world, tensor_parallel_config=cfg, sharded=False)
    with torch.no_grad():
        ref = block.to(DEV).float()(x.to(DEV).float())
        out = model_tp(x.to(DEV))
    torch.testing.assert_close(out.float(), ref, rtol=2e-2, atol=2e-2 * ref.std().item())


def test_opt_125m_tensor_parallel_logits():
    """BASELINE config 1: OPT-125m architecture, fp32, N(0, 0.02) weights from seed 0, W = 2 through
    tp.tensor_parallel, batch 2 x seq 64; final logits against the unsplit model."""
    from transformers import OPTConfig, OPTForCausalLM

    torch.manual_seed(0)
    model = OPTForCausalLM(OPTConfig()).eval()
    with torch.no_grad():
        for p in model.parameters():
            p.normal_(0.0, 0.02)
    ids = torch.randint(0, 50272, (2, 64), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        ref = model(input_ids=ids, use_cache=False).logits
    model_tp = tp.tensor_parallel(deepcopy(model), [DEV, DEV])
    assert isinstance(model_tp, tp.TensorParallelPreTrainedModel)
    shard0 = model_tp.wrapped_model.module_shards[0]
    assert shard0.model.decoder.layers[0].fc1.tp_wrapped_module.weight.shape == (1536, 768)
    assert shard0.model.decoder.embed_tokens.tp_wrapped_module.weight.shape == (50272, 384)
    for r, shard in enumerate(model_tp.wrapped_model.module_shards):  # rank shards are the oracle's slices
        w = shard.model.decoder.layers[3].fc2.tp_wrapped_module.weight
        assert torch.equal(w.cpu(), torch.tensor_split(model.model.decoder.layers[3].fc2.weight, 2, dim=0)[r])
    with torch.no_grad():
        out = model_tp(input_ids=ids.to(DEV), use_cache=False).logits
    assert out.shape == (2, 64, 50272)
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-5, atol=3e-3)
    assert (out.cpu() - ref).abs().max().item() < 1e-3


def test_delay_init_parks_shards_on_the_host_until_the_first_forward():
    """`delay_init=True` (reference tensor_parallel.py:33,80-81,140-143): after construction the shards hold no device
    memory, the first forward moves every rank's shard to its device, and the result equals the eager build's."""
    torch.manual_seed(0)
    model = torch.nn.Sequential(torch.nn.Embedding(50, 32), torch.nn.Linear(32, 64), torch.nn.ReLU(), torch.nn.Linear(64, 24))
    ids = torch.randint(0, 50, (3, 7))
    devices = ["cuda:0", "cuda:0"]
    eager = tp.TensorParallel(model, devices, sharded=False)
    lazy = tp.TensorParallel(model, devices, sharded=False, delay_init=True)
    assert lazy.need_delayed_init
    assert all(p.device.type == "cpu" for shard in lazy.module_shards for p in shard.parameters())
    for a, b in zip(eager.module_shards.parameters(), lazy.module_shards.parameters()):
        assert torch.equal(a.cpu(), b)
    out = lazy(ids.to("cuda:0"))
    assert not lazy.need_delayed_init
    assert all(p.device == torch.device("cuda", 0) for shard in lazy.module_shards for p in shard.parameters())
    assert torch.equal(out, eager(ids.to("cuda:0")))
    torch.testing.assert_close(out.cpu(), model(ids), rtol=1e-5, atol=1e-5)


def test_gated_mlp_fusion_is_checked_at_the_first_forward_and_respects_hooks():
    """The fused gate/up forward takes over only where it reproduces the block's own forward: a block that looks the
    same but computes something else, and a block whose gate_proj carries a hook, keep their own forward."""
    from tensor_parallel_amd.shard_modules import _gated_mlp_forward, install_shard_kernels

    class Odd(LlamaMLP):  # same children, another formula
        def forward(self, x):
            return self.down_proj(self.act_fn(self.up_proj(x)) * self.gate_proj(x))

    torch.manual_seed(0)
    x = torch.randn(5, 64).to(torch.bfloat16).to(DEV)
    plain, odd, hooked = LlamaMLP(64, 96), Odd(64, 96), LlamaMLP(64, 96)
    seen = []
    hooked.gate_proj.register_forward_hook(lambda m, i, o: seen.append(1))
    holder = nn.ModuleList([plain, odd, hooked]).to(torch.bfloat16).to(DEV)
    want = [m(x) for m in holder]
    install_shard_kernels(holder)
    for m in holder:
        assert type(m.gate_proj) is ShardLinear
    with torch.no_grad():
        got = [m(x) for m in holder] + [m(x) for m in holder]  # the second pass runs what the first pass settled on
    for i in range(6):
        torch.testing.assert_close(got[i].float(), want[i % 3].float(), rtol=2e-2, atol=2e-2 * want[i % 3].float().std().item())
    assert getattr(plain.forward, "__func__", None) is _gated_mlp_forward
    assert "forward" not in odd.__dict__ and "forward" not in hooked.__dict__
    assert len(seen) == 3  # the reference call and both passes went through gate_proj's hook
