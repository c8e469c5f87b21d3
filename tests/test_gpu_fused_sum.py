"""The "sum" output rule folded into the row-parallel Linear that feeds it: through tp.TensorParallel the last-arriving
rank's Linear adds the waiting partial in its epilogue (tpamd_linear_add) and no reduction kernel runs; the result is
the reduction kernel's, bit for bit."""
from copy import deepcopy
from types import SimpleNamespace

import pytest
import torch
from torch import nn

import tensor_parallel_amd as tp
from tensor_parallel_amd import _native, collectives
from tensor_parallel_amd.slicing_configs import get_llama_config

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


class LlamaMLP(nn.Module):
    def __init__(self, d, f):
        super().__init__()
        self.gate_proj, self.up_proj, self.down_proj = nn.Linear(d, f, bias=False), nn.Linear(d, f, bias=False), nn.Linear(f, d, bias=False)
        self.act_fn = nn.SiLU()

    def forward(self, x):
        return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))


class Block(nn.Module):
    def __init__(self, d, f, mlp=LlamaMLP):
        super().__init__()
        self.mlp = mlp(d, f)

    def forward(self, x):
        return self.mlp(x)


class Counter:
    """Counts the library calls of a forward by wrapping the binding's functions."""

    def __init__(self, monkeypatch):
        self.fused = self.plain = self.reductions = 0
        linear, reduce_partials = _native.linear, _native.reduce_partials

        def counted_linear(*args, **kwargs):
            if kwargs.get("addend") is not None:
                self.fused += 1
            else:
                self.plain += 1
            return linear(*args, **kwargs)

        def counted_reduce(*args, **kwargs):
            self.reductions += 1
            return reduce_partials(*args, **kwargs)

        monkeypatch.setattr(_native, "linear", counted_linear)
        monkeypatch.setattr(_native, "reduce_partials", counted_reduce)

    def reset(self):
        self.fused = self.plain = self.reductions = 0


def build(world, dtype=torch.bfloat16, mlp=LlamaMLP, d=256, f=768):
    torch.manual_seed(0)
    block = Block(d, f, mlp)
    for p in block.parameters():
        nn.init.normal_(p, std=0.05)
    block = block.to(dtype)
    cfg = get_llama_config(SimpleNamespace(model_type="llama", hidden_size=d, num_attention_heads=4, num_key_value_heads=4), [DEV] * world)
    return block, tp.TensorParallel(deepcopy(block), [DEV] * world, tensor_parallel_config=cfg, sharded=False)


@pytest.mark.parametrize("tokens", [5, 300])
def test_two_ranks_fold_the_sum_into_the_down_projection(monkeypatch, tokens):
    block, model_tp = build(2)
    x = torch.randn(2, tokens, 256).to(torch.bfloat16).to(DEV)
    monkeypatch.setattr(collectives, "FUSE_SUM", False)
    with torch.no_grad():
        want = model_tp(x)  # the sum in its own kernel; also settles the fused gate/up forward of the blocks
        want2 = model_tp(x)
    assert torch.equal(want, want2)
    monkeypatch.setattr(collectives, "FUSE_SUM", True)
    count = Counter(monkeypatch)
    with torch.no_grad():
        first = model_tp(x)   # the op sees which Linear produced the value it is handed
        assert count.fused == 0 and count.reductions == 1
        count.reset()
        outs = [model_tp(x) for _ in range(3)]
    # per forward: rank A's down projection plain, rank B's with the addend, no reduction launch
    assert count.fused == 3 and count.plain == 3 and count.reductions == 0
    for out in [first] + outs:
        assert torch.equal(out, want)
    ref = block.float()(x.float().cpu())
    torch.testing.assert_close(outs[0].float().cpu(), ref, rtol=2e-2, atol=2e-2 * ref.std().item())


@pytest.mark.parametrize("world", [3, 4])
def test_more_ranks_keep_the_rank_ordered_sum(monkeypatch, world):
    """Whatever order the rank threads arrive in, the value equals the rank-ordered stepwise sum of the reduction kernel:
    a Linear only adds a running sum that starts at rank 0 and ends just below its own rank."""
    _, model_tp = build(world)
    x = torch.randn(1, 40, 256).to(torch.bfloat16).to(DEV)
    monkeypatch.setattr(collectives, "FUSE_SUM", False)
    with torch.no_grad():
        model_tp(x)
        want = model_tp(x)
    monkeypatch.setattr(collectives, "FUSE_SUM", True)
    count = Counter(monkeypatch)
    with torch.no_grad():
        outs = [model_tp(x) for _ in range(6)]
    for out in outs:
        assert torch.equal(out, want)
    assert count.fused + count.plain == 6 * world


def test_a_module_that_touches_the_linear_output_keeps_the_separate_sum(monkeypatch):
    class Doubling(LlamaMLP):
        def forward(self, x):
            return super().forward(x) * 2

    block, model_tp = build(2, mlp=Doubling)
    x = torch.randn(3, 7, 256).to(torch.bfloat16).to(DEV)
    count = Counter(monkeypatch)
    with torch.no_grad():
        outs = [model_tp(x) for _ in range(4)]
    assert count.fused == 0 and count.reductions == 4
    ref = block.float()(x.float().cpu())
    for out in outs:
        torch.testing.assert_close(out.float().cpu(), ref, rtol=2e-2, atol=2e-2 * ref.std().item())


def test_fp32_linear_with_bias_under_a_sum_rule(monkeypatch):
    """A row-parallel fp32 Linear with a bias (divided by the world size on every rank) whose own output is summed."""
    torch.manual_seed(0)
    model = nn.Sequential(nn.Linear(48, 96), nn.ReLU(), nn.Linear(96, 24))
    world = 2
    cfg = tp.Config(
        state_rules={r"^0\.weight$": tp.Split(world, 0), r"^0\.bias$": tp.Split(world, 0), r"^2\.weight$": tp.Split(world, 1),
                     r"^2\.bias$": tp.Scale(world)},
        input_rules={}, output_rules={r"^2$": {0: "sum"}}, attr_rules={})
    model_tp = tp.TensorParallel(deepcopy(model), [DEV] * world, tensor_parallel_config=cfg, sharded=False)
    x = torch.randn(9, 48)
    monkeypatch.setattr(collectives, "FUSE_SUM", False)
    with torch.no_grad():
        want = model_tp(x.to(DEV))
    monkeypatch.setattr(collectives, "FUSE_SUM", True)
    count = Counter(monkeypatch)
    with torch.no_grad():
        outs = [model_tp(x.to(DEV)) for _ in range(3)]
    assert count.fused == 2 and count.reductions == 1
    for out in outs:
        assert torch.equal(out, want)
    torch.testing.assert_close(outs[-1].cpu(), model(x), rtol=1e-5, atol=1e-5)


def test_two_summed_outputs_of_one_module_share_the_op(monkeypatch):
    """A module that returns two row-parallel products, both under a "sum" rule (one op object serves both): the Linear
    behind output 0 folds its sum, output 1 goes through the reduction kernel, and neither is taken for the other."""
    class Pair(nn.Module):
        def __init__(self, d):
            super().__init__()
            self.a, self.b = nn.Linear(d, d, bias=False), nn.Linear(d, 2 * d, bias=False)

        def forward(self, x):
            second = self.a(x)
            first = self.b(x)
            return first, second

    torch.manual_seed(0)
    d, world = 128, 2
    model = nn.Sequential(Pair(d)).to(torch.bfloat16)
    cfg = tp.Config(state_rules={r"^0\.a\.weight$": tp.Split(world, 1), r"^0\.b\.weight$": tp.Split(world, 1)},
                    input_rules={r"^0$": {0: "split -1"}}, output_rules={r"^0$": {0: "sum", 1: "sum"}}, attr_rules={})
    model_tp = tp.TensorParallel(deepcopy(model), [DEV] * world, tensor_parallel_config=cfg, sharded=False)
    x = torch.randn(33, d).to(torch.bfloat16).to(DEV)
    monkeypatch.setattr(collectives, "FUSE_SUM", False)
    with torch.no_grad():
        want = model_tp(x)
    monkeypatch.setattr(collectives, "FUSE_SUM", True)
    count = Counter(monkeypatch)
    with torch.no_grad():
        outs = [model_tp(x) for _ in range(3)]
    # first forward: two reductions; then output 0 is folded into b's epilogue and only output 1 is reduced
    assert count.reductions == 2 + 1 + 1 and count.fused == 2
    for out in outs:
        assert torch.equal(out[0], want[0]) and torch.equal(out[1], want[1])
    ref = model.float()(x.float().cpu())
    for got, r in zip(outs[-1], ref):
        torch.testing.assert_close(got.float().cpu(), r, rtol=2e-2, atol=2e-2 * r.std().item())
