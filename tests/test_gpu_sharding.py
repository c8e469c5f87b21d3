"""ZeRO-3 side-car on the device: flat shards and their recombination against the oracle (bit-exact), the reference's
own assertions about it (tests/test_basic.py:33-57, 110-135; tests/test_saving.py:19-88; tests/test_legacy.py), and
what a changed flat shard does to the next forward."""
from copy import deepcopy

import numpy as np
import pytest
import torch
from torch import nn

import tensor_parallel_amd as tp
from oracle import sharding as osh

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def toy(emb_cls=nn.Embedding):
    torch.manual_seed(0)
    return nn.Sequential(emb_cls(num_embeddings=1337, embedding_dim=64), nn.LayerNorm(64), nn.Linear(64, 128), nn.ReLU(), nn.Linear(128, 10))


@pytest.mark.parametrize("world", [1, 2, 3])
def test_sharded_num_params(world):
    model = toy()
    original = sum(p.numel() for p in model.parameters())
    model_tp = tp.TensorParallel(deepcopy(model), [DEV] * world, sharded=False)
    before = sum(p.numel() for p in model_tp.parameters())
    model_tp.apply_sharding()
    after = sum(p.numel() for p in model_tp.parameters())
    assert after < before or world == 1
    assert after == original + (0 if world < 3 else 4)


@pytest.mark.parametrize("world", [2, 3, 4])
def test_flat_shards_and_recombination_match_the_oracle(world):
    model = toy()
    with torch.no_grad():
        model[1].weight.copy_(torch.randn(64))
        model[1].bias.copy_(torch.randn(64))
    model_tp = tp.TensorParallel(deepcopy(model), [DEV] * world, sharded=True)
    manager = model_tp.sharding_manager
    assert manager.sharded_param_names == ("1.weight", "1.bias")
    params = [model[1].weight.detach().numpy(), model[1].bias.detach().numpy()]
    flat, sizes = osh.make_flat_shards([params] * world, world)
    assert manager._shard_sizes_with_pad == sizes
    for mine, want in zip(manager.flat_shards, flat):
        assert np.array_equal(mine.detach().cpu().numpy().view(np.uint32), want.view(np.uint32))
    for shard in model_tp.module_shards:  # the originals are gone until the first synchronisation
        assert shard[1].weight is None and "weight" not in shard[1]._parameters
    manager.synchronize_weights(True)
    want = osh.combine_shards(flat, sizes, [(64,), (64,)])
    for shard in model_tp.module_shards:
        assert np.array_equal(shard[1].weight.cpu().numpy(), want[0]) and np.array_equal(shard[1].bias.cpu().numpy(), want[1])
        assert shard[1].weight.data_ptr() % 256 == 0 and shard[1].bias.data_ptr() % 256 == 0
    # one recombined copy serves every rank
    assert len({shard[1].weight.data_ptr() for shard in model_tp.module_shards}) == 1


@pytest.mark.parametrize("world", [2, 3])
def test_forward_with_sharding_equals_forward_without(world):
    model = toy()
    ids = torch.randint(1, 1000, size=(4, 10), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        ref = model(ids)
        plain = tp.TensorParallel(deepcopy(model), [DEV] * world, sharded=False)(ids.to(DEV))
        sharded_tp = tp.TensorParallel(deepcopy(model), [DEV] * world, sharded=True)
        out = sharded_tp(ids.to(DEV))
        again = sharded_tp(ids.to(DEV))
    assert torch.equal(out, plain) and torch.equal(again, out)
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-5, atol=1e-5)


def test_a_written_flat_shard_reaches_the_next_forward():
    model = toy()
    ids = torch.randint(1, 1000, size=(2, 6), generator=torch.Generator().manual_seed(1))
    model_tp = tp.TensorParallel(deepcopy(model), [DEV] * 2, sharded=True)
    with torch.no_grad():
        first = model_tp(ids.to(DEV))
        saved = deepcopy(model_tp.state_dict())
        for flat in model_tp.sharding_manager.flat_shards:
            flat.mul_(2.0)  # LayerNorm's weight and bias doubled: its output doubles
        model[1].weight.mul_(2.0)
        model[1].bias.mul_(2.0)
        doubled = model_tp(ids.to(DEV))
        torch.testing.assert_close(doubled.cpu(), model(ids), rtol=1e-5, atol=1e-5)
        assert not torch.equal(doubled, first)
        model_tp.load_state_dict(saved)  # copies into the flat shards in place
        assert torch.equal(model_tp(ids.to(DEV)), first)


def test_sharding_twice_is_an_error_and_meta_is_refused():
    model_tp = tp.TensorParallel(toy(), [DEV] * 2, sharded=True)
    with pytest.raises(Exception, match="second time"):
        model_tp.apply_sharding()
    with torch.device("meta"):
        meta = nn.Sequential(nn.Linear(8, 8), nn.LayerNorm(8))
    with pytest.raises(RuntimeError, match="meta"):
        tp.TensorParallel(meta, [DEV] * 2, sharded=True)


def test_factory_default_is_unsharded_and_legacy_spelling_applies_it():
    model_tp = tp.tensor_parallel(toy(), [DEV, DEV])
    assert model_tp.sharding_manager is None
    assert tp.tensor_parallel(toy(), [DEV, DEV], sharded=True).sharding_manager is not None
    same = tp.Sharded(model_tp)
    assert same is model_tp and model_tp.sharding_manager is not None
    with torch.no_grad():
        model_tp(torch.zeros(1, 8, dtype=torch.long, device=DEV))


def test_named_subset_and_tied_parameters():
    class Tied(nn.Module):
        def __init__(self):
            super().__init__()
            self.emb = nn.Embedding(50, 16)
            self.norm = nn.LayerNorm(16)
            self.proj = nn.Linear(16, 16)
            self.head = nn.Linear(16, 50, bias=False)
            self.head.weight = self.emb.weight

        def forward(self, ids):
            return self.head(self.proj(self.norm(self.emb(ids))))

    torch.manual_seed(0)
    model = Tied()
    ids = torch.randint(0, 50, (3, 5), generator=torch.Generator().manual_seed(2))
    with torch.no_grad():
        ref = model(ids)
    # nothing is tensor parallel: ZeRO-3 alone, on the tied table and the norm only
    model_tp = tp.TensorParallel(deepcopy(model), [DEV] * 3, tensor_parallel_config=tp.Config({}, {}, {}, {}), sharded=True,
                                 sharded_param_names=["emb.weight", "norm.weight"])
    shard = model_tp.module_shards[0]
    assert "weight" not in shard.emb._parameters and "weight" not in shard.head._parameters and "bias" in shard.norm._parameters
    with torch.no_grad():
        out = model_tp(ids.to(DEV))
    assert shard.head.weight.data_ptr() == shard.emb.weight.data_ptr()
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-5, atol=1e-5)


def _tiny_bert():
    from transformers import BertConfig, BertModel

    torch.manual_seed(0)
    return BertModel(BertConfig(hidden_size=64, num_attention_heads=4, num_hidden_layers=2, intermediate_size=128, vocab_size=128,
                                max_position_embeddings=64)).eval()


@pytest.mark.parametrize("world", [2, 3])
@pytest.mark.parametrize("tensor_parallel", [False, True])
def test_saved_state_dict_is_the_original_models(world, tensor_parallel):
    """tests/test_saving.py:19-88 of the reference on a random tiny BERT: ZeRO-3 alone (empty rule table) and ZeRO-3 with
    the BERT table; under save_tensor_parallel the state dict has the original names and values. Splitting and
    recombining move elements, so values must come back bit-exact, except what the table scales (divided by W on the
    way in, multiplied on the way out: exact for W = 2, rounding for W = 3)."""
    model = _tiny_bert()
    want = {k: v.clone() for k, v in model.state_dict().items()}
    if tensor_parallel:
        model_tp = tp.TensorParallelPreTrainedModel(model, [DEV] * world, sharded=True)
    else:
        model_tp = tp.TensorParallel(model, [DEV] * world, tensor_parallel_config=tp.Config({}, {}, {}, {}), sharded=True)
    with tp.save_tensor_parallel(model_tp):
        got = model_tp.state_dict()
    assert sorted(got) == sorted(want)
    for name, value in want.items():
        assert got[name].shape == value.shape, name
        if world == 2 or not name.endswith("output.dense.bias"):
            assert torch.equal(got[name].cpu(), value), name
        else:
            torch.testing.assert_close(got[name].cpu(), value, rtol=1e-6, atol=1e-7)
    with torch.no_grad():  # and the model still runs afterwards
        model_tp(input_ids=torch.zeros(1, 8, dtype=torch.long, device=DEV))


def test_parameters_of_a_minority_dtype_stay_replicated():
    """fp32 norms beside bf16 weights: the flat shards hold the dtype most of the replicated elements have; the rest
    stays whole on every rank and the model computes what it computed before."""
    torch.manual_seed(0)
    model = nn.Sequential(nn.Linear(16, 16), nn.LayerNorm(16), nn.LayerNorm(16), nn.Linear(16, 4)).to(torch.bfloat16)
    model[1].float()  # the first norm's 32 elements are fp32, the second norm's stay bf16
    x = torch.randn(3, 16)

    class Cast(nn.Module):
        def __init__(self, inner):
            super().__init__()
            self.inner = inner

        def forward(self, t):
            t = self.inner[0](t)
            t = self.inner[1](t.float()).to(torch.bfloat16)
            return self.inner[3](self.inner[2](t))

    wrapped = Cast(model)
    extra = nn.Parameter(torch.zeros(64, dtype=torch.bfloat16))  # makes bf16 the majority among the replicated parameters
    wrapped.register_parameter("extra", extra)
    with torch.no_grad():
        want = wrapped(x.to(torch.bfloat16))
    model_tp = tp.TensorParallel(deepcopy(wrapped), [DEV] * 2, sharded=True)
    names = set(model_tp.sharding_manager.sharded_param_names)
    assert "inner.2.weight" in names and "extra" in names and "inner.1.weight" not in names
    norm32 = model_tp.module_shards[1].inner[1]
    assert isinstance(norm32.weight, nn.Parameter) and norm32.weight.dtype == torch.float32
    with torch.no_grad():
        got = model_tp(x.to(torch.bfloat16).to(DEV))
    torch.testing.assert_close(got.float().cpu(), want.float(), rtol=2e-2, atol=2e-2)
