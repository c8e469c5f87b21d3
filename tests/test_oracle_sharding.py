"""Pins for oracle/sharding.py and for the product's host-side layout arithmetic (no device needed)."""
import numpy as np
import pytest
import torch
from torch import nn

from oracle import sharding as osh
from tensor_parallel_amd.sharding import find_all_occurences, flat_layout


def ragged(seed, sizes, dtype=np.int64):
    rng = np.random.default_rng(seed)
    return [rng.integers(-1000, 1000, size=s).astype(dtype) for s in sizes]


@pytest.mark.parametrize("world", [1, 2, 3, 4, 7])
def test_combine_inverts_make(world):
    shapes = [(5, 7), (1,), (13,), (2, 3, 4), (0,), (6, 1)]
    params = ragged(world, shapes)
    flat, sizes = osh.make_flat_shards([params] * world, world)
    assert len({f.size for f in flat}) == 1
    assert all(sum(s) == flat[0].size for s in sizes)
    back = osh.combine_shards(flat, sizes, shapes)
    for a, b in zip(params, back):
        assert a.shape == b.shape and np.array_equal(a, b)


def test_rank_sections_come_from_that_ranks_copy():
    """Rank r's flat shard reads rank r's copy (sharding.py:143-146): distinct copies must show up in distinct shards."""
    world = 3
    copies = [[np.full(10, r, dtype=np.int64), np.full(4, 10 + r, dtype=np.int64)] for r in range(world)]
    flat, sizes = osh.make_flat_shards(copies, world)
    assert sizes == [[4, 2, 0], [3, 1, 2], [3, 1, 2]]
    assert flat[0].tolist() == [0] * 4 + [10] * 2
    assert flat[1].tolist() == [1] * 3 + [11] + [0, 0]
    assert flat[2].tolist() == [2] * 3 + [12] + [0, 0]


@pytest.mark.parametrize("world,padding", [(1, 0), (2, 0), (3, 4)])
def test_parameter_counts_of_the_reference_test(world, padding):
    """tests/test_basic.py:110-135 of the reference: Embedding(1337, 64), LayerNorm(64), Linear(64, 128), Linear(128, 10)
    under the default rules leave LayerNorm's weight and bias replicated; after ZeRO-3 the model holds the original
    parameter count, plus 4 at W = 3."""
    replicated = ragged(0, [(64,), (64,)])
    flat, _ = osh.make_flat_shards([replicated] * world, world)
    assert sum(f.size for f in flat) == 128 + padding


@pytest.mark.parametrize("n", range(0, 23))
@pytest.mark.parametrize("world", [1, 2, 3, 5, 8])
def test_section_lengths_are_tensor_split(n, world):
    want = [t.numel() for t in torch.tensor_split(torch.empty(n), world)]
    got = [osh.extract_param_shards([np.arange(n)], r, world)[0].size for r in range(world)]
    assert got == want


@pytest.mark.parametrize("world", [1, 2, 3, 4, 7])
def test_product_layout_agrees_with_the_oracle(world):
    shapes = [(5, 7), (1,), (13,), (2, 3, 4), (0,), (6, 1), (1025,)]
    params = ragged(3, shapes)
    _, sizes = osh.make_flat_shards([params] * world, world)
    sections, pads, flat_len = flat_layout([p.size for p in params], world)
    assert [[length for _, length in sec] + [pad] for sec, pad in zip(sections, pads)] == sizes
    assert all(sum(s) == flat_len for s in sizes)
    for i, p in enumerate(params):  # the sections of one parameter tile it in rank order
        at = 0
        for r in range(world):
            start, length = sections[r][i]
            assert start == at
            at += length
        assert at == p.size


def test_occurences_include_tied_parameters():
    class Tied(nn.Module):
        def __init__(self):
            super().__init__()
            self.emb = nn.Embedding(10, 4)
            self.norm = nn.LayerNorm(4)
            self.head = nn.Linear(4, 10, bias=False)
            self.head.weight = self.emb.weight

    model = Tied()
    names = [n for n, _ in model.named_parameters()]
    assert names == ["emb.weight", "norm.weight", "norm.bias"]
    found = find_all_occurences(model, names)
    assert [(type(m).__name__, n) for m, n in found[0]] == [("Embedding", "weight"), ("Linear", "weight")]
    assert [(type(m).__name__, n) for m, n in found[1]] == [("LayerNorm", "weight")]
    with pytest.raises(AssertionError):
        find_all_occurences(model, ["missing.weight"])
