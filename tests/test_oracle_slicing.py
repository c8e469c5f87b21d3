"""Pins oracle/slicing.py: the reference's docstring vectors, torch.tensor_split, brute force, invariants."""
import itertools

import numpy as np
import pytest
import torch

from oracle import slicing as osl


def chars(s):
    return np.frombuffer(s.replace(" ", "").encode(), dtype=np.uint8)


def text(a):
    return bytes(a.tolist()).decode()


def test_docstring_vector_split():
    # state_actions.py:40  XXXXXXXXXXXXXXX -> (world_size = 3) -> [XXXXX, XXXXX, XXXXX]
    a = chars("XXXXXXXXXXXXXXX")
    assert [text(osl.split(a, 3, 0, r)) for r in range(3)] == ["XXXXX"] * 3
    b = chars("ABCDEFGHIJKLMNO")
    assert [text(osl.split(b, 3, 0, r)) for r in range(3)] == ["ABCDE", "FGHIJ", "KLMNO"]


def test_docstring_vector_split_in_chunks():
    # state_actions.py:67  AAABBBCCCDDDEEE -> (world_size = 3, chunk_size = 3) -> [AAABBB, CCCDDD, EEE]
    a = chars("AAABBBCCCDDDEEE")
    assert [text(osl.split_in_chunks(a, 3, 0, 3, r)) for r in range(3)] == ["AAABBB", "CCCDDD", "EEE"]


def test_docstring_vector_split_in_grouped_chunks():
    # state_actions.py:94
    a = chars("AABBCCDDEE AABBCCDDEE AABBCCDDEE")
    got = [text(osl.split_in_grouped_chunks(a, 3, 0, 3, 2, r)) for r in range(3)]
    assert got == ["AABBAABBAABB", "CCDDCCDDCCDD", "EEEEEE"]
    parts = [osl.split_in_grouped_chunks(a, 3, 0, 3, 2, r) for r in range(3)]
    assert text(osl.split_in_grouped_chunks_undo(parts, 0, 3)) == "AABBCCDDEE" * 3


@pytest.mark.parametrize("n", range(0, 40))
@pytest.mark.parametrize("world", range(1, 10))
def test_tensor_split_matches_torch(n, world):
    a = np.arange(n * 3).reshape(n, 3)
    want = torch.tensor_split(torch.from_numpy(a), world, dim=0)
    got = osl.tensor_split(a, world, 0)
    assert len(got) == world
    for g, w in zip(got, want):
        assert np.array_equal(g, w.numpy())
    # closed form quoted by the survey: q = n // W, m = n % W, start = r*q + min(r, m), len = q + (r < m)
    q, m = divmod(n, world)
    for r in range(world):
        assert got[r].shape[0] == q + (r < m)
        if got[r].size:
            assert got[r][0, 0] == (r * q + min(r, m)) * 3


@pytest.mark.parametrize("dim", [0, 1, 2, -1, -2])
@pytest.mark.parametrize("world", [1, 2, 3, 4])
def test_split_in_chunks_brute_force(dim, world):
    rng = np.random.default_rng(0)
    shape = [6, 12, 8]
    a = rng.integers(0, 1 << 16, size=shape).astype(np.uint16)
    d = dim % 3
    chunk = {0: 2, 1: 3, 2: 4}[d]
    n_chunks = shape[d] // chunk
    for r in range(world):
        got = osl.split_in_chunks(a, world, dim, chunk, r)
        owned = np.array_split(np.arange(n_chunks), world)[r]
        idx = [c * chunk + j for c in owned for j in range(chunk)]
        want = np.take(a, idx, axis=d)
        assert np.array_equal(got, want)
    parts = [osl.split_in_chunks(a, world, dim, chunk, r) for r in range(world)]
    assert np.array_equal(osl.split_undo(parts, d), a)


@pytest.mark.parametrize("dim", [0, 1])
@pytest.mark.parametrize("world", [1, 2, 3, 5])
@pytest.mark.parametrize("groups,chunk", [(3, 2), (3, 1), (2, 4), (1, 2)])
def test_grouped_chunks_brute_force(dim, world, groups, chunk):
    rng = np.random.default_rng(1)
    per_group_chunks = 5
    n = groups * per_group_chunks * chunk
    shape = [n, 7] if dim == 0 else [7, n]
    a = rng.integers(0, 255, size=shape).astype(np.uint8)
    for r in range(world):
        got = osl.split_in_grouped_chunks(a, world, dim, groups, chunk, r)
        owned = np.array_split(np.arange(per_group_chunks), world)[r]
        idx = [g * per_group_chunks * chunk + c * chunk + j for g in range(groups) for c in owned for j in range(chunk)]
        assert np.array_equal(got, np.take(a, idx, axis=dim))
    parts = [osl.split_in_grouped_chunks(a, world, dim, groups, chunk, r) for r in range(world)]
    assert np.array_equal(osl.split_in_grouped_chunks_undo(parts, dim, groups), a)


def test_grouped_chunks_is_qkv_interleave():
    # GPT-2 c_attn: [in, 3*hidden] with q | k | v side by side; a rank must get its heads of q, of k and of v
    hidden, heads, world = 12, 3, 3
    head_dim = hidden // heads
    q, k, v = (np.full((2, hidden), fill) + np.arange(hidden) // head_dim for fill in (100, 200, 300))
    fused = np.concatenate([q, k, v], axis=1)
    for r in range(world):
        got = osl.split_in_grouped_chunks(fused, world, 1, 3, head_dim, r)
        assert got.shape == (2, 3 * head_dim)
        assert np.array_equal(got[0], np.repeat([100 + r, 200 + r, 300 + r], head_dim))


def test_scale_and_attr_math():
    a = np.array([3.0, -7.5, 0.0], dtype=np.float32)
    assert np.array_equal(osl.scale(a, 2), np.array([1.5, -3.75, 0.0], dtype=np.float32))
    # aux_actions.py:34-36: never 0
    assert [osl.split_num_heads(8, r, 3) for r in range(3)] == [3, 3, 2]
    assert [osl.split_num_heads(2, r, 4) for r in range(4)] == [1, 1, 1, 1]
    # Falcon-40B shape at W=2: 8 kv groups -> 4, query heads 16 * 4 = 64
    assert osl.split_num_heads(8, 0, 2) == 4
    assert 16 * osl.split_num_heads(128 // 16, 0, 2) == 64
    assert osl.split_inner_dim(4096, 1, 32, 8) == 512


def test_baseline_shapes():
    """Shard shapes of the Llama-2-7B and Falcon-40B tensors (element movement checked on thin stand-ins: the
    non-split axis is shortened to 2, the split axis has its real length)."""
    for world, rows in ((2, 5504), (4, 2752), (8, 1376)):
        gate = np.zeros((11008, 2), np.uint8)
        assert osl.split(gate, world, 0, 0).shape == (rows, 2)
        down = np.zeros((2, 11008), np.uint8)
        assert osl.split(down, world, 1, world - 1).shape == (2, rows)
    for world, rows in ((2, 2048), (4, 1024), (8, 512)):
        qw = np.zeros((4096, 2), np.uint8)
        assert osl.split_in_chunks(qw, world, 0, 128, 0).shape == (rows, 2)
        emb = np.zeros((3, 4096), np.uint8)
        assert osl.split(emb, world, 1, 1).shape == (3, rows)
    qkv = np.arange(9216, dtype=np.int32).reshape(9216, 1)
    r0 = osl.split_in_chunks(qkv, 2, 0, (2 + 16) * 64, 0)
    assert r0.shape == (4608, 1) and r0[0, 0] == 0 and r0[-1, 0] == 4607
    dense = np.arange(8192, dtype=np.int32).reshape(1, 8192)
    assert osl.split_in_chunks(dense, 2, 1, 16 * 64, 0).shape == (1, 4096)
