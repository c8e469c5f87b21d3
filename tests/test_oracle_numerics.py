"""Pins oracle/reduce.py, oracle/shard_forward.py and oracle/quant.py."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import to_bits
from oracle import quant as oq
from oracle import reduce as ored
from oracle import shard_forward as ofw


def _special_bf16():
    vals = [0.0, -0.0, 1.0, -1.0, 1.0078125, 3.3895313892515355e38, 1e-40, float("inf"), -float("inf"), float("nan"), 65280.0, 0.1]
    return torch.tensor(vals, dtype=torch.float32).to(torch.bfloat16)


@pytest.mark.parametrize("world", [2, 3, 4, 8])
def test_bf16_stepwise_matches_torch_sum(world):
    g = torch.Generator().manual_seed(world)
    parts = [torch.randn(4097, generator=g).to(torch.bfloat16) for _ in range(world)]
    parts[0][: _special_bf16().numel()] = _special_bf16()
    want = sum(parts)  # the reference's expression, cross_device_ops.py:49
    got = ored.sum_bf16_stepwise([to_bits(p) for p in parts])
    w = to_bits(want)
    nan = np.isnan(ored.bf16_to_f32(w))
    assert np.array_equal(got[~nan], w[~nan])
    assert np.isnan(ored.bf16_to_f32(got[nan])).all()


def test_bf16_rounding_ties_to_even():
    # 1 + 2^-8 is exactly between two bf16 values around 1.0: ties go to the even mantissa
    x = np.array([1.0 + 2.0**-8, 1.0 + 3 * 2.0**-8, 1.0 + 2.0**-8 + 2.0**-20], dtype=np.float32)
    got = ored.bf16_to_f32(ored.f32_to_bf16(x))
    assert got.tolist() == [1.0, 1.015625, 1.0078125]
    assert np.array_equal(ored.f32_to_bf16(x), to_bits(torch.from_numpy(x).to(torch.bfloat16)))


def test_w2_both_modes_agree_and_order_free():
    g = torch.Generator().manual_seed(0)
    a, b = (to_bits(torch.randn(1000, generator=g).to(torch.bfloat16)) for _ in range(2))
    assert np.array_equal(ored.sum_bf16_stepwise([a, b]), ored.sum_bf16_f32acc([a, b]))
    assert np.array_equal(ored.sum_bf16_stepwise([a, b]), ored.sum_bf16_stepwise([b, a]))


def test_f16_and_f32_sums_match_torch():
    g = torch.Generator().manual_seed(3)
    parts = [torch.randn(513, generator=g).to(torch.float16) for _ in range(3)]
    assert np.array_equal(ored.sum_f16_stepwise([p.numpy() for p in parts]), sum(parts).numpy())
    parts32 = [torch.randn(513, generator=g) for _ in range(4)]
    assert np.array_equal(ored.sum_f32([p.numpy() for p in parts32]), sum(parts32).numpy())


@pytest.mark.parametrize("world", [2, 3, 4])
def test_shards_recombine_to_unsplit_linear(world):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 24, generator=g, dtype=torch.float64)
    w = torch.randn(18, 24, generator=g, dtype=torch.float64)
    b = torch.randn(18, generator=g, dtype=torch.float64)
    full = F.linear(x, w, b)
    cols = torch.cat([ofw.column_parallel_linear(x, w, b, world, r) for r in range(world)], dim=-1)
    torch.testing.assert_close(cols, full, rtol=1e-12, atol=1e-12)
    rows = ofw.reduce_sum([ofw.row_parallel_linear(x, w, world, r) for r in range(world)]) + b
    torch.testing.assert_close(rows, full, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("threads", [False, True])
def test_tp_mlp_equals_unsplit_mlp(threads):
    g = torch.Generator().manual_seed(1)
    d, ffn = 16, 44
    x = torch.randn(3, d, generator=g, dtype=torch.float64)
    wg, wu = (torch.randn(ffn, d, generator=g, dtype=torch.float64) * 0.1 for _ in range(2))
    wd = torch.randn(d, ffn, generator=g, dtype=torch.float64) * 0.1
    full = ofw.gated_mlp_shard(x, wg, wu, wd)
    for world in (2, 3):
        torch.testing.assert_close(ofw.llama_mlp_tp_forward(x, wg, wu, wd, world, threads), full, rtol=1e-12, atol=1e-12)


def test_quantizer_definition():
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((12, 64)) * 0.02).astype(np.float32)
    cols = np.sort(rng.permutation(64)[:5])
    w[:, cols] *= 50  # outlier columns must not influence the scales
    q, scale, w_out = oq.quantize_rows(w, cols)
    assert q.dtype == np.int8 and np.abs(q).max() == 127 and (q[:, cols] == 0).all()
    keep = np.setdiff1d(np.arange(64), cols)
    assert np.allclose(scale, np.abs(w[:, keep]).max(axis=1) / 127, rtol=0, atol=0)
    assert (np.abs(q[:, keep] * scale[:, None] - w[:, keep]) <= scale[:, None] / 2 + 1e-12).all()
    assert np.array_equal(w_out, w[:, cols])
    # ties to even: 0.5 -> 0, 1.5 -> 2, 2.5 -> 2
    wt = np.array([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5]], dtype=np.float32)
    qt, st, _ = oq.quantize_rows(wt, np.array([], dtype=np.int64))
    assert st[0] == 1.0 and qt[0].tolist() == [127, 0, 2, 2, 0, -2]
    x = rng.standard_normal((3, 64)).astype(np.float32)
    y = oq.linear_w8_f64(x, q, scale, cols, w_out)
    exact = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(y - exact).max() < 0.02
