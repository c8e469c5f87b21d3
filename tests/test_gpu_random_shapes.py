"""Seeded random shapes through the default dispatch of the shard Linears (1 to 70 rows, where the choice of kernel
depends on M, N and K) against fp32 torch on the host: catches a kernel that is chosen for a shape it mishandles."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import shard_forward as ofw
from tensor_parallel_amd import _native

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)
RTOL = 2e-2


def draw(seed):
    g = torch.Generator().manual_seed(seed)
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))  # noqa: E731
    M = pick(1, 70)
    K = 8 * pick(1, 1100)
    # a few sizes around the tile-count thresholds of a 256-CU part, otherwise anything
    N = 4 * pick(1, 1200) if pick(0, 2) else [2048, 4096, 4100, 5504, 8192][pick(0, 4)]
    dtype = [torch.bfloat16, torch.float16][pick(0, 1)]
    return g, M, N, K, dtype


@pytest.mark.parametrize("seed", range(60))
def test_linear_random_shape(seed):
    g, M, N, K, dtype = draw(seed)
    x = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.02).to(dtype)
    b = (torch.randn(N, generator=g) * 0.1).to(dtype) if seed % 2 else None
    act = _native.ACT_GELU if seed % 3 == 0 else _native.ACT_NONE
    got = _native.linear(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV), act=act)
    want = F.linear(x.float(), w.float(), None if b is None else b.float())
    if act == _native.ACT_GELU:
        want = F.gelu(want)
    sigma = 0.02 * math.sqrt(K)
    torch.testing.assert_close(got.float().cpu(), want, rtol=RTOL, atol=RTOL * sigma, msg=lambda m: f"M={M} N={N} K={K} {dtype}: {m}")


@pytest.mark.parametrize("seed", range(100, 140))
def test_gated_pair_random_shape(seed):
    g, M, N, K, dtype = draw(seed)
    x = torch.randn(M, K, generator=g).to(dtype)
    wg = (torch.randn(N, K, generator=g) * 0.02).to(dtype)
    wu = (torch.randn(N, K, generator=g) * 0.02).to(dtype)
    got = _native.swiglu_up(x.to(DEV), wg.to(DEV), wu.to(DEV))
    want = ofw.gated_mlp_hidden(x.float(), wg.float(), wu.float())
    sigma = (0.02 * math.sqrt(K)) ** 2
    torch.testing.assert_close(got.float().cpu(), want, rtol=RTOL, atol=RTOL * sigma, msg=lambda m: f"M={M} N={N} K={K} {dtype}: {m}")


@pytest.mark.parametrize("seed", range(200, 230))
def test_int8_linear_random_shape(seed):
    """int8 weights with outlier columns: rows 1 to 64, matrices on both sides of the size from which K is split over blocks."""
    import numpy as np

    from oracle import quant as oq

    g = torch.Generator().manual_seed(seed)
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))  # noqa: E731
    M = pick(1, 64)
    big = seed % 3 == 0
    N, K = (16 * pick(260, 520), 16 * pick(256, 520)) if big else (4 * pick(1, 600), 16 * pick(2, 350))
    n_out = [0, 5, 41, 100][pick(0, 3)]
    dtype = [torch.bfloat16, torch.float16][pick(0, 1)]
    w = (torch.randn(N, K, generator=g) * 0.02).to(dtype).float().numpy()
    x = torch.randn(M, K, generator=g)
    cols = np.sort(torch.randperm(K, generator=g)[:n_out].numpy())
    x[:, cols] *= 20
    x = x.to(dtype)
    wq, scale, w_out = oq.quantize_rows(w, cols)
    got = _native.linear_w8(x.to(DEV), torch.from_numpy(wq).to(DEV), torch.from_numpy(scale).to(DEV),
                            torch.from_numpy(cols.astype(np.int32)).to(DEV) if n_out else None,
                            torch.from_numpy(w_out).to(dtype).to(DEV) if n_out else None)
    want = oq.linear_w8_f64(x.float().numpy(), wq, scale, cols, w_out)
    sigma = 0.02 * math.sqrt(K + 400 * n_out)
    torch.testing.assert_close(got.double().cpu(), torch.from_numpy(want), rtol=RTOL, atol=RTOL * sigma, msg=lambda m: f"M={M} N={N} K={K} n_out={n_out} {dtype}: {m}")
