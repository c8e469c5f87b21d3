"""tpamd_linear_add: the shard Linear with one step of the partial-sum reduction in its epilogue.

The reference sums rank partials with `sum([...])` over same-dtype tensors (src/tensor_parallel/cross_device_ops.py:49),
i.e. torch's elementwise add: fp32 sum of the widened values, one rounding. The fused form must give exactly
`linear(x, w) + addend` as torch computes it on the host, whichever kernel the shape selects."""
import numpy as np
import pytest
import torch

from oracle import reduce as ored
from tensor_parallel_amd import _native
from tests.conftest import to_bits

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def rnd(shape, seed, std=1.0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype)


def check_fused(x, w, b, a, act=_native.ACT_NONE):
    plain = _native.linear(x, w, b, act=act)
    fused = _native.linear(x, w, b, act=act, addend=a)
    want = plain.cpu() + a.cpu()  # torch's host add: the reference's arithmetic
    assert torch.equal(fused.cpu(), want)
    if x.dtype == torch.bfloat16:  # and the oracle's bit-level restatement of that add
        assert np.array_equal(to_bits(fused), ored.sum_bf16_stepwise([to_bits(plain), to_bits(a)]))
    elif x.dtype == torch.float16:
        f16 = lambda t: t.cpu().numpy()  # noqa: E731
        assert np.array_equal(f16(fused), ored.sum_f16_stepwise([f16(plain), f16(a)]))
    return fused


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [1, 3, 8, 16, 17, 40, 130, 300])
@pytest.mark.parametrize("N,K", [(64, 64), (132, 200), (512, 1024), (260, 72)])
def test_fused_add_equals_linear_then_add(dtype, M, N, K):
    x, w, b = rnd((M, K), 1, 1.0, dtype).to(DEV), rnd((N, K), 0, 0.05, dtype).to(DEV), rnd((N,), 2, 0.1, dtype).to(DEV)
    a = rnd((M, N), 5, 1.0, dtype).to(DEV)
    check_fused(x, w, b, a)
    check_fused(x, w, None, a, act=_native.ACT_GELU)


@pytest.mark.parametrize("M", [17, 32, 40, 64])
def test_fused_add_on_the_weight_streaming_kernel_above_16_rows(M):
    """Few output tiles per CU: 17 to 64 rows of a single matrix stay on the weight-streaming kernel."""
    x, w, a = rnd((M, 4096), 1).to(DEV), rnd((1024, 4096), 0, 0.05).to(DEV), rnd((M, 1024), 5).to(DEV)
    check_fused(x, w, None, a)


@pytest.mark.parametrize("M,N,K", [(5, 7, 3), (70, 10, 36), (33, 130, 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fused_add_on_the_scalar_kernel(dtype, M, N, K):
    x, w, a = rnd((M, K), 1, 1.0, dtype).to(DEV), rnd((N, K), 0, 0.1, dtype).to(DEV), rnd((M, N), 5, 1.0, dtype).to(DEV)
    check_fused(x, w, None, a)


@pytest.mark.parametrize("tile,splits,waves", [("256", 1, 4), ("256", 1, 8), ("256", 2, 4), ("128", 1, 4), ("128", 3, 4)])
def test_fused_add_on_every_tiled_kernel(tile, splits, waves, tune):
    M, N, K = 384, 640, 1024
    tune("TPAMD_GEMM_TILE", tile)
    tune("TPAMD_GEMM_W4", "1" if waves == 4 else "0")
    tune("TPAMD_GEMM_SPLITK256" if tile == "256" else "TPAMD_GEMM_SPLITK", splits)
    x, w, a = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.05).to(DEV), rnd((M, N), 5).to(DEV)
    check_fused(x, w, None, a)
    # ragged edge tiles and an 8-byte-aligned, strided addend
    big = rnd((M, N + 12), 6).to(DEV)
    a2 = big[:300, 4 : 4 + 636]
    x2, w2 = x[:300], w[:636]
    fused = _native.linear(x2, w2, addend=a2)
    assert torch.equal(fused.cpu(), _native.linear(x2, w2).cpu() + a2.cpu())


def test_accumulating_in_place_gives_the_rank_ordered_sum():
    """y += x_r . w_r^T over the ranks of a row-parallel layer: ((p0 + p1) + p2) + p3 with a rounding per step, the
    reference's `sum` over rank partials in rank order."""
    M, N, K, W = 130, 256, 2048, 4
    x, w = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV)
    xs, ws = torch.tensor_split(x, W, 1), torch.tensor_split(w, W, 1)
    parts = [_native.linear(xs[r], ws[r]) for r in range(W)]
    y = parts[0].clone()
    for r in range(1, W):
        _native.linear(xs[r], ws[r], addend=y, out=y)
    want = parts[0].cpu()
    for r in range(1, W):
        want = want + parts[r].cpu()
    assert torch.equal(y.cpu(), want)
    assert torch.equal(y, _native.reduce_partials(parts))


def test_llama_down_projection_with_the_other_ranks_partial():
    """BASELINE config 2 at M = 4096: the down projection of the rank-0 shard with rank 1's partial as the addend
    equals down projection, then the 2-partial reduce kernel, bit for bit."""
    M, d, f = 4096, 4096, 5504
    h, wd, other = rnd((M, f), 1, 0.2).to(DEV), rnd((d, f), 0, 0.02).to(DEV), rnd((M, d), 3, 0.3).to(DEV)
    fused = _native.linear(h, wd, addend=other)
    p = _native.linear(h, wd)
    assert torch.equal(fused, _native.reduce_partials([p, other]))
    assert torch.equal(fused.cpu(), p.cpu() + other.cpu())


def test_argument_errors():
    x, w = rnd((8, 64), 1).to(DEV), rnd((32, 64), 0).to(DEV)
    with pytest.raises(ValueError):
        _native.linear(x, w, addend=rnd((8, 16), 2).to(DEV))
    with pytest.raises(ValueError):
        _native.linear(x, w, addend=rnd((8, 32), 2, dtype=torch.float16).to(DEV))
    with pytest.raises(ValueError):
        _native.linear(x, w, addend=rnd((8, 32), 2))  # host tensor
