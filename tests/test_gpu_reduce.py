"""Partial-sum reduction on the GPU against the oracle: bit-exact in both accumulation modes."""
import numpy as np
import pytest
import torch

from conftest import to_bits
from oracle import reduce as ored
from tensor_parallel_amd import _native

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def parts_for(world, n, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(n, generator=g) * 3).to(dtype) for _ in range(world)]


@pytest.mark.parametrize("world", [1, 2, 3, 4, 8, 16])
@pytest.mark.parametrize("n", [1, 7, 8, 4096, 4096 * 16 + 5])
def test_bf16_bit_exact(world, n):
    parts = parts_for(world, n, torch.bfloat16, world)
    bits = [to_bits(p) for p in parts]
    dev = [p.to(DEV) for p in parts]
    got = to_bits(_native.reduce_partials(dev, accum=_native.ACCUM_STEPWISE))
    assert np.array_equal(got, ored.sum_bf16_stepwise(bits))
    got32 = to_bits(_native.reduce_partials(dev, accum=_native.ACCUM_F32))
    assert np.array_equal(got32, ored.sum_bf16_f32acc(bits))
    # the reference's own expression on the host (cross_device_ops.py:49)
    assert torch.equal(_native.reduce_partials(dev).cpu(), sum(parts))


@pytest.mark.parametrize("world", [2, 3, 5])
def test_f16_and_f32_bit_exact(world):
    p16 = parts_for(world, 10007, torch.float16, 1)
    got = _native.reduce_partials([p.to(DEV) for p in p16]).cpu()
    assert np.array_equal(got.numpy(), ored.sum_f16_stepwise([p.numpy() for p in p16]))
    p32 = parts_for(world, 10007, torch.float32, 2)
    got = _native.reduce_partials([p.to(DEV) for p in p32]).cpu()
    assert np.array_equal(got.numpy(), ored.sum_f32([p.numpy() for p in p32]))
    assert torch.equal(got, sum(p32))


def test_shapes_specials_and_aliasing():
    a = torch.tensor([1.0, float("inf"), -float("inf"), float("nan"), 65280.0, 1e-40, -0.0], dtype=torch.bfloat16)
    b = torch.tensor([1.0078125, 1.0, float("inf"), 1.0, 65280.0, 1e-40, 0.0], dtype=torch.bfloat16)
    got = _native.reduce_partials([a.to(DEV), b.to(DEV)]).cpu()
    want = a + b
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    assert torch.equal(got[~torch.isnan(got)], want[~torch.isnan(want)])
    # [M, N] partials, result written over partial 0
    parts = [p.view(16, 256).to(DEV) for p in parts_for(2, 4096, torch.bfloat16, 9)]
    want = (parts[0] + parts[1]).cpu()
    out = _native.reduce_partials(parts, out=parts[0])
    assert out.data_ptr() == parts[0].data_ptr() and torch.equal(out.cpu(), want)
    with pytest.raises(ValueError):
        _native.reduce_partials([parts[0], parts[1][:8]])
    with pytest.raises(ValueError):
        _native.reduce_partials([parts[0]] * 17)


def test_full_size_properties():
    """C2 prefill size, [4096, 4096] bf16, W = 2: order-independent, and equal to the host sum on a sample."""
    g = torch.Generator(device=DEV).manual_seed(0)
    a, b = (torch.randn(4096, 4096, generator=g, device=DEV).to(torch.bfloat16) for _ in range(2))
    ab, ba = _native.reduce_partials([a, b]), _native.reduce_partials([b, a])
    assert torch.equal(ab, ba)
    rows = torch.tensor([0, 1, 2047, 4095])
    assert torch.equal(ab[rows.to(DEV)].cpu(), a[rows.to(DEV)].cpu() + b[rows.to(DEV)].cpu())
    zero = torch.zeros_like(a)
    assert torch.equal(_native.reduce_partials([a, zero]), a)
