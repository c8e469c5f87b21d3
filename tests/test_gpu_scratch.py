"""The K-split kernels keep their fp32 partial results in scratch memory that belongs to one (device, stream): work on
two streams of a device must never meet in one buffer."""
import pytest
import torch

from tensor_parallel_amd import _native

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def rnd(shape, seed, std=1.0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype)


def test_each_stream_gets_its_own_buffer(tune):
    tune("TPAMD_GEMM_TILE", "128")
    tune("TPAMD_GEMM_SPLITK", "4")
    M, N, K = 256, 512, 4096
    x, w = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV)
    x2, w2 = rnd((M, K), 3).to(DEV), rnd((N, K), 4, 0.02).to(DEV)
    tune("TPAMD_GEMM_SPLITK", "1")
    want, want2 = _native.linear(x, w), _native.linear(x2, w2)  # unsplit
    tune("TPAMD_GEMM_SPLITK", "4")
    torch.cuda.synchronize()
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    assert _native.scratch_of_stream(DEV, a.cuda_stream) == (None, 0)
    outs = []
    for _ in range(20):  # interleaved K-split launches on both streams, nothing orders the streams
        with torch.cuda.stream(a):
            outs.append((_native.linear(x, w), want))
        with torch.cuda.stream(b):
            outs.append((_native.linear(x2, w2), want2))
    torch.cuda.synchronize()
    pa, na = _native.scratch_of_stream(DEV, a.cuda_stream)
    pb, nb = _native.scratch_of_stream(DEV, b.cuda_stream)
    assert pa is not None and pb is not None and pa != pb
    assert na >= 4 * (M // 128) * (N // 128) * 128 * 128 * 4 and nb == na
    for got, ref in outs:
        torch.testing.assert_close(got.float(), ref.float(), rtol=2e-2, atol=2e-2)
    # a stream keeps its buffer
    with torch.cuda.stream(a):
        _native.linear(x, w)
    assert _native.scratch_of_stream(DEV, a.cuda_stream) == (pa, na)


def test_first_use_under_capture_runs_unsplit_and_allocates_nothing(tune):
    tune("TPAMD_GEMM_TILE", "128")
    tune("TPAMD_GEMM_SPLITK", "4")
    M, N, K = 256, 512, 4096
    x, w = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV)
    eager = _native.linear(x, w)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    out = None
    with torch.cuda.graph(graph, stream=side):
        out = _native.linear(x, w)
    assert _native.scratch_of_stream(DEV, side.cuda_stream) == (None, 0)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        torch.testing.assert_close(out.float(), eager.float(), rtol=2e-2, atol=2e-2)
