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


def test_a_capturing_stream_takes_the_spare_buffer(tune):
    """Nothing is allocated under capture; a stream that captures K-split work without having run any gets the spare
    buffer that the device's first allocation set aside, and the graph replays to the eager (split) result."""
    tune("TPAMD_GEMM_TILE", "128")
    tune("TPAMD_GEMM_SPLITK", "4")
    M, N, K = 256, 512, 4096
    x, w = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV)
    eager = _native.linear(x, w)  # allocates the default stream's buffer and, the first time on this device, the spare
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    assert _native.scratch_of_stream(DEV, side.cuda_stream) == (None, 0)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out = _native.linear(x, w)
    taken = _native.scratch_of_stream(DEV, side.cuda_stream)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        assert torch.equal(_native.linear(x, w), eager)  # eager K-split work on another stream between the replays
        torch.cuda.synchronize()
        if taken[0] is not None:
            assert torch.equal(out, eager) and taken[0] != _native.scratch_of_stream(DEV)[0]
        else:  # an earlier capture in this process took the spare: the call ran unsplit
            torch.testing.assert_close(out.float(), eager.float(), rtol=2e-2, atol=2e-2)


def test_a_retired_stream_gives_its_buffer_back(tune):
    """tpamd_scratch_release: the stream's buffer is freed (the device's free memory grows by about its size) and the stream
    has none afterwards; K-split work on the stream later simply gets a new one."""
    tune("TPAMD_GEMM_TILE", "128")
    tune("TPAMD_GEMM_SPLITK", "4")
    M, N, K = 256, 512, 4096
    x, w = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV)
    want = _native.linear(x, w)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        got = _native.linear(x, w)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    ptr, nbytes = _native.scratch_of_stream(DEV, stream.cuda_stream)
    assert ptr is not None and nbytes > 0
    free_before = torch.cuda.mem_get_info(DEV)[0]
    _native.release_scratch(DEV, stream.cuda_stream)
    assert _native.scratch_of_stream(DEV, stream.cuda_stream) == (None, 0)
    assert torch.cuda.mem_get_info(DEV)[0] >= free_before + nbytes // 2  # the driver accounts in its own granules
    _native.release_scratch(DEV, stream.cuda_stream)  # a stream without a buffer: nothing to do
    with torch.cuda.stream(stream):
        again = _native.linear(x, w)
    torch.cuda.synchronize()
    assert torch.equal(again, want)
    assert _native.scratch_of_stream(DEV, stream.cuda_stream)[0] is not None
