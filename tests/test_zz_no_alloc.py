"""tpamd_linear_noalloc: the shard Linear that allocates no device memory (its K-split partial tiles go into a fixed
array inside the library). It runs the same kernels with the same choices as tpamd_linear, so its output must be
that entry point's bit for bit. Called through the C ABI with raw pointers."""
import ctypes

import pytest
import torch

from tensor_parallel_amd import _native

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def rnd(shape, seed, std=1.0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype)


def call(name, x, w, b, y, act=0):
    lib = _native.lib()
    fn = getattr(lib, name)
    M, K = x.shape
    N = w.shape[0]
    stream = ctypes.c_void_p(torch.cuda.current_stream(DEV).cuda_stream)
    return fn(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(w.data_ptr()), ctypes.c_void_p(b.data_ptr()) if b is not None else None,
              ctypes.c_void_p(y.data_ptr()), M, N, K, x.stride(0), w.stride(0), y.stride(0), _native.dtype_code(x.dtype), act, stream)


def both(M, N, K, dtype=torch.bfloat16, bias=True):
    x, w = rnd((M, K), 1, 1.0, dtype).to(DEV), rnd((N, K), 0, 0.02, dtype).to(DEV)
    b = rnd((N,), 2, 0.1, dtype).to(DEV) if bias else None
    y_ref = torch.full((M, N), 7.0, dtype=dtype, device=DEV)
    y_new = torch.full((M, N), -7.0, dtype=dtype, device=DEV)
    assert call("tpamd_linear", x, w, b, y_ref) == 0, _native.lib().tpamd_last_error()
    assert call("tpamd_linear_noalloc", x, w, b, y_new) == 0, _native.lib().tpamd_last_error()
    torch.cuda.synchronize()
    assert torch.equal(y_ref, y_new), f"M={M} N={N} K={K}: tpamd_linear_noalloc differs from tpamd_linear"
    return y_new


def test_two_calls_in_a_row_the_second_smaller():
    """Both shapes split K (few output tiles, long K), so both calls use the fixed array; the second, smaller call
    finds the first one's partial tiles in it and must not be disturbed by them."""
    assert _native.lib().tpamd_noalloc_scratch_bytes() == 32 << 20
    both(512, 4096, 5504)   # Llama-7B down projection shard at 512 tokens: 128 x 128 tiles, K split 4 ways = 32 MiB
    both(200, 1024, 4096)
    both(512, 4096, 5504)   # and the large one again, after the small one


def test_every_batch_size_class():
    """Decode-sized calls (no scratch memory at all), K-split mid-sized ones, and a prefill-sized one."""
    for M in (1, 8, 16, 40, 300, 1024):
        both(M, 1024, 2048, torch.float16)
    both(1024, 4096, 4096, bias=False)


def test_a_shape_whose_partial_tiles_do_not_fit_is_refused():
    """M = 1024, N = 4608, K = 8192 (Falcon-40B qkv shard at 1024 tokens) runs on 256 x 256 tiles with K split 3 ways:
    54 MiB of partial tiles against a 32 MiB array. The call must fail with a message and launch nothing."""
    M, N, K = 1024, 4608, 8192
    x, w = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV)
    y = torch.full((M, N), 3.0, dtype=torch.bfloat16, device=DEV)
    rc = call("tpamd_linear_noalloc", x, w, None, y)
    torch.cuda.synchronize()
    assert rc == -2
    assert b"fixed array" in _native.lib().tpamd_last_error()
    assert bool((y == 3.0).all())
    assert call("tpamd_linear", x, w, None, y) == 0  # the allocating entry point takes it
    torch.cuda.synchronize()


def test_inside_a_hip_graph():
    """A stream capture may not allocate: tpamd_linear_noalloc still splits K there. Replayed three times with eager
    work in between, each replay checked against the eager result."""
    M, N, K = 384, 2048, 4096
    x, w = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV)
    y_ref = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
    y = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
    assert call("tpamd_linear", x, w, None, y_ref) == 0
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        assert call("tpamd_linear_noalloc", x, w, None, y) == 0
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        assert call("tpamd_linear_noalloc", x, w, None, y) == 0
    for _ in range(3):
        y.fill_(0)
        both(200, 1024, 4096)  # eager work that uses the same array between the replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, y_ref)
