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
    assert _native.lib().tpamd_noalloc_scratch_bytes() == 64 << 20
    both(512, 4096, 5504)   # Llama-7B down projection shard at 512 tokens: 128 x 128 tiles, K split 4 ways = 32 MiB
    both(1024, 4608, 8192)  # Falcon-40B qkv shard at 1024 tokens: 256 x 256 tiles, K split 3 ways = 54 MiB
    both(200, 1024, 4096)
    both(512, 4096, 5504)   # and the large one again, after the small one


def test_every_batch_size_class():
    """Decode-sized calls (no scratch memory at all), K-split mid-sized ones, and a prefill-sized one."""
    for M in (1, 8, 16, 40, 300, 1024):
        both(M, 1024, 2048, torch.float16)
    both(1024, 4096, 4096, bias=False)


def test_a_split_whose_partial_tiles_do_not_fit_is_refused(tune):
    """The array holds what a stream's buffer holds on this part, so the library's own choices fit. A K split forced
    beyond that (256 tiles of 128 x 128 split 8 ways: 128 MiB) must fail with a message and launch nothing."""
    tune("TPAMD_GEMM_TILE", "128")
    tune("TPAMD_GEMM_SPLITK", "8")
    M, N, K = 1024, 4096, 4096
    x, w = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV)
    y = torch.full((M, N), 3.0, dtype=torch.bfloat16, device=DEV)
    rc = call("tpamd_linear_noalloc", x, w, None, y)
    torch.cuda.synchronize()
    assert rc == -2
    assert b"fixed array" in _native.lib().tpamd_last_error()
    assert bool((y == 3.0).all())
    assert call("tpamd_linear", x, w, None, y) == 0  # the allocating entry point takes it (unsplit if its buffer is too small)
    torch.cuda.synchronize()


def test_nothing_is_allocated():
    """A first call on a fresh stream, with a K-split shape: the device's free memory does not move and the stream gets
    no scratch buffer of its own (the allocating entry point would give it 64 MiB). The stream has run one unrelated
    kernel before, so that what the HIP runtime itself sets up for a stream's first launch (2 MiB here) is not counted."""
    M, N, K = 384, 2048, 4096
    x, w = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV)
    y = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
    fresh = torch.cuda.Stream()
    with torch.cuda.stream(fresh):
        y.zero_()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(DEV)[0]
    with torch.cuda.stream(fresh):
        assert call("tpamd_linear_noalloc", x, w, None, y) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(DEV)[0] == free_before
    assert _native.scratch_of_stream(DEV, fresh.cuda_stream) == (None, 0)


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
    assert _native.scratch_of_stream(DEV, side.cuda_stream) == (None, 0)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        assert call("tpamd_linear_noalloc", x, w, None, y) == 0
    for _ in range(3):
        y.fill_(0)
        both(200, 1024, 4096)  # eager work that uses the same array between the replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, y_ref)


FIRST_USE_UNDER_CAPTURE = r"""
import ctypes, sys, torch
sys.path.insert(0, sys.argv[1])
from tensor_parallel_amd import _native
dev = torch.device("cuda", 0)
g = torch.Generator().manual_seed(0)
M, N, K = 384, 2048, 4096
x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(dev)
w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16).to(dev)
y = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
y_ref = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
lib = _native.lib()
def call(name, out):
    s = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    return getattr(lib, name)(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(w.data_ptr()), None, ctypes.c_void_p(out.data_ptr()),
                              M, N, K, K, K, N, _native.BF16, 0, s)
torch.cuda.synchronize()
graph = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph):  # the library's very first call in this process happens under capture
    rc = call("tpamd_linear_noalloc", y)
assert rc == 0, lib.tpamd_last_error()
for _ in range(3):
    y.zero_()
    graph.replay()
    torch.cuda.synchronize()
    assert call("tpamd_linear", y_ref) == 0
    torch.cuda.synchronize()
    assert torch.equal(y, y_ref)
print("first use under capture ok")
"""


def test_first_use_under_capture_in_a_fresh_process():
    """The address of the fixed array is looked up at the entry point's first call on a device. In a fresh process
    that first call is made while a stream is being captured: the lookup must not disturb the capture, and the graph
    replays to the eager result."""
    import subprocess
    import sys
    from pathlib import Path

    root = str(Path(__file__).resolve().parent.parent)
    res = subprocess.run([sys.executable, "-c", FIRST_USE_UNDER_CAPTURE, root], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0 and "first use under capture ok" in res.stdout, res.stdout + res.stderr
