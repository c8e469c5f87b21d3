"""int8 weight-only shard Linear with 16-bit outlier columns against its closed-form definition (oracle/quant.py,
evaluated in float64). The reference has no such path: parity is against the definition, not the reference."""
import math

import numpy as np
import pytest
import torch

from oracle import quant as oq
from tensor_parallel_amd import _native

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def make_case(M, N, K, n_out, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(N, K, generator=g) * 0.02).to(dtype).float().numpy()
    x = torch.randn(M, K, generator=g)
    cols = np.sort(torch.randperm(K, generator=torch.Generator().manual_seed(2))[:n_out].numpy())
    x[:, cols] *= 20
    x = x.to(dtype)
    wq, scale, w_out = oq.quantize_rows(w, cols)
    return x, wq, scale, cols, w_out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 2, 5, 16, 17, 33, 64, 70])
@pytest.mark.parametrize("N,K,n_out", [(64, 256, 0), (48, 512, 3), (128, 1024, 41), (36, 272, 33)])
def test_linear_w8_matches_definition(dtype, M, N, K, n_out):
    x, wq, scale, cols, w_out = make_case(M, N, K, n_out, dtype)
    want = oq.linear_w8_f64(x.float().numpy(), wq, scale, cols, w_out)
    got = _native.linear_w8(
        x.to(DEV), torch.from_numpy(wq).to(DEV), torch.from_numpy(scale).to(DEV),
        torch.from_numpy(cols.astype(np.int32)).to(DEV) if n_out else None,
        torch.from_numpy(w_out).to(dtype).to(DEV) if n_out else None,
    )
    sigma = 0.02 * math.sqrt(K + 400 * n_out)
    torch.testing.assert_close(got.double().cpu(), torch.from_numpy(want), rtol=2e-2, atol=2e-2 * sigma)


def test_int8_conversion_is_exact_for_every_code():
    """Every int8 code -127..127 (and -128) through the in-register conversion: x = one-hot rows pick out
    single weights, scale 1, so the output must equal the integer exactly."""
    K = 256
    codes = torch.arange(-128, 128, dtype=torch.int16).to(torch.int8)  # one row holding every code once
    wq = torch.stack([codes, codes.flip(0)] * 8)  # N = 16
    x = torch.eye(K)[:64]
    for dtype in (torch.float16, torch.bfloat16):
        for m0 in range(0, K, 64):
            xs = torch.eye(K)[m0 : m0 + 64].to(dtype)
            got = _native.linear_w8(xs.to(DEV), wq.to(DEV), torch.ones(16, device=DEV), None, None)
            want = wq[:, m0 : m0 + 64].t().float()
            assert torch.equal(got.float().cpu(), want)


def test_falcon_mlp_shard_full_shape():
    """BASELINE config 5 at its real shape: up [16384 x 8192] + GELU, down [8192 x 16384], fp16, batch 4."""
    M, d, f = 4, 8192, 16384
    x, wq1, s1, c1, o1 = make_case(M, f, d, 41, torch.float16, 0)
    up = _native.linear_w8(x.to(DEV), torch.from_numpy(wq1).to(DEV), torch.from_numpy(s1).to(DEV),
                           torch.from_numpy(c1.astype(np.int32)).to(DEV), torch.from_numpy(o1).half().to(DEV), act=_native.ACT_GELU)
    want_up = oq.linear_w8_f64(x.float().numpy(), wq1, s1, c1, o1)
    want_up = torch.nn.functional.gelu(torch.from_numpy(want_up))
    torch.testing.assert_close(up.double().cpu(), want_up, rtol=2e-2, atol=2e-2 * 0.02 * math.sqrt(d + 400 * 41))
    h, wq2, s2, c2, o2 = make_case(M, d, f, 82, torch.float16, 1)
    h = up.cpu()  # feed the device's own hidden forward
    down = _native.linear_w8(up, torch.from_numpy(wq2).to(DEV), torch.from_numpy(s2).to(DEV),
                             torch.from_numpy(c2.astype(np.int32)).to(DEV), torch.from_numpy(o2).half().to(DEV))
    want_down = oq.linear_w8_f64(h.float().numpy(), wq2, s2, c2, o2)
    scale_y = float(np.abs(want_down).std())
    torch.testing.assert_close(down.double().cpu(), torch.from_numpy(want_down), rtol=2e-2, atol=2e-2 * scale_y)


@pytest.mark.parametrize("M", [1, 2, 4, 16, 32, 64])
def test_falcon_mlp_shard_full_shape_every_decode_batch(M):
    """BASELINE config 5 at its real shape through the DEFAULT dispatch at batch 1, 16, 32 and 64 (the row-streaming
    kernel at 1, the K-split kernel whose wavefronts own columns from 2 rows on at this size): both matrices against the closed-form definition in
    float64. The down projection is fed the device's own hidden activations."""
    d, f = 8192, 16384
    x, wq1, s1, c1, o1 = make_case(M, f, d, 41, torch.float16, 0)
    dev = lambda a, dt=None: (torch.from_numpy(a) if dt is None else torch.from_numpy(a).to(dt)).to(DEV)  # noqa: E731
    up = _native.linear_w8(x.to(DEV), dev(wq1), dev(s1), dev(c1.astype(np.int32)), dev(o1, torch.float16), act=_native.ACT_GELU)
    want_up = torch.nn.functional.gelu(torch.from_numpy(oq.linear_w8_f64(x.float().numpy(), wq1, s1, c1, o1)))
    torch.testing.assert_close(up.double().cpu(), want_up, rtol=2e-2, atol=2e-2 * 0.02 * math.sqrt(d + 400 * 41))
    del wq1, want_up
    _, wq2, s2, c2, o2 = make_case(1, d, f, 82, torch.float16, 1)
    down = _native.linear_w8(up, dev(wq2), dev(s2), dev(c2.astype(np.int32)), dev(o2, torch.float16))
    want_down = oq.linear_w8_f64(up.cpu().float().numpy(), wq2, s2, c2, o2)
    torch.testing.assert_close(down.double().cpu(), torch.from_numpy(want_down), rtol=2e-2, atol=2e-2 * float(np.abs(want_down).std()))


@pytest.fixture
def column_groups(tune):
    """Forces the number of 16-column groups per block of the decode kernel (a debugging knob of the library;
    by default it is chosen from the shape and only large N gets more than one)."""
    def use(cg):
        tune("TPAMD_SKINNY_CG", str(cg))
    return use


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [5, 16, 17, 32, 40, 64])
@pytest.mark.parametrize("cg", [2, 4])
def test_linear_w8_column_groups_do_not_change_the_result(dtype, M, cg, column_groups):
    """The same chunks meet the same MFMAs in the same order whatever the grouping: bit-identical results, and
    both within tolerance of the definition."""
    N, K, n_out = 192, 1296, 41  # K: 5 whole 256-element chunks and a ragged one
    x, wq, scale, cols, w_out = make_case(M, N, K, n_out, dtype, seed=3)
    args = (x.to(DEV), torch.from_numpy(wq).to(DEV), torch.from_numpy(scale).to(DEV),
            torch.from_numpy(cols.astype(np.int32)).to(DEV), torch.from_numpy(w_out).to(dtype).to(DEV))
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(5)) * 0.1).to(dtype).to(DEV)
    column_groups(1)
    one = _native.linear_w8(*args, bias=bias, act=_native.ACT_GELU)
    column_groups(cg)
    grouped = _native.linear_w8(*args, bias=bias, act=_native.ACT_GELU)
    assert torch.equal(one, grouped)
    want = oq.linear_w8_f64(x.float().numpy(), wq, scale, cols, w_out) + bias.double().cpu().numpy()
    want = 0.5 * want * (1.0 + np.vectorize(math.erf)(want / math.sqrt(2.0)))
    sigma = 0.02 * math.sqrt(K + 400 * n_out)
    torch.testing.assert_close(grouped.double().cpu(), torch.from_numpy(want), rtol=2e-2, atol=2e-2 * sigma)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [4, 16, 25, 32])
@pytest.mark.parametrize("cg", [2, 4])
def test_16bit_decode_kernels_column_groups(dtype, M, cg, column_groups):
    N, K = 128, 840
    g = torch.Generator().manual_seed(7)
    x = torch.randn(M, K, generator=g).to(dtype).to(DEV)
    w1, w2 = ((torch.randn(N, K, generator=g) * 0.05).to(dtype).to(DEV) for _ in range(2))
    column_groups(1)
    lin1, sw1 = _native.linear(x, w1), _native.swiglu_up(x, w1, w2)
    column_groups(cg)
    lin, sw = _native.linear(x, w1), _native.swiglu_up(x, w1, w2)  # the gated pair uses at most 2 groups
    assert torch.equal(lin, lin1) and torch.equal(sw, sw1)
    torch.testing.assert_close(lin.float(), torch.nn.functional.linear(x.float(), w1.float()), rtol=2e-2, atol=2e-2 * 0.05 * math.sqrt(K))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [9, 16, 17, 32, 33, 64, 70])
@pytest.mark.parametrize("N,K,n_out", [(64, 4096, 0), (200, 4128, 5), (1000, 8192, 41), (528, 6144, 33), (48, 16384, 256)])
def test_k_split_kernel(dtype, M, N, K, n_out, tune):
    """The int8 kernel that splits K over blocks and keeps its x fragments in registers (forced; by default it
    serves 12 or more rows on matrices the column-owning kernel does not take): 1, 2 and 4 row tiles, a single split and several, a last split that
    is partly or wholly past the end of K, column ranges whose last tile is masked, outlier columns on wavefronts
    0 to 7 of split 0, more than 64 rows (slabs), bias and GELU. Same products as the unsplit kernel in another
    order: both are compared with the definition, and with each other."""
    x, wq, scale, cols, w_out = make_case(M, N, K, n_out, dtype, seed=4)
    args = (x.to(DEV), torch.from_numpy(wq).to(DEV), torch.from_numpy(scale).to(DEV),
            torch.from_numpy(cols.astype(np.int32)).to(DEV) if n_out else None,
            torch.from_numpy(w_out).to(dtype).to(DEV) if n_out else None)
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(5)) * 0.1).to(dtype).to(DEV)
    tune("TPAMD_W8_SPLIT", "1")
    got = _native.linear_w8(*args, bias=bias, act=_native.ACT_GELU)
    tune("TPAMD_W8_SPLIT", "0")
    plain = _native.linear_w8(*args, bias=bias, act=_native.ACT_GELU)
    want = oq.linear_w8_f64(x.float().numpy(), wq, scale, cols, w_out) + bias.double().cpu().numpy()
    want = 0.5 * want * (1.0 + np.vectorize(math.erf)(want / math.sqrt(2.0)))
    sigma = 0.02 * math.sqrt(K + 400 * n_out)
    torch.testing.assert_close(got.double().cpu(), torch.from_numpy(want), rtol=2e-2, atol=2e-2 * sigma)
    torch.testing.assert_close(got.float(), plain.float(), rtol=2e-2, atol=2e-2 * sigma)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 9, 16, 17, 32, 33, 48, 49, 64])
@pytest.mark.parametrize("N,K,n_out", [(64, 4096, 0), (200, 4128, 5), (1000, 8192, 41), (528, 6144, 33), (48, 16384, 256),
                                       (256, 1024, 0), (2068, 1040, 7)])
def test_k_split_kernel_whose_wavefronts_own_columns(dtype, M, N, K, n_out, tune):
    """The int8 kernel that keeps the x rows of its K split in LDS and gives every wavefront whole 16-row weight tiles
    (forced; by default it serves 2 or more rows on large matrices): 1 to 4 row tiles of x, one K plane (results
    stored directly) and several, a last plane that is partly past the end of K, column ranges with fewer tiles than
    wavefronts and with a ragged last tile, N not a multiple of 4, the outlier plane with 1 to 8 groups of 32
    columns, bias and GELU. Compared with the definition, and with the unsplit kernel."""
    x, wq, scale, cols, w_out = make_case(M, N, K, n_out, dtype, seed=4)
    args = (x.to(DEV), torch.from_numpy(wq).to(DEV), torch.from_numpy(scale).to(DEV),
            torch.from_numpy(cols.astype(np.int32)).to(DEV) if n_out else None,
            torch.from_numpy(w_out).to(dtype).to(DEV) if n_out else None)
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(5)) * 0.1).to(dtype).to(DEV)
    tune("TPAMD_W8_COLS", "1")
    got = _native.linear_w8(*args, bias=bias, act=_native.ACT_GELU)
    tune("TPAMD_W8_COLS", "0")
    tune("TPAMD_W8_SPLIT", "0")
    plain = _native.linear_w8(*args, bias=bias, act=_native.ACT_GELU)
    want = oq.linear_w8_f64(x.float().numpy(), wq, scale, cols, w_out) + bias.double().cpu().numpy()
    want = 0.5 * want * (1.0 + np.vectorize(math.erf)(want / math.sqrt(2.0)))
    sigma = 0.02 * math.sqrt(K + 400 * n_out)
    torch.testing.assert_close(got.double().cpu(), torch.from_numpy(want), rtol=2e-2, atol=2e-2 * sigma)
    torch.testing.assert_close(got.float(), plain.float(), rtol=2e-2, atol=2e-2 * sigma)


@pytest.mark.parametrize("M,N,K", [(2, 11024, 2048), (24, 11024, 3072), (24, 5504, 4096), (16, 8192, 4096), (48, 4352, 5504), (48, 8192, 4096),
                                   (4, 8192, 11264), (64, 3072, 11008)])
def test_int8_kernel_chosen_by_shape(M, N, K):
    """The library's own choice among the three int8 kernels for 2 to 64 rows, on a shape from every branch of the rule
    (wide matrices with short rows, K = 4096 at 24 rows off and on whole rounds of tiles, few columns with long rows):
    against the definition."""
    x, wq, scale, cols, w_out = make_case(M, N, K, 9, torch.bfloat16, seed=6)
    got = _native.linear_w8(x.to(DEV), torch.from_numpy(wq).to(DEV), torch.from_numpy(scale).to(DEV),
                            torch.from_numpy(cols.astype(np.int32)).to(DEV), torch.from_numpy(w_out).to(torch.bfloat16).to(DEV))
    want = oq.linear_w8_f64(x.float().numpy(), wq, scale, cols, w_out)
    sigma = 0.02 * math.sqrt(K + 400 * 9)
    torch.testing.assert_close(got.double().cpu(), torch.from_numpy(want), rtol=2e-2, atol=2e-2 * sigma)


@pytest.mark.parametrize("knob", ["TPAMD_W8_SPLIT", "TPAMD_W8_COLS"])
def test_k_split_kernel_inside_a_hip_graph(knob, tune):
    """Either K-split int8 kernel and its finishing pass (two launches sharing the library's scratch buffer) recorded
    into a HIP graph after a warm-up call: every replay gives the eager result, with eager work in between."""
    tune(knob, "1")
    M, N, K, n_out = 32, 200, 8192, 41
    x, wq, scale, cols, w_out = make_case(M, N, K, n_out, torch.float16, seed=6)
    args = (x.to(DEV), torch.from_numpy(wq).to(DEV), torch.from_numpy(scale).to(DEV),
            torch.from_numpy(cols.astype(np.int32)).to(DEV), torch.from_numpy(w_out).half().to(DEV))
    eager = _native.linear_w8(*args)
    torch.cuda.synchronize()
    out = torch.empty_like(eager)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on the capture stream: a stream's scratch buffer is allocated at its first use
        assert torch.equal(_native.linear_w8(*args), eager)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out.copy_(_native.linear_w8(*args))
    for i in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        assert torch.equal(_native.linear_w8(*args), eager)  # eager work between replays


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 2, 3])
@pytest.mark.parametrize("N,K,n_out", [(2048, 1024, 0), (2100, 2064, 7), (4096, 4096, 41)])
def test_int8_row_streaming_kernel_on_wide_matrices(dtype, M, N, K, n_out):
    x, wq, scale, cols, w_out = make_case(M, N, K, n_out, dtype, seed=4)
    args = (x.to(DEV), torch.from_numpy(wq).to(DEV), torch.from_numpy(scale).to(DEV),
            torch.from_numpy(cols.astype(np.int32)).to(DEV) if n_out else None, torch.from_numpy(w_out).to(dtype).to(DEV) if n_out else None)
    got = _native.linear_w8(*args)
    want = oq.linear_w8_f64(x.float().numpy(), wq, scale, cols, w_out)
    torch.testing.assert_close(got.double().cpu(), torch.from_numpy(want), rtol=2e-2, atol=2e-2 * 0.02 * math.sqrt(K + 400 * n_out))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K,n_out", [
    (129, 64, 256, 0),       # just above the slabs, one ragged 128 x 128 tile, no outliers
    (200, 300, 528, 41),     # ragged in M, N and K (K: 8 tiles of 64 and a quarter), outliers in one staged tile
    (260, 132, 1040, 70),    # outliers over two staged tiles
    (700, 36, 272, 256),     # the most outlier columns the kernels take
])
def test_linear_w8_prefill_sizes_match_definition(dtype, M, N, K, n_out):
    """More rows than the weight-streaming kernels take in two passes: the weights go through the matrix pipe once,
    dequantised on their way into LDS; scales, outlier columns, bias and GELU as at every other size."""
    x, wq, scale, cols, w_out = make_case(M, N, K, n_out, dtype, seed=M)
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(5)) * 0.1).to(dtype)
    args = (x.to(DEV), torch.from_numpy(wq).to(DEV), torch.from_numpy(scale).to(DEV),
            torch.from_numpy(cols.astype(np.int32)).to(DEV) if n_out else None,
            torch.from_numpy(w_out).to(dtype).to(DEV) if n_out else None)
    want = oq.linear_w8_f64(x.float().numpy(), wq, scale, cols, w_out)
    sigma = 0.02 * math.sqrt(K + 400 * n_out)
    got = _native.linear_w8(*args)
    torch.testing.assert_close(got.double().cpu(), torch.from_numpy(want), rtol=2e-2, atol=2e-2 * sigma)
    want_b = want + bias.double().numpy()
    want_b = 0.5 * want_b * (1.0 + np.vectorize(math.erf)(want_b / math.sqrt(2.0)))
    got = _native.linear_w8(*args, bias=bias.to(DEV), act=_native.ACT_GELU)
    torch.testing.assert_close(got.double().cpu(), torch.from_numpy(want_b), rtol=2e-2, atol=2e-2 * sigma)
    # the first 64 rows through the weight-streaming kernels: the same sums in another order
    few = _native.linear_w8(args[0][:64].contiguous(), *args[1:])
    torch.testing.assert_close(few.float().cpu(), _native.linear_w8(*args)[:64].float().cpu(), rtol=2e-2, atol=2e-2 * sigma)


def test_falcon_mlp_shard_full_shape_at_prefill():
    """BASELINE config 5's matrices at 1024 tokens (256 x 256 tiles fill the part): sampled rows against the definition."""
    M, d, f = 1024, 8192, 16384
    x, wq1, s1, c1, o1 = make_case(M, f, d, 41, torch.float16, 0)
    dev = lambda a, dt=None: (torch.from_numpy(a) if dt is None else torch.from_numpy(a).to(dt)).to(DEV)  # noqa: E731
    up = _native.linear_w8(x.to(DEV), dev(wq1), dev(s1), dev(c1.astype(np.int32)), dev(o1, torch.float16), act=_native.ACT_GELU)
    rows = [0, 1, 255, 256, 511, 777, 1023]
    want_up = torch.nn.functional.gelu(torch.from_numpy(oq.linear_w8_f64(x[rows].float().numpy(), wq1, s1, c1, o1)))
    torch.testing.assert_close(up[rows].double().cpu(), want_up, rtol=2e-2, atol=2e-2 * 0.02 * math.sqrt(d + 400 * 41))
    assert torch.isfinite(up.float()).all()
    del wq1, want_up
    _, wq2, s2, c2, o2 = make_case(1, d, f, 82, torch.float16, 1)
    down = _native.linear_w8(up, dev(wq2), dev(s2), dev(c2.astype(np.int32)), dev(o2, torch.float16))
    want_down = oq.linear_w8_f64(up[rows].cpu().float().numpy(), wq2, s2, c2, o2)
    torch.testing.assert_close(down[rows].double().cpu(), torch.from_numpy(want_down), rtol=2e-2, atol=2e-2 * float(np.abs(want_down).std()))
