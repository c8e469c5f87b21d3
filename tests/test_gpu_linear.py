"""Rank-shard Linears on the GPU against the oracle (torch on CPU).

Tolerances: bf16/fp16 results are compared with the fp32 CPU product of the same bf16/fp16 inputs at
rtol 2e-2 (atol scaled to the typical output magnitude), fp32 results at rtol 1e-5."""
import ctypes
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import shard_forward as ofw
from tensor_parallel_amd import _native

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)
RTOL_HALF = 2e-2
RTOL_F32 = 1e-5


def rnd(shape, seed, std=1.0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype)


def check_half(got, want_f32, K, x_std=1.0, w_std=0.02):
    """rtol 2e-2 plus an absolute floor of 2e-2 output standard deviations (entries near zero)."""
    sigma = x_std * w_std * math.sqrt(K)
    torch.testing.assert_close(got.float().cpu(), want_f32, rtol=RTOL_HALF, atol=RTOL_HALF * sigma)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [1, 3, 16, 17, 32, 33, 64, 130, 256, 300])
@pytest.mark.parametrize("N,K", [(64, 64), (132, 200), (260, 72), (512, 1024)])
def test_linear_half(dtype, M, N, K):
    x, w, b = rnd((M, K), 1, 1.0, dtype), rnd((N, K), 0, 0.02, dtype), rnd((N,), 2, 0.1, dtype)
    want = F.linear(x.float(), w.float(), b.float())
    got = _native.linear(x.to(DEV), w.to(DEV), b.to(DEV))
    assert got.shape == (M, N) and got.dtype == dtype
    check_half(got, want, K)
    got_nb = _native.linear(x.to(DEV), w.to(DEV))
    check_half(got_nb, F.linear(x.float(), w.float()), K)
    # leading dimensions are kept
    if M % 2 == 0:
        got3 = _native.linear(x.view(2, M // 2, K).to(DEV), w.to(DEV))
        assert got3.shape == (2, M // 2, N) and torch.equal(got3.view(M, N), got_nb)


@pytest.mark.parametrize("M", [1, 5, 16, 31, 40, 128, 257])
@pytest.mark.parametrize("N,K", [(64, 64), (100, 136), (344, 128), (256, 512)])
def test_swiglu_matches_oracle(M, N, K):
    x, wg, wu = rnd((M, K), 1), rnd((N, K), 0, 0.05), rnd((N, K), 3, 0.05)
    got = _native.swiglu_up(x.to(DEV), wg.to(DEV), wu.to(DEV))
    want32 = ofw.gated_mlp_hidden(x.float(), wg.float(), wu.float())
    sigma = (0.05 * math.sqrt(K)) ** 2
    torch.testing.assert_close(got.float().cpu(), want32, rtol=RTOL_HALF, atol=RTOL_HALF * sigma)
    # against the reference's own bf16 op chain on the host: same roundings, so differences are a few ulp
    want_bf16 = ofw.gated_mlp_hidden(x, wg, wu).float()
    torch.testing.assert_close(got.float().cpu(), want_bf16, rtol=RTOL_HALF, atol=RTOL_HALF * sigma)


@pytest.mark.parametrize("M,N,K", [(1, 10, 16), (7, 33, 50), (64, 64, 64), (130, 70, 129), (128, 768, 3072)])
def test_linear_fp32(M, N, K):
    x, w, b = rnd((M, K), 1, 1.0, torch.float32), rnd((N, K), 0, 0.02, torch.float32), rnd((N,), 2, 0.1, torch.float32)
    got = _native.linear(x.to(DEV), w.to(DEV), b.to(DEV)).cpu()
    want = F.linear(x.double(), w.double(), b.double()).float()
    torch.testing.assert_close(got, want, rtol=RTOL_F32, atol=RTOL_F32 * 0.02 * math.sqrt(K))


@pytest.mark.parametrize("M,N,K", [(130, 72, 132), (64, 4, 4), (1000, 4100, 72), (2048, 2048, 100), (128, 50272, 384)])
def test_linear_fp32_on_the_matrix_pipe(M, N, K):
    """fp32 operands whose rows take 16-byte accesses run on v_mfma_f32_32x32x2_f32: 64 x 64 tiles while those do not
    fill the CUs, 128 x 128 tiles above (the third and fourth shapes), ragged tiles in M, N and K, a row-parallel
    slice of x (leading dimension above K), bias, GELU and the addend of the fused partial sum. The last shape is the
    tied head of BASELINE config 1 (OPT-125m at W = 2: 128 tokens, K = 384 of 768 columns)."""
    full = rnd((M, K + 8), 1, 1.0, torch.float32)
    w, b = rnd((N, K), 0, 0.02, torch.float32), rnd((N,), 2, 0.1, torch.float32)
    other = rnd((M, N), 3, 0.5, torch.float32)
    xd = full.to(DEV)[:, 4:4 + K]  # rows 16-byte aligned, not contiguous
    x = full[:, 4:4 + K]
    atol = RTOL_F32 * 0.02 * math.sqrt(K)
    want = F.linear(x.double(), w.double(), b.double())
    got = _native.linear(xd, w.to(DEV), b.to(DEV)).cpu()
    torch.testing.assert_close(got, want.float(), rtol=RTOL_F32, atol=atol)
    got = _native.linear(xd, w.to(DEV), b.to(DEV), addend=other.to(DEV)).cpu()
    torch.testing.assert_close(got, (want + other.double()).float(), rtol=RTOL_F32, atol=atol)
    got = _native.linear(xd, w.to(DEV), None, act=_native.ACT_GELU).cpu()
    torch.testing.assert_close(got, F.gelu(F.linear(x.double(), w.double())).float(), rtol=RTOL_F32, atol=atol)


def test_gelu_epilogue_and_argument_errors():
    x, w = rnd((40, 64), 1, 1.0, torch.float16), rnd((64, 64), 0, 0.1, torch.float16)
    for M in (8, 40):
        got = _native.linear(x[:M].to(DEV), w.to(DEV), act=_native.ACT_GELU)
        want = F.gelu(F.linear(x[:M].float(), w.float()))
        torch.testing.assert_close(got.float().cpu(), want, rtol=RTOL_HALF, atol=2e-2)
    with pytest.raises(ValueError):
        _native.linear(x.to(DEV), rnd((64, 60), 0, 0.1, torch.float16).to(DEV))  # K mismatch
    with pytest.raises(TypeError):
        _native.linear(x.to(DEV), w.to(DEV).bfloat16())
    assert _native.linear(torch.empty(0, 64, dtype=torch.float16, device=DEV), w.to(DEV)).shape == (0, 64)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", [(4, 8, 12), (6, 256, 172), (70, 10, 36), (33, 130, 8), (5, 7, 3)])
def test_unaligned_shapes_take_the_scalar_kernel(dtype, M, N, K):
    """K not a multiple of 8 or N not a multiple of 4 (what an uneven split of a small model produces)."""
    x, w, b = rnd((M, K), 1, 1.0, dtype), rnd((N, K), 0, 0.1, dtype), rnd((N,), 2, 0.1, dtype)
    got = _native.linear(x.to(DEV), w.to(DEV), b.to(DEV))
    torch.testing.assert_close(got.float().cpu(), F.linear(x.float(), w.float(), b.float()), rtol=RTOL_HALF, atol=2e-2)
    w2 = rnd((N, K), 5, 0.1, dtype)
    h = _native.swiglu_up(x.to(DEV), w.to(DEV), w2.to(DEV))
    torch.testing.assert_close(h.float().cpu(), ofw.gated_mlp_hidden(x.float(), w.float(), w2.float()), rtol=RTOL_HALF, atol=2e-2)


def test_swiglu_fp32():
    x, wg, wu = rnd((9, 40), 1, 1.0, torch.float32), rnd((24, 40), 0, 0.1, torch.float32), rnd((24, 40), 3, 0.1, torch.float32)
    got = _native.swiglu_up(x.to(DEV), wg.to(DEV), wu.to(DEV)).cpu()
    torch.testing.assert_close(got, ofw.gated_mlp_hidden(x, wg, wu), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("world", [2, 4])
def test_shards_recombine(world):
    """Column-parallel shard outputs are the columns of the unsplit product bit for bit (same kernel, same K
    order); row-parallel partials reduced on the device agree with the unsplit product within tolerance."""
    M, N, K = 96, 256, 512
    x, w = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV)
    full = _native.linear(x, w)
    cols = [_native.linear(x, torch.tensor_split(w, world, 0)[r].contiguous()) for r in range(world)]
    assert torch.equal(torch.cat(cols, dim=-1), full)
    parts = [_native.linear(torch.tensor_split(x, world, 1)[r].contiguous(), torch.tensor_split(w, world, 1)[r].contiguous()) for r in range(world)]
    summed = _native.reduce_partials(parts)
    check_half(summed, F.linear(x.float().cpu(), w.float().cpu()), K)
    # strided (non-copied) column slices of x and w are accepted as they are: leading dimension > K
    xs, ws = torch.tensor_split(x, world, 1)[1], torch.tensor_split(w, world, 1)[1]
    assert not xs.is_contiguous()
    assert torch.equal(_native.linear(xs, ws), parts[1])


@pytest.mark.parametrize("M", [1, 16, 512])
def test_llama_mlp_shard_full_shape(M):
    """BASELINE config 2: rank-0 shard at W=2 of a Llama-7B MLP, d=4096, ffn shard 5504, bf16."""
    d, f = 4096, 5504
    x, wg, wu, wd = rnd((M, d), 1), rnd((f, d), 0, 0.02), rnd((f, d), 3, 0.02), rnd((d, f), 4, 0.02)
    xd, gd, ud, dd = (t.to(DEV) for t in (x, wg, wu, wd))
    h = _native.swiglu_up(xd, gd, ud)
    y = _native.linear(h, dd)
    h_want = ofw.gated_mlp_hidden(x.float(), wg.float(), wu.float())
    sig_h = (0.02 * math.sqrt(d)) ** 2
    torch.testing.assert_close(h.float().cpu(), h_want, rtol=RTOL_HALF, atol=RTOL_HALF * sig_h)
    y_want = F.linear(h.float().cpu(), wd.float())  # the down projection of the hidden the device produced
    sig_y = 0.5 * sig_h * 0.02 * math.sqrt(f)
    torch.testing.assert_close(y.float().cpu(), y_want, rtol=RTOL_HALF, atol=RTOL_HALF * sig_y)
    if M <= 16:  # the reference's op chain in bf16 on the host, end to end
        y_ref = ofw.gated_mlp_shard(x, wg, wu, wd).float()
        torch.testing.assert_close(y.float().cpu(), y_ref, rtol=RTOL_HALF, atol=2 * RTOL_HALF * sig_y)


def test_llama_mlp_shard_prefill_4096_sampled_rows():
    """M = 4096 at the full shape: 96 sampled rows against the host, all rows for finiteness, and row
    independence: a row's result does not depend on which other rows share the launch, up to the last bit of
    the 16-bit result (a smaller batch may be served by another tiling, which may split K and so add the same
    products in another order)."""
    d, f, M = 4096, 5504, 4096
    g = torch.Generator(device=DEV).manual_seed(0)
    x = torch.randn(M, d, generator=g, device=DEV).to(torch.bfloat16)
    wg, wu = ((torch.randn(f, d, generator=g, device=DEV) * 0.02).to(torch.bfloat16) for _ in range(2))
    wd = (torch.randn(d, f, generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    h = _native.swiglu_up(x, wg, wu)
    y = _native.linear(h, wd)
    assert torch.isfinite(y.float()).all()
    rows = torch.cat([torch.arange(0, 32), torch.arange(2030, 2062), torch.arange(4064, 4096)])
    xs = x[rows.to(DEV)].cpu()
    h_want = ofw.gated_mlp_hidden(xs.float(), wg.float().cpu(), wu.float().cpu())
    sig_h = (0.02 * math.sqrt(d)) ** 2
    torch.testing.assert_close(h[rows.to(DEV)].float().cpu(), h_want, rtol=RTOL_HALF, atol=RTOL_HALF * sig_h)
    y_want = F.linear(h[rows.to(DEV)].float().cpu(), wd.float().cpu())
    sig_y = 0.5 * sig_h * 0.02 * math.sqrt(f)
    torch.testing.assert_close(y[rows.to(DEV)].float().cpu(), y_want, rtol=RTOL_HALF, atol=RTOL_HALF * sig_y)
    h_sub = _native.swiglu_up(x[1024:1536].contiguous(), wg, wu)
    torch.testing.assert_close(h_sub.float(), h[1024:1536].float(), rtol=2.0 ** -7, atol=2.0 ** -7 * sig_h)
    assert (h_sub != h[1024:1536]).float().mean().item() < 0.01
    sub = _native.linear(h[1024:1536].contiguous(), wd)
    torch.testing.assert_close(sub.float(), y[1024:1536].float(), rtol=2.0 ** -7, atol=2.0 ** -7 * sig_y)
    assert (sub != y[1024:1536]).float().mean().item() < 0.01
    # the same tiling twice: bit-identical
    assert torch.equal(_native.linear(h[1024:1536].contiguous(), wd), sub)


def test_llama_mlp_shard_prefill_4096_every_output():
    """BASELINE config 2 at M = 4096: all 4096 x 5504 hidden values and all 4096 x 4096 outputs against fp32 products of
    the same bf16 inputs on the host (rtol 2e-2, absolute floor 2e-2 output standard deviations), then the fused sum
    with the other rank's partial against torch's host add, bit for bit."""
    d, f, M = 4096, 5504, 4096
    x, wg, wu, wd = rnd((M, d), 1), rnd((f, d), 0, 0.02), rnd((f, d), 3, 0.02), rnd((d, f), 4, 0.02)
    h = _native.swiglu_up(x.to(DEV), wg.to(DEV), wu.to(DEV))
    y = _native.linear(h, wd.to(DEV))
    h_cpu, y_cpu = h.cpu(), y.cpu()
    h_want = ofw.gated_mlp_hidden(x.float(), wg.float(), wu.float())
    sig_h = (0.02 * math.sqrt(d)) ** 2
    torch.testing.assert_close(h_cpu.float(), h_want, rtol=RTOL_HALF, atol=RTOL_HALF * sig_h)
    del h_want
    y_want = F.linear(h_cpu.float(), wd.float())  # the down projection of the hidden the device produced
    sig_y = 0.5 * sig_h * 0.02 * math.sqrt(f)
    torch.testing.assert_close(y_cpu.float(), y_want, rtol=RTOL_HALF, atol=RTOL_HALF * sig_y)
    other = rnd((M, d), 9, 0.3)
    fused = _native.linear(h, wd.to(DEV), addend=other.to(DEV))
    assert torch.equal(fused.cpu(), y_cpu + other)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", [(40, 136, 5504), (130, 260, 1536), (300, 64, 2048), (17, 512, 1024)])
@pytest.mark.parametrize("splits", [1, 3, 8])
def test_split_k_tiles(dtype, M, N, K, splits, tune):
    """The 128 x 128 tiling with K split `splits` ways (forced through the library's debugging knob; by default
    the split is chosen from the tile count): ragged last split, tile rows past M, tile columns past N, bias and
    GELU applied by the finishing pass."""
    tune("TPAMD_GEMM_SPLITK", str(splits))
    tune("TPAMD_GEMM_TILE", "128")
    x, w, b = rnd((M, K), 1, 1.0, dtype), rnd((N, K), 0, 0.02, dtype), rnd((N,), 2, 0.1, dtype)
    got = _native.linear(x.to(DEV), w.to(DEV), b.to(DEV), act=_native.ACT_GELU)
    want = F.gelu(F.linear(x.float(), w.float(), b.float()))
    check_half(got, want, K)
    w2 = rnd((N, K), 5, 0.02, dtype)
    h = _native.swiglu_up(x.to(DEV), w.to(DEV), w2.to(DEV))
    sigma = (0.02 * math.sqrt(K)) ** 2
    torch.testing.assert_close(h.float().cpu(), ofw.gated_mlp_hidden(x.float(), w.float(), w2.float()), rtol=RTOL_HALF, atol=RTOL_HALF * sigma)


def test_mid_sized_linear_inside_a_hip_graph():
    """A split-K GEMM recorded into a HIP graph after a warm-up call on the capture stream (which allocates that
    stream's scratch buffer) replays to the eager result every time, with eager work in between."""
    M, N, K = 64, 512, 4096
    x, w = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV)
    eager = _native.linear(x, w)
    torch.cuda.synchronize()
    out = torch.empty_like(eager)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        assert torch.equal(_native.linear(x, w), eager)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out.copy_(_native.linear(x, w))
    for i in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        assert torch.equal(_native.linear(x, w), eager)  # eager work between replays


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", [(300, 520, 128), (513, 260, 192), (700, 1028, 320), (256, 256, 64), (1030, 772, 1088)])
@pytest.mark.parametrize("waves", [4, 8])
def test_256_tiles_on_ragged_shapes(dtype, M, N, K, waves, tune):
    """The 256 x 256 tiling (forced through the library's debugging knobs; by default it is taken when a cost model
    predicts it to be faster) with 4 and with 8 wavefronts per block: two-tile K (the pipeline's minimum), tile rows past M, tile
    columns past N, bias and GELU, the gated pair, and a strided x. K = 64 is always served by the 8-wavefront
    kernel. Blocks that walk through several tiles are covered by the next test and by the full-shape tests."""
    tune("TPAMD_GEMM_TILE", "256")
    tune("TPAMD_GEMM_W4", "1" if waves == 4 else "0")
    x, w, b = rnd((M, K), 1, 1.0, dtype), rnd((N, K), 0, 0.02, dtype), rnd((N,), 2, 0.1, dtype)
    got = _native.linear(x.to(DEV), w.to(DEV), b.to(DEV), act=_native.ACT_GELU)
    check_half(got, F.gelu(F.linear(x.float(), w.float(), b.float())), K)
    w2 = rnd((N, K), 5, 0.02, dtype)
    h = _native.swiglu_up(x.to(DEV), w.to(DEV), w2.to(DEV))
    sigma = (0.02 * math.sqrt(K)) ** 2
    torch.testing.assert_close(h.float().cpu(), ofw.gated_mlp_hidden(x.float(), w.float(), w2.float()), rtol=RTOL_HALF, atol=RTOL_HALF * sigma)
    wide = rnd((M, 2 * K), 3, 1.0, dtype).to(DEV)
    strided = wide[:, K:]  # row pitch 2K: what a row-parallel shard sees of an unsplit activation
    got = _native.linear(strided, w.to(DEV))
    check_half(got, F.linear(strided.float().cpu(), w.float()), K)


def test_both_256_tile_kernels_agree_bit_for_bit(tune):
    """Same products added in the same order: the 4- and the 8-wavefront kernel must give identical results, also
    when a block walks through several tiles (3 x 96 = 288 tiles on at most 256 blocks)."""
    M, N, K = 700, 24500, 256
    x, w = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV)
    tune("TPAMD_GEMM_TILE", "256")
    tune("TPAMD_GEMM_W4", "1")
    four = _native.linear(x, w)
    tune("TPAMD_GEMM_W4", "0")
    eight = _native.linear(x, w)
    assert torch.equal(four, eight)
    check_half(four[:, :512], F.linear(x.float().cpu(), w[:512].float().cpu()), K)
    check_half(four[:, -512:], F.linear(x.float().cpu(), w[-512:].float().cpu()), K)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K,splits", [(300, 520, 256, 2), (513, 260, 320, 2), (700, 1028, 448, 3), (256, 256, 576, 4), (1030, 772, 1088, 8), (130, 8, 704, 5)])
def test_256_tiles_split_over_k(dtype, M, N, K, splits, tune):
    """The 4-wavefront 256 x 256 kernel with K split over several blocks per tile (forced; by default the cost model
    decides): splits of unequal length, the shortest allowed (2 K tiles), a last split that would be a single K tile
    (K = 448 = 7 tiles in 3 splits: the library lengthens the splits instead), an odd number of 128 x 128 partial
    tiles along M and N, bias and GELU applied by the finishing pass, and the gated pair."""
    tune("TPAMD_GEMM_TILE", "256")
    tune("TPAMD_GEMM_SPLITK256", str(splits))
    x, w, b = rnd((M, K), 1, 1.0, dtype), rnd((N, K), 0, 0.02, dtype), rnd((N,), 2, 0.1, dtype)
    got = _native.linear(x.to(DEV), w.to(DEV), b.to(DEV), act=_native.ACT_GELU)
    check_half(got, F.gelu(F.linear(x.float(), w.float(), b.float())), K)
    w2 = rnd((N, K), 5, 0.02, dtype)
    h = _native.swiglu_up(x.to(DEV), w.to(DEV), w2.to(DEV))
    sigma = (0.02 * math.sqrt(K)) ** 2
    torch.testing.assert_close(h.float().cpu(), ofw.gated_mlp_hidden(x.float(), w.float(), w2.float()), rtol=RTOL_HALF, atol=RTOL_HALF * sigma)
    # the unsplit launch adds the same products in another order
    tune("TPAMD_GEMM_SPLITK256", "1")
    unsplit = _native.linear(x.to(DEV), w.to(DEV), b.to(DEV), act=_native.ACT_GELU)
    torch.testing.assert_close(got.float(), unsplit.float(), rtol=RTOL_HALF, atol=RTOL_HALF * 0.02 * math.sqrt(K))


def test_mid_sized_shapes_choose_a_correct_path():
    """Shapes on which the dispatch takes the 256 x 256 tiling with K split (few tiles, long K) and without."""
    for M, N, K in [(1024, 4608, 8192), (768, 8192, 8192), (1024, 5504, 4096)]:
        x, w = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV)
        got = _native.linear(x, w)
        check_half(got[:, :256], F.linear(x.float().cpu(), w[:256].float().cpu()), K)
        check_half(got[-300:, -300:], F.linear(x[-300:].float().cpu(), w[-300:].float().cpu()), K)


@pytest.mark.parametrize("tile", ["128", "256"])
@pytest.mark.parametrize("N,ldy,shift", [(260, 264, 0), (260, 264, 4), (256, 260, 0), (520, 528, 8), (132, 136, 4)])
def test_strided_and_8_byte_aligned_outputs_through_the_c_abi(tile, N, ldy, shift, tune):
    """y with a row pitch above N and a base that is 8- but not 16-byte aligned (shift = 4 elements): the epilogues
    choose between 16- and 8-byte stores by the alignment of y and its pitch, and a row's last 4 columns (N % 8 == 4)
    are always an 8-byte store. The columns between N and the pitch must stay untouched."""
    import ctypes

    tune("TPAMD_GEMM_TILE", tile)
    M, K = 300, 256
    x, w, b = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV), rnd((N,), 2, 0.1).to(DEV)
    w2 = rnd((N, K), 5, 0.02).to(DEV)
    buf = torch.full((M * ldy + 16,), 7.0, dtype=torch.bfloat16, device=DEV)
    y = buf[shift: shift + M * ldy].view(M, ldy)
    stream = ctypes.c_void_p(torch.cuda.current_stream(DEV).cuda_stream)
    rc = _native.lib().tpamd_linear(x.data_ptr(), w.data_ptr(), b.data_ptr(), y.data_ptr(), M, N, K, K, K, ldy,
                                    _native.dtype_code(torch.bfloat16), _native.ACT_NONE, stream)
    assert rc == 0
    check_half(y[:, :N], F.linear(x.float().cpu(), w.float().cpu(), b.float().cpu()), K)
    assert bool((y[:, N:] == 7.0).all()) and bool((buf[:shift] == 7.0).all()) and bool((buf[shift + M * ldy:] == 7.0).all())
    buf.fill_(7.0)
    rc = _native.lib().tpamd_swiglu_up(x.data_ptr(), w.data_ptr(), w2.data_ptr(), y.data_ptr(), M, N, K, K, K, ldy,
                                       _native.dtype_code(torch.bfloat16), stream)
    assert rc == 0
    sigma = (0.02 * math.sqrt(K)) ** 2
    want = ofw.gated_mlp_hidden(x.float().cpu(), w.float().cpu(), w2.float().cpu())
    torch.testing.assert_close(y[:, :N].float().cpu(), want, rtol=RTOL_HALF, atol=RTOL_HALF * sigma)
    assert bool((y[:, N:] == 7.0).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [4, 9, 16])
@pytest.mark.parametrize("N,K", [(64, 64), (132, 200), (1028, 1000), (2740, 4096), (520, 5504), (300, 8192), (260, 7000)])
def test_x_resident_weight_streaming_kernel(dtype, M, N, K, tune):
    """The weight-streaming kernel that keeps its x fragments in registers and walks a range of columns per block
    (forced; by default it serves 9 to 16 rows when there are enough weight tiles per CU): fewer tiles than CUs,
    several tiles per block with a masked last tile (2740 columns over 256 blocks), column ranges that do not start
    on a multiple of 8, a ragged last K chunk, K above 4096 and above 6144 (6 and 8 chunks per wavefront), bias and
    GELU, the gated pair."""
    tune("TPAMD_SKINNY_RESIDENT", "1")
    tune("TPAMD_SKINNY_XLDS", "0")  # the gated pair would otherwise go to the kernel that stages x in LDS
    x, w, b = rnd((M, K), 1, 1.0, dtype), rnd((N, K), 0, 0.02, dtype), rnd((N,), 2, 0.1, dtype)
    got = _native.linear(x.to(DEV), w.to(DEV), b.to(DEV), act=_native.ACT_GELU)
    check_half(got, F.gelu(F.linear(x.float(), w.float(), b.float())), K)
    w2 = rnd((N, K), 5, 0.02, dtype)
    h = _native.swiglu_up(x.to(DEV), w.to(DEV), w2.to(DEV))
    sigma = (0.02 * math.sqrt(K)) ** 2
    torch.testing.assert_close(h.float().cpu(), ofw.gated_mlp_hidden(x.float(), w.float(), w2.float()), rtol=RTOL_HALF, atol=RTOL_HALF * sigma)
    tune("TPAMD_SKINNY_RESIDENT", "0")
    plain = _native.swiglu_up(x.to(DEV), w.to(DEV), w2.to(DEV))
    torch.testing.assert_close(h.float(), plain.float(), rtol=RTOL_HALF, atol=RTOL_HALF * sigma)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [17, 31, 32, 33, 48, 64])
@pytest.mark.parametrize("N,K", [(2048, 4096), (4096, 5504), (1000, 2056), (132, 8192), (3072, 3072)])
def test_single_matrix_with_few_tiles_at_17_to_64_rows(dtype, M, N, K):
    """A single 16-bit matrix with at most one 16-column tile per CU stays on the weight-streaming kernel up to 32 rows
    (up to 64 with rows of at most 3072 elements; not at all with long rows on few tiles, which the tiled kernels split
    over K): two and four row tiles of x, a partly filled last one, a ragged last K chunk, bias and GELU."""
    x, w, b = rnd((M, K), 1, 1.0, dtype), rnd((N, K), 0, 0.02, dtype), rnd((N,), 2, 0.1, dtype)
    got = _native.linear(x.to(DEV), w.to(DEV), b.to(DEV), act=_native.ACT_GELU)
    check_half(got, F.gelu(F.linear(x.float(), w.float(), b.float())), K)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [17, 20, 32, 33, 50, 64])
@pytest.mark.parametrize("N,K", [(4608, 4096), (5504, 4096), (4100, 2048)])
def test_k_split_tiles_with_part_of_the_x_tile(tune, dtype, M, N, K):
    """17 to 64 rows of a single matrix with more than one 16-column tile per CU go to the K-split 128 x 128 kernel, which
    then loads only the quarter or half of the x tile that exists and lets the two wavefronts of the missing rows only
    load: against the fp32 host product, and bit for bit what the kernel with whole tiles gives (bias, GELU and the
    fused addend included; a ragged last column tile)."""
    x, w, b = rnd((M, K), 1, 1.0, dtype).to(DEV), rnd((N, K), 0, 0.02, dtype).to(DEV), rnd((N,), 2, 0.1, dtype).to(DEV)
    other = rnd((M, N), 7, 1.0, dtype).to(DEV)
    part = _native.linear(x, w, b, act=_native.ACT_GELU)
    part_sum = _native.linear(x, w, None, addend=other)
    check_half(part, F.gelu(F.linear(x.float().cpu(), w.float().cpu(), b.float().cpu())), K)
    tune("TPAMD_GEMM_PART_X", "0")
    assert torch.equal(_native.linear(x, w, b, act=_native.ACT_GELU), part)
    assert torch.equal(_native.linear(x, w, None, addend=other), part_sum)


@pytest.mark.parametrize("M", [24, 128, 300])
@pytest.mark.parametrize("N,K", [(2048, 4096), (4096, 5504), (1028, 1088)])
def test_k_split_tiles_with_two_and_four_lds_stages(tune, M, N, K):
    """The K-split 128 x 128 kernel keeps four K tiles in LDS where every block has a CU to itself, two otherwise: the same
    bits either way, for the single matrix (with its part tiles of x at few rows) and for the gated pair, also with the
    four stages forced on a launch that has more blocks than CUs."""
    x, w, w2 = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV), rnd((N, K), 5, 0.02).to(DEV)
    tune("TPAMD_SKINNY_MAX_M", "16")
    lin, pair = _native.linear(x, w), _native.swiglu_up(x, w, w2)
    check_half(lin, F.linear(x.float().cpu(), w.float().cpu()), K)
    for stages in ("2", "4"):
        tune("TPAMD_GEMM_STAGES", stages)
        assert torch.equal(_native.linear(x, w), lin) and torch.equal(_native.swiglu_up(x, w, w2), pair)
    tune("TPAMD_GEMM_SPLITK", "8")  # 8 splits: more blocks than CUs on the larger shapes, still four stages
    tune("TPAMD_GEMM_TILE", "128")
    forced = _native.linear(x, w)
    tune("TPAMD_GEMM_STAGES", "2")
    assert torch.equal(_native.linear(x, w), forced)
    check_half(forced, F.linear(x.float().cpu(), w.float().cpu()), K)


def test_rows_limit_of_the_weight_streaming_kernels_can_be_forced(tune):
    """TPAMD_SKINNY_MAX_M = 64 sends 17 to 64 rows of any single 16-bit matrix to the weight-streaming kernel, 16 sends
    them to the tiled kernels: same result within rounding."""
    M, N, K = 40, 4608, 4096
    x, w = rnd((M, K), 1), rnd((N, K), 0, 0.02)
    tune("TPAMD_SKINNY_MAX_M", "64")
    streamed = _native.linear(x.to(DEV), w.to(DEV))
    tune("TPAMD_SKINNY_MAX_M", "16")
    tiled = _native.linear(x.to(DEV), w.to(DEV))
    check_half(streamed, F.linear(x.float(), w.float()), K)
    check_half(tiled, F.linear(x.float(), w.float()), K)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [4, 7, 12, 16])
@pytest.mark.parametrize("N,K", [(8, 64), (64, 64), (133, 200), (1028, 1000), (2740, 4096), (520, 5504), (4100, 2048), (300, 8192), (260, 7000),
                                 (16400, 512)])
def test_gated_pair_with_x_staged_in_lds(dtype, M, N, K, tune):
    """The gated-pair kernel for 4 to 16 rows that stages x in LDS chunk by chunk (forced on every shape): one tile, fewer
    tiles than CUs, several tiles per block, column counts that are not multiples of 8, K that is not a multiple of the
    64-element unit, one partly filled chunk of K, several chunks with a ragged last one, 8 tiles per CU (16400 columns:
    2050 tiles on 256 CUs), and x with a row pitch above K. Against the oracle's gated hidden state and against the older
    kernels."""
    tune("TPAMD_SKINNY_XLDS", "1")
    x_wide = rnd((M, K + 24), 1, 1.0, dtype).to(DEV)
    x = x_wide[:, 8:K + 8]
    w, w2 = rnd((N, K), 0, 0.02, dtype), rnd((N, K), 5, 0.02, dtype)
    h = _native.swiglu_up(x, w.to(DEV), w2.to(DEV))
    sigma = (0.02 * math.sqrt(K)) ** 2
    torch.testing.assert_close(h.float().cpu(), ofw.gated_mlp_hidden(x.float().cpu(), w.float(), w2.float()), rtol=RTOL_HALF, atol=RTOL_HALF * sigma)
    tune("TPAMD_SKINNY_XLDS", "0")
    older = _native.swiglu_up(x, w.to(DEV), w2.to(DEV))
    torch.testing.assert_close(h.float(), older.float(), rtol=RTOL_HALF, atol=RTOL_HALF * sigma)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [17, 24, 31, 32])
@pytest.mark.parametrize("N,K", [(1376, 4096), (2048, 2048), (1000, 2056), (132, 5504)])
def test_gated_pair_with_few_tiles_at_17_to_32_rows(dtype, M, N, K, tune):
    """A gated pair with at most one 8-column tile per CU stays on the weight-streaming kernel up to 32 rows (two row
    tiles of x, the second partly filled; a ragged last K chunk; a column count that is not a multiple of 8): against
    the oracle's gated hidden state, and against the tiled kernels that take these rows on wider matrices."""
    x, w, w2 = rnd((M, K), 1, 1.0, dtype).to(DEV), rnd((N, K), 0, 0.02, dtype).to(DEV), rnd((N, K), 5, 0.02, dtype).to(DEV)
    h = _native.swiglu_up(x, w, w2)
    sigma = (0.02 * math.sqrt(K)) ** 2
    torch.testing.assert_close(h.float().cpu(), ofw.gated_mlp_hidden(x.float().cpu(), w.float().cpu(), w2.float().cpu()), rtol=RTOL_HALF, atol=RTOL_HALF * sigma)
    tune("TPAMD_SKINNY_MAX_M", "16")
    tiled = _native.swiglu_up(x, w, w2)
    torch.testing.assert_close(h.float(), tiled.float(), rtol=RTOL_HALF, atol=RTOL_HALF * sigma)


def test_gated_pair_with_x_staged_in_lds_leaves_rows_past_m_and_columns_past_n_alone(tune):
    tune("TPAMD_SKINNY_XLDS", "1")
    M, N, K, ldy = 5, 1001, 4096, 1016
    x, w, w2 = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV), rnd((N, K), 5, 0.02).to(DEV)
    buf = torch.full((8 * ldy,), 7.0, dtype=torch.bfloat16, device=DEV)
    y = buf[ldy:ldy + M * ldy].view(M, ldy)
    rc = _native.lib().tpamd_swiglu_up(x.data_ptr(), w.data_ptr(), w2.data_ptr(), y.data_ptr(), M, N, K, K, K, ldy, _native.dtype_code(torch.bfloat16),
                                       ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    sigma = (0.02 * math.sqrt(K)) ** 2
    torch.testing.assert_close(y[:, :N].float().cpu(), ofw.gated_mlp_hidden(x.float().cpu(), w.float().cpu(), w2.float().cpu()), rtol=RTOL_HALF, atol=RTOL_HALF * sigma)
    assert bool((y[:, N:] == 7.0).all()) and bool((buf[:ldy] == 7.0).all()) and bool((buf[ldy + M * ldy:] == 7.0).all())


@pytest.mark.parametrize("case", ["tiles256_split", "resident_pair", "resident_single", "xlds_pair"])
def test_other_dispatch_paths_inside_a_hip_graph(case, tune):
    """The 256 x 256 tiling with K split over blocks (two launches sharing the scratch buffer) and the x-resident
    weight-streaming kernel, recorded into a HIP graph after a warm-up call: every replay gives the eager result,
    with eager work in between."""
    if case == "tiles256_split":
        tune("TPAMD_GEMM_TILE", "256")
        tune("TPAMD_GEMM_SPLITK256", "3")
        M, N, K = 300, 520, 1088
    elif case == "xlds_pair":
        tune("TPAMD_SKINNY_XLDS", "1")
        M, N, K = 13, 2740, 5504
    else:
        tune("TPAMD_SKINNY_RESIDENT", "1")
        tune("TPAMD_SKINNY_XLDS", "0")
        M, N, K = 16, 2740, 4096
    x, w, w2 = rnd((M, K), 1).to(DEV), rnd((N, K), 0, 0.02).to(DEV), rnd((N, K), 5, 0.02).to(DEV)
    fn = (lambda: _native.swiglu_up(x, w, w2)) if case in ("resident_pair", "xlds_pair") else (lambda: _native.linear(x, w))
    eager = fn()
    torch.cuda.synchronize()
    out = torch.empty_like(eager)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on the capture stream: a stream's scratch buffer is allocated at its first use
        assert torch.equal(fn(), eager)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out.copy_(fn())
    for i in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        assert torch.equal(fn(), eager)  # eager work between replays


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [1, 2, 3])
@pytest.mark.parametrize("N,K", [(2048, 512), (2053, 520), (4100, 5504), (6000, 1032), (3000, 8192), (4096, 4096), (8192, 6656), (8200, 4096), (4608, 8192), (1376, 6144)])
def test_row_streaming_kernel_on_wide_matrices(dtype, M, N, K):
    """M <= 3 and thousands of output columns (ragged column count, ragged last K step): against the fp32 host
    product, the gated pair against the oracle, the fused sum bit for bit. The shapes reach every choice of the rule
    for these row counts: blocks of 4, 8 and 16 wavefronts, the general row kernel, the MFMA kernels at 2 rows."""
    x, w, w2, b = rnd((M, K), 1, 1.0, dtype).to(DEV), rnd((N, K), 0, 0.02, dtype).to(DEV), rnd((N, K), 5, 0.02, dtype).to(DEV), rnd((N,), 2, 0.1, dtype).to(DEV)
    lin = _native.linear(x, w, b)
    check_half(lin, F.linear(x.float().cpu(), w.float().cpu(), b.float().cpu()), K)
    sw = _native.swiglu_up(x, w, w2)
    sigma = (0.02 * math.sqrt(K)) ** 2
    torch.testing.assert_close(sw.float().cpu(), ofw.gated_mlp_hidden(x.float().cpu(), w.float().cpu(), w2.float().cpu()), rtol=RTOL_HALF, atol=RTOL_HALF * sigma)
    other = rnd((M, N), 7, 1.0, dtype).to(DEV)
    assert torch.equal(_native.linear(x, w, b, addend=other).cpu(), lin.cpu() + other.cpu())
