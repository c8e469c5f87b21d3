"""Seeded random shapes through the default dispatch of the shard Linears (1 to 70 rows, and mid-sized problems up to 1500
rows, where the choice of kernel depends on M, N and K) against fp32 torch on the host: catches a kernel that is chosen for
a shape it mishandles."""
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


@pytest.mark.parametrize("seed", range(300, 324))
def test_mid_sized_random_shape_on_sampled_columns(seed):
    """17 to 1500 rows of matrices with thousands of columns and long rows: where the tiling (128 x 128 or 256 x 256), the
    K split, the number of LDS stages and the part of the x tile that is loaded are chosen by cost models. The single
    matrix (bias, and the fused addend on odd seeds) and the gated pair, on 96 sampled output columns against fp32 on the
    host (whole matrices of this size would take the host minutes)."""
    g = torch.Generator().manual_seed(seed)
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))  # noqa: E731
    M = [pick(17, 64), pick(65, 300), pick(301, 1500)][pick(0, 2)]
    N = 64 * pick(16, 224)
    K = 64 * pick(32, 128)
    dtype = [torch.bfloat16, torch.float16][pick(0, 1)]
    x = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.02).to(dtype)
    w2 = (torch.randn(N, K, generator=g) * 0.02).to(dtype)
    b = (torch.randn(N, generator=g) * 0.1).to(dtype)
    other = torch.randn(M, N, generator=g).to(dtype) if seed % 2 else None
    cols = torch.randperm(N, generator=g)[:96]
    xd, wd, w2d = x.to(DEV), w.to(DEV), w2.to(DEV)
    got = _native.linear(xd, wd, b.to(DEV), addend=None if other is None else other.to(DEV)).float().cpu()[:, cols]
    want = F.linear(x.float(), w[cols].float(), b[cols].float())
    if other is not None:
        want = want.to(dtype).float() + other[:, cols].float()  # the sum is rounded once more, as the fused epilogue does
    sigma = 0.02 * math.sqrt(K)
    torch.testing.assert_close(got, want, rtol=RTOL, atol=RTOL * max(sigma, 1.0 if other is not None else 0.0), msg=lambda m: f"linear M={M} N={N} K={K} {dtype}: {m}")
    pair = _native.swiglu_up(xd, wd, w2d).float().cpu()[:, cols]
    want = ofw.gated_mlp_hidden(x.float(), w[cols].float(), w2[cols].float())
    torch.testing.assert_close(pair, want, rtol=RTOL, atol=RTOL * sigma ** 2, msg=lambda m: f"pair M={M} N={N} K={K} {dtype}: {m}")


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


@pytest.mark.parametrize("seed", range(300, 330))
def test_fp32_linear_random_shape(seed):
    """fp32 operands, mostly with rows that 16-byte accesses can take (the matrix-pipe kernel in its three tilings), some
    without (the scalar kernel); bias, GELU and the addend of the folded partial sum in turn. rtol 1e-5."""
    g = torch.Generator().manual_seed(seed)
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))  # noqa: E731
    aligned = seed % 5 != 0
    M = pick(1, 700)
    K = 4 * pick(1, 400) if aligned else pick(1, 900)
    N = 4 * pick(1, 700) if aligned else pick(1, 900)
    if seed % 7 == 0:  # enough 128 x 128 tiles for the large tiling
        M, N = 128 * pick(9, 14), 128 * pick(20, 24) + 4 * pick(0, 8)
    x = torch.randn(M, K, generator=g)
    w = torch.randn(N, K, generator=g) * 0.02
    b = torch.randn(N, generator=g) * 0.1 if seed % 2 else None
    add = torch.randn(M, N, generator=g) if seed % 3 == 1 else None
    act = _native.ACT_GELU if seed % 3 == 0 else _native.ACT_NONE
    got = _native.linear(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV), act=act, addend=None if add is None else add.to(DEV))
    want = F.linear(x.double(), w.double(), None if b is None else b.double())
    if act == _native.ACT_GELU:
        want = F.gelu(want)
    if add is not None:
        want = want + add.double()
    torch.testing.assert_close(got.cpu(), want.float(), rtol=1e-5, atol=1e-5 * 0.02 * math.sqrt(K) + 1e-6,
                               msg=lambda m: f"M={M} N={N} K={K} aligned={aligned}: {m}")


@pytest.mark.parametrize("seed", range(400, 416))
def test_int8_linear_random_shape_at_prefill_sizes(seed):
    """More rows than the weight-streaming kernels take: the tiled kernel that converts the weights on their way into LDS
    (both tilings), and the slabs of 64 rows where the matrix has too few tiles."""
    import numpy as np

    from oracle import quant as oq

    g = torch.Generator().manual_seed(seed)
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))  # noqa: E731
    M = pick(129, 900)
    N, K = 4 * pick(8, 1100), 16 * pick(2, 260)
    if seed % 4 == 0:
        M, N = 256 * pick(4, 6) + pick(0, 40), 256 * pick(16, 20) + 4 * pick(0, 20)  # fills the 256 x 256 tiling
    n_out = [0, 7, 41, 130, 256][pick(0, 4)]
    n_out = min(n_out, K // 2)
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
    torch.testing.assert_close(got.double().cpu(), torch.from_numpy(want), rtol=RTOL, atol=RTOL * sigma,
                               msg=lambda m: f"M={M} N={N} K={K} n_out={n_out} {dtype}: {m}")


@pytest.mark.parametrize("seed", range(500, 520))
def test_rope_append_random_shape(seed):
    """Random batch, positions, head counts and cache offsets, q / k / v as strided views of one fused buffer: bit for bit
    against the oracle."""
    from oracle import rope as orp

    g = torch.Generator().manual_seed(seed)
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))  # noqa: E731
    B, S, Hkv, per = pick(1, 5), pick(1, 40), pick(1, 5), pick(1, 9)
    D = [64, 128][pick(0, 1)]
    dtype = [torch.bfloat16, torch.float16][pick(0, 1)]
    pos0 = pick(0, 50)
    L = pos0 + S + pick(0, 7)
    fused = torch.randn(B, S, Hkv, per + 2, D, generator=g).to(dtype)
    cos, sin = orp.angles(torch.arange(pos0, pos0 + S), D, dtype=dtype)
    kc = torch.randn(B, Hkv, L, D, generator=g).to(dtype)
    vc = torch.randn(B, Hkv, L, D, generator=g).to(dtype)
    want_q, want_kc, want_vc = orp.rope_append(fused[:, :, :, :per].reshape(B, S, Hkv * per, D), fused[:, :, :, per], fused[:, :, :, per + 1],
                                               cos[None], sin[None], kc, vc, pos0)
    fd, kcd, vcd = fused.to(DEV), kc.to(DEV), vc.to(DEV)
    got_q = _native.rope_append(fd[:, :, :, :per], fd[:, :, :, per], fd[:, :, :, per + 1], cos.to(DEV), sin.to(DEV), kcd, vcd, pos0)
    as_bits = lambda t: t.detach().cpu().contiguous().view(torch.int16)  # noqa: E731
    assert torch.equal(as_bits(got_q), as_bits(want_q)), f"B={B} S={S} Hkv={Hkv} per={per} D={D} pos0={pos0}"
    assert torch.equal(as_bits(kcd), as_bits(want_kc)) and torch.equal(as_bits(vcd), as_bits(want_vc))


@pytest.mark.parametrize("seed", range(600, 650))
def test_attention_random_shape(seed):
    """Random batch, head grouping, new positions, key counts (up to 5000: one block per range, split ranges, and ranges
    long enough for the kernel that keeps several tiles in flight), head_dim and mask through the default dispatch, q / k /
    v as strided views of wider buffers, against the float64 oracle."""
    from oracle import attention as oat

    g = torch.Generator().manual_seed(seed)
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))  # noqa: E731
    B, Hkv, G = pick(1, 4), pick(1, 4), [1, 2, 4, 8, 16][pick(0, 4)]
    D = [64, 128][pick(0, 1)]
    decode = pick(0, 2) > 0
    Sq = 1 if decode else pick(2, 150)
    Skv = pick(max(Sq, 1), 5000 if decode else 700)
    causal = bool(pick(0, 1))
    dtype = [torch.bfloat16, torch.float16][pick(0, 1)]
    Hq = Hkv * G
    pad = 8 * pick(0, 2)
    q_wide = torch.randn(B, Hq, Sq, D + pad, generator=g).to(dtype)
    k_wide = torch.randn(B, Hkv, Skv + pick(0, 5), D, generator=g).to(dtype)
    v_wide = torch.randn(B, Hkv, Skv, D + pad, generator=g).to(dtype)
    views = lambda qw, kw, vw: (qw[..., :D], kw[:, :, :Skv], vw[..., pad:])  # noqa: E731
    q, k, v = views(q_wide, k_wide, v_wide)
    scale = D ** -0.5 * [1.0, 0.5, 3.0][pick(0, 2)]
    got = _native.attention(*views(q_wide.to(DEV), k_wide.to(DEV), v_wide.to(DEV)), scale=scale, causal=causal)
    want = torch.from_numpy(oat.attention_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), scale, causal))
    torch.testing.assert_close(got.double().cpu(), want, rtol=RTOL, atol=RTOL * want.std().item(),
                               msg=lambda m: f"B={B} Hq={Hq} Hkv={Hkv} Sq={Sq} Skv={Skv} D={D} causal={causal} {dtype}: {m}")


@pytest.mark.parametrize("seed", range(700, 730))
def test_decode_with_folded_rotary_random_shape(seed):
    """One new position on caches of random length (0 to 3000 positions), random batch and head grouping: cache rows bit for
    bit against the oracle's rotary step, the output against its attention in float64."""
    from oracle import attention as oat
    from oracle import rope as orp

    g = torch.Generator().manual_seed(seed)
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))  # noqa: E731
    B, Hkv, per = pick(1, 6), pick(1, 4), [1, 2, 4, 8, 16][pick(0, 4)]
    D = [64, 128][pick(0, 1)]
    dtype = [torch.bfloat16, torch.float16][pick(0, 1)]
    pos0 = [0, 1, pick(2, 200), pick(200, 3000)][pick(0, 3)]
    L = pos0 + 1 + pick(0, 9)
    on_device = seed % 2 == 1  # every other case: the count read by the kernels, in caches with room for up to 1500 more positions
    if on_device:
        L = pos0 + 1 + pick(0, 1500)
    fused = torch.randn(B, 1, Hkv, per + 2, D, generator=g).to(dtype)
    kc = torch.randn(B, Hkv, L, D, generator=g).to(dtype)
    vc = torch.randn(B, Hkv, L, D, generator=g).to(dtype)
    cos, sin = orp.angles(torch.tensor([pos0]), D, dtype=dtype)
    q = fused[:, :, :, :per].reshape(B, 1, Hkv * per, D)
    q_rot, want_kc, want_vc = orp.rope_append(q, fused[:, :, :, per], fused[:, :, :, per + 1], cos[None], sin[None], kc.clone(), vc.clone(), pos0)
    scale = D ** -0.5
    want = torch.from_numpy(oat.attention_f64(q_rot.float().numpy(), want_kc[:, :, :pos0 + 1].float().numpy(),
                                              want_vc[:, :, :pos0 + 1].float().numpy(), scale, True))
    fd, kcd, vcd = fused.to(DEV), kc.to(DEV), vc.to(DEV)
    pos = torch.tensor([pos0], dtype=torch.int64, device=DEV) if on_device else pos0
    got = _native.attention_decode_rope(fd[:, :, :, :per], fd[:, :, :, per], fd[:, :, :, per + 1], cos.to(DEV), sin.to(DEV), kcd, vcd, pos)
    as_bits = lambda t: t.detach().cpu().contiguous().view(torch.int16)  # noqa: E731
    tag = f"B={B} Hkv={Hkv} per={per} D={D} pos0={pos0} L={L} count on the device={on_device} {dtype}"
    assert torch.equal(as_bits(kcd), as_bits(want_kc)) and torch.equal(as_bits(vcd), as_bits(want_vc)), tag
    torch.testing.assert_close(got.double().cpu(), want, rtol=RTOL, atol=RTOL * want.std().item(), msg=lambda m: f"{tag}: {m}")
