"""tpamd_rope_append on the GPU against the oracle, bit for bit: rotated queries in the attention layout, rotated keys and
the values at their cache positions, every other cache position untouched."""
import pytest
import torch

from oracle import attention as oat
from oracle import rope as orp
from tensor_parallel_amd import _native

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def bits(t):
    return t.detach().cpu().contiguous().view(torch.int16)


def fused_qkv(B, S, Hq, Hkv, D, dtype, seed):
    """q / k / v as views of one fused projection output laid out [B, S, Hkv, Hq/Hkv + 2, D] (the Falcon-40B shard's
    query_key_value: per key/value head its query heads, then the key, then the value)."""
    g = torch.Generator().manual_seed(seed)
    per = Hq // Hkv
    fused = torch.randn(B, S, Hkv, per + 2, D, generator=g).to(dtype)
    return fused


def run_case(B, S, Hq, Hkv, D, dtype, pos0, L, shared_angles=True, seed=0, by_group=False):
    fused = fused_qkv(B, S, Hq, Hkv, D, dtype, seed)
    per = Hq // Hkv
    pos = torch.arange(pos0, pos0 + S)
    cos, sin = orp.angles(pos, D, dtype=dtype)
    if shared_angles:
        cos, sin = cos[None], sin[None]
    else:  # a different position offset per batch entry
        tables = [orp.angles(pos + 3 * b, D, dtype=dtype) for b in range(B)]
        cos, sin = torch.stack([t[0] for t in tables]), torch.stack([t[1] for t in tables])
    g = torch.Generator().manual_seed(seed + 1)
    kc = torch.randn(B, Hkv, L, D, generator=g).to(dtype)
    vc = torch.randn(B, Hkv, L, D, generator=g).to(dtype)
    # host: the oracle on contiguous copies of the three parts
    q_h = fused[:, :, :, :per].reshape(B, S, Hq, D)
    k_h, v_h = fused[:, :, :, per], fused[:, :, :, per + 1]
    want_q, want_kc, want_vc = orp.rope_append(q_h, k_h, v_h, cos, sin, kc, vc, pos0)
    # device: strided views of the fused tensor, no copies. The query heads of one key/value head are contiguous rows of
    # D and the groups are (per + 2) * D apart: a 5-d view [B, S, Hkv, per, D]; a plain 4-d view exists with one group
    # or one query head per group; `by_group` passes the groups one by one with q_out views instead
    fd = fused.to(DEV)
    kcd, vcd = kc.to(DEV), vc.to(DEV)
    cd, sd = cos.to(DEV), sin.to(DEV)
    if not by_group:
        qv = fd[:, :, :, :per]
        if Hkv == 1:
            qv = qv.reshape(B, S, Hq, D)
        elif per == 1:
            qv = fd[:, :, :, 0]
        got_q = _native.rope_append(qv, fd[:, :, :, per], fd[:, :, :, per + 1], cd, sd, kcd, vcd, pos0)
    else:
        got_q = torch.empty(B, Hq, S, D, dtype=dtype, device=DEV)
        for gi in range(Hkv):
            _native.rope_append(fd[:, :, gi, :per], fd[:, :, gi:gi + 1, per], fd[:, :, gi:gi + 1, per + 1], cd, sd,
                                kcd[:, gi:gi + 1], vcd[:, gi:gi + 1], pos0, q_out=got_q[:, gi * per:(gi + 1) * per])
    assert torch.equal(bits(got_q), bits(want_q))
    assert torch.equal(bits(kcd), bits(want_kc))
    assert torch.equal(bits(vcd), bits(want_vc))
    return got_q, kcd, vcd


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,S,Hq,Hkv,D,pos0,L", [
    (2, 1, 4, 4, 64, 5, 16),        # decode, equal heads
    (1, 7, 8, 1, 64, 0, 7),         # prefill filling the cache exactly, one key/value head
    (3, 5, 8, 2, 128, 9, 20),       # grouped heads as a 5-d view of the fused output, head_dim 128
    (2, 33, 2, 2, 128, 31, 64),     # more rows than one block of lanes
])
def test_rope_append_bit_exact(dtype, B, S, Hq, Hkv, D, pos0, L):
    run_case(B, S, Hq, Hkv, D, dtype, pos0, L)


def test_groups_one_by_one_into_views_of_the_output():
    run_case(2, 3, 12, 3, 64, torch.float16, 2, 8, seed=9, by_group=True)


def test_per_batch_angles():
    run_case(3, 2, 4, 4, 64, torch.bfloat16, 4, 12, shared_angles=False, seed=5)


def test_falcon_40b_rank_shard_decode_step_pieces():
    """BASELINE config 4 at W = 2, decode: batch 8, one new position on 2047 cached ones, 4 key/value heads with 16
    query heads each, head_dim 64. The cache after the append feeds the attention core; its output equals the oracle's
    attention over the oracle's cache."""
    B, S, Hq, Hkv, D, pos0, L = 8, 1, 64, 4, 64, 2047, 2048
    got_q, kcd, vcd = run_case(B, S, Hq, Hkv, D, torch.bfloat16, pos0, L, seed=7)
    out = _native.attention(got_q, kcd, vcd, causal=True)
    want = oat.attention_f64(got_q.float().cpu().numpy(), kcd.float().cpu().numpy(), vcd.float().cpu().numpy(), D ** -0.5, True)
    want = torch.from_numpy(want)
    torch.testing.assert_close(out.double().cpu(), want, rtol=2e-2, atol=2e-2 * want.std().item())


def test_argument_errors():
    B, S, Hq, Hkv, D = 1, 2, 2, 2, 64
    q = torch.zeros(B, S, Hq, D, dtype=torch.bfloat16, device=DEV)
    k = torch.zeros(B, S, Hkv, D, dtype=torch.bfloat16, device=DEV)
    cos = torch.zeros(1, S, D, dtype=torch.bfloat16, device=DEV)
    cache = torch.zeros(B, Hkv, 4, D, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):
        _native.rope_append(q, k, k, cos, cos, cache, cache.clone(), 3)  # positions 3, 4 of a cache of 4
    with pytest.raises(ValueError):
        _native.rope_append(q, k, k, cos[:, :1], cos[:, :1], cache, cache.clone(), 0)  # angles for one position only
    with pytest.raises(TypeError):
        _native.rope_append(q.float(), k.float(), k.float(), cos.float(), cos.float(), cache.float(), cache.float(), 0)
    q32 = torch.zeros(B, S, Hq, 32, dtype=torch.bfloat16, device=DEV)
    c32 = torch.zeros(1, S, 32, dtype=torch.bfloat16, device=DEV)
    cache32 = torch.zeros(B, Hkv, 4, 32, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError):
        _native.rope_append(q32, q32, q32, c32, c32, cache32, cache32.clone(), 0)  # head_dim 32: no kernel
