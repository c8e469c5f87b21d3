"""Pins oracle/rope.py: transformers' apply_rotary_pos_emb bit for bit, the complex-rotation closed form in float64,
norm preservation, and the identity at position 0."""
import pytest
import torch

from oracle import rope as orp


def inputs(B, S, Hq, Hkv, D, dtype, seed=0, pos0=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, S, Hq, D, generator=g).to(dtype)
    k = torch.randn(B, S, Hkv, D, generator=g).to(dtype)
    v = torch.randn(B, S, Hkv, D, generator=g).to(dtype)
    cos, sin = orp.angles(torch.arange(pos0, pos0 + S), D, dtype=dtype)
    return q, k, v, cos[None], sin[None]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("B,S,Hq,Hkv,D,pos0", [(1, 5, 2, 1, 8, 0), (2, 3, 4, 2, 64, 7), (1, 1, 16, 1, 128, 2047)])
def test_rotation_equals_the_library_routine_bit_for_bit(dtype, B, S, Hq, Hkv, D, pos0):
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb

    q, k, v, cos, sin = inputs(B, S, Hq, Hkv, D, dtype, seed=S, pos0=pos0)
    want_q, want_k = apply_rotary_pos_emb(q.transpose(1, 2), k.transpose(1, 2), cos, sin)  # [B, H, S, D] layout
    L = pos0 + S + 3
    kc = torch.full((B, Hkv, L, D), 5.0, dtype=dtype)
    vc = torch.full((B, Hkv, L, D), 6.0, dtype=dtype)
    got_q, got_kc, got_vc = orp.rope_append(q, k, v, cos, sin, kc, vc, pos0)
    assert torch.equal(got_q, want_q)
    assert torch.equal(got_kc[:, :, pos0:pos0 + S], want_k)
    assert torch.equal(got_vc[:, :, pos0:pos0 + S], v.transpose(1, 2))
    # every other position of the caches is untouched
    assert bool((got_kc[:, :, :pos0] == 5.0).all()) and bool((got_kc[:, :, pos0 + S:] == 5.0).all())
    assert bool((got_vc[:, :, :pos0] == 6.0).all()) and bool((got_vc[:, :, pos0 + S:] == 6.0).all())


def test_closed_form_complex_rotation():
    """(x[j] + i x[j + D/2]) * exp(i pos theta_j): a dropped sign or swapped halves fails this."""
    B, S, H, D, pos0 = 1, 6, 3, 16, 11
    g = torch.Generator().manual_seed(1)
    x = torch.randn(B, S, H, D, generator=g, dtype=torch.float64)
    cos, sin = orp.angles(torch.arange(pos0, pos0 + S), D, dtype=torch.float64)
    got = orp.rotate(x, cos[None, :, None, :], sin[None, :, None, :])
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float64) / D))
    theta = torch.arange(pos0, pos0 + S, dtype=torch.float64)[:, None] * inv[None, :]
    z = torch.complex(x[..., : D // 2], x[..., D // 2:]) * torch.polar(torch.ones_like(theta), theta)[None, :, None, :]
    want = torch.cat((z.real, z.imag), dim=-1)
    torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-12)


def test_invariants():
    q, k, v, cos, sin = inputs(2, 9, 4, 2, 32, torch.float32, seed=3, pos0=100)
    rot = orp.rotate(q, cos.unsqueeze(2), sin.unsqueeze(2))
    half = 16
    before = q[..., :half] ** 2 + q[..., half:] ** 2
    after = rot[..., :half] ** 2 + rot[..., half:] ** 2
    torch.testing.assert_close(after, before, rtol=1e-5, atol=1e-6)
    q0, _, _, cos0, sin0 = inputs(1, 1, 2, 1, 32, torch.bfloat16, seed=4, pos0=0)
    assert torch.equal(orp.rotate(q0, cos0.unsqueeze(2), sin0.unsqueeze(2)), q0)
