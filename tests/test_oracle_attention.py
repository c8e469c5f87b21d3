"""Pins oracle/attention.py: against torch's CPU scaled_dot_product_attention where that routine covers the case,
against explicit loops where it does not, and against two invariants."""
import numpy as np
import pytest
import torch

from oracle import attention as oat


def rnd(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,H,S,D", [(1, 1, 5, 4), (2, 3, 17, 8), (1, 2, 64, 16)])
def test_matches_torch_sdpa_equal_heads(B, H, S, D, causal):
    q, k, v = rnd((B, H, S, D), 0), rnd((B, H, S, D), 1), rnd((B, H, S, D), 2)
    want = torch.nn.functional.scaled_dot_product_attention(torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v),
                                                            is_causal=causal, scale=0.3).transpose(1, 2).numpy()
    np.testing.assert_allclose(oat.attention_f64(q, k, v, 0.3, causal), want, rtol=1e-10, atol=1e-12)


def test_grouped_heads_equal_repeated_heads_through_torch():
    B, Hq, Hkv, Sq, Skv, D = 2, 6, 2, 7, 11, 8
    q, k, v = rnd((B, Hq, Sq, D), 0), rnd((B, Hkv, Skv, D), 1), rnd((B, Hkv, Skv, D), 2)
    kr, vr = np.repeat(k, Hq // Hkv, axis=1), np.repeat(v, Hq // Hkv, axis=1)  # head h -> h // group, as repeat_kv does
    want = torch.nn.functional.scaled_dot_product_attention(torch.from_numpy(q), torch.from_numpy(kr), torch.from_numpy(vr),
                                                            scale=0.5).transpose(1, 2).numpy()
    np.testing.assert_allclose(oat.attention_f64(q, k, v, 0.5, False), want, rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("Sq,Skv", [(1, 6), (3, 7), (5, 5)])
def test_causal_is_aligned_to_the_end_of_the_keys(Sq, Skv):
    """Explicit loops, and torch with an explicit boolean mask (its is_causal flag aligns to the start instead)."""
    B, Hq, Hkv, D = 1, 4, 2, 3
    q, k, v = rnd((B, Hq, Sq, D), 3), rnd((B, Hkv, Skv, D), 4), rnd((B, Hkv, Skv, D), 5)
    got = oat.attention_f64(q, k, v, 0.7, True)
    loops = np.array(oat.attention_loops(q.tolist(), k.tolist(), v.tolist(), 0.7, True))
    np.testing.assert_allclose(got, loops, rtol=1e-10, atol=1e-12)
    mask = torch.arange(Skv)[None, :] <= torch.arange(Sq)[:, None] + (Skv - Sq)
    kr, vr = np.repeat(k, 2, axis=1), np.repeat(v, 2, axis=1)
    want = torch.nn.functional.scaled_dot_product_attention(torch.from_numpy(q), torch.from_numpy(kr), torch.from_numpy(vr),
                                                            attn_mask=mask, scale=0.7).transpose(1, 2).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-12)


def test_invariants():
    B, Hq, Hkv, Sq, Skv, D = 1, 4, 1, 9, 9, 5
    q, k = rnd((B, Hq, Sq, D), 6), rnd((B, Hkv, Skv, D), 7)
    ones = np.ones((B, Hkv, Skv, D))
    np.testing.assert_allclose(oat.attention_f64(q, k, ones, 1.0, True), np.ones((B, Sq, Hq, D)), rtol=1e-12)
    v = rnd((B, Hkv, Skv, D), 8)
    first = oat.attention_f64(q, k, v, 1.0, True)[:, 0]  # position 0 sees key 0 only
    np.testing.assert_allclose(first, np.broadcast_to(v[:, 0, 0][:, None, :], first.shape), rtol=1e-12)
