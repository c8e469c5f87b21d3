"""Rotary position embedding of new query / key rows and their hand-over to a rank-local key/value cache, on the CPU.

TEST INFRASTRUCTURE ONLY (see the package docstring).

The reference has no rotary or cache-append code of its own: every rank runs the wrapped transformers attention module
on its share of the heads (src/tensor_parallel/wrapper.py:69-72; Falcon-40B shard: fused query_key_value split by
src/tensor_parallel/slicing_configs.py:430-432, head counts by :455-461), and only routes the cache tensors that module
returns (select_kv_for_rank / gather_kv, src/tensor_parallel/aux_actions.py:7-15). What is restated here is therefore
the operation that module performs, in its arithmetic: element j < D/2 of a row pairs with element j + D/2,

    out[j]       = r(r(x[j] * cos[j])             + r(-x[j + D/2] * sin[j]))
    out[j + D/2] = r(r(x[j + D/2] * cos[j + D/2]) + r( x[j]       * sin[j + D/2]))

with r = rounding to the tensor dtype after each of the three torch operations, then the rotated keys and the values
are written at positions pos0 .. pos0 + S - 1 of the cache.

Pinned (tests/test_oracle_rope.py) by transformers' apply_rotary_pos_emb (a library routine) bit for bit in bfloat16,
float16 and float32, by the closed form (x[j] + i x[j + D/2]) * exp(i theta_j) in float64, by the invariant that a
rotation keeps the norm of every pair, and by position 0 (cos = 1, sin = 0) returning its input.
"""
import torch


def rotate(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [..., S, H, D], cos / sin broadcastable to [..., S, 1, D]; every operation in x's dtype."""
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    c1, c2 = cos[..., :half], cos[..., half:]
    s1, s2 = sin[..., :half], sin[..., half:]
    first = (x1 * c1) + ((-x2) * s1)
    second = (x2 * c2) + (x1 * s2)
    return torch.cat((first, second), dim=-1)


def rope_append(q, k, v, cos, sin, k_cache, v_cache, pos0: int):
    """q [B, S, Hq, D], k / v [B, S, Hkv, D], cos / sin [B or 1, S, D], caches [B, Hkv, L, D] (updated copies are
    returned). Returns (rotated q as [B, Hq, S, D], new key cache, new value cache)."""
    S = q.shape[1]
    c, s = cos.unsqueeze(2), sin.unsqueeze(2)
    q_rot = rotate(q, c, s).transpose(1, 2).contiguous()
    k_cache, v_cache = k_cache.clone(), v_cache.clone()
    k_cache[:, :, pos0:pos0 + S] = rotate(k, c, s).transpose(1, 2)
    v_cache[:, :, pos0:pos0 + S] = v.transpose(1, 2)
    return q_rot, k_cache, v_cache


def angles(positions: torch.Tensor, dim: int, base: float = 10000.0, dtype=torch.float32):
    """cos / sin tables [S, D] as rotary embeddings build them: theta_j = pos * base^(-2j / D), both halves alike."""
    inv = 1.0 / (base ** (torch.arange(0, dim, 2, dtype=torch.float64) / dim))
    freqs = positions.to(torch.float64)[:, None] * inv[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)
