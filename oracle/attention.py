"""Rank-local attention core on the CPU, float64: softmax(scale * q k^T + causal mask) v with grouped-query heads.

TEST INFRASTRUCTURE ONLY (see the package docstring).

The reference has no attention code of its own: a rank runs the wrapped transformers module on its share of the
heads (src/tensor_parallel/wrapper.py:69-72; head counts divided by the attr rules of
src/tensor_parallel/slicing_configs.py:382-389 and :414-433). What this function restates is therefore the
textbook operation those modules perform, in the layout they use: q [B, Hq, Sq, D], k / v [B, Hkv, Skv, D],
result [B, Sq, Hq, D]. Query head h reads key/value head h // (Hq // Hkv). With `causal`, the Sq queries are the
LAST Sq positions of the Skv keys: query i sees keys j <= i + Skv - Sq.

Pinned (tests/test_oracle_attention.py) by torch.nn.functional.scaled_dot_product_attention on the CPU (a library
routine) for the cases it covers (equal head counts or repeated heads, Sq == Skv causal, non-causal), by a
triple-loop evaluation on tiny inputs for the grouped and the Sq < Skv causal cases, and by two invariants:
rows of the probabilities sum to one (v = ones gives ones) and a single visible key returns that key's value.
"""
import numpy as np


def attention_f64(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, causal: bool) -> np.ndarray:
    q, k, v = (np.asarray(t, dtype=np.float64) for t in (q, k, v))
    B, Hq, Sq, D = q.shape
    _, Hkv, Skv, _ = k.shape
    assert Hq % Hkv == 0 and v.shape == k.shape and k.shape[0] == B and k.shape[3] == D
    group = Hq // Hkv
    out = np.empty((B, Sq, Hq, D), dtype=np.float64)
    visible = None
    if causal:
        i = np.arange(Sq)[:, None]
        j = np.arange(Skv)[None, :]
        visible = j <= i + (Skv - Sq)
    for b in range(B):
        for h in range(Hq):
            kv = h // group
            s = (q[b, h] @ k[b, kv].T) * scale
            if visible is not None:
                s = np.where(visible, s, -np.inf)
            s = s - s.max(axis=1, keepdims=True)
            p = np.exp(s)
            p /= p.sum(axis=1, keepdims=True)
            out[b, :, h, :] = p @ v[b, kv]
    return out


def attention_loops(q, k, v, scale: float, causal: bool):
    """The same by explicit loops over every (batch, head, query, key): for tiny inputs only."""
    import math

    B, Hq, Sq, D = len(q), len(q[0]), len(q[0][0]), len(q[0][0][0])
    Hkv, Skv = len(k[0]), len(k[0][0])
    group = Hq // Hkv
    out = [[[[0.0] * D for _ in range(Hq)] for _ in range(Sq)] for _ in range(B)]
    for b in range(B):
        for h in range(Hq):
            kv = h // group
            for i in range(Sq):
                scores = []
                for j in range(Skv):
                    if causal and j > i + (Skv - Sq):
                        continue
                    scores.append((j, scale * sum(q[b][h][i][d] * k[b][kv][j][d] for d in range(D))))
                top = max(s for _, s in scores)
                weights = [(j, math.exp(s - top)) for j, s in scores]
                total = sum(w for _, w in weights)
                for d in range(D):
                    out[b][i][h][d] = sum(w * v[b][kv][j][d] for j, w in weights) / total
    return out
