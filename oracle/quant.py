"""Closed-form definition of the int8 weight-only shard Linear with outlier columns kept in 16 bits.

NOT in the reference (its README only links to LLM.int8 notebooks; bitsandbytes is neither pinned nor
installed): PARITY UNPINNED against the reference. The definition:

  O        = the outlier input columns (sorted)
  scale[n] = max over k not in O of |W[n,k]| / 127          (1.0 where that max is 0)
  Wq[n,k]  = clamp(round_half_even(W[n,k] / scale[n]), -127, 127) for k not in O, 0 for k in O
  y        = x . (Wq * scale[:,None])^T  +  x[:, O] . W[:, O]^T
"""
from __future__ import annotations

from typing import Tuple

import numpy as np


def quantize_rows(w: np.ndarray, outlier_cols: np.ndarray) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """w: float32 [N,K]. Returns (wq int8 [N,K], scale float32 [N], w_out float32 [N, n_out])."""
    w = np.asarray(w, dtype=np.float32)
    outlier_cols = np.asarray(outlier_cols, dtype=np.int64)
    keep = np.ones(w.shape[1], dtype=bool)
    keep[outlier_cols] = False
    absmax = np.abs(w[:, keep]).max(axis=1) if keep.any() else np.zeros(w.shape[0], np.float32)
    scale = (absmax / np.float32(127.0)).astype(np.float32)
    scale[scale == 0] = 1.0
    q = np.rint(w / scale[:, None])  # rint: ties to even
    q = np.clip(q, -127, 127).astype(np.int8)
    q[:, ~keep] = 0
    return q, scale, w[:, outlier_cols].copy()


def linear_w8_f64(x: np.ndarray, wq: np.ndarray, scale: np.ndarray, outlier_cols: np.ndarray, w_out: np.ndarray) -> np.ndarray:
    """The definition evaluated in float64."""
    x = np.asarray(x, dtype=np.float64)
    main = x @ (wq.astype(np.float64) * scale.astype(np.float64)[:, None]).T
    if len(outlier_cols):
        main = main + x[:, np.asarray(outlier_cols, dtype=np.int64)] @ np.asarray(w_out, dtype=np.float64).T
    return main
