"""Oracle for the "sum" rule: `sum([p_0, ..., p_{W-1}])` over same-dtype tensors, i.e. Python's left fold
starting from 0 (src/tensor_parallel/cross_device_ops.py:49). For bf16/fp16 tensors every `+` rounds its
result to the tensor dtype; that is restated here at bit level on uint16 arrays."""
from __future__ import annotations

from typing import Sequence

import numpy as np


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """Round to nearest, ties to even; NaN stays NaN."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = (u + (0x7FFF + ((u >> 16) & 1))) >> 16
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    return np.where(nan, (u >> 16) | 0x0040, rounded).astype(np.uint16)


def sum_bf16_stepwise(parts: Sequence[np.ndarray]) -> np.ndarray:
    """((p0 + p1) + p2) + ... with a bf16 rounding after every add. Inputs and output: uint16 bit patterns."""
    acc = np.asarray(parts[0], dtype=np.uint16)
    for p in parts[1:]:
        acc = f32_to_bf16(bf16_to_f32(acc) + bf16_to_f32(np.asarray(p, dtype=np.uint16)))
    return acc


def sum_bf16_f32acc(parts: Sequence[np.ndarray]) -> np.ndarray:
    """fp32 running sum in rank order, one rounding at the end."""
    acc = bf16_to_f32(np.asarray(parts[0], dtype=np.uint16)).copy()
    for p in parts[1:]:
        acc = acc + bf16_to_f32(np.asarray(p, dtype=np.uint16))
    return f32_to_bf16(acc)


def sum_f16_stepwise(parts: Sequence[np.ndarray]) -> np.ndarray:
    """fp16 inputs as np.float16; each add is done in fp32 and rounded to fp16 (what torch does on CPU)."""
    acc = np.asarray(parts[0], dtype=np.float16)
    for p in parts[1:]:
        acc = (acc.astype(np.float32) + np.asarray(p, dtype=np.float16).astype(np.float32)).astype(np.float16)
    return acc


def sum_f32(parts: Sequence[np.ndarray]) -> np.ndarray:
    acc = np.asarray(parts[0], dtype=np.float32).copy()
    for p in parts[1:]:
        acc = acc + np.asarray(p, dtype=np.float32)
    return acc
