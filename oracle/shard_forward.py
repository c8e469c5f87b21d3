"""Oracle for the forward side of the hot path, torch on CPU: what a rank's shard computes with the
reference's machinery - `torch.nn.functional.linear` on the sliced weight inside the wrapped module
(src/tensor_parallel/wrapper.py:69-72 with weights from shard.py:160), the module's own activation code,
and the thread-rendezvous sum (communications.py:103-139 + cross_device_ops.py:49)."""
from __future__ import annotations

import threading
from typing import List, Optional, Sequence

import torch
import torch.nn.functional as F


def tensor_split_rank(t: torch.Tensor, world_size: int, dim: int, rank: int) -> torch.Tensor:
    return torch.tensor_split(t, world_size, dim=dim)[rank]


def column_parallel_linear(x, w_full, b_full, world_size: int, rank: int) -> torch.Tensor:
    """Shard of a Linear split on its output axis (Split(dim=0) on weight and bias)."""
    w = tensor_split_rank(w_full, world_size, 0, rank)
    b = None if b_full is None else tensor_split_rank(b_full, world_size, 0, rank)
    return F.linear(x, w, b)


def row_parallel_linear(x_full, w_full, world_size: int, rank: int) -> torch.Tensor:
    """Shard of a Linear split on its input axis (Split(dim=1)); consumes the matching slice of x; the
    result is a partial sum."""
    w = tensor_split_rank(w_full, world_size, 1, rank)
    x = tensor_split_rank(x_full, world_size, -1, rank)
    return F.linear(x, w)


def conv1d_shard(x: torch.Tensor, w_in_out: torch.Tensor, bias) -> torch.Tensor:
    """transformers' Conv1D on one rank's sliced weight, the module the reference's GPT-2 shards run
    (slicing_configs.py:192-201; called through wrapper.py:69-72): addmm(bias, x2d, w) with w of shape [in, out]."""
    out = x.reshape(-1, x.shape[-1]) @ w_in_out
    if bias is not None:
        out = out + bias
    return out.reshape(*x.shape[:-1], w_in_out.shape[1])


def gated_mlp_shard(x: torch.Tensor, wg: torch.Tensor, wu: torch.Tensor, wd: torch.Tensor) -> torch.Tensor:
    """Llama MLP on one rank's weights: down(silu(gate(x)) * up(x)), every op in the tensors' dtype."""
    return F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)


def gated_mlp_hidden(x: torch.Tensor, wg: torch.Tensor, wu: torch.Tensor) -> torch.Tensor:
    return F.silu(F.linear(x, wg)) * F.linear(x, wu)


def reduce_sum(parts: Sequence[torch.Tensor]) -> torch.Tensor:
    """reduce_add on non-cuda devices: Python's sum of the partials (cross_device_ops.py:49)."""
    return sum(list(parts))


def llama_mlp_tp_forward(x: torch.Tensor, wg: torch.Tensor, wu: torch.Tensor, wd: torch.Tensor, world_size: int,
                         threads: bool = True) -> torch.Tensor:
    """The whole tensor-parallel MLP as the reference runs it on ['cpu'] * W: W shards, one thread each
    (tensor_parallel.py:237-287), then the sum. Weights are the FULL matrices; they are sliced here by the
    Llama rules (gate/up dim 0, down dim 1, slicing_configs.py:376-378)."""
    shards = []
    for r in range(world_size):
        shards.append((
            tensor_split_rank(wg, world_size, 0, r).clone(),
            tensor_split_rank(wu, world_size, 0, r).clone(),
            tensor_split_rank(wd, world_size, 1, r).clone(),
        ))
    return run_mlp_shards(x, shards, threads)


def run_mlp_shards(x: torch.Tensor, shards: Sequence[Sequence[torch.Tensor]], threads: bool = True) -> torch.Tensor:
    partials: List[Optional[torch.Tensor]] = [None] * len(shards)

    def work(r):
        g, u, d = shards[r]
        partials[r] = gated_mlp_shard(x, g, u, d)

    if threads and len(shards) > 1:
        ts = [threading.Thread(target=work, args=(r,)) for r in range(len(shards))]
        for t in ts:
            t.start()
        for t in ts:
            t.join()
    else:
        for r in range(len(shards)):
            work(r)
    return reduce_sum(partials)
