"""Slicing engine, host side: turns "take these index ranges of axis d" into 2-D byte-region copy jobs for
the HIP mover, for one tensor or for a whole state dict times all ranks in one launch.

A split of a contiguous tensor of shape S on axis d keeps, for every one of outer = prod(S[:d]) slabs, the
index ranges [start, start+len) of that axis. With inner = prod(S[d+1:]) each kept range is one region of
`outer` rows of len*inner*itemsize bytes, read at pitch S[d]*inner*itemsize and written at the pitch of the
shard. The inverse direction (undo of a split, gather of column-parallel outputs) swaps source and
destination pitches.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import _native

Segment = Tuple[int, int]  # (start, length) on the split axis


def tensor_split_range(n: int, world_size: int, rank: int) -> Segment:
    """Index range that `torch.tensor_split(t, world_size, dim)[rank]` keeps on an axis of length n."""
    if world_size <= 0:
        raise ValueError(f"world_size must be positive, got {world_size}")
    if not 0 <= rank < world_size:
        raise IndexError(f"rank {rank} out of range for world_size {world_size}")
    q, m = divmod(n, world_size)
    start = rank * q + min(rank, m)
    return start, q + (1 if rank < m else 0)


@dataclass(frozen=True)
class SliceSpec:
    """Which ranges of axis `dim` of a tensor of shape `shape` one shard keeps, in output order."""

    shape: Tuple[int, ...]
    dim: int
    segments: Tuple[Segment, ...]

    @property
    def out_shape(self) -> Tuple[int, ...]:
        s = list(self.shape)
        s[self.dim] = sum(length for _, length in self.segments)
        return tuple(s)

    @property
    def outer(self) -> int:
        return math.prod(self.shape[: self.dim])

    @property
    def inner(self) -> int:
        return math.prod(self.shape[self.dim + 1 :])


def normalize_dim(dim: int, ndim: int) -> int:
    if not -ndim <= dim < ndim:
        raise IndexError(f"Dimension out of range (expected to be in range of [{-ndim}, {ndim - 1}], but got {dim})")
    return dim % ndim


def copy_jobs(spec: SliceSpec, itemsize: int, full_ptr: int, shard_ptr: int, scatter: bool = False) -> List[tuple]:
    """Copy jobs that move `spec`'s segments between the full tensor at `full_ptr` and the shard at `shard_ptr`.

    scatter=False: full -> shard (slice). scatter=True: shard -> full (undo / gather).
    """
    n = spec.shape[spec.dim]
    inner_b = spec.inner * itemsize
    full_pitch = n * inner_b
    shard_len = sum(length for _, length in spec.segments)
    shard_pitch = shard_len * inner_b
    rows = spec.outer
    jobs = []
    done = 0
    for start, length in spec.segments:
        if length == 0 or rows == 0 or inner_b == 0:
            done += length
            continue
        full_at = full_ptr + start * inner_b
        shard_at = shard_ptr + done * inner_b
        row_bytes = length * inner_b
        if scatter:
            jobs.append((shard_at, full_at, rows, row_bytes, shard_pitch, full_pitch))
        else:
            jobs.append((full_at, shard_at, rows, row_bytes, full_pitch, shard_pitch))
        done += length
    return jobs


def transpose_jobs(spec: SliceSpec, itemsize: int, full_ptr: int, out_ptr: int) -> List[tuple]:
    """Transposing-mover jobs that cut `spec`'s segments out of a row-major 2-D tensor at `full_ptr` and write the
    shard with its axes swapped: the shard of logical shape (R, C) is stored at `out_ptr` as C rows of R elements."""
    if len(spec.shape) != 2:
        raise ValueError(f"transposed slicing needs a 2-D tensor, got shape {spec.shape}")
    rows, cols = spec.shape
    out_rows = spec.out_shape[0]
    jobs, done = [], 0
    for start, length in spec.segments:
        if length and rows and cols:
            if spec.dim == 1:  # columns [start, start + length) become stored rows done ... done + length
                jobs.append((full_ptr + start * itemsize, out_ptr + done * out_rows * itemsize, rows, length, cols * itemsize, out_rows * itemsize))
            else:  # rows [start, start + length) become stored columns done ... done + length
                jobs.append((full_ptr + start * cols * itemsize, out_ptr + done * itemsize, length, cols, cols * itemsize, out_rows * itemsize))
        done += length
    return jobs


def is_k_major(t: torch.Tensor) -> bool:
    """True for a 2-D tensor stored with its first axis fastest: `t.t()` is row-major contiguous."""
    return t.dim() == 2 and t.stride(0) == 1 and t.stride(1) == t.shape[0]


def _device_source(t: torch.Tensor, device: Optional[torch.device]) -> torch.Tensor:
    """The tensor, contiguous, on the HIP device the kernels will run on (uploaded if it lives on the host)."""
    if t.device.type == "cuda":
        if is_k_major(t) and not t.is_contiguous() and t.element_size() in (1, 2, 4):
            return _native.transpose_regions(t.t(), [(0, t.shape[0])])
        return t.contiguous()
    if t.device.type != "cpu":
        raise _native.NativeLibraryError(f"cannot slice a tensor on {t.device}")
    if device is None:
        if not torch.cuda.is_available():
            raise _native.NativeLibraryError(
                "slicing runs on a HIP device and none is visible; tensor_parallel_amd has no host implementation"
            )
        device = torch.device("cuda", torch.cuda.current_device())
    return t.contiguous().to(device, non_blocking=False)


def apply_spec(t: torch.Tensor, spec: SliceSpec, device: Optional[torch.device] = None) -> torch.Tensor:
    """One shard of one tensor, as a fresh contiguous tensor (meta tensors stay meta: shapes only)."""
    if tuple(t.shape) != spec.shape:
        raise ValueError(f"spec was made for shape {spec.shape}, tensor has {tuple(t.shape)}")
    if t.device.type == "meta":
        return torch.empty(spec.out_shape, dtype=t.dtype, device="meta")
    src = _device_source(t, device)
    out = torch.empty(spec.out_shape, dtype=t.dtype, device=src.device)
    jobs = copy_jobs(spec, t.element_size(), src.data_ptr(), out.data_ptr())
    _native.run_copy_jobs(jobs, src.device)
    return out


def concat_specs(parts: Sequence[torch.Tensor], specs: Sequence[SliceSpec], copies: int = 1):
    """Inverse of slicing: scatter every part back to the ranges its spec names, giving the full tensor. With
    `copies` > 1: a list of that many separate full tensors (one per rank of a gather), written by as few launches as
    their jobs fit into."""
    if len(parts) != len(specs) or not parts:
        raise ValueError("concat_specs: need one spec per part")
    full_shape = specs[0].shape
    first = parts[0]
    if first.device.type == "meta":
        outs = [torch.empty(full_shape, dtype=first.dtype, device="meta") for _ in range(copies)]
        return outs[0] if copies == 1 else outs
    dev_parts = [_device_source(p, None if first.device.type != "cuda" else first.device) for p in parts]
    device = dev_parts[0].device
    for p, spec in zip(dev_parts, specs):
        if tuple(p.shape) != spec.out_shape:
            raise ValueError(f"part has shape {tuple(p.shape)}, its spec expects {spec.out_shape}")
        if p.device != device or p.dtype != first.dtype:
            raise ValueError("concat_specs: parts must share device and dtype")
    outs = [torch.empty(full_shape, dtype=first.dtype, device=device) for _ in range(copies)]
    jobs: List[tuple] = []
    for out in outs:
        mine: List[tuple] = []
        for p, spec in zip(dev_parts, specs):
            mine += copy_jobs(spec, p.element_size(), out.data_ptr(), p.data_ptr(), scatter=True)
        # the jobs of several copies share a launch while they fit the kernel's argument list
        if jobs and len(jobs) + len(mine) > _native.SMALL_COPY_MAX_JOBS:
            _native.run_copy_jobs(jobs, device)
            jobs = []
        jobs += mine
    _native.run_copy_jobs(jobs, device)
    return outs[0] if copies == 1 else outs


def concat_dim(parts: Sequence[torch.Tensor], dim: int, copies: int = 1):
    """torch.cat(parts, dim) through the region mover (parts may have different lengths on `dim`); `copies` as in
    concat_specs."""
    first = parts[0]
    d = normalize_dim(dim, first.dim())
    total = sum(p.shape[d] for p in parts)
    full_shape = list(first.shape)
    full_shape[d] = total
    specs, at = [], 0
    for p in parts:
        specs.append(SliceSpec(tuple(full_shape), d, ((at, p.shape[d]),)))
        at += p.shape[d]
    return concat_specs(parts, specs, copies)


class BatchSlicer:
    """Collects (tensor, spec) requests and serves all of them with ONE kernel launch."""

    def __init__(self, device: Optional[torch.device] = None):
        self.device = device
        self._sources: Dict[int, torch.Tensor] = {}  # id(original) -> device-resident contiguous source
        self._keep: List[torch.Tensor] = []
        self._jobs: List[tuple] = []
        self._transposing: Dict[int, List[tuple]] = {}  # element size -> jobs of the transposing mover
        self.plan: Optional[_native.CopyPlan] = None

    def add(self, t: torch.Tensor, spec: SliceSpec, k_major: bool = False) -> torch.Tensor:
        """Queue one shard of `t`. With `k_major` (2-D tensors) the shard is written with its first axis fastest: it has
        the shape `spec.out_shape` and the memory of its transpose, which is how `tpamd_linear` wants a weight that the
        model code keeps as [in, out]; slicing and transposing are one pass of the transposing mover."""
        if tuple(t.shape) != spec.shape:
            raise ValueError(f"spec was made for shape {spec.shape}, tensor has {tuple(t.shape)}")
        if t.device.type == "meta":
            return torch.empty(spec.out_shape, dtype=t.dtype, device="meta")
        k_major = k_major and t.dim() == 2 and t.element_size() in (1, 2, 4)
        src = self._sources.get(id(t))
        if src is None:
            src = _device_source(t, self.device)
            self._sources[id(t)] = src
            self._keep.append(t)  # keeps id(t) unique while the batch is open
            if self.device is None:
                self.device = src.device
        if src.device != self.device:
            raise ValueError(f"batch is on {self.device}, tensor on {src.device}")
        if k_major:
            stored = torch.empty(spec.out_shape[::-1], dtype=t.dtype, device=src.device)
            self._transposing.setdefault(t.element_size(), []).extend(transpose_jobs(spec, t.element_size(), src.data_ptr(), stored.data_ptr()))
            return stored.t()
        out = torch.empty(spec.out_shape, dtype=t.dtype, device=src.device)
        self._jobs += copy_jobs(spec, t.element_size(), src.data_ptr(), out.data_ptr())
        return out

    def build(self) -> Optional[_native.CopyPlan]:
        if self.plan is None and self._jobs:
            self.plan = _native.CopyPlan(self._jobs, self.device)
        return self.plan

    def run(self) -> int:
        """Launch the batch; returns the bytes moved one way."""
        moved = 0
        for itemsize, jobs in self._transposing.items():
            _native.run_transpose_jobs(jobs, itemsize, self.device)
            moved += sum(j[2] * j[3] for j in jobs) * itemsize
        plan = self.build()
        if plan is None:
            return moved
        plan.run()
        return moved + plan.nbytes

    def close(self) -> None:
        if self.plan is not None:
            self.plan.close()
            self.plan = None
        self._sources.clear()
        self._keep.clear()
        self._jobs = []
        self._transposing = {}
