"""ctypes binding of `libtpamd.so` (include/tpamd.h).

The library is loaded when this module is imported. If it cannot be loaded, importing still succeeds (so
that rule tables and shape arithmetic can be used on a machine without the build), but every compute
entry point raises `NativeLibraryError`: there is no other implementation to fall back to.
"""
from __future__ import annotations

import ctypes
import os
from pathlib import Path
from typing import Optional, Sequence

import torch  # imported first on purpose: the library binds to the HIP runtime torch has loaded

LIB_PATH = Path(__file__).resolve().parent / "_lib" / "libtpamd.so"

EXPORTS = (
    "tpamd_abi_version",
    "tpamd_last_error",
    "tpamd_copy_plan_create",
    "tpamd_copy_plan_run",
    "tpamd_copy_plan_bytes",
    "tpamd_copy_plan_destroy",
    "tpamd_copy_jobs_run",
    "tpamd_transpose_jobs_run",
    "tpamd_scale",
    "tpamd_reduce_partials",
    "tpamd_tuning_reload",
    "tpamd_scratch_query",
    "tpamd_scratch_release",
    "tpamd_linear",
    "tpamd_linear_add",
    "tpamd_linear_noalloc",
    "tpamd_noalloc_scratch_bytes",
    "tpamd_swiglu_up",
    "tpamd_linear_w8",
    "tpamd_attention",
    "tpamd_rope_append",
    "tpamd_attention_decode_rope",
    "tpamd_attention_decode_rope_devpos",
)

ABI_VERSION = 5

BF16, F16, F32 = 0, 1, 2
ACCUM_STEPWISE, ACCUM_F32 = 0, 1
ACT_NONE, ACT_GELU = 0, 1

_DTYPES = {torch.bfloat16: BF16, torch.float16: F16, torch.float32: F32}


class NativeLibraryError(RuntimeError):
    pass


class CopyJob(ctypes.Structure):
    _fields_ = [
        ("src", ctypes.c_void_p),
        ("dst", ctypes.c_void_p),
        ("rows", ctypes.c_uint64),
        ("row_bytes", ctypes.c_uint64),
        ("src_pitch", ctypes.c_uint64),
        ("dst_pitch", ctypes.c_uint64),
    ]


class TransposeJob(ctypes.Structure):
    _fields_ = [
        ("src", ctypes.c_void_p),
        ("dst", ctypes.c_void_p),
        ("rows", ctypes.c_uint64),
        ("cols", ctypes.c_uint64),
        ("src_pitch", ctypes.c_uint64),
        ("dst_pitch", ctypes.c_uint64),
    ]


_lib: Optional[ctypes.CDLL] = None
_load_error: Optional[str] = None


def _declare(lib: ctypes.CDLL) -> None:
    c = ctypes
    i64, u64, vp, ci = c.c_int64, c.c_uint64, c.c_void_p, c.c_int
    lib.tpamd_abi_version.restype = ci
    lib.tpamd_abi_version.argtypes = []
    lib.tpamd_last_error.restype = c.c_char_p
    lib.tpamd_last_error.argtypes = []
    lib.tpamd_copy_plan_create.restype = ci
    lib.tpamd_copy_plan_create.argtypes = [c.POINTER(CopyJob), c.c_size_t, c.POINTER(vp)]
    lib.tpamd_copy_plan_run.restype = ci
    lib.tpamd_copy_plan_run.argtypes = [vp, vp]
    lib.tpamd_copy_plan_bytes.restype = u64
    lib.tpamd_copy_plan_bytes.argtypes = [vp]
    lib.tpamd_copy_plan_destroy.restype = ci
    lib.tpamd_copy_plan_destroy.argtypes = [vp]
    lib.tpamd_copy_jobs_run.restype = ci
    lib.tpamd_copy_jobs_run.argtypes = [c.POINTER(CopyJob), c.c_size_t, vp]
    lib.tpamd_transpose_jobs_run.restype = ci
    lib.tpamd_transpose_jobs_run.argtypes = [c.POINTER(TransposeJob), c.c_size_t, ci, vp]
    lib.tpamd_scale.restype = ci
    lib.tpamd_scale.argtypes = [vp, vp, u64, ci, ci, ci, vp]
    lib.tpamd_reduce_partials.restype = ci
    lib.tpamd_reduce_partials.argtypes = [c.POINTER(vp), ci, vp, u64, ci, ci, vp]
    lib.tpamd_linear.restype = ci
    lib.tpamd_linear.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, ci, vp]
    lib.tpamd_linear_add.restype = ci
    lib.tpamd_linear_add.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, ci, ci, vp]
    lib.tpamd_linear_noalloc.restype = ci
    lib.tpamd_linear_noalloc.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, ci, vp]
    lib.tpamd_noalloc_scratch_bytes.restype = u64
    lib.tpamd_noalloc_scratch_bytes.argtypes = []
    lib.tpamd_tuning_reload.restype = None
    lib.tpamd_tuning_reload.argtypes = []
    lib.tpamd_scratch_query.restype = ci
    lib.tpamd_scratch_query.argtypes = [vp, c.POINTER(vp), c.POINTER(u64)]
    lib.tpamd_scratch_release.restype = ci
    lib.tpamd_scratch_release.argtypes = [vp]
    lib.tpamd_swiglu_up.restype = ci
    lib.tpamd_swiglu_up.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, vp]
    lib.tpamd_attention.restype = ci
    lib.tpamd_attention.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, c.POINTER(i64), c.c_float, ci, ci, vp]
    lib.tpamd_attention_decode_rope.restype = ci
    lib.tpamd_attention_decode_rope.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, c.POINTER(i64), c.c_float, ci, vp]
    lib.tpamd_attention_decode_rope_devpos.restype = ci
    lib.tpamd_attention_decode_rope_devpos.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, vp, i64, c.POINTER(i64), c.c_float, ci, vp]
    lib.tpamd_rope_append.restype = ci
    lib.tpamd_rope_append.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, c.POINTER(i64), ci, vp]
    lib.tpamd_linear_w8.restype = ci
    lib.tpamd_linear_w8.argtypes = [vp, vp, vp, vp, vp, i64, vp, vp, i64, i64, i64, i64, i64, i64, i64, ci, ci, vp]


def _load() -> None:
    global _lib, _load_error
    path = Path(os.environ.get("TPAMD_LIB", str(LIB_PATH)))
    if not path.exists():
        _load_error = f"{path} does not exist; build it with `python -m tensor_parallel_amd.build`"
        return
    try:
        lib = ctypes.CDLL(str(path))
        for name in EXPORTS:
            getattr(lib, name)
        _declare(lib)
        got = lib.tpamd_abi_version()
        if got != ABI_VERSION:
            raise OSError(f"ABI version {got}, expected {ABI_VERSION}")
        _lib = lib
    except (OSError, AttributeError) as e:  # pragma: no cover - depends on the machine
        _load_error = f"cannot load {path}: {e}"


_load()


def available() -> bool:
    return _lib is not None


def load_error() -> Optional[str]:
    return _load_error


def lib() -> ctypes.CDLL:
    if _lib is None:
        raise NativeLibraryError(f"the HIP library of tensor_parallel_amd is not available: {_load_error}")
    return _lib


def _check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().tpamd_last_error().decode("utf-8", "replace")
        if rc == -1:
            raise ValueError(f"{what}: {msg}")
        raise RuntimeError(f"{what} failed (status {rc}): {msg}")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise TypeError(f"tensor_parallel_amd kernels support bfloat16, float16 and float32, got {dtype}") from None


def require_device(t: torch.Tensor, what: str) -> None:
    if t.device.type != "cuda":
        raise NativeLibraryError(
            f"{what}: expected a tensor on a HIP device, got {t.device}. tensor_parallel_amd computes on the GPU only."
        )


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream_ptr(device: torch.device) -> int:
    """Handle of torch's current stream on `device` (the stream every kernel of a call is enqueued on)."""
    if _raw_stream is not None:
        index = device.index
        return _raw_stream(torch.cuda.current_device() if index is None else index)
    return torch.cuda.current_stream(device).cuda_stream


class _on_device:
    """`with _on_device(dev):` makes `dev` the current HIP device for the call; costs nothing when it already is."""

    __slots__ = ("index", "prev")

    def __init__(self, device: torch.device):
        self.index = device.index

    def __enter__(self):
        self.prev = None
        if self.index is not None:
            cur = torch.cuda.current_device()
            if cur != self.index:
                self.prev = cur
                torch.cuda.set_device(self.index)

    def __exit__(self, *exc):
        if self.prev is not None:
            torch.cuda.set_device(self.prev)
        return False


class CopyPlan:
    """A device-resident table of 2-D byte-region copies, run as one kernel launch."""

    def __init__(self, jobs: Sequence[tuple], device: torch.device):
        # jobs: (src_ptr, dst_ptr, rows, row_bytes, src_pitch, dst_pitch)
        self._handle = ctypes.c_void_p()
        self.device = device
        arr = (CopyJob * max(len(jobs), 1))()
        for i, j in enumerate(jobs):
            arr[i] = CopyJob(*j)
        with _on_device(device):
            _check(lib().tpamd_copy_plan_create(arr, len(jobs), ctypes.byref(self._handle)), "tpamd_copy_plan_create")
        self.n_jobs = len(jobs)

    @property
    def nbytes(self) -> int:
        return int(lib().tpamd_copy_plan_bytes(self._handle))

    def run(self, stream_ptr: Optional[int] = None) -> None:
        with _on_device(self.device):
            if stream_ptr is None:
                stream_ptr = current_stream_ptr(self.device)
            _check(lib().tpamd_copy_plan_run(self._handle, ctypes.c_void_p(stream_ptr)), "tpamd_copy_plan_run")

    def close(self) -> None:
        if self._handle:
            h, self._handle = self._handle, ctypes.c_void_p()
            if _lib is not None:
                _lib.tpamd_copy_plan_destroy(h)

    def __del__(self):  # noqa: D105
        try:
            self.close()
        except Exception:
            pass


SMALL_COPY_MAX_JOBS = 16


def run_copy_jobs(jobs: Sequence[tuple], device: torch.device) -> None:
    """Launch up to 16 copy jobs without building a plan (nothing allocated, nothing to keep alive); more jobs go
    through a plan, which is destroyed once its launch has finished."""
    if not jobs:
        return
    with _on_device(device):
        if len(jobs) <= SMALL_COPY_MAX_JOBS:
            arr = (CopyJob * len(jobs))(*[CopyJob(*j) for j in jobs])
            _check(lib().tpamd_copy_jobs_run(arr, len(jobs), ctypes.c_void_p(current_stream_ptr(device))), "tpamd_copy_jobs_run")
            return
    plan = CopyPlan(jobs, device)
    plan.run()
    torch.cuda.current_stream(device).synchronize()  # the plan's tile table must outlive the launch
    plan.close()


TRANSPOSE_MAX_JOBS = 16


def run_transpose_jobs(jobs: Sequence[tuple], elem_bytes: int, device: torch.device) -> None:
    """Launch transposing region moves: jobs are (src_ptr, dst_ptr, rows, cols, src_pitch, dst_pitch) with the extent
    in elements of the source region and the pitches in bytes; 16 jobs per launch."""
    with _on_device(device):
        for at in range(0, len(jobs), TRANSPOSE_MAX_JOBS):
            part = jobs[at:at + TRANSPOSE_MAX_JOBS]
            arr = (TransposeJob * len(part))(*[TransposeJob(*j) for j in part])
            _check(lib().tpamd_transpose_jobs_run(arr, len(part), elem_bytes, ctypes.c_void_p(current_stream_ptr(device))),
                   "tpamd_transpose_jobs_run")


def transpose_regions(src: torch.Tensor, col_ranges: Sequence[tuple], row_range: Optional[tuple] = None,
                      out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`cat([src[r0:r1, a:b] for a, b in col_ranges], dim=1).t()` as a fresh contiguous tensor, in one launch: column
    ranges (and one row range) are cut out of the row-major 2-D tensor `src` and land transposed, one below the other.
    With the whole tensor as its only range this is `src.t().contiguous()`."""
    require_device(src, "transpose_regions")
    if src.dim() != 2 or src.stride(1) != 1 or src.element_size() not in (1, 2, 4):
        raise ValueError(f"transpose_regions: a row-major 2-D tensor of 1-, 2- or 4-byte elements is needed, got shape {tuple(src.shape)} "
                         f"strides {src.stride()} {src.dtype}")
    r0, r1 = (0, src.shape[0]) if row_range is None else row_range
    if not (0 <= r0 <= r1 <= src.shape[0]) or any(not (0 <= a <= b <= src.shape[1]) for a, b in col_ranges):
        raise ValueError(f"transpose_regions: ranges {row_range} x {list(col_ranges)} outside shape {tuple(src.shape)}")
    es, n_out = src.element_size(), sum(b - a for a, b in col_ranges)
    if out is None:
        out = torch.empty((n_out, r1 - r0), dtype=src.dtype, device=src.device)
    elif out.shape != (n_out, r1 - r0) or out.dtype != src.dtype or out.device != src.device or not out.is_contiguous():
        raise ValueError("transpose_regions: out must be a contiguous tensor of the result's shape, dtype and device")
    pitch, jobs, at = src.stride(0) * es, [], 0
    for a, b in col_ranges:
        if b > a and r1 > r0:
            jobs.append((src.data_ptr() + r0 * pitch + a * es, out.data_ptr() + at * out.stride(0) * es, r1 - r0, b - a, pitch, out.stride(0) * es))
        at += b - a
    run_transpose_jobs(jobs, es, src.device)
    return out


def scale(inp: torch.Tensor, world_size: int, multiply: bool = False) -> torch.Tensor:
    require_device(inp, "scale")
    src = inp.contiguous()
    out = torch.empty_like(src)
    with _on_device(src.device):
        _check(
            lib().tpamd_scale(src.data_ptr(), out.data_ptr(), src.numel(), dtype_code(src.dtype), world_size,
                              1 if multiply else 0, ctypes.c_void_p(current_stream_ptr(src.device))),
            "tpamd_scale",
        )
    return out


def reduce_partials(parts: Sequence[torch.Tensor], accum: int = ACCUM_STEPWISE, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    if len(parts) == 0:
        raise ValueError("reduce_partials: no partials")
    first = parts[0]
    require_device(first, "reduce_partials")
    keep = []
    for p in parts:
        if p.shape != first.shape or p.dtype != first.dtype or p.device != first.device:
            raise ValueError("reduce_partials: partials must agree in shape, dtype and device")
        keep.append(p.contiguous())
    if out is None:
        out = torch.empty_like(keep[0])
    ptrs = (ctypes.c_void_p * len(keep))(*[p.data_ptr() for p in keep])
    with _on_device(first.device):
        _check(
            lib().tpamd_reduce_partials(ptrs, len(keep), out.data_ptr(), first.numel(), dtype_code(first.dtype), accum,
                                        ctypes.c_void_p(current_stream_ptr(first.device))),
            "tpamd_reduce_partials",
        )
    return out


def _as_2d(x: torch.Tensor) -> torch.Tensor:
    if x.dim() == 2 and x.is_contiguous():
        return x
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(-1) != 1 or (x2.shape[0] > 1 and x2.stride(0) < x2.shape[1]):
        x2 = x2.contiguous()
    return x2


def _ld(t: torch.Tensor) -> int:
    return t.stride(0) if t.shape[0] > 1 else max(t.shape[1], 1)


def reload_tuning() -> None:
    """Make the library read its TPAMD_* environment variables again (it reads them once, at load time)."""
    lib().tpamd_tuning_reload()


def scratch_of_stream(device: torch.device, stream_ptr: Optional[int] = None) -> tuple:
    """(address, bytes) of the K-split scratch buffer that work on the stream uses, (None, 0) while it has none."""
    ptr, nbytes = ctypes.c_void_p(), ctypes.c_uint64()
    with _on_device(device):
        if stream_ptr is None:
            stream_ptr = current_stream_ptr(device)
        _check(lib().tpamd_scratch_query(ctypes.c_void_p(stream_ptr), ctypes.byref(ptr), ctypes.byref(nbytes)), "tpamd_scratch_query")
    return ptr.value, int(nbytes.value)


def release_scratch(device: torch.device, stream_ptr: Optional[int] = None) -> None:
    """Free the K-split scratch buffer of a stream that is about to be retired (it is synchronised first)."""
    with _on_device(device):
        if stream_ptr is None:
            stream_ptr = current_stream_ptr(device)
        _check(lib().tpamd_scratch_release(ctypes.c_void_p(stream_ptr)), "tpamd_scratch_release")


def linear(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, act: int = ACT_NONE,
           addend: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = act(x @ w.T + bias) with w of shape [N, K]; leading dimensions of x are kept. With `addend` (same shape
    and dtype as y): y = (that result, rounded to the dtype) + addend, one step of the sum over rank partials, in the
    same launch. `out` (contiguous, may be `addend`) receives the result."""
    require_device(x, "linear")
    require_device(w, "linear")
    if x.dtype != w.dtype:
        raise TypeError(f"linear: x is {x.dtype} but w is {w.dtype}")
    if w.dim() != 2 or x.shape[-1] != w.shape[1]:
        raise ValueError(f"linear: x has {x.shape[-1]} input features, w is {tuple(w.shape)}")
    if w.device != x.device:
        raise ValueError(f"linear: x is on {x.device}, w on {w.device}")
    N, K = w.shape
    M = x.numel() // K if K else 0
    if bias is not None and (bias.shape != (N,) or bias.dtype != x.dtype or bias.device != x.device):
        raise ValueError("linear: bias must have shape [N], the dtype of x and live on its device")
    if addend is not None and (addend.dtype != x.dtype or addend.device != x.device or addend.numel() != M * N
                               or addend.shape[-1] != N):
        raise ValueError("linear: addend must have the shape, dtype and device of the result")
    if out is not None and (out.dtype != x.dtype or out.device != x.device or out.numel() != M * N or not out.is_contiguous()):
        raise ValueError("linear: out must be a contiguous tensor of the result's size, dtype and device")
    x2, w2 = _as_2d(x), _as_2d(w)
    M = x2.shape[0]
    y = torch.empty((M, N), dtype=x.dtype, device=x.device) if out is None else out.view(M, N)
    b = bias.contiguous() if bias is not None else None
    a2 = _as_2d(addend) if addend is not None else None
    with _on_device(x.device):
        stream = ctypes.c_void_p(current_stream_ptr(x.device))
        if a2 is None:
            _check(
                lib().tpamd_linear(x2.data_ptr(), w2.data_ptr(), b.data_ptr() if b is not None else None, y.data_ptr(),
                                   M, N, K, _ld(x2), _ld(w2), N, dtype_code(x.dtype), act, stream),
                "tpamd_linear",
            )
        else:
            _check(
                lib().tpamd_linear_add(x2.data_ptr(), w2.data_ptr(), b.data_ptr() if b is not None else None, a2.data_ptr(),
                                       y.data_ptr(), M, N, K, _ld(x2), _ld(w2), _ld(a2), N, dtype_code(x.dtype), act, stream),
                "tpamd_linear_add",
            )
    return y.view(*x.shape[:-1], N)


def swiglu_up(x: torch.Tensor, wg: torch.Tensor, wu: torch.Tensor) -> torch.Tensor:
    """h = silu(x @ wg.T) * (x @ wu.T)."""
    require_device(x, "swiglu_up")
    if not (x.dtype == wg.dtype == wu.dtype):
        raise TypeError("swiglu_up: x, wg, wu must share one dtype")
    if wg.dim() != 2 or wg.shape != wu.shape or x.shape[-1] != wg.shape[1]:
        raise ValueError("swiglu_up: shape mismatch")
    if wg.device != x.device or wu.device != x.device:
        raise ValueError(f"swiglu_up: x is on {x.device}, wg on {wg.device}, wu on {wu.device}")
    x2, g2, u2 = _as_2d(x), _as_2d(wg), _as_2d(wu)
    if _ld(g2) != _ld(u2):
        u2 = u2.contiguous()
        g2 = g2.contiguous()
    M, K = x2.shape
    N = g2.shape[0]
    h = torch.empty((M, N), dtype=x.dtype, device=x.device)
    with _on_device(x.device):
        _check(
            lib().tpamd_swiglu_up(x2.data_ptr(), g2.data_ptr(), u2.data_ptr(), h.data_ptr(), M, N, K, _ld(x2), _ld(g2), N,
                                  dtype_code(x.dtype), ctypes.c_void_p(current_stream_ptr(x.device))),
            "tpamd_swiglu_up",
        )
    return h.view(*x.shape[:-1], N)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: Optional[float] = None, causal: bool = True,
              out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """softmax(scale * q k^T [+ causal]) v. q [B, Hq, Sq, D], k / v [B, Hkv, Skv, D] -> [B, Sq, Hq, D] (the layout the
    attention output projection consumes). Grouped-query heads when Hq > Hkv; causal is aligned to the END of the key
    range (query i sees keys j <= i + Skv - Sq). `out`, if given, is a [B, Sq, Hq, D] tensor (or view) of q's dtype and
    device whose rows are contiguous and start on 8-byte boundaries."""
    require_device(q, "attention")
    if not (q.dtype == k.dtype == v.dtype) or q.dtype not in (torch.bfloat16, torch.float16):
        raise TypeError("attention: q, k, v must share bfloat16 or float16")
    if q.dim() != 4 or k.dim() != 4 or v.shape != k.shape or q.shape[0] != k.shape[0] or q.shape[3] != k.shape[3]:
        raise ValueError(f"attention: shapes q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)} do not fit")
    if k.device != q.device or v.device != q.device:
        raise ValueError(f"attention: q is on {q.device}, k on {k.device}, v on {v.device}")
    B, Hq, Sq, D = q.shape
    Hkv, Skv = k.shape[1], k.shape[2]
    q, k, v = (t if t.stride(3) == 1 else t.contiguous() for t in (q, k, v))
    if out is None:
        out = torch.empty((B, Sq, Hq, D), dtype=q.dtype, device=q.device)
    elif out.shape != (B, Sq, Hq, D) or out.dtype != q.dtype or out.device != q.device or out.stride(3) != 1:
        raise ValueError(f"attention: out must be a [{B}, {Sq}, {Hq}, {D}] {q.dtype} tensor on {q.device} with contiguous rows")
    strides = (ctypes.c_int64 * 12)(q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
                                    v.stride(0), v.stride(1), v.stride(2), out.stride(0), out.stride(1), out.stride(2))
    with _on_device(q.device):
        _check(
            lib().tpamd_attention(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), B, Hq, Hkv, Sq, Skv, D, strides,
                                  float(scale if scale is not None else D ** -0.5), 1 if causal else 0, dtype_code(q.dtype),
                                  ctypes.c_void_p(current_stream_ptr(q.device))),
            "tpamd_attention",
        )
    return out


def rope_append(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                k_cache: torch.Tensor, v_cache: torch.Tensor, pos0: int, q_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rotary embedding of the new rows and their hand-over to the rank-local cache, one launch.
    q [B, S, Hq, D] or [B, S, Hkv, Hq / Hkv, D] (the query heads of each key/value head, as a fused projection that
    interleaves them with their key and value lays them out), k / v [B, S, Hkv, D] (all views of a projection output),
    cos / sin [B or 1, S, D];
    k_cache / v_cache [B, Hkv, L, D] are written in place at positions pos0 .. pos0 + S - 1 (rotated k, v);
    returns the rotated q as [B, Hq, S, D], the layout `attention` takes."""
    require_device(q, "rope_append")
    if not (q.dtype == k.dtype == v.dtype == cos.dtype == sin.dtype == k_cache.dtype == v_cache.dtype) or q.dtype not in (
            torch.bfloat16, torch.float16):
        raise TypeError("rope_append: every tensor must share bfloat16 or float16")
    if q.dim() not in (4, 5) or k.dim() != 4 or v.shape != k.shape or q.shape[:2] != k.shape[:2] or q.shape[-1] != k.shape[3] or (
            q.dim() == 5 and q.shape[2] != k.shape[2]):
        raise ValueError(f"rope_append: shapes q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)} do not fit")
    B, S, Hkv, D = k.shape
    Hq = q.shape[2] if q.dim() == 4 else q.shape[2] * q.shape[3]
    if Hq % Hkv:
        raise ValueError(f"rope_append: {Hq} query heads over {Hkv} key/value heads")
    q_head, q_group = (q.stride(2), q.stride(2) * (Hq // Hkv)) if q.dim() == 4 else (q.stride(3), q.stride(2))
    if cos.dim() == 2:
        cos, sin = cos.unsqueeze(0), sin.unsqueeze(0)
    if cos.shape != sin.shape or cos.dim() != 3 or cos.shape[0] not in (1, B) or cos.shape[1:] != (S, D):
        raise ValueError(f"rope_append: cos / sin must be [{B} or 1, {S}, {D}], got {tuple(cos.shape)} / {tuple(sin.shape)}")
    if k_cache.dim() != 4 or v_cache.shape != k_cache.shape or k_cache.shape[0] != B or k_cache.shape[1] != Hkv or k_cache.shape[3] != D:
        raise ValueError(f"rope_append: caches must be [{B}, {Hkv}, L, {D}], got {tuple(k_cache.shape)} / {tuple(v_cache.shape)}")
    for name, t in (("k", k), ("v", v), ("cos", cos), ("sin", sin), ("k_cache", k_cache), ("v_cache", v_cache)):
        if t.device != q.device:
            raise ValueError(f"rope_append: q is on {q.device}, {name} on {t.device}")
        if t.stride(-1) != 1:
            raise ValueError(f"rope_append: {name} must have contiguous rows")
    if q.stride(-1) != 1:
        raise ValueError("rope_append: q must have contiguous rows")
    if sin.stride() != cos.stride():
        sin = sin.contiguous()
        cos = cos.contiguous()
    if q_out is None:
        q_out = torch.empty((B, Hq, S, D), dtype=q.dtype, device=q.device)
    elif q_out.shape != (B, Hq, S, D) or q_out.dtype != q.dtype or q_out.device != q.device or q_out.stride(3) != 1:
        raise ValueError(f"rope_append: q_out must be a [{B}, {Hq}, {S}, {D}] {q.dtype} tensor on {q.device} with contiguous rows")
    strides = (ctypes.c_int64 * 21)(q.stride(0), q.stride(1), q_head, k.stride(0), k.stride(1), k.stride(2),
                                    v.stride(0), v.stride(1), v.stride(2), cos.stride(0) if cos.shape[0] > 1 else 0, cos.stride(1),
                                    q_out.stride(0), q_out.stride(1), q_out.stride(2), k_cache.stride(0), k_cache.stride(1),
                                    k_cache.stride(2), v_cache.stride(0), v_cache.stride(1), v_cache.stride(2), q_group)
    with _on_device(q.device):
        _check(
            lib().tpamd_rope_append(q.data_ptr(), k.data_ptr(), v.data_ptr(), cos.data_ptr(), sin.data_ptr(), q_out.data_ptr(),
                                    k_cache.data_ptr(), v_cache.data_ptr(), B, S, Hq, Hkv, D, int(pos0), k_cache.shape[2], strides,
                                    dtype_code(q.dtype), ctypes.c_void_p(current_stream_ptr(q.device))),
            "tpamd_rope_append",
        )
    return q_out


def attention_decode_rope(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                          k_cache: torch.Tensor, v_cache: torch.Tensor, pos0, scale: Optional[float] = None,
                          out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`rope_append` and `attention` for one new position per sequence, in two launches instead of three.
    q [B, 1, Hq, D] or [B, 1, Hkv, Hq / Hkv, D], k / v [B, 1, Hkv, D] (views of the projection output), cos / sin [B or 1, 1, D]
    (or [1, D] / [D]); the caches [B, Hkv, L, D] hold pos0 positions and receive the new one at pos0. Returns [B, 1, Hq, D].
    Where the library has no scratch buffer for the stream (first use under graph capture) the two calls are made instead.

    `pos0` may also be an int64 tensor of one element on the device: the kernels then read the count when they run
    (`tpamd_attention_decode_rope_devpos`), the launches are laid out for the L positions the caches can hold, and the call
    can sit in a HIP graph that is replayed for every decode step. The caller advances the count."""
    require_device(q, "attention_decode_rope")
    if not (q.dtype == k.dtype == v.dtype == cos.dtype == sin.dtype == k_cache.dtype == v_cache.dtype) or q.dtype not in (
            torch.bfloat16, torch.float16):
        raise TypeError("attention_decode_rope: every tensor must share bfloat16 or float16")
    if q.dim() not in (4, 5) or k.dim() != 4 or v.shape != k.shape or q.shape[:2] != k.shape[:2] or k.shape[1] != 1 or \
            q.shape[-1] != k.shape[3] or (q.dim() == 5 and q.shape[2] != k.shape[2]):
        raise ValueError(f"attention_decode_rope: shapes q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)} do not fit one new position")
    B, _, Hkv, D = k.shape
    Hq = q.shape[2] if q.dim() == 4 else q.shape[2] * q.shape[3]
    if Hq % Hkv:
        raise ValueError(f"attention_decode_rope: {Hq} query heads over {Hkv} key/value heads")
    q_head, q_group = (q.stride(2), q.stride(2) * (Hq // Hkv)) if q.dim() == 4 else (q.stride(3), q.stride(2))
    cos, sin = cos.reshape(-1, D), sin.reshape(-1, D)
    if cos.shape != sin.shape or cos.shape[0] not in (1, B):
        raise ValueError(f"attention_decode_rope: cos / sin must hold [{B} or 1] rows of {D}, got {tuple(cos.shape)} / {tuple(sin.shape)}")
    if k_cache.dim() != 4 or v_cache.shape != k_cache.shape or k_cache.shape[0] != B or k_cache.shape[1] != Hkv or k_cache.shape[3] != D:
        raise ValueError(f"attention_decode_rope: caches must be [{B}, {Hkv}, L, {D}], got {tuple(k_cache.shape)} / {tuple(v_cache.shape)}")
    for name, t in (("q", q), ("k", k), ("v", v), ("cos", cos), ("sin", sin), ("k_cache", k_cache), ("v_cache", v_cache)):
        if t.device != q.device:
            raise ValueError(f"attention_decode_rope: q is on {q.device}, {name} on {t.device}")
        if t.stride(-1) != 1:
            raise ValueError(f"attention_decode_rope: {name} must have contiguous rows")
    if sin.stride() != cos.stride():
        sin, cos = sin.contiguous(), cos.contiguous()
    if out is None:
        out = torch.empty((B, 1, Hq, D), dtype=q.dtype, device=q.device)
    elif out.shape != (B, 1, Hq, D) or out.dtype != q.dtype or out.device != q.device or out.stride(3) != 1:
        raise ValueError(f"attention_decode_rope: out must be a [{B}, 1, {Hq}, {D}] {q.dtype} tensor on {q.device} with contiguous rows")
    strides = (ctypes.c_int64 * 16)(q.stride(0), q_head, q_group, k.stride(0), k.stride(2), v.stride(0), v.stride(2),
                                    cos.stride(0) if cos.shape[0] > 1 else 0, k_cache.stride(0), k_cache.stride(1), k_cache.stride(2),
                                    v_cache.stride(0), v_cache.stride(1), v_cache.stride(2), out.stride(0), out.stride(2))
    if isinstance(pos0, torch.Tensor):
        if pos0.dtype != torch.int64 or pos0.numel() != 1 or pos0.device != q.device:
            raise ValueError(f"attention_decode_rope: a position on the device must be one int64 element on {q.device}, "
                             f"got {tuple(pos0.shape)} {pos0.dtype} on {pos0.device}")
        with _on_device(q.device):
            rc = lib().tpamd_attention_decode_rope_devpos(q.data_ptr(), k.data_ptr(), v.data_ptr(), cos.data_ptr(), sin.data_ptr(),
                                                          k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), B, Hq, Hkv, D,
                                                          ctypes.c_void_p(pos0.data_ptr()), k_cache.shape[2], strides,
                                                          float(scale if scale is not None else D ** -0.5), dtype_code(q.dtype),
                                                          ctypes.c_void_p(current_stream_ptr(q.device)))
        _check(rc, "tpamd_attention_decode_rope_devpos")
        return out
    with _on_device(q.device):
        rc = lib().tpamd_attention_decode_rope(q.data_ptr(), k.data_ptr(), v.data_ptr(), cos.data_ptr(), sin.data_ptr(),
                                               k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), B, Hq, Hkv, D, int(pos0),
                                               k_cache.shape[2], strides, float(scale if scale is not None else D ** -0.5),
                                               dtype_code(q.dtype), ctypes.c_void_p(current_stream_ptr(q.device)))
    if rc == -2 and B > 0 and D in (64, 128):  # no scratch buffer for this stream: the two-call sequence needs none
        q_rot = rope_append(q, k, v, cos.unsqueeze(1), sin.unsqueeze(1), k_cache, v_cache, pos0)
        return attention(q_rot, k_cache[:, :, :pos0 + 1], v_cache[:, :, :pos0 + 1], scale=scale, causal=True, out=out)
    _check(rc, "tpamd_attention_decode_rope")
    return out


def linear_w8(x: torch.Tensor, wq: torch.Tensor, scale_: torch.Tensor, outlier_idx: Optional[torch.Tensor],
              w_out: Optional[torch.Tensor], bias: Optional[torch.Tensor] = None, act: int = ACT_NONE) -> torch.Tensor:
    """Weight-only int8 Linear with outlier columns kept in the activation dtype."""
    require_device(x, "linear_w8")
    if wq.dtype != torch.int8 or scale_.dtype != torch.float32:
        raise TypeError("linear_w8: wq must be int8 and scale float32")
    if x.dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"linear_w8: x must be bfloat16 or float16, got {x.dtype}")
    x2 = _as_2d(x)
    M, K = x2.shape
    if wq.dim() != 2 or wq.shape[1] != K:
        raise ValueError(f"linear_w8: x has {K} input features, wq is {tuple(wq.shape)}")
    N = wq.shape[0]
    if scale_.shape != (N,):
        raise ValueError(f"linear_w8: scale must have shape [{N}], got {tuple(scale_.shape)}")
    for name, t in (("wq", wq), ("scale", scale_), ("outlier_idx", outlier_idx), ("w_out", w_out), ("bias", bias)):
        if t is not None and t.device != x.device:
            raise ValueError(f"linear_w8: x is on {x.device}, {name} on {t.device}")
    if bias is not None and (bias.shape != (N,) or bias.dtype != x.dtype):
        raise ValueError("linear_w8: bias must have shape [N] and the dtype of x")
    wq = wq.contiguous()
    n_out = 0 if outlier_idx is None else int(outlier_idx.numel())
    if n_out:
        if outlier_idx.dtype != torch.int32 or w_out is None or w_out.shape != (N, n_out) or w_out.dtype != x.dtype:
            raise ValueError("linear_w8: outlier_idx must be int32 [n_out] and w_out [N, n_out] in the dtype of x")
        if n_out > K:
            raise ValueError(f"linear_w8: {n_out} outlier columns for K = {K}")
        w_out = w_out.contiguous()
        outlier_idx = outlier_idx.contiguous()
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    b = bias.contiguous() if bias is not None else None
    with _on_device(x.device):
        _check(
            lib().tpamd_linear_w8(x2.data_ptr(), wq.data_ptr(), scale_.contiguous().data_ptr(),
                                  outlier_idx.data_ptr() if n_out else None, w_out.data_ptr() if n_out else None, n_out,
                                  b.data_ptr() if b is not None else None, y.data_ptr(), M, N, K, _ld(x2), K, max(n_out, 1), N,
                                  dtype_code(x.dtype), act, ctypes.c_void_p(current_stream_ptr(x.device))),
            "tpamd_linear_w8",
        )
    return y.view(*x.shape[:-1], N)
