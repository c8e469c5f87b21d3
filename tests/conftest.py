import sys
from pathlib import Path

import numpy as np
import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (run on the MI355X box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no HIP device")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def to_bits(t: torch.Tensor) -> np.ndarray:
    """Raw element bits of a CPU tensor as a numpy array (bf16/fp16 -> uint16, fp32 -> uint32, ints as is)."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.float32:
        return t.view(torch.int32).numpy().view(np.uint32)
    return t.numpy()


def run_jobs_on_host(jobs, buffers):
    """Execute 2-D byte-region copy jobs on numpy byte buffers. `buffers`: {base_address: np.uint8 array}; job
    addresses are base + offset. Used to check the job tables the product builds without a GPU."""
    bases = sorted(buffers)

    def locate(addr):
        for b in reversed(bases):
            if addr >= b:
                assert addr - b <= buffers[b].size, "address outside every buffer"
                return buffers[b], addr - b
        raise AssertionError("address below every buffer")

    for src, dst, rows, row_bytes, sp, dp in jobs:
        sbuf, soff = locate(src)
        dbuf, doff = locate(dst)
        for r in range(rows):
            s0 = soff + r * (sp if rows > 1 else 0)
            d0 = doff + r * (dp if rows > 1 else 0)
            assert s0 + row_bytes <= sbuf.size and d0 + row_bytes <= dbuf.size
            dbuf[d0 : d0 + row_bytes] = sbuf[s0 : s0 + row_bytes]


@pytest.fixture
def tune(monkeypatch):
    """Sets a TPAMD_* tuning knob for one test: the library reads its environment once, so it is told to read it again,
    and once more when the variable is gone."""
    from tensor_parallel_amd import _native

    def set_knob(name, value):
        monkeypatch.setenv(name, str(value))
        _native.reload_tuning()

    yield set_knob
    monkeypatch.undo()
    if _native.available():
        _native.reload_tuning()
