"""Validation, output allocation and device-memory budget for the kernel-vector drivers.

Same rules as falkon/mmv_ops/utils.py:36-58,124-155.
"""
from typing import Optional, Sequence, Tuple

import time

import torch

from ..utils.tensor_helpers import create_C, create_fortran, create_same_stride, is_contig

__all__ = ("check_contiguity", "create_output_mat", "usable_gpu_memory", "retry_with_fresh_memory_report")


def check_contiguity(*args: Tuple[Optional[torch.Tensor], str]) -> None:
    """Every given tensor needs a unit stride (falkon/mmv_ops/utils.py:36-39)."""
    for tensor, name in args:
        if tensor is not None and not is_contig(tensor):
            raise ValueError(f"Tensor '{name}' must be memory contiguous")


def create_output_mat(out: Optional[torch.Tensor], data_devs: Sequence[torch.device], shape: Tuple[int, int],
                      dtype: torch.dtype, other_mat: torch.Tensor, output_stride: Optional[str] = None) -> torch.Tensor:
    """Return ``out`` if given, else a new matrix on the first GPU the data lives on (the host,
    pinned, if all data is on the host) laid out like ``other_mat``
    (falkon/mmv_ops/utils.py:124-155)."""
    if out is not None:
        return out
    out_dev = torch.device("cpu")
    for ddev in data_devs:
        if ddev.type == "cuda":
            out_dev = ddev
            break
    pin = out_dev.type != "cuda"
    if output_stride is None:
        return create_same_stride(shape, other_mat, dtype, device=out_dev, pin_memory=pin)
    if output_stride == "F":
        return create_fortran(shape, dtype, device=out_dev, pin_memory=pin)
    return create_C(shape, dtype, device=out_dev, pin_memory=pin)


# Asking the driver for the free memory takes longer (about 12 microseconds) than the host side of everything else in
# a small product, so a call that needs at most 1/8 of what the driver reported within the last 50 ms reuses that
# report; the value returned is then 1/8 of it, which such a call fits unless somebody allocated seven eighths of the
# free memory in between.  Reading the allocator's counters to notice that would cost more than the report itself, so
# the drivers guard the other end instead: a product that runs out of memory on a plan made from a reused report is
# planned again from a fresh one (retry_with_fresh_memory_report).
_recent_free = {}
_reused = set()        # devices whose last budget came from a reused report
_FREE_MEMORY_TTL = 0.05
_SMALL_CALL_MARGIN = 8.0


def usable_gpu_memory(dev: torch.device, max_gpu_mem: float, slack: float, enough: float = float("inf")) -> float:
    """Bytes a call may use on ``dev``: ``slack * min(free, max_gpu_mem)``
    (falkon/mmv_ops/utils.py:47-58; free memory counts what torch's allocator holds cached,
    falkon/utils/devices.py:84-96).  Raises MemoryError when nothing is left.

    ``enough`` is what the caller needs at most: when the memory the driver reports free already covers it, the
    allocator's statistics (by far the slowest part of a small call: two passes over a few hundred counters) are
    not read, and the value returned is a lower bound of the usable memory that is at least ``enough``."""
    key = (dev.type, dev.index)
    seen = _recent_free.get(key)
    now = time.monotonic()
    if seen is not None and now - seen[1] < _FREE_MEMORY_TTL and _SMALL_CALL_MARGIN * enough <= seen[0] * slack:
        _reused.add(key)
        return min(seen[0] * slack / _SMALL_CALL_MARGIN, max_gpu_mem * slack)
    _reused.discard(key)
    free, _total = torch.cuda.mem_get_info(dev)
    _recent_free[key] = (free, now)
    usable = min(free * slack, max_gpu_mem * slack)
    if usable >= enough:
        return usable
    cached = torch.cuda.memory_reserved(dev) - torch.cuda.memory_allocated(dev)
    usable = min((free + cached) * slack, max_gpu_mem * slack)
    if usable < 0:
        raise MemoryError(f"Usable memory on device {dev} is less than 0. Either there is no free memory "
                          f"available, or the `max_gpu_mem` setting is too low.")
    return usable


def retry_with_fresh_memory_report(run):
    """``run()``; if it runs out of device memory on a plan that was made from a reused free-memory report, forget the
    reports and run it once more (the second plan asks the driver, sees what is really free and splits the rows)."""
    try:
        return run()
    except torch.cuda.OutOfMemoryError:
        if not _reused:
            raise
        _reused.clear()
        _recent_free.clear()
        return run()
