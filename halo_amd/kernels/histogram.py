"""Sync-free histograms for MoE routing (no host readback; counts are exact).

Mirrors the reference's ``halo/kernels/histogram.py:9-26``; the kernels are behind ``hmoe_bincount`` in
``csrc/route_sort.hip`` (LDS counters; many workgroups for large inputs, any number of bins).
"""

from __future__ import annotations

import torch

from halo_amd import _lib
from halo_amd.kernels import _cpu


def sync_free_bincount(
    indices: torch.Tensor, size: int, *, dtype: torch.dtype = torch.float32, weights: torch.Tensor | None = None
) -> torch.Tensor:
    """Counts (or weight sums) of each value in ``[0, size)``; values outside the range are ignored.  ``dtype`` is
    fp32 where counts feed metric math, int64 where they become offsets."""
    if not indices.is_cuda:
        return _cpu.bincount(indices, size, dtype, weights)
    device = _lib.require_device(indices, weights)
    flat = indices.flatten().long().contiguous()
    native = torch.int64 if (weights is None and not dtype.is_floating_point) else torch.float32
    w = None if weights is None else weights.flatten().float().contiguous()
    out = torch.empty(size, dtype=native, device=device)
    with _lib.on_device(device):
        _lib.call("hmoe_bincount", _lib.ptr(flat), _lib.ptr(w), flat.numel(), size, int(native == torch.int64),
                  _lib.ptr(out), _lib.stream_ptr(device))
    return out if out.dtype == dtype else out.to(dtype)


def accumulate_bincount(
    counter: torch.Tensor | None, indices: torch.Tensor, size: int, *, weights: torch.Tensor | None = None
) -> torch.Tensor:
    """Adds this call's histogram into ``counter`` in place and returns it; with no counter yet (None before the first
    forward that routes) the histogram itself becomes the counter."""
    fresh = sync_free_bincount(indices, size, weights=weights)
    if counter is None:
        return fresh
    return counter.add_(fresh)
