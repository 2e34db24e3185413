"""Grouped GEMM over rows stacked by expert, with its two gradients, on hand-written MFMA kernels
(``csrc/grouped_gemm.hip``).

Mirrors the reference's ``halo/kernels/grouped_mm.py`` (``grouped_mm`` ``:50-51``, ``grouped_mm_grads`` ``:16-27``,
``_GroupedMMFunction`` ``:30-47``), whose arithmetic is torch's ``F.grouped_mm``: ``mat_a [R, K]`` times
``mat_b [G, K, N]`` with ``offs`` the int32 inclusive group ends; the output carries ``mat_a``'s dtype.
"""

from __future__ import annotations

import torch
from torch.autograd import Function

from halo_amd import _lib

# Every operand row must start on a 16-byte boundary (8 bf16), as for torch's grouped GEMM.
GROUPED_MM_STRIDE_ALIGNMENT_BYTES = 16
# Kept for API parity: the reference warms two CUTLASS tiles picked around this row count; one binary serves here.
GROUPED_MM_SMALL_TILE_DIM = 128


def _rows(t: torch.Tensor) -> torch.Tensor:
    """A 2-D operand with unit inner stride (row stride free)."""
    return t if t.stride(-1) == 1 and t.stride(0) >= t.shape[1] else t.contiguous()


def _offs_arg(offs: torch.Tensor | None, groups: int):
    if offs is None:
        if groups != 1:
            raise ValueError("grouped_mm without offs takes a single group (mat_b [1, K, N])")
        return None
    if offs.numel() != groups:
        raise ValueError(f"{offs.numel()} group ends for {groups} groups")
    return offs.to(torch.int32).contiguous()


def _forward(mat_a: torch.Tensor, mat_b: torch.Tensor, offs: torch.Tensor | None) -> torch.Tensor:
    device = _lib.require_device(mat_a, mat_b, offs)
    if mat_a.dtype != mat_b.dtype:
        raise TypeError(f"grouped_mm operands must share a dtype, got {mat_a.dtype} and {mat_b.dtype}")
    if mat_a.dim() != 2 or mat_b.dim() != 3 or mat_a.shape[1] != mat_b.shape[1]:
        raise ValueError(f"expected [R, K] x [G, K, N], got {tuple(mat_a.shape)} x {tuple(mat_b.shape)}")
    groups, k, n = mat_b.shape
    rows = mat_a.shape[0]
    out = torch.empty((rows, n), dtype=mat_a.dtype, device=device)
    if rows == 0 or n == 0:
        return out
    mat_a = _rows(mat_a)
    offs32 = _offs_arg(offs, groups)
    dtype = _lib.dtype_id(mat_a.dtype)
    with _lib.on_device(device):
        if mat_b.is_contiguous():
            _lib.call("hmoe_grouped_gemm_fwd", _lib.ptr(mat_a), mat_a.stride(0), _lib.ptr(mat_b), _lib.ptr(offs32),
                      rows, groups, k, n, dtype, _lib.ptr(out), out.stride(0), _lib.stream_ptr(device))
        elif mat_b.transpose(-2, -1).is_contiguous():
            # mat_b is a transposed view of a contiguous [G, N, K] weight: out = A @ W^T, the dgrad kernel's form
            w = mat_b.transpose(-2, -1)
            _lib.call("hmoe_grouped_gemm_dgrad", _lib.ptr(mat_a), mat_a.stride(0), _lib.ptr(w), _lib.ptr(offs32),
                      rows, groups, n, k, dtype, _lib.ptr(out), out.stride(0), _lib.stream_ptr(device))
        else:
            w = mat_b.contiguous()
            _lib.call("hmoe_grouped_gemm_fwd", _lib.ptr(mat_a), mat_a.stride(0), _lib.ptr(w), _lib.ptr(offs32),
                      rows, groups, k, n, dtype, _lib.ptr(out), out.stride(0), _lib.stream_ptr(device))
    return out


def grouped_wgrad(mat_a: torch.Tensor, grad_output: torch.Tensor, offs: torch.Tensor | None,
                  groups: int) -> torch.Tensor:
    """``[groups, K, N]``: ``A[s:e]^T @ dO[s:e]`` per group, contiguous; an empty group's slice is exact zeros."""
    device = _lib.require_device(mat_a, grad_output, offs)
    if grad_output.dtype != mat_a.dtype:
        raise TypeError("grouped_wgrad operands must share a dtype")
    rows, k = mat_a.shape
    n = grad_output.shape[1]
    a = _rows(mat_a)
    grad_output = _rows(grad_output) if grad_output.numel() else grad_output.new_empty(grad_output.shape)
    offs32 = _offs_arg(offs, groups)
    grad_b = torch.empty((groups, k, n), dtype=mat_a.dtype, device=device)
    if k and n:
        with _lib.on_device(device):
            _lib.call("hmoe_grouped_gemm_wgrad", _lib.ptr(a), a.stride(0) if rows else k, _lib.ptr(grad_output),
                      grad_output.stride(0) if rows else n, _lib.ptr(offs32), rows, groups, k, n,
                      _lib.dtype_id(mat_a.dtype), _lib.ptr(grad_b), _lib.stream_ptr(device))
    return grad_b


def grouped_mm_grads(mat_a, mat_b, grad_output, offs, needs_a: bool, needs_b: bool):
    """``(grad_a, grad_b)``: ``dO @ B^T`` per group and ``A^T @ dO`` per group (an empty group's weight gradient is
    exact zeros).  ``grad_output`` and the operands must share a dtype.  A broadcast (zero-stride) gradient is
    materialised first."""
    device = _lib.require_device(mat_a, mat_b, grad_output, offs)
    if grad_output.dtype != mat_a.dtype or mat_b.dtype != mat_a.dtype:
        raise TypeError("grouped_mm_grads operands must share a dtype")
    groups, k, n = mat_b.shape
    rows = mat_a.shape[0]
    grad_output = _rows(grad_output) if grad_output.numel() else grad_output.new_empty(grad_output.shape)
    offs32 = _offs_arg(offs, groups)
    dtype = _lib.dtype_id(mat_a.dtype)
    grad_a = grad_b = None
    with _lib.on_device(device):
        if needs_a:
            grad_a = torch.empty((rows, k), dtype=mat_a.dtype, device=device)
            if rows and k:
                w = mat_b
                if w.is_contiguous():
                    _lib.call("hmoe_grouped_gemm_dgrad", _lib.ptr(grad_output), grad_output.stride(0), _lib.ptr(w),
                              _lib.ptr(offs32), rows, groups, k, n, dtype, _lib.ptr(grad_a), grad_a.stride(0),
                              _lib.stream_ptr(device))
                elif w.transpose(-2, -1).is_contiguous():
                    # B = W^T with W [G, N, K] contiguous: dA = dO @ W, the forward kernel's form
                    wt = w.transpose(-2, -1)
                    _lib.call("hmoe_grouped_gemm_fwd", _lib.ptr(grad_output), grad_output.stride(0), _lib.ptr(wt),
                              _lib.ptr(offs32), rows, groups, n, k, dtype, _lib.ptr(grad_a), grad_a.stride(0),
                              _lib.stream_ptr(device))
                else:
                    w = w.contiguous()
                    _lib.call("hmoe_grouped_gemm_dgrad", _lib.ptr(grad_output), grad_output.stride(0), _lib.ptr(w),
                              _lib.ptr(offs32), rows, groups, k, n, dtype, _lib.ptr(grad_a), grad_a.stride(0),
                              _lib.stream_ptr(device))
        if needs_b:
            grad_b = grouped_wgrad(mat_a, grad_output, offs32, groups)
            if not mat_b.is_contiguous() and mat_b.transpose(-2, -1).is_contiguous():
                # keep the gradient in the parameter's own layout
                grad_b = grad_b.transpose(-2, -1).contiguous().transpose(-2, -1)
    return grad_a, grad_b


class _GroupedMMFunction(Function):
    """The output carries ``mat_a``'s dtype (no autocast), and ``backward`` hands ``grad_output`` on uncast."""

    @staticmethod
    def forward(ctx, mat_a, mat_b, offs):
        if offs is not None:
            offs = offs.to(torch.int32)
        ctx.save_for_backward(mat_a, mat_b, offs)
        return _forward(mat_a, mat_b, offs)

    @staticmethod
    def backward(ctx, grad_output):
        mat_a, mat_b, offs = ctx.saved_tensors
        grad_mat_a, grad_mat_b = grouped_mm_grads(
            mat_a, mat_b, grad_output, offs, ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        )
        return grad_mat_a, grad_mat_b, None


def grouped_mm(mat_a, mat_b, *, offs=None):
    return _GroupedMMFunction.apply(mat_a, mat_b, offs)
