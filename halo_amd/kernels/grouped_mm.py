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
from halo_amd.kernels import _cpu

# Every operand row must start on a 16-byte boundary (8 bf16), as for torch's grouped GEMM.
GROUPED_MM_STRIDE_ALIGNMENT_BYTES = 16
# Kept for API parity: the reference warms two CUTLASS tiles picked around this row count; one binary serves here.
GROUPED_MM_SMALL_TILE_DIM = 128


_GEMM_TILES = {"auto": 0, "mono": 1, "duo": 2, "small": 3}


class gemm_tile:
    """Forces one of the bf16 grouped GEMM's three tile configurations for every product of the process, as a context
    manager or by ``gemm_tile.set(name)``: ``"mono"`` is the 256 x 256 tile on one workgroup per compute unit, ``"duo"``
    the 128 x 256 tile on two, ``"small"`` the 128 x 128 tile on three, ``"auto"`` (the default) the largest of which
    the product has a tile per compute unit.  All give the same bits; a
    tuning and test switch with no counterpart in the reference (``HALO_GEMM_TILE`` sets the initial value)."""

    def __init__(self, name: str):
        self.name = name
        self.before = None

    @staticmethod
    def set(name: str) -> str:
        if name not in _GEMM_TILES:
            raise ValueError(f"unknown tile configuration {name!r}; expected one of {sorted(_GEMM_TILES)}")
        before = _lib.load().hmoe_set_gemm_tile(_GEMM_TILES[name])
        return next(k for k, v in _GEMM_TILES.items() if v == before)

    def __enter__(self):
        self.before = gemm_tile.set(self.name)
        return self

    def __exit__(self, *exc):
        gemm_tile.set(self.before)
        return False


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
    if mat_a.dtype != mat_b.dtype:
        raise TypeError(f"grouped_mm operands must share a dtype, got {mat_a.dtype} and {mat_b.dtype}")
    if mat_a.dim() != 2 or mat_b.dim() != 3 or mat_a.shape[1] != mat_b.shape[1]:
        raise ValueError(f"expected [R, K] x [G, K, N], got {tuple(mat_a.shape)} x {tuple(mat_b.shape)}")
    if not mat_a.is_cuda:
        return _cpu.grouped_forward(mat_a, mat_b, _offs_arg(offs, mat_b.shape[0]))
    device = _lib.require_device(mat_a, mat_b, offs)
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


grouped_mm_forward = _forward  # the forward product alone (no autograd node), for callers that build their own


def grouped_wgrad(mat_a: torch.Tensor, grad_output: torch.Tensor, offs: torch.Tensor | None,
                  groups: int) -> torch.Tensor:
    """``[groups, K, N]``: ``A[s:e]^T @ dO[s:e]`` per group, contiguous; an empty group's slice is exact zeros."""
    if grad_output.dtype != mat_a.dtype:
        raise TypeError("grouped_wgrad operands must share a dtype")
    if not mat_a.is_cuda:
        return _cpu.grouped_wgrad(mat_a, grad_output, _offs_arg(offs, groups), groups)
    device = _lib.require_device(mat_a, grad_output, offs)
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
    if grad_output.dtype != mat_a.dtype or mat_b.dtype != mat_a.dtype:
        raise TypeError("grouped_mm_grads operands must share a dtype")
    if not mat_a.is_cuda:
        offs32 = _offs_arg(offs, mat_b.shape[0])
        return (_cpu.grouped_dgrad(grad_output, mat_b, offs32) if needs_a else None,
                _cpu.grouped_wgrad(mat_a, grad_output, offs32, mat_b.shape[0]) if needs_b else None)
    device = _lib.require_device(mat_a, mat_b, grad_output, offs)
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
        a, b, offs = ctx.saved_tensors
        want_a, want_b = ctx.needs_input_grad[:2]
        return (*grouped_mm_grads(a, b, grad_output, offs, want_a, want_b), None)


def grouped_mm(mat_a, mat_b, *, offs=None):
    return _GroupedMMFunction.apply(mat_a, mat_b, offs)


# ------------------------------------------------------------------------------------ expert bias in the epilogue

def bias_fusable(mat_a: torch.Tensor, mat_b, bias) -> bool:
    """Whether ``grouped_mm_bias`` can take these operands: a plain contiguous ``[G, K, N]`` weight and a ``[G, N]``
    bias on the device, all of ``mat_a``'s dtype (bf16 or fp32)."""
    return (isinstance(mat_b, torch.Tensor) and isinstance(bias, torch.Tensor) and mat_a.is_cuda
            and mat_a.dtype in (torch.bfloat16, torch.float32) and mat_b.dtype == mat_a.dtype
            and bias.dtype == mat_a.dtype and mat_a.dim() == 2 and mat_b.dim() == 3 and mat_b.is_contiguous()
            and bias.dim() == 2 and bias.shape == (mat_b.shape[0], mat_b.shape[2]) and mat_a.shape[1] == mat_b.shape[1])


class _GroupedMMBias(Function):
    """``grouped_mm(mat_a, mat_b, offs) + bias[eids]`` as one node: the GEMM's epilogue adds the expert's bias row
    (``hmoe_grouped_gemm_fwd_bias``), rounding the product first and the sum again as the two tensor operations do
    (reference ``families/gpt_oss.py:153-159``: ``_expert_proj`` then ``+ MoEExpertBiasGather.apply(bias, eids)``), so
    neither the gathered ``[R, N]`` bias nor the sum's extra pass exists.  The bias gradient is the per-expert column
    sum of ``grad_output``, as ``MoEExpertBiasGather.backward`` computes it."""

    @staticmethod
    def forward(ctx, mat_a, mat_b, bias, offs, eids):
        device = _lib.require_device(mat_a, mat_b, bias, offs, eids)
        groups, k, n = mat_b.shape
        rows = mat_a.shape[0]
        offs32 = _offs_arg(offs, groups)
        ctx.save_for_backward(mat_a, mat_b, offs32, eids)
        out = torch.empty((rows, n), dtype=mat_a.dtype, device=device)
        if rows == 0 or n == 0:
            return out
        a = _rows(mat_a)
        bias = bias.contiguous()
        with _lib.on_device(device):
            _lib.call("hmoe_grouped_gemm_fwd_bias", _lib.ptr(a), a.stride(0), _lib.ptr(mat_b), _lib.ptr(bias),
                      _lib.ptr(offs32), rows, groups, k, n, _lib.dtype_id(mat_a.dtype), _lib.ptr(out), out.stride(0),
                      _lib.stream_ptr(device))
        return out

    @staticmethod
    def backward(ctx, grad_output):
        from halo_amd.kernels.moe_permute import expert_bias_grad

        mat_a, mat_b, offs32, eids = ctx.saved_tensors
        grad_a, grad_b = grouped_mm_grads(mat_a, mat_b, grad_output, offs32, ctx.needs_input_grad[0],
                                          ctx.needs_input_grad[1])
        grad_bias = expert_bias_grad(grad_output, eids, mat_b.shape[0]) if ctx.needs_input_grad[2] else None
        return grad_a, grad_b, grad_bias, None, None


def grouped_mm_bias(mat_a, mat_b, bias, *, offs, eids):
    """``grouped_mm(mat_a, mat_b, offs=offs) + bias[eids]`` with ``eids`` the sorted expert id of every row (the ids
    ``offs`` are the ends of); see ``bias_fusable`` for the operands it takes."""
    return _GroupedMMBias.apply(mat_a, mat_b, bias, offs, eids)


# --------------------------------------------------------------------------- a scaled product added to a tensor

class _GroupedMMAddTo(Function):
    """``addend + scale * grouped_mm(mat_a, mat_b, offs)`` as one node: the product's epilogue multiplies by ``scale``
    and adds ``addend`` (``hmoe_grouped_gemm_fwd_addto``), rounding where the tensor operations round, so the result
    carries their bits and neither the product nor its multiple is written.  The adapted expert projection of the
    reference, ``out + scaling * grouped_mm(hidden, lora_b)`` (``compute.py:283-294``), with ``mat_a`` the adapter's
    low-rank activations.  The gradients are those operations' own: ``grad_addend = grad_out``, and the product's two
    gradients over ``scale * grad_out``."""

    @staticmethod
    def forward(ctx, mat_a, mat_b, addend, scale, offs):
        device = _lib.require_device(mat_a, mat_b, addend, offs)
        groups, k, n = mat_b.shape
        rows = mat_a.shape[0]
        offs32 = _offs_arg(offs, groups)
        ctx.scale = float(scale)
        ctx.save_for_backward(mat_a, mat_b, offs32)
        out = torch.empty((rows, n), dtype=mat_a.dtype, device=device)
        if rows == 0 or n == 0:
            return out
        a, base = _rows(mat_a), _rows(addend)
        with _lib.on_device(device):
            _lib.call("hmoe_grouped_gemm_fwd_addto", _lib.ptr(a), a.stride(0), _lib.ptr(mat_b), _lib.ptr(offs32), rows,
                      groups, k, n, _lib.dtype_id(mat_a.dtype), _lib.ptr(base), base.stride(0), ctx.scale,
                      _lib.ptr(out), out.stride(0), _lib.stream_ptr(device))
        return out

    @staticmethod
    def backward(ctx, grad_output):
        mat_a, mat_b, offs32 = ctx.saved_tensors
        grad_a = grad_b = None
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            scaled = grad_output * ctx.scale  # the gradient of `scale * product`, rounded as autograd rounds it
            grad_a, grad_b = grouped_mm_grads(mat_a, mat_b, scaled, offs32, ctx.needs_input_grad[0],
                                              ctx.needs_input_grad[1])
        return grad_a, grad_b, grad_output if ctx.needs_input_grad[2] else None, None, None


def addto_fusable(mat_a: torch.Tensor, mat_b, addend) -> bool:
    """Whether :func:`grouped_mm_addto` can take these operands: a plain contiguous ``[G, K, N]`` weight and an
    ``[R, N]`` addend on the device, all of ``mat_a``'s dtype (bf16 or fp32), rows of 16-byte multiples in bf16."""
    if not (isinstance(mat_b, torch.Tensor) and isinstance(addend, torch.Tensor) and isinstance(mat_a, torch.Tensor)
            and mat_a.is_cuda and mat_a.dtype in (torch.bfloat16, torch.float32) and mat_b.dtype == mat_a.dtype
            and addend.dtype == mat_a.dtype and mat_a.dim() == 2 and mat_b.dim() == 3 and mat_b.is_contiguous()
            and addend.dim() == 2 and addend.shape == (mat_a.shape[0], mat_b.shape[2])
            and mat_a.shape[1] == mat_b.shape[1]):
        return False
    return mat_a.dtype == torch.float32 or (mat_b.shape[1] % 8 == 0 and mat_b.shape[2] % 8 == 0)


def grouped_mm_addto(mat_a, mat_b, addend, scale: float, *, offs):
    """``addend + scale * grouped_mm(mat_a, mat_b, offs=offs)``; see :class:`_GroupedMMAddTo` and
    :func:`addto_fusable`."""
    return _GroupedMMAddTo.apply(mat_a, mat_b, addend, scale, offs)


# ------------------------------------------------------------------------------------- permute folded into the GEMM

def gather_fusable(tokens: torch.Tensor, mat_b) -> bool:
    """Whether ``gather_grouped_mm`` can take these operands: bf16 rows of 16-byte multiples on the device and a plain
    contiguous ``[G, K, N]`` weight of the same dtype."""
    return (isinstance(mat_b, torch.Tensor) and tokens.is_cuda and tokens.dtype == torch.bfloat16
            and mat_b.dtype == torch.bfloat16 and mat_b.dim() == 3 and mat_b.is_contiguous() and tokens.dim() == 2
            and tokens.stride(-1) == 1 and tokens.stride(0) % 8 == 0 and tokens.shape[1] % 8 == 0
            and mat_b.shape[2] % 8 == 0 and tokens.shape[1] == mat_b.shape[1])


def _gather_forward(tokens, row_index, mat_b, bias, offs32) -> torch.Tensor:
    """``tokens[row_index] @ mat_b (+ bias row of the row's group)`` through the gathering forward kernel."""
    device = tokens.device
    groups, k, n = mat_b.shape
    rows = row_index.shape[0]
    out = torch.empty((rows, n), dtype=tokens.dtype, device=device)
    if rows and n:
        with _lib.on_device(device):
            if bias is None:
                _lib.call("hmoe_grouped_gemm_fwd_gather", _lib.ptr(tokens), tokens.stride(0), tokens.shape[0],
                          _lib.ptr(row_index), _lib.ptr(mat_b), _lib.ptr(offs32), rows, groups, k, n,
                          _lib.dtype_id(tokens.dtype), _lib.ptr(out), out.stride(0), _lib.stream_ptr(device))
            else:
                _lib.call("hmoe_grouped_gemm_fwd_gather_bias", _lib.ptr(tokens), tokens.stride(0), tokens.shape[0],
                          _lib.ptr(row_index), _lib.ptr(mat_b), _lib.ptr(bias), _lib.ptr(offs32), rows, groups, k, n,
                          _lib.dtype_id(tokens.dtype), _lib.ptr(out), out.stride(0), _lib.stream_ptr(device))
    return out


def _gather_wgrad(tokens, row_index, grad_output, offs32, groups: int) -> torch.Tensor:
    """``[groups, K, N]``: ``tokens[row_index][s:e]^T @ grad_output[s:e]`` per group, the rows fetched by index."""
    device = tokens.device
    rows, k, n = row_index.shape[0], tokens.shape[1], grad_output.shape[1]
    grad_b = torch.empty((groups, k, n), dtype=tokens.dtype, device=device)
    if k and n:
        with _lib.on_device(device):
            _lib.call("hmoe_grouped_gemm_wgrad_gather", _lib.ptr(tokens), tokens.stride(0), tokens.shape[0],
                      _lib.ptr(row_index), _lib.ptr(grad_output), grad_output.stride(0) if rows else n,
                      _lib.ptr(offs32), rows, groups, k, n, _lib.dtype_id(tokens.dtype), _lib.ptr(grad_b),
                      _lib.stream_ptr(device))
    return grad_b


class _GatherGroupedMM(Function):
    """``grouped_mm(tokens[row_index], mat_b, offs)`` without the permuted copy: the GEMM's loader and its weight
    gradient's fetch the rows through ``row_index`` (``hmoe_grouped_gemm_fwd_gather`` / ``_wgrad_gather``).  This is
    ``MoEGatherPermute`` followed by ``grouped_mm`` (reference ``moe_permute.py:130-141`` + ``grouped_mm.py:30-47``)
    as one autograd node; the gradient for ``tokens`` is the dgrad scattered back with the atomic-free gather-reduce
    over ``inv_map``, exactly as ``MoEGatherPermute.backward`` does."""

    @staticmethod
    def forward(ctx, tokens, row_index, inv_map, mat_b, offs):
        _lib.require_device(tokens, row_index, inv_map, mat_b, offs)
        row_index = row_index.long().contiguous()
        offs32 = _offs_arg(offs, mat_b.shape[0])
        ctx.save_for_backward(tokens, row_index, inv_map, mat_b, offs32)
        return _gather_forward(tokens, row_index, mat_b, None, offs32)

    @staticmethod
    def backward(ctx, grad_output):
        from halo_amd.kernels.moe_permute import gather_reduce_rows

        tokens, row_index, inv_map, mat_b, offs32 = ctx.saved_tensors
        groups, k, n = mat_b.shape
        rows = row_index.shape[0]
        grad_output = _rows(grad_output) if grad_output.numel() else grad_output.new_empty(grad_output.shape)
        grad_tokens = grad_b = None
        if ctx.needs_input_grad[0]:
            shape_only = grad_output.new_empty((1, k)).expand(rows, k)  # dgrad reads mat_a's shape and dtype only
            grad_sorted, _ = grouped_mm_grads(shape_only, mat_b, grad_output, offs32, True, False)
            grad_tokens = gather_reduce_rows(grad_sorted, inv_map)
        if ctx.needs_input_grad[3]:
            grad_b = _gather_wgrad(tokens, row_index, grad_output, offs32, groups)
        return grad_tokens, None, None, grad_b, None


def gather_grouped_mm(tokens, row_index, inv_map, mat_b, *, offs):
    """``grouped_mm(tokens[row_index], mat_b, offs=offs)``; see :class:`_GatherGroupedMM`.  The caller checks
    :func:`gather_fusable` first."""
    return _GatherGroupedMM.apply(tokens, row_index, inv_map, mat_b, offs)


def pair_fusable(tokens: torch.Tensor, mat_b1, bias1, mat_b2, bias2) -> bool:
    """Whether :func:`gather_grouped_mm_pair` can take these operands: both weights as :func:`gather_fusable` asks,
    and both biases either absent or ``[G, N]`` of the rows' dtype."""
    def bias_ok(bias, mat_b):
        return bias is None or (isinstance(bias, torch.Tensor) and bias.dtype == tokens.dtype and bias.is_cuda
                                and bias.dim() == 2 and bias.shape == (mat_b.shape[0], mat_b.shape[2]))

    return (gather_fusable(tokens, mat_b1) and gather_fusable(tokens, mat_b2) and mat_b1.shape[0] == mat_b2.shape[0]
            and bias_ok(bias1, mat_b1) and bias_ok(bias2, mat_b2))


class _GatherGroupedMMPair(Function):
    """Two projections of the same gathered rows as one node: ``(tokens[row_index] @ w1 + b1[eids],
    tokens[row_index] @ w2 + b2[eids])``, the gate and up projections of a layer that stores them apart (reference
    ``families/gpt_oss.py:139-160``).  Both fetch the rows through ``row_index`` and add their bias in the epilogue, so
    the permuted copy is never written.  In backward the reference's autograd adds the two projections' input
    gradients at the rows' node and then scatters the sum back (``moe_permute.py:138-141``); here the second input
    gradient joins the first in its epilogue (``hmoe_grouped_gemm_dgrad_addto``: each product rounded, then the sum,
    as the tensor addition rounds), and one gather-reduce follows: the same bits without the ``[R, K]`` pass that adds
    them."""

    @staticmethod
    def forward(ctx, tokens, row_index, inv_map, w1, b1, w2, b2, offs, eids):
        _lib.require_device(tokens, row_index, inv_map, w1, b1, w2, b2, offs, eids)
        row_index = row_index.long().contiguous()
        offs32 = _offs_arg(offs, w1.shape[0])
        ctx.save_for_backward(tokens, row_index, inv_map, w1, w2, offs32, eids)
        return (_gather_forward(tokens, row_index, w1, None if b1 is None else b1.contiguous(), offs32),
                _gather_forward(tokens, row_index, w2, None if b2 is None else b2.contiguous(), offs32))

    @staticmethod
    def backward(ctx, grad1, grad2):
        from halo_amd.kernels.moe_permute import expert_bias_grad, gather_reduce_rows

        tokens, row_index, inv_map, w1, w2, offs32, eids = ctx.saved_tensors
        device = tokens.device
        groups, k = w1.shape[0], w1.shape[1]
        rows = row_index.shape[0]
        grad1 = _rows(grad1) if grad1.numel() else grad1.new_empty(grad1.shape)
        grad2 = _rows(grad2) if grad2.numel() else grad2.new_empty(grad2.shape)
        need = ctx.needs_input_grad
        grad_tokens = None
        if need[0]:
            shape_only = grad1.new_empty((1, k)).expand(rows, k)  # dgrad reads mat_a's shape and dtype only
            grad_sorted, _ = grouped_mm_grads(shape_only, w1, grad1, offs32, True, False)
            if rows and k:
                with _lib.on_device(device):
                    _lib.call("hmoe_grouped_gemm_dgrad_addto", _lib.ptr(grad2), grad2.stride(0), _lib.ptr(w2),
                              _lib.ptr(offs32), rows, groups, k, w2.shape[2], _lib.dtype_id(tokens.dtype),
                              _lib.ptr(grad_sorted), grad_sorted.stride(0), _lib.ptr(grad_sorted),
                              grad_sorted.stride(0), _lib.stream_ptr(device))
            grad_tokens = gather_reduce_rows(grad_sorted, inv_map)
        grad_w1 = _gather_wgrad(tokens, row_index, grad1, offs32, groups) if need[3] else None
        grad_w2 = _gather_wgrad(tokens, row_index, grad2, offs32, groups) if need[5] else None
        grad_b1 = expert_bias_grad(grad1, eids, groups) if need[4] else None
        grad_b2 = expert_bias_grad(grad2, eids, groups) if need[6] else None
        return grad_tokens, None, None, grad_w1, grad_b1, grad_w2, grad_b2, None, None


def gather_grouped_mm_pair(tokens, row_index, inv_map, mat_b1, bias1, mat_b2, bias2, *, offs, eids):
    """``(grouped_mm(tokens[row_index], mat_b1) + bias1[eids], grouped_mm(tokens[row_index], mat_b2) + bias2[eids])``
    (a bias may be None); see :class:`_GatherGroupedMMPair`.  The caller checks :func:`pair_fusable` first."""
    return _GatherGroupedMMPair.apply(tokens, row_index, inv_map, mat_b1, bias1, mat_b2, bias2, offs, eids)


# ------------------------------------------------------------------------- down projection + plain combine

def combine_fusable(mat_a: torch.Tensor, mat_b, hidden_dtype: torch.dtype) -> bool:
    """Whether :func:`grouped_mm_combine` can take these operands: bf16 rows of 16-byte multiples on the device and a
    plain contiguous ``[G, K, N]`` bf16 weight, the layer's output in bf16 as well."""
    return (isinstance(mat_b, torch.Tensor) and isinstance(mat_a, torch.Tensor) and mat_a.is_cuda
            and mat_a.dtype == torch.bfloat16 and mat_b.dtype == torch.bfloat16 and hidden_dtype == torch.bfloat16
            and mat_b.dim() == 3 and mat_b.is_contiguous() and mat_a.dim() == 2 and mat_a.shape[1] == mat_b.shape[1]
            and mat_b.shape[1] % 8 == 0 and mat_b.shape[2] % 8 == 0)


class _GroupedMMCombine(Function):
    """``out[t] = sum over the sorted rows j of token t of (mat_a @ mat_b)[j]  (+ scale[t] * addend[t])``: a grouped
    product whose output rows are summed per token through ``inv_map`` without weights (``mat_a``'s rows already
    carry the gate weights).  One autograd node, so the ``[R, N]`` product is not kept and its gradient never exists:
    ``grad_a = grad_out[row_index] @ mat_b^T`` and ``grad_b = mat_a^T @ grad_out[row_index]`` fetch the token
    gradient's rows through ``row_index`` (``hmoe_grouped_gemm_dgrad_gather`` / ``_wgrad_gather_grad``).  Replaces
    the reference's ``grouped_mm`` (``grouped_mm.py:30-47``) + ``MoEWeightedUnpermute`` (``moe_permute.py:144-189``)
    pair on the down projection; ``addend`` / ``scale`` as in ``MoEWeightedUnpermuteAdd``."""

    @staticmethod
    def forward(ctx, mat_a, mat_b, offs, row_index, inv_map, addend, scale):
        from halo_amd.kernels.moe_permute import gather_reduce_rows

        offs32 = _offs_arg(offs, mat_b.shape[0])
        row_index = row_index.long().contiguous()
        product = _forward(mat_a, mat_b, offs32)
        ctx.scaled = scale is not None
        ctx.scale_shape = scale.shape if ctx.scaled else None
        ctx.tokens = inv_map.shape[0]
        ctx.save_for_backward(mat_a, mat_b, offs32, row_index,
                              addend if ctx.scaled and ctx.needs_input_grad[6] else None, scale)
        return gather_reduce_rows(product, inv_map, None, addend=addend, addend_scale=scale)

    @staticmethod
    def backward(ctx, grad_out):
        from halo_amd.kernels.moe_permute import _unpermute_backward

        mat_a, mat_b, offs32, row_index, addend, scale = ctx.saved_tensors
        device = mat_a.device
        groups, k, n = mat_b.shape
        rows = mat_a.shape[0]
        # under EP the gradient arrives as a row-strided view of the padded transport buffer, read in place
        if grad_out.stride(-1) != 1 or grad_out.stride(0) % 8 or grad_out.data_ptr() % 16:
            grad_out = grad_out.contiguous()
        grad_a = grad_b = grad_addend = grad_scale = None
        dtype = _lib.dtype_id(mat_a.dtype)
        with _lib.on_device(device):
            if ctx.needs_input_grad[0]:
                grad_a = torch.empty((rows, k), dtype=mat_a.dtype, device=device)
                if rows and k:
                    _lib.call("hmoe_grouped_gemm_dgrad_gather", _lib.ptr(grad_out), grad_out.stride(0),
                              grad_out.shape[0], _lib.ptr(row_index), _lib.ptr(mat_b), _lib.ptr(offs32), rows, groups,
                              k, n, dtype, _lib.ptr(grad_a), grad_a.stride(0), _lib.stream_ptr(device))
            if ctx.needs_input_grad[1]:
                grad_b = torch.empty((groups, k, n), dtype=mat_a.dtype, device=device)
                a = _rows(mat_a)
                if k and n:
                    _lib.call("hmoe_grouped_gemm_wgrad_gather_grad", _lib.ptr(a), a.stride(0) if rows else k,
                              _lib.ptr(grad_out), grad_out.stride(0) if grad_out.shape[0] else n, grad_out.shape[0],
                              _lib.ptr(row_index), _lib.ptr(offs32), rows, groups, k, n, dtype, _lib.ptr(grad_b),
                              _lib.stream_ptr(device))
        if not ctx.scaled:
            grad_addend = grad_out if ctx.needs_input_grad[5] else None
        elif ctx.needs_input_grad[5] or ctx.needs_input_grad[6]:
            # every row its own token: scale[r] * grad_out[r] and <grad_out[r], addend[r]>
            own = torch.arange(grad_out.shape[0], device=device)
            want_scale = ctx.needs_input_grad[6]
            grad_addend, grad_scale = _unpermute_backward(grad_out, addend, scale.reshape(-1), own, want_scale)
            if want_scale:
                grad_scale = grad_scale.to(scale.dtype).view(ctx.scale_shape)
        return grad_a, grad_b, None, None, None, grad_addend, grad_scale


def grouped_mm_combine(mat_a, mat_b, *, offs, row_index, inv_map, addend=None, scale=None):
    """``gather_reduce_rows(grouped_mm(mat_a, mat_b, offs=offs), inv_map) (+ scale[:, None] * addend)``; see
    :class:`_GroupedMMCombine`.  The caller checks :func:`combine_fusable` first."""
    return _GroupedMMCombine.apply(mat_a, mat_b, offs, row_index, inv_map, addend, scale)


class GatheredRows:
    """``tokens[row_index]`` that nobody has copied yet: what the sort hands to the first expert projection when that
    projection can fetch the rows itself (:func:`gather_grouped_mm`).  A consumer that cannot calls
    :meth:`materialize`, which is ``MoEGatherPermute`` (reference ``moe_permute.py:130-141``), once."""

    def __init__(self, tokens: torch.Tensor, row_index: torch.Tensor, inv_map: torch.Tensor):
        self.tokens, self.row_index, self.inv_map = tokens, row_index, inv_map
        self._rows = None

    @property
    def shape(self):
        return torch.Size((self.row_index.shape[0], self.tokens.shape[1]))

    @property
    def dtype(self):
        return self.tokens.dtype

    @property
    def device(self):
        return self.tokens.device

    def to(self, dtype: torch.dtype) -> "GatheredRows":
        return self if dtype == self.tokens.dtype else GatheredRows(self.tokens.to(dtype), self.row_index, self.inv_map)

    def materialize(self) -> torch.Tensor:
        if self._rows is None:
            from halo_amd.kernels.moe_permute import MoEGatherPermute

            self._rows = MoEGatherPermute.apply(self.tokens, self.row_index, self.inv_map)
        return self._rows

    def grouped_mm(self, mat_b, *, offs) -> torch.Tensor | None:
        """The projection through the gathering kernels, or None when these operands do not qualify."""
        if not gather_fusable(self.tokens, mat_b):
            return None
        return gather_grouped_mm(self.tokens, self.row_index, self.inv_map, mat_b, offs=offs)

    def grouped_mm_pair(self, mat_b1, bias1, mat_b2, bias2, *, offs, eids):
        """Two biased projections of these rows through the gathering kernels as one node, or None when the operands
        do not qualify."""
        if not pair_fusable(self.tokens, mat_b1, bias1, mat_b2, bias2):
            return None
        return gather_grouped_mm_pair(self.tokens, self.row_index, self.inv_map, mat_b1, bias1, mat_b2, bias2,
                                      offs=offs, eids=eids)

