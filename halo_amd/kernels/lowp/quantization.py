"""Block-scaled quantisation for the expert GEMM: e4m3 (MXFP8) or e2m1 (MXFP4) elements plus one e8m0 power-of-two
scale per 32 values along the contraction axis, or e2m1 elements with an e4m3 scale per 16 values and one fp32 scale
per tensor (NVFP4); the straight-through fake-quant, and the per-step weight cache.

Mirrors ``halo/kernels/lowp/quantization.py`` of the reference for its three formats:
``BlockScaledTensor`` (:104-117), ``quantize_mxfp8`` (:236-245), ``quantize_mxfp4`` (:248-266), ``dequantize``
(:277-297), ``fake_quant`` (:350-365), ``WeightVersionCache`` / ``cached_fake_quant`` (:368-422).  The MXFP8 kernels are
``csrc/mxfp8.hip``; they write the operands in the layout the GEMM kernel loads (:class:`MxRows`, :class:`MxWeight`),
and the reference's logical layout is a byte permutation of those.  The MXFP4 kernels are ``csrc/mxfp4.hip``; they
write the reference's layout (two codes per byte along the quantised axis), the matrix kernel's operands
(:class:`Mx4Rows`, :class:`Mx4Weight`) and the round trip's bf16 result in one pass.  The NVFP4 kernels are
``csrc/nvfp4.hip`` (``quantize_nvfp4``, :209-226, :269-270): the reference's layout and the round trip, after a
reduction of the tensor's largest magnitude.
"""

from __future__ import annotations

import os
import weakref
from dataclasses import dataclass

import torch

from halo_amd import _lib
from halo_amd.kernels.lowp.spec import FORMAT_BLOCK_SIZE, require_implemented

E4M3_MAX = 448.0
BLOCK = FORMAT_BLOCK_SIZE["mxfp8"]
PANEL = 64  # contraction values that lie together in the GEMM's operand layout


@dataclass(frozen=True)
class BlockScaledTensor:
    """``data`` holds ``float8_e4m3fn`` elements in the source's shape, or, when ``packed``, two ``e2m1`` codes per byte
    (uint8, ``axis`` halved, the even element in the low nibble); ``scales`` one entry per block of ``block_size`` along
    ``axis``: an ``e8m0`` biased exponent (uint8) when ``pow2_scale`` (MX), an ``e4m3`` value otherwise (NVFP4).  An
    element is ``code x 2^(scales - 127)``, or ``code x scales x global_scale`` for NVFP4."""

    data: torch.Tensor
    scales: torch.Tensor
    block_size: int
    axis: int
    packed: bool = False
    pow2_scale: bool = True
    global_scale: torch.Tensor | None = None


@dataclass(frozen=True)
class MxRows:
    """Activation rows ``[R, K]`` as the GEMM loads them: ``q`` uint8 ``[ceil(K / 64), R, 64]`` (e4m3 codes in panels
    of 64 contraction values) and ``scales`` uint8 ``[K / 32, R]``."""

    q: torch.Tensor
    scales: torch.Tensor
    k: int

    @property
    def rows(self) -> int:
        return self.q.shape[1]


@dataclass(frozen=True)
class MxWeight:
    """Expert weights ``[G, K, N]`` quantised along K: ``q`` uint8 ``[G, ceil(K / 64), N, 64]``, ``scales`` uint8
    ``[G, K / 32, N]``, and ``dequant`` the round trip's bf16 ``[G, K, N]`` (None unless asked for)."""

    q: torch.Tensor
    scales: torch.Tensor
    dequant: torch.Tensor | None
    k: int


@dataclass(frozen=True)
class Mx4Rows:
    """Activation rows ``[R, K]`` as the e2m1 matrix kernel loads them: ``q`` uint8 ``[ceil(K / 128), R, 64]`` (two
    codes per byte, panels of 128 contraction values, zeros past K) and ``scales`` uint8 ``[ceil(K / 128), R, 4]``."""

    q: torch.Tensor
    scales: torch.Tensor
    k: int

    @property
    def rows(self) -> int:
        return self.q.shape[1]


@dataclass(frozen=True)
class Mx4Weight:
    """Expert weights ``[G, K, N]`` quantised along K: ``q`` uint8 ``[G, ceil(K / 128), N, 64]``, ``scales`` uint8
    ``[G, ceil(K / 128), N, 4]``, and ``dequant`` the round trip's bf16 ``[G, K, N]`` (None unless asked for)."""

    q: torch.Tensor
    scales: torch.Tensor
    dequant: torch.Tensor | None
    k: int


def _native_input(t: torch.Tensor) -> torch.Tensor:
    return t if t.dtype in (torch.bfloat16, torch.float32) else t.float()


def quantize_rows_mxfp8(x: torch.Tensor, row_index: torch.Tensor | None = None) -> MxRows:
    """``x [R, K]`` (bf16 or fp32, K a multiple of 32) to :class:`MxRows`; with ``row_index`` (int64 ``[R']``) the rows
    quantised are ``x[row_index]``, fetched by the kernel itself."""
    device = _lib.require_device(x, row_index)
    if x.dim() != 2:
        raise ValueError(f"expected [R, K], got {tuple(x.shape)}")
    x = _native_input(x)
    k = x.shape[1]
    if k % BLOCK:
        raise ValueError(f"axis 1 size {k} not divisible by block_size {BLOCK}")
    if row_index is not None:
        row_index = row_index.to(torch.int64).contiguous()
    rows = x.shape[0] if row_index is None else row_index.numel()
    if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
        if x.stride(0) % 8:  # a row length that is no multiple of 8 cannot happen (K % 32 == 0); a 1-row view can
            x = x.clone()
    q = torch.empty((-(-k // PANEL), rows, PANEL), dtype=torch.uint8, device=device)
    scales = torch.empty((k // BLOCK, rows), dtype=torch.uint8, device=device)
    if k % PANEL:
        q[-1, :, BLOCK:].zero_()  # the half panel no value belongs to
    with _lib.on_device(device):
        _lib.call("hmoe_quantize_rows_mxfp8", _lib.ptr(x), _lib.dtype_id(x.dtype), x.stride(0), _lib.ptr(row_index),
                  x.shape[0], rows, k, _lib.ptr(q), _lib.ptr(scales), rows, _lib.stream_ptr(device))
    return MxRows(q, scales, k)


def dequantize_rows_mxfp8(rows: MxRows) -> torch.Tensor:
    """bf16 ``[R, K]``: ``code * 2^(scale - 127)`` for every element of an :class:`MxRows`."""
    device = _lib.require_device(rows.q, rows.scales)
    out = torch.empty((rows.rows, rows.k), dtype=torch.bfloat16, device=device)
    with _lib.on_device(device):
        _lib.call("hmoe_dequantize_rows_mxfp8", _lib.ptr(rows.q), _lib.ptr(rows.scales), rows.rows, rows.rows, rows.k,
                  _lib.ptr(out), out.stride(0) if rows.rows else rows.k, _lib.stream_ptr(device))
    return out


def quantize_weight_mxfp8(w: torch.Tensor, with_dequant: bool = False) -> MxWeight:
    """``w [G, K, N]`` (bf16 or fp32, K a multiple of 32) quantised along K to :class:`MxWeight`."""
    device = _lib.require_device(w)
    if w.dim() != 3:
        raise ValueError(f"expected [G, K, N], got {tuple(w.shape)}")
    w = _native_input(w).contiguous()
    g, k, n = w.shape
    if k % BLOCK:
        raise ValueError(f"axis 1 size {k} not divisible by block_size {BLOCK}")
    q = torch.empty((g, -(-k // PANEL), n, PANEL), dtype=torch.uint8, device=device)
    scales = torch.empty((g, k // BLOCK, n), dtype=torch.uint8, device=device)
    dequant = torch.empty((g, k, n), dtype=torch.bfloat16, device=device) if with_dequant else None
    if k % PANEL:
        q[:, -1, :, BLOCK:].zero_()
    with _lib.on_device(device):
        _lib.call("hmoe_quantize_weight_mxfp8", _lib.ptr(w), _lib.dtype_id(w.dtype), g, k, n, _lib.ptr(q),
                  _lib.ptr(scales), _lib.ptr(dequant), _lib.stream_ptr(device))
    return MxWeight(q, scales, dequant, k)


def _aligned_rows(x: torch.Tensor) -> torch.Tensor:
    if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
        if x.stride(0) % 8:
            x = x.clone()
    return x


def mxfp4_rows(x: torch.Tensor, row_index: torch.Tensor | None = None, *, codes: bool = True,
               round_trip: bool = False) -> tuple[torch.Tensor | None, torch.Tensor | None, torch.Tensor | None]:
    """``x [R, K]`` (bf16 or fp32, K a multiple of 32) along its last axis in one launch: ``(packed uint8 [R, K / 2],
    scales uint8 [R, K / 32], round trip bf16 [R, K])``, the first two None unless ``codes``, the last unless
    ``round_trip``.  With ``row_index`` (int64 ``[R']``) the rows taken are ``x[row_index]``, fetched by the kernel."""
    device = _lib.require_device(x, row_index)
    if x.dim() != 2:
        raise ValueError(f"expected [R, K], got {tuple(x.shape)}")
    if not (codes or round_trip):
        raise ValueError("nothing to compute: neither codes nor round_trip asked for")
    x = _aligned_rows(_native_input(x))
    k = x.shape[1]
    if k % BLOCK:
        raise ValueError(f"axis 1 size {k} not divisible by block_size {BLOCK}")
    if row_index is not None:
        row_index = row_index.to(torch.int64).contiguous()
    rows = x.shape[0] if row_index is None else row_index.numel()
    packed = torch.empty((rows, k // 2), dtype=torch.uint8, device=device) if codes else None
    scales = torch.empty((rows, k // BLOCK), dtype=torch.uint8, device=device) if codes else None
    out = torch.empty((rows, k), dtype=torch.bfloat16, device=device) if round_trip else None
    with _lib.on_device(device):
        _lib.call("hmoe_mxfp4_rows", _lib.ptr(x), _lib.dtype_id(x.dtype), x.stride(0) if x.shape[0] else k,
                  _lib.ptr(row_index), x.shape[0], rows, k, _lib.ptr(packed), _lib.ptr(scales), _lib.ptr(out), k,
                  _lib.stream_ptr(device))
    return packed, scales, out


def mxfp4_weight(w: torch.Tensor, *, codes: bool = True, round_trip: bool = False
                 ) -> tuple[torch.Tensor | None, torch.Tensor | None, torch.Tensor | None]:
    """``w [G, K, N]`` (bf16 or fp32, K a multiple of 32) along K in one launch: ``(packed uint8 [G, K / 2, N], scales
    uint8 [G, K / 32, N], round trip bf16 [G, K, N])``, selected as in :func:`mxfp4_rows`."""
    device = _lib.require_device(w)
    if w.dim() != 3:
        raise ValueError(f"expected [G, K, N], got {tuple(w.shape)}")
    if not (codes or round_trip):
        raise ValueError("nothing to compute: neither codes nor round_trip asked for")
    w = _native_input(w).contiguous()
    g, k, n = w.shape
    if k % BLOCK:
        raise ValueError(f"axis 1 size {k} not divisible by block_size {BLOCK}")
    packed = torch.empty((g, k // 2, n), dtype=torch.uint8, device=device) if codes else None
    scales = torch.empty((g, k // BLOCK, n), dtype=torch.uint8, device=device) if codes else None
    out = torch.empty((g, k, n), dtype=torch.bfloat16, device=device) if round_trip else None
    with _lib.on_device(device):
        _lib.call("hmoe_mxfp4_weight", _lib.ptr(w), _lib.dtype_id(w.dtype), g, k, n, _lib.ptr(packed), _lib.ptr(scales),
                  _lib.ptr(out), _lib.stream_ptr(device))
    return packed, scales, out


def quantize_rows_mxfp4(x: torch.Tensor, row_index: torch.Tensor | None = None) -> Mx4Rows:
    """``x [R, K]`` (bf16 or fp32, K a multiple of 32) to :class:`Mx4Rows`; with ``row_index`` (int64 ``[R']``) the rows
    quantised are ``x[row_index]``, fetched by the kernel itself."""
    device = _lib.require_device(x, row_index)
    if x.dim() != 2:
        raise ValueError(f"expected [R, K], got {tuple(x.shape)}")
    x = _aligned_rows(_native_input(x))
    k = x.shape[1]
    if k % BLOCK:
        raise ValueError(f"axis 1 size {k} not divisible by block_size {BLOCK}")
    if row_index is not None:
        row_index = row_index.to(torch.int64).contiguous()
    rows = x.shape[0] if row_index is None else row_index.numel()
    panels = -(-k // 128)
    q = torch.empty((panels, rows, 64), dtype=torch.uint8, device=device)
    scales = torch.empty((panels, rows, 4), dtype=torch.uint8, device=device)
    with _lib.on_device(device):
        _lib.call("hmoe_mxfp4_rows_panels", _lib.ptr(x), _lib.dtype_id(x.dtype), x.stride(0) if x.shape[0] else k,
                  _lib.ptr(row_index), x.shape[0], rows, k, _lib.ptr(q), _lib.ptr(scales), rows,
                  _lib.stream_ptr(device))
    return Mx4Rows(q, scales, k)


def dequantize_rows_mxfp4(rows: Mx4Rows) -> torch.Tensor:
    """bf16 ``[R, K]``: ``level * sign * 2^(scale - 127)`` for every element of an :class:`Mx4Rows`."""
    device = _lib.require_device(rows.q, rows.scales)
    out = torch.empty((rows.rows, rows.k), dtype=torch.bfloat16, device=device)
    with _lib.on_device(device):
        _lib.call("hmoe_mxfp4_dequantize_panels", _lib.ptr(rows.q), _lib.ptr(rows.scales), rows.rows, rows.rows,
                  rows.k, _lib.ptr(out), rows.k, _lib.stream_ptr(device))
    return out


def quantize_weight_mxfp4(w: torch.Tensor, with_dequant: bool = False) -> Mx4Weight:
    """``w [G, K, N]`` (bf16 or fp32, K a multiple of 32) quantised along K to :class:`Mx4Weight`."""
    device = _lib.require_device(w)
    if w.dim() != 3:
        raise ValueError(f"expected [G, K, N], got {tuple(w.shape)}")
    w = _native_input(w).contiguous()
    g, k, n = w.shape
    if k % BLOCK:
        raise ValueError(f"axis 1 size {k} not divisible by block_size {BLOCK}")
    panels = -(-k // 128)
    q = torch.empty((g, panels, n, 64), dtype=torch.uint8, device=device)
    scales = torch.empty((g, panels, n, 4), dtype=torch.uint8, device=device)
    dequant = torch.empty((g, k, n), dtype=torch.bfloat16, device=device) if with_dequant else None
    with _lib.on_device(device):
        _lib.call("hmoe_mxfp4_weight_panels", _lib.ptr(w), _lib.dtype_id(w.dtype), g, k, n, _lib.ptr(q),
                  _lib.ptr(scales), _lib.ptr(dequant), _lib.stream_ptr(device))
    return Mx4Weight(q, scales, dequant, k)


NVFP4_BLOCK = FORMAT_BLOCK_SIZE["nvfp4"]


def _tensor_amax(t: torch.Tensor) -> torch.Tensor:
    """The largest magnitude of ``t`` as one fp32 value on the device (NaN if ``t`` holds one): the reduction NVFP4's
    per-tensor scale needs before any block can be scaled."""
    if t.numel() == 0:
        return torch.zeros((), dtype=torch.float32, device=t.device)
    return t.detach().abs().amax().float()


def nvfp4_rows(x: torch.Tensor, *, codes: bool = True, round_trip: bool = False, amax: torch.Tensor | None = None):
    """``x [R, K]`` (bf16 or fp32, K a multiple of 16) along its last axis in one launch: ``(packed uint8 [R, K / 2],
    scales float8_e4m3fn [R, K / 16], round trip bf16 [R, K], global scale fp32 [])``, the first two None unless
    ``codes``, the third unless ``round_trip``.  ``amax``: the tensor's largest magnitude when the caller has it."""
    device = _lib.require_device(x, amax)
    if x.dim() != 2:
        raise ValueError(f"expected [R, K], got {tuple(x.shape)}")
    if not (codes or round_trip):
        raise ValueError("nothing to compute: neither codes nor round_trip asked for")
    x = _aligned_rows(_native_input(x))
    rows, k = x.shape
    if k % NVFP4_BLOCK:
        raise ValueError(f"axis 1 size {k} not divisible by block_size {NVFP4_BLOCK}")
    amax = _tensor_amax(x) if amax is None else amax.float().reshape(())
    packed = torch.empty((rows, k // 2), dtype=torch.uint8, device=device) if codes else None
    scales = torch.empty((rows, k // NVFP4_BLOCK), dtype=torch.uint8, device=device) if codes else None
    out = torch.empty((rows, k), dtype=torch.bfloat16, device=device) if round_trip else None
    global_scale = torch.ones((), dtype=torch.float32, device=device)
    with _lib.on_device(device):
        _lib.call("hmoe_nvfp4_rows", _lib.ptr(x), _lib.dtype_id(x.dtype), x.stride(0) if rows else k, None, rows, rows,
                  k, _lib.ptr(amax), _lib.ptr(packed), _lib.ptr(scales), _lib.ptr(out), k, _lib.ptr(global_scale),
                  _lib.stream_ptr(device))
    return packed, None if scales is None else scales.view(torch.float8_e4m3fn), out, global_scale


def nvfp4_weight(w: torch.Tensor, *, codes: bool = True, round_trip: bool = False):
    """``w [G, K, N]`` (bf16 or fp32, K a multiple of 16) along K under one scale for the whole bank: ``(packed uint8
    [G, K / 2, N], scales float8_e4m3fn [G, K / 16, N], round trip bf16 [G, K, N], global scale fp32 [])``."""
    device = _lib.require_device(w)
    if w.dim() != 3:
        raise ValueError(f"expected [G, K, N], got {tuple(w.shape)}")
    if not (codes or round_trip):
        raise ValueError("nothing to compute: neither codes nor round_trip asked for")
    w = _native_input(w).contiguous()
    g, k, n = w.shape
    if k % NVFP4_BLOCK:
        raise ValueError(f"axis 1 size {k} not divisible by block_size {NVFP4_BLOCK}")
    amax = _tensor_amax(w)
    packed = torch.empty((g, k // 2, n), dtype=torch.uint8, device=device) if codes else None
    scales = torch.empty((g, k // NVFP4_BLOCK, n), dtype=torch.uint8, device=device) if codes else None
    out = torch.empty((g, k, n), dtype=torch.bfloat16, device=device) if round_trip else None
    global_scale = torch.ones((), dtype=torch.float32, device=device)
    with _lib.on_device(device):
        _lib.call("hmoe_nvfp4_weight", _lib.ptr(w), _lib.dtype_id(w.dtype), g, k, n, _lib.ptr(amax), _lib.ptr(packed),
                  _lib.ptr(scales), _lib.ptr(out), _lib.ptr(global_scale), _lib.stream_ptr(device))
    return packed, None if scales is None else scales.view(torch.float8_e4m3fn), out, global_scale


def quantize_nvfp4(t: torch.Tensor, axis: int = -1) -> BlockScaledTensor:
    """The reference's layout (``quantization.py:218-226, 248-270``): ``data`` uint8 with ``axis`` halved, ``scales``
    float8_e4m3fn with ``axis`` divided by 16, ``global_scale`` a 0-dim fp32 tensor."""
    if t.dim() == 0:
        raise ValueError("quantize_nvfp4 expects at least one axis")
    kind, axis = _axis_layout(t, axis)
    k = t.shape[axis]
    if k % NVFP4_BLOCK:
        raise ValueError(f"axis {axis} size {k} not divisible by block_size {NVFP4_BLOCK}")
    if kind == "moved":
        inner = quantize_nvfp4(t.transpose(axis, -1).contiguous(), -1)
        return BlockScaledTensor(inner.data.transpose(axis, -1).contiguous(),
                                 inner.scales.view(torch.uint8).transpose(axis, -1).contiguous().view(torch.float8_e4m3fn),
                                 NVFP4_BLOCK, axis, packed=True, pow2_scale=False, global_scale=inner.global_scale)
    if kind == "rows":
        lead = t.shape[:-1]
        packed, scales, _, gs = nvfp4_rows(t.reshape(-1, k))
        return BlockScaledTensor(packed.reshape(*lead, k // 2), scales.reshape(*lead, k // NVFP4_BLOCK), NVFP4_BLOCK,
                                 axis, packed=True, pow2_scale=False, global_scale=gs)
    lead, n = t.shape[:-2], t.shape[-1]
    packed, scales, _, gs = nvfp4_weight(t.reshape(-1, k, n))
    return BlockScaledTensor(packed.reshape(*lead, k // 2, n), scales.reshape(*lead, k // NVFP4_BLOCK, n), NVFP4_BLOCK,
                             axis, packed=True, pow2_scale=False, global_scale=gs)


def _dequantize_nvfp4(q: BlockScaledTensor) -> torch.Tensor:
    data, axis = q.data, q.axis % q.data.dim()
    scales = q.scales.view(torch.uint8)
    if axis != data.dim() - 1:
        moved = BlockScaledTensor(data.transpose(axis, -1).contiguous(),
                                  scales.transpose(axis, -1).contiguous().view(torch.float8_e4m3fn), NVFP4_BLOCK, -1,
                                  packed=True, pow2_scale=False, global_scale=q.global_scale)
        return _dequantize_nvfp4(moved).transpose(axis, -1).contiguous()
    device = _lib.require_device(data, scales, q.global_scale)
    k = data.shape[-1] * 2
    if k % NVFP4_BLOCK or scales.shape[-1] != k // NVFP4_BLOCK:
        raise ValueError(f"packed axis of {data.shape[-1]} bytes does not match {scales.shape[-1]} scales of {NVFP4_BLOCK}")
    flat = data.reshape(-1, k // 2).contiguous()
    flat_scales = scales.reshape(-1, k // NVFP4_BLOCK).contiguous()
    gs = q.global_scale.float().reshape(()).contiguous()
    out = torch.empty((flat.shape[0], k), dtype=torch.bfloat16, device=device)
    with _lib.on_device(device):
        _lib.call("hmoe_nvfp4_dequantize_rows", _lib.ptr(flat), _lib.ptr(flat_scales), _lib.ptr(gs), flat.shape[0], k,
                  _lib.ptr(out), k, _lib.stream_ptr(device))
    return out.reshape(*data.shape[:-1], k)


def _axis_layout(t: torch.Tensor, axis: int) -> tuple[str, int]:
    axis = axis % t.dim()
    if axis == t.dim() - 1:
        return "rows", axis
    if axis == t.dim() - 2:
        return "weight", axis
    return "moved", axis


def quantize_mxfp8(t: torch.Tensor, axis: int = -1) -> BlockScaledTensor:
    """The reference's layout (``quantization.py:236-245``): ``data`` float8_e4m3fn of ``t``'s shape, ``scales`` uint8
    with ``axis`` divided by 32.  Quantised by the same kernels as the GEMM's operands; the panels are unfolded."""
    if t.dim() == 0:
        raise ValueError("quantize_mxfp8 expects at least one axis")
    kind, axis = _axis_layout(t, axis)
    k = t.shape[axis]
    if k % BLOCK:
        raise ValueError(f"axis {axis} size {k} not divisible by block_size {BLOCK}")
    if kind == "moved":
        inner = quantize_mxfp8(t.transpose(axis, -1).contiguous(), -1)
        return BlockScaledTensor(inner.data.transpose(axis, -1).contiguous(),
                                 inner.scales.transpose(axis, -1).contiguous(), BLOCK, axis)
    if kind == "rows":
        lead = t.shape[:-1]
        rows = quantize_rows_mxfp8(t.reshape(-1, k))
        data = rows.q.permute(1, 0, 2).reshape(rows.rows, -1)[:, :k].reshape(*lead, k)
        scales = rows.scales.t().reshape(*lead, k // BLOCK)
    else:
        lead, n = t.shape[:-2], t.shape[-1]
        w = quantize_weight_mxfp8(t.reshape(-1, k, n))
        data = w.q.permute(0, 1, 3, 2).reshape(w.q.shape[0], -1, n)[:, :k].reshape(*lead, k, n)
        scales = w.scales.reshape(*lead, k // BLOCK, n)
    return BlockScaledTensor(data.contiguous().view(torch.float8_e4m3fn), scales.contiguous(), BLOCK, axis)


def quantize_mxfp4(t: torch.Tensor, axis: int = -1) -> BlockScaledTensor:
    """The reference's layout (``quantization.py:248-266``): ``data`` uint8 with ``axis`` halved (two e2m1 codes per
    byte, the even element low), ``scales`` uint8 with ``axis`` divided by 32."""
    if t.dim() == 0:
        raise ValueError("quantize_mxfp4 expects at least one axis")
    kind, axis = _axis_layout(t, axis)
    k = t.shape[axis]
    if k % BLOCK:
        raise ValueError(f"axis {axis} size {k} not divisible by block_size {BLOCK}")
    if kind == "moved":
        inner = quantize_mxfp4(t.transpose(axis, -1).contiguous(), -1)
        return BlockScaledTensor(inner.data.transpose(axis, -1).contiguous(),
                                 inner.scales.transpose(axis, -1).contiguous(), BLOCK, axis, packed=True)
    if kind == "rows":
        lead = t.shape[:-1]
        packed, scales, _ = mxfp4_rows(t.reshape(-1, k))
        return BlockScaledTensor(packed.reshape(*lead, k // 2), scales.reshape(*lead, k // BLOCK), BLOCK, axis,
                                 packed=True)
    lead, n = t.shape[:-2], t.shape[-1]
    packed, scales, _ = mxfp4_weight(t.reshape(-1, k, n))
    return BlockScaledTensor(packed.reshape(*lead, k // 2, n), scales.reshape(*lead, k // BLOCK, n), BLOCK, axis,
                             packed=True)


QUANTIZERS = {"mxfp8": quantize_mxfp8, "mxfp4": quantize_mxfp4, "nvfp4": quantize_nvfp4}


def _dequantize_packed(q: BlockScaledTensor) -> torch.Tensor:
    data, axis = q.data, q.axis % q.data.dim()
    if axis != data.dim() - 1:
        moved = BlockScaledTensor(data.transpose(axis, -1).contiguous(), q.scales.transpose(axis, -1).contiguous(),
                                  BLOCK, -1, packed=True)
        return _dequantize_packed(moved).transpose(axis, -1).contiguous()
    device = _lib.require_device(data, q.scales)
    k = data.shape[-1] * 2
    if k % BLOCK or q.scales.shape[-1] != k // BLOCK:
        raise ValueError(f"packed axis of {data.shape[-1]} bytes does not match {q.scales.shape[-1]} scales of {BLOCK}")
    flat = data.reshape(-1, k // 2).contiguous()
    scales = q.scales.reshape(-1, k // BLOCK).contiguous()
    out = torch.empty((flat.shape[0], k), dtype=torch.bfloat16, device=device)
    with _lib.on_device(device):
        _lib.call("hmoe_mxfp4_dequantize_rows", _lib.ptr(flat), _lib.ptr(scales), flat.shape[0], k, _lib.ptr(out), k,
                  _lib.stream_ptr(device))
    return out.reshape(*data.shape[:-1], k)


def dequantize(q: BlockScaledTensor) -> torch.Tensor:
    """bf16 ``code * 2^(scales - 127)`` (MX) or ``code * scales * global_scale`` (NVFP4) in the source's shape
    (``quantization.py:277-297``)."""
    if not q.pow2_scale and q.packed and q.block_size == NVFP4_BLOCK and q.global_scale is not None:
        return _dequantize_nvfp4(q)
    if not q.pow2_scale or q.block_size != BLOCK or q.global_scale is not None:
        raise NotImplementedError("only the MX formats and NVFP4 are built on this path")
    if q.packed:
        return _dequantize_packed(q)
    data = q.data.view(torch.uint8)
    axis = q.axis % data.dim()
    if axis != data.dim() - 1:
        moved = BlockScaledTensor(data.transpose(axis, -1).contiguous(), q.scales.transpose(axis, -1).contiguous(),
                                  BLOCK, -1)
        return dequantize(moved).transpose(axis, -1).contiguous()
    k = data.shape[-1]
    flat = data.reshape(-1, k)
    rows = flat.shape[0]
    panels = -(-k // PANEL)
    padded = flat if k % PANEL == 0 else torch.nn.functional.pad(flat, (0, panels * PANEL - k))
    packed = MxRows(padded.reshape(rows, panels, PANEL).permute(1, 0, 2).contiguous(),
                    q.scales.reshape(rows, k // BLOCK).t().contiguous(), k)
    return dequantize_rows_mxfp8(packed).reshape(data.shape)


def _round_trip(t: torch.Tensor, fmt: str, axis: int) -> torch.Tensor:
    """Quantise then dequantise, bf16 (``quantization.py:307-311``): one launch, except MXFP8 rows, which take two."""
    require_implemented(fmt)
    kind, axis = _axis_layout(t, axis)
    if t.shape[axis] % FORMAT_BLOCK_SIZE[fmt]:
        raise ValueError(f"axis {axis} size {t.shape[axis]} not divisible by block_size {FORMAT_BLOCK_SIZE[fmt]}")
    if kind == "moved":
        return _round_trip(t.transpose(axis, -1).contiguous(), fmt, -1).transpose(axis, -1).contiguous()
    if kind == "rows":
        flat = t.reshape(-1, t.shape[-1])
        if fmt == "nvfp4":
            return nvfp4_rows(flat, codes=False, round_trip=True)[2].reshape(t.shape)
        if fmt == "mxfp4":
            return mxfp4_rows(flat, codes=False, round_trip=True)[2].reshape(t.shape)
        return dequantize_rows_mxfp8(quantize_rows_mxfp8(flat)).reshape(t.shape)
    banks = t.reshape(-1, *t.shape[-2:])
    if fmt == "nvfp4":
        return nvfp4_weight(banks, codes=False, round_trip=True)[2].reshape(t.shape)
    if fmt == "mxfp4":
        return mxfp4_weight(banks, codes=False, round_trip=True)[2].reshape(t.shape)
    return quantize_weight_mxfp8(banks, with_dequant=True).dequant.reshape(t.shape)


class _FakeQuant(torch.autograd.Function):
    """Straight-through estimator: forward quantise -> dequantise, identity backward to the master
    (``quantization.py:350-360``)."""

    @staticmethod
    def forward(ctx, t: torch.Tensor, fmt: str, axis: int) -> torch.Tensor:
        return _round_trip(t, fmt, axis).to(t.dtype)

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None, None


def fake_quant(t: torch.Tensor, fmt: str = "mxfp8", axis: int = -1) -> torch.Tensor:
    """The axis must divide by the format's block size.  Expert weights use :func:`cached_fake_quant`."""
    return _FakeQuant.apply(t, fmt, axis)


class WeightVersionCache:
    """Keyed by tensor identity plus a caller fingerprint, for values derived once per optimizer step.  A ``weakref``
    finalizer evicts a collected weight's entry, so a reused ``id`` never serves a stale hit
    (``quantization.py:368-394``)."""

    def __init__(self) -> None:
        self._entries: dict[int, tuple[weakref.ref, tuple, object]] = {}

    def get(self, weight: torch.Tensor, fingerprint: tuple):
        entry = self._entries.get(id(weight))
        if entry is None:
            return None
        ref, cached_fingerprint, value = entry
        if ref() is not weight or cached_fingerprint != fingerprint:
            return None
        return value

    def put(self, weight: torch.Tensor, fingerprint: tuple, value) -> None:
        wid = id(weight)
        entries = self._entries
        ref = weakref.ref(weight, lambda _ref, wid=wid: entries.pop(wid, None))
        entries[wid] = (ref, fingerprint, value)

    def __len__(self) -> int:
        return len(self._entries)


_weight_dequant_cache = WeightVersionCache()
_weight_round_trip_cache = WeightVersionCache()
_weight_operand_cache = WeightVersionCache()


def weight_cache_enabled() -> bool:
    """``HALO_LOWP_WEIGHT_CACHE`` (default on), the reference's switch (``quantization.py:414``)."""
    return os.environ.get("HALO_LOWP_WEIGHT_CACHE", "1").strip().lower() not in ("0", "false", "no", "off", "")


class _CachedFakeQuant(torch.autograd.Function):
    """Cloned per call so the shared entry never meets autograd's one-grad_fn-per-tensor rule
    (``quantization.py:397-407``)."""

    @staticmethod
    def forward(ctx, weight: torch.Tensor, cached_dequant: torch.Tensor) -> torch.Tensor:
        return cached_dequant.clone()

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None


def cached_fake_quant(weight: torch.Tensor, fmt: str = "mxfp8", axis: int = -1) -> torch.Tensor:
    """:func:`fake_quant` for an expert weight, quantised once per optimizer step (keyed on ``weight._version``); only
    leaf parameters cache (``quantization.py:410-422``)."""
    require_implemented(fmt)
    if not weight.is_leaf or not weight_cache_enabled():
        return fake_quant(weight, fmt, axis)
    fingerprint = (weight._version, fmt, axis)
    dequant = _weight_dequant_cache.get(weight, fingerprint)
    if dequant is None:
        with torch.no_grad():
            dequant = _round_trip(weight, fmt, axis).to(weight.dtype)
        _weight_dequant_cache.put(weight, fingerprint, dequant)
    return _CachedFakeQuant.apply(weight, dequant)


def expert_weight_round_trip(weight: torch.Tensor, fmt: str, cacheable: bool) -> torch.Tensor:
    """The bf16 round trip of ``[G, K, N]`` expert weights along K, detached: what the fake-quant route multiplies by
    in the forward and in the input gradient.  Computed once per optimizer step for a leaf parameter when
    ``cacheable``; the caller must not write to it."""
    require_implemented(fmt)
    if not (cacheable and weight.is_leaf and weight_cache_enabled()):
        with torch.no_grad():
            return _round_trip(weight.detach(), fmt, 1).to(torch.bfloat16)
    fingerprint = (weight._version, fmt, 1)
    value = _weight_round_trip_cache.get(weight, fingerprint)
    if value is None:
        with torch.no_grad():
            value = _round_trip(weight.detach(), fmt, 1).to(torch.bfloat16)
        _weight_round_trip_cache.put(weight, fingerprint, value)
    return value


def expert_weight_operand(weight: torch.Tensor, cacheable: bool, fmt: str = "mxfp8"):
    """``[G, K, N]`` expert weights as the matrix kernel's operand in ``fmt`` (:class:`MxWeight` or
    :class:`Mx4Weight`) together with the round trip's bf16 copy (which the backward products read), quantised once per
    optimizer step for a leaf parameter when ``cacheable``."""
    quantise = {"mxfp8": quantize_weight_mxfp8, "mxfp4": quantize_weight_mxfp4}[fmt]
    if not (cacheable and weight.is_leaf and weight_cache_enabled()):
        with torch.no_grad():
            return quantise(weight.detach(), with_dequant=True)
    fingerprint = (weight._version, fmt, 1)
    operand = _weight_operand_cache.get(weight, fingerprint)
    if operand is None:
        with torch.no_grad():
            operand = quantise(weight.detach(), with_dequant=True)
        _weight_operand_cache.put(weight, fingerprint, operand)
    return operand
