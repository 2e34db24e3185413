"""Grouped GEMM for MoE expert FFNs, by weight format: bf16/fp32 (the training path), or block-fp8 weights (the
quantised-weight serving configuration, forward only).

Mirrors the dispatch seam of the reference's ``halo/kernels/expert_gemm.py:14-38``.  The reference's other
``quant_format`` values name its fake-quant QAT formats (mxfp8 / mxfp4 / nvfp4), which are not part of this path.
"""

from __future__ import annotations

import torch

from halo_amd import _lib
from halo_amd.kernels.grouped_mm import GatheredRows, _offs_arg, _rows, grouped_mm


# rows per expert (on average) from which the dequantised-copy route is taken
_CACHED_MIN_ROWS = 64


class BlockFp8Weight:
    """Expert weights ``[G, K, N]`` as float8_e4m3fn with one fp32 power-of-two scale per 128x128 block
    (``halo_amd.kernels.lowp.block_fp8.quantize_block_fp8`` of the matmul-convention weight)."""

    def __init__(self, q: torch.Tensor, scale_inv: torch.Tensor):
        if q.dim() != 3 or scale_inv.dim() != 3:
            raise ValueError("expected q [G, K, N] and scale_inv [G, ceil(K/128), ceil(N/128)]")
        g, k, n = q.shape
        if tuple(scale_inv.shape) != (g, -(-k // 128), -(-n // 128)):
            raise ValueError(f"scale grid {tuple(scale_inv.shape)} does not match weight {tuple(q.shape)}")
        self.q = q.contiguous()
        self.scale_inv = scale_inv.float().contiguous()
        self._bf16 = None
        self._panels = None

    @property
    def shape(self):
        return self.q.shape

    def dequantized(self) -> torch.Tensor:
        """The weights as bf16 ``[G, K, N]`` (``q * scale`` per block, exact: the scales are powers of two), made once
        and kept: twice the fp8 bytes again in device memory, for the bf16 kernel's speed on compute-bound batches."""
        if self._bf16 is None:
            from halo_amd.kernels.lowp.block_fp8 import dequantize_block_fp8

            self._bf16 = dequantize_block_fp8(self.q, self.scale_inv)
        return self._bf16


    def panels(self) -> torch.Tensor:
        """The e4m3 bytes as ``[G, K / 64, N, 64]``: the contraction contiguous within a panel of 64 values and a
        tile's columns of one panel in one run, which is how the fp8 MFMA kernel loads them.  Made once and kept: the
        fp8 bytes once more in device memory."""
        if self._panels is None:
            g, k, n = self.q.shape
            self._panels = self.q.view(torch.uint8).view(g, k // 64, 64, n).permute(0, 1, 3, 2).contiguous()
        return self._panels


def expert_gemm(
    mat_a: torch.Tensor,
    mat_b,
    *,
    offs: torch.Tensor | None = None,
    quant_format=None,
    weight_cacheable: bool = True,
    fp8_activations: bool = False,
) -> torch.Tensor:
    """``[total_tokens, K]`` activations stacked by expert times ``[num_experts, K, N]`` weights.  ``mat_b`` may be a
    :class:`BlockFp8Weight` (or ``quant_format == "block_fp8"`` with ``mat_b = (q, scale_inv)``): bf16 activations
    against fp8 weights dequantised on their way into the MFMA tiles, forward only.  ``fp8_activations=True``
    quantises the activations too (per row and 128 values, power-of-two scales) and multiplies on the e4m3 MFMA:
    twice the bf16 rate and half the bytes, at e4m3 precision on both sides instead of one."""
    if isinstance(mat_b, BlockFp8Weight) or quant_format == "block_fp8":
        weight = mat_b if isinstance(mat_b, BlockFp8Weight) else BlockFp8Weight(*mat_b)
        if fp8_activations:
            return _fp8_mfma_forward(mat_a, weight, offs)
        # Two routes with bit-identical results (the dequantisation is exact).  The kernel that reads the fp8 bytes
        # moves half the weight traffic, which is what counts while a batch is small; once an expert sees enough rows
        # to be compute-bound the bf16 kernel over a dequantised copy kept with the weight is faster (configuration 5:
        # 1.1 PFLOP/s against 0.65).  ``weight_cacheable=False`` (weights that change under the caller) always takes
        # the first.
        if weight_cacheable and isinstance(mat_b, BlockFp8Weight) and mat_a.shape[0] >= _CACHED_MIN_ROWS * weight.shape[0]:
            if mat_a.requires_grad and torch.is_grad_enabled():
                raise RuntimeError("the block-fp8 expert GEMM is forward only")
            with torch.no_grad():
                return grouped_mm(mat_a, weight.dequantized(), offs=offs)
        return _fp8w_forward(mat_a, weight, offs)
    if quant_format is not None:
        raise NotImplementedError(
            f"quant_format={quant_format!r}: the reference's fake-quant QAT formats are not part of the expert path"
        )
    return grouped_mm(mat_a, mat_b, offs=offs)


def _fp8w_forward(mat_a: torch.Tensor, weight: BlockFp8Weight, offs: torch.Tensor | None) -> torch.Tensor:
    device = _lib.require_device(mat_a, weight.q, weight.scale_inv, offs)
    if mat_a.dtype != torch.bfloat16:
        raise TypeError(f"block-fp8 expert GEMM takes bf16 activations, got {mat_a.dtype}")
    if mat_a.requires_grad and torch.is_grad_enabled():
        raise RuntimeError("the block-fp8 expert GEMM is forward only")
    groups, k, n = weight.shape
    rows = mat_a.shape[0]
    out = torch.empty((rows, n), dtype=torch.bfloat16, device=device)
    if rows == 0 or n == 0:
        return out
    mat_a = _rows(mat_a)
    offs32 = _offs_arg(offs, groups)
    q = weight.q.view(torch.uint8)
    with _lib.on_device(device):
        _lib.call("hmoe_grouped_gemm_fwd_fp8w", _lib.ptr(mat_a), mat_a.stride(0), _lib.ptr(q),
                  _lib.ptr(weight.scale_inv), _lib.ptr(offs32), rows, groups, k, n, _lib.ptr(out), out.stride(0),
                  _lib.stream_ptr(device))
    return out


def fp8_mfma_usable(k: int, n: int) -> bool:
    """Whether the e4m3 MFMA kernel takes a ``[*, K] x [G, K, N]`` product: whole 128-value scale blocks along K,
    16-byte output rows."""
    return k > 0 and k % 128 == 0 and n % 8 == 0


def _fp8_mfma_forward(mat_a: torch.Tensor, weight: BlockFp8Weight, offs: torch.Tensor | None) -> torch.Tensor:
    """Activations to e4m3 (one launch, which also fetches the rows when ``mat_a`` is a :class:`GatheredRows`: the
    permuted bf16 copy is never written; none at all when ``mat_a`` already is a ``QuantizedRows``), then the grouped GEMM on the scaled e4m3 MFMA against the weight's bytes in
    panels and its fp32 block scales."""
    from halo_amd.kernels.lowp.block_fp8 import QuantizedRows, quantize_rows_fp8

    gathered = isinstance(mat_a, GatheredRows)
    quantized = isinstance(mat_a, QuantizedRows)
    source = mat_a.tokens if gathered else (mat_a.q if quantized else mat_a)
    device = _lib.require_device(source, weight.q, weight.scale_inv, offs)
    if quantized:
        source = mat_a  # its dtype and gradient flag stand for the bf16 rows it was made from
    if source.dtype != torch.bfloat16:
        raise TypeError(f"block-fp8 expert GEMM takes bf16 activations, got {source.dtype}")
    if source.requires_grad and torch.is_grad_enabled():
        raise RuntimeError("the block-fp8 expert GEMM is forward only")
    groups, k, n = weight.shape
    if len(mat_a.shape) != 2 or mat_a.shape[1] != k:
        raise ValueError(f"expected [R, {k}] activations, got {tuple(mat_a.shape)}")
    if not fp8_mfma_usable(k, n):
        raise ValueError(f"the fp8 MFMA product needs K % 128 == 0 and N % 8 == 0, got K = {k}, N = {n}")
    rows = mat_a.shape[0]
    out = torch.empty((rows, n), dtype=torch.bfloat16, device=device)
    if rows == 0 or n == 0:
        return out
    offs32 = _offs_arg(offs, groups)
    if quantized:
        a_q, a_scale = mat_a.q, mat_a.scale_exponents
    else:
        a_q, a_scale = quantize_rows_fp8(source, mat_a.row_index if gathered else None)
    w_panels = weight.panels()
    with _lib.on_device(device):
        _lib.call("hmoe_grouped_gemm_fwd_fp8", _lib.ptr(a_q), _lib.ptr(a_scale), rows, _lib.ptr(w_panels),
                  _lib.ptr(weight.scale_inv), _lib.ptr(offs32), rows, groups, k, n, _lib.ptr(out), out.stride(0),
                  _lib.stream_ptr(device))
    return out
