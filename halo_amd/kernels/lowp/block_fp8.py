"""DeepSeek-style block FP8 for served weights: float8_e4m3fn values with one fp32 power-of-two scale per 128x128
block, stored beside the weight as ``<weight>_scale_inv``.

Mirrors the reference's ``halo/kernels/lowp/block_fp8.py:16-34`` and the dequantiser of
``halo/checkpoint/tools/fp8_dequant.py:153-170``; the kernels are ``csrc/quant.hip``.
"""

from __future__ import annotations

import torch

from halo_amd import _lib

BLOCK = 128
SCALE_SUFFIX = "_scale_inv"
E4M3_MAX = 448.0


def quantize_block_fp8(weight: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``(q, scale_inv)`` for ``weight`` ``[..., N, K]``: ``q`` has its shape in float8_e4m3fn, ``scale_inv`` is fp32
    ``[..., ceil(N/128), ceil(K/128)]`` and ``q * scale_inv`` (broadcast over blocks) reconstructs the weight."""
    device = _lib.require_device(weight)
    if weight.dim() < 2:
        raise ValueError("quantize_block_fp8 expects at least a 2-D weight")
    if weight.dtype not in (torch.float32, torch.bfloat16):
        weight = weight.float()
    weight = weight.contiguous()
    n, k = weight.shape[-2:]
    lead = weight.shape[:-2]
    batch = 1
    for d in lead:
        batch *= d
    q = torch.empty(weight.shape, dtype=torch.uint8, device=device)
    scale = torch.empty((*lead, -(-n // BLOCK), -(-k // BLOCK)), dtype=torch.float32, device=device)
    with _lib.on_device(device):
        _lib.call("hmoe_quantize_block_fp8", _lib.ptr(weight), _lib.dtype_id(weight.dtype), batch, n, k, _lib.ptr(q),
                  _lib.ptr(scale), _lib.stream_ptr(device))
    return q.view(torch.float8_e4m3fn), scale


def dequantize_block_fp8(weight: torch.Tensor, scale_inv: torch.Tensor, dtype: torch.dtype = torch.bfloat16
                         ) -> torch.Tensor:
    """``weight * scale_inv`` per 128x128 block in fp32, rounded once to ``dtype``."""
    device = _lib.require_device(weight, scale_inv)
    weight = weight.contiguous()
    n, k = weight.shape[-2:]
    lead = weight.shape[:-2]
    batch = 1
    for d in lead:
        batch *= d
    if tuple(scale_inv.shape) != (*lead, -(-n // BLOCK), -(-k // BLOCK)):
        raise ValueError(f"scale grid {tuple(scale_inv.shape)} does not match weight {tuple(weight.shape)}")
    out = torch.empty(weight.shape, dtype=dtype, device=device)
    scale_inv = scale_inv.float().contiguous()
    with _lib.on_device(device):
        _lib.call("hmoe_dequantize_block_fp8", _lib.ptr(weight.view(torch.uint8)), _lib.ptr(scale_inv), batch, n, k,
                  _lib.dtype_id(dtype), _lib.ptr(out), _lib.stream_ptr(device))
    return out


class QuantizedRows:
    """Activation rows already in the fp8 expert GEMM's operand form: ``q`` e4m3 panels ``[K / 64, R, 64]`` and
    ``scale_exponents`` uint8 ``[K / 128, R]`` as :func:`quantize_rows_fp8` returns them.  Stands where a bf16
    ``[R, K]`` tensor would (``shape``, ``dtype``, ``device``) for a producer that quantises as it writes."""

    def __init__(self, q: torch.Tensor, scale_exponents: torch.Tensor):
        self.q, self.scale_exponents = q, scale_exponents

    @property
    def shape(self):
        return torch.Size((self.q.shape[1], self.q.shape[0] * self.q.shape[2]))

    dtype = torch.bfloat16  # the precision the values were rounded to before they were scaled
    requires_grad = False

    @property
    def device(self):
        return self.q.device


def quantize_rows_fp8(x: torch.Tensor, row_index: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """``(q, scale_exponents)`` for bf16 activations ``x [R, K]`` (K a multiple of 128): ``q`` float8_e4m3fn
    ``[K / 64, R, 64]`` (panels of 64 values, as the fp8 expert GEMM reads them: ``q.permute(1, 0, 2)`` is
    ``[R, K / 64, 64]``) and uint8 ``[K / 128, R]``, the biased exponent ``e + 127`` of each row's power-of-two
    scale ``2^e`` per 128 values (the smallest that brings the block's largest magnitude to 448 or below; 0 for an
    all-zero block).  ``q * 2^e`` reconstructs ``x`` to e4m3 precision.  With ``row_index`` (int64 ``[R]``) the rows
    quantised are ``x[row_index]``, fetched by the kernel itself.  This is the
    "dynamic" activation scheme of :func:`block_fp8_quantization_config`, with scales the matrix instruction takes
    as they are."""
    device = _lib.require_device(x, row_index)
    if x.dim() != 2 or x.dtype != torch.bfloat16:
        raise TypeError(f"quantize_rows_fp8 takes bf16 [R, K], got {x.dtype} {tuple(x.shape)}")
    k = x.shape[1]
    if row_index is not None:
        row_index = row_index.to(torch.int64).contiguous()
    rows = x.shape[0] if row_index is None else row_index.numel()
    if k % BLOCK:
        raise ValueError(f"K = {k} is not a multiple of {BLOCK}")
    if x.stride(1) != 1 or x.stride(0) % 8:
        x = x.contiguous()
    q = torch.empty((k // 64, rows, 64), dtype=torch.uint8, device=device)
    scale = torch.empty((k // BLOCK, rows), dtype=torch.uint8, device=device)
    with _lib.on_device(device):
        _lib.call("hmoe_quantize_rows_fp8", _lib.ptr(x), x.stride(0), _lib.ptr(row_index), x.shape[0], rows, k,
                  _lib.ptr(q), _lib.ptr(scale), rows, _lib.stream_ptr(device))
    return q.view(torch.float8_e4m3fn), scale


def block_fp8_quantization_config(modules_to_not_convert: list[str]) -> dict:
    """The ``config.json`` ``quantization_config`` serving engines read for such a checkpoint."""
    return {
        "quant_method": "fp8",
        "fmt": "e4m3",
        "activation_scheme": "dynamic",
        "weight_block_size": [BLOCK, BLOCK],
        "modules_to_not_convert": sorted(modules_to_not_convert),
    }
