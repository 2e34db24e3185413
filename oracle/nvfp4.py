"""Oracle (test infrastructure): NVFP4 block-scaled quantisation (e2m1 elements, two per byte, one e4m3 scale per 16
values along the contraction axis and one fp32 power-of-two scale per tensor), its dequantiser, the fake-quant round
trip and the fake-quantised expert GEMM, in numpy.

Follows the eager CPU path of ``halo/kernels/lowp/quantization.py``: ``nvfp4_global_scale`` (:209-215), ``_nvfp4_core``
(:218-226), ``_e2m1_codes`` (:201-205), ``_e2m1_round`` (:191-198), ``_quantize_fp4`` (:248-263), ``dequantize``
(:277-297); the expert GEMM is ``halo/kernels/expert_gemm.py:33-38``.  The e4m3 codec is the explicit one of
``oracle.block_fp8``; the e2m1 rounding is ``oracle.mxfp4.e2m1_round``.

The global scale ``exp2(ceil(log2(max(amax, tiny) / 2688)))`` is evaluated in integer arithmetic on the operand's
exponent and mantissa (2688 = 0.65625 * 2^12); for a tensor whose amax / 2688 lies within an ulp of a power of two the
reference's result depends on its fp32 ``log2`` rounding, and such inputs are outside what this oracle pins.
"""

from __future__ import annotations

import numpy as np
import torch

from oracle.block_fp8 import decode_e4m3fn, encode_e4m3fn
from oracle.mxfp4 import E2M1_LEVELS, e2m1_round, unpack_codes
from oracle.mxfp8 import AMAX_FLOOR, _round_to_bf16

BLOCK = 16
E2M1_MAX = 6.0
E4M3_MAX = 448.0
GLOBAL_SCALE_DIVISOR = E4M3_MAX * E2M1_MAX  # the tensor amax is lifted to the largest e4m3 scale times the largest level


def global_scale(amax) -> np.float32:
    """The per-tensor fp32 scale (``quantization.py:209-215``): the smallest power of two ``>= max(amax, tiny) / 2688``;
    NaN for a NaN amax, inf for an infinite one."""
    amax = np.float32(amax)
    if np.isnan(amax):
        return np.float32(np.nan)
    if np.isinf(amax):
        return np.float32(np.inf)
    mantissa, exponent = np.frexp(np.float64(max(amax, AMAX_FLOOR)))  # mantissa in [0.5, 1)
    e = int(exponent) - 12 + (1 if mantissa > 0.65625 else 0)
    return np.float32(np.ldexp(1.0, e))  # down to 2^-137, a subnormal fp32, as torch.exp2 returns it


def _encode_scale(x: np.ndarray) -> np.ndarray:
    """fp32 block scales (not negative, at most 448, or NaN) to e4m3fn bits; NaN takes the format's NaN pattern."""
    nan = np.isnan(x)
    return np.where(nan, np.uint8(0x7F), encode_e4m3fn(np.where(nan, np.float32(0.0), x))).astype(np.uint8)


def _decode_scale(bits: np.ndarray) -> np.ndarray:
    return np.where((bits & 0x7F) == 0x7F, np.float32(np.nan), decode_e4m3fn(bits)).astype(np.float32)


def quantize_nvfp4(t: np.ndarray, axis: int = -1) -> tuple[np.ndarray, np.ndarray, np.float32]:
    """``(data uint8 with the axis halved, two codes per byte, the even element in the low nibble; scales uint8 e4m3fn
    bits with the axis divided by 16; the tensor's global scale)`` (``quantization.py:218-226, 248-263``)."""
    t = np.asarray(t, dtype=np.float32)
    axis = axis % t.ndim
    if t.shape[axis] % BLOCK:
        raise ValueError(f"axis {axis} size {t.shape[axis]} not divisible by block_size {BLOCK}")
    work = np.moveaxis(t, axis, -1)
    blocks = work.reshape(*work.shape[:-1], work.shape[-1] // BLOCK, BLOCK)
    with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
        g = global_scale(np.abs(blocks).max()) if blocks.size else np.float32(1.0)
        amax = np.abs(blocks).max(axis=-1)
        ratio = (amax / np.float32(E2M1_MAX)).astype(np.float32) / g  # two fp32 divisions, as the reference's
        ratio = np.where(np.isnan(ratio), ratio, np.minimum(ratio, np.float32(E4M3_MAX))).astype(np.float32)
        scale_bits = _encode_scale(ratio)
        divisor = (_decode_scale(scale_bits) * g).astype(np.float32)
        divisor = np.where(divisor == 0, np.float32(1.0), divisor)
        scaled = (blocks / divisor[..., None]).astype(np.float32)
    code = e2m1_round(scaled).reshape(work.shape)
    packed = (code[..., 0::2] | (code[..., 1::2] << 4)).astype(np.uint8)
    return (np.ascontiguousarray(np.moveaxis(packed, -1, axis)), np.ascontiguousarray(np.moveaxis(scale_bits, -1, axis)),
            np.float32(g))


def dequantize_nvfp4(data: np.ndarray, scales: np.ndarray, g, axis: int = -1) -> np.ndarray:
    """``level * sign * (scale * global)`` in fp32, rounded to bf16 as the reference returns it
    (``quantization.py:277-297``); returned as fp32 holding bf16 values."""
    axis = axis % data.ndim
    codes = np.moveaxis(unpack_codes(data, axis), axis, -1)
    elems = E2M1_LEVELS[codes & 7] * (1 - 2 * (codes >> 3).astype(np.float32))
    with np.errstate(invalid="ignore", over="ignore"):
        s = (_decode_scale(np.moveaxis(scales, axis, -1)) * np.float32(g)).astype(np.float32)
        out = (elems.reshape(*elems.shape[:-1], elems.shape[-1] // BLOCK, BLOCK) * s[..., None]).reshape(elems.shape)
    return np.ascontiguousarray(np.moveaxis(_round_to_bf16(out.astype(np.float32)), -1, axis))


def fake_quant_nvfp4(t: np.ndarray, axis: int = -1) -> np.ndarray:
    """Quantise then dequantise (``quantization.py:307-311``): fp32 holding bf16 values."""
    data, scales, g = quantize_nvfp4(t, axis)
    return dequantize_nvfp4(data, scales, g, axis)


def expert_gemm_nvfp4(a: np.ndarray, b: np.ndarray, offs, acc_dtype=np.float64) -> np.ndarray:
    """``grouped_mm(fake_quant(a, axis=-1), fake_quant(b, axis=1))`` (``expert_gemm.py:33-38``) accumulated in
    ``acc_dtype``.  ``a [R, K]``, ``b [G, K, N]`` (one global scale for the whole bank), ``offs`` the inclusive group
    ends."""
    aq = fake_quant_nvfp4(a, -1).astype(acc_dtype)
    bq = fake_quant_nvfp4(b, 1).astype(acc_dtype)
    out = np.zeros((a.shape[0], b.shape[2]), dtype=acc_dtype)
    start = 0
    for g, end in enumerate(np.asarray(offs).tolist()):
        if end > start:
            out[start:end] = aq[start:end] @ bq[g]
        start = end
    return out


class _FakeQuantSTE(torch.autograd.Function):
    """The round trip on a CPU tensor with the identity backward (``quantization.py:350-360``)."""

    @staticmethod
    def forward(ctx, t, axis):
        out = fake_quant_nvfp4(t.detach().float().numpy(), axis)
        return torch.from_numpy(out).to(t.dtype)

    @staticmethod
    def backward(ctx, grad):
        return grad, None


def fake_quant_ste(t: torch.Tensor, axis: int = -1) -> torch.Tensor:
    """``fake_quant(t, "nvfp4", axis)`` for CPU tensors inside an autograd graph."""
    return _FakeQuantSTE.apply(t, axis)
