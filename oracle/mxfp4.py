"""Oracle (test infrastructure): MXFP4 block-scaled quantisation (e2m1 elements, two per byte, one e8m0 power-of-two
scale per 32 values along the contraction axis), its dequantiser, the fake-quant round trip and the fake-quantised
expert GEMM, in numpy.

Follows the eager CPU path of ``halo/kernels/lowp/quantization.py``: ``_e8m0_scale`` (:154-160), ``_e8m0_scale_down``
(:167-180), ``_e2m1_round`` (:191-198), ``_mxfp4_core`` (:208-211), ``_quantize_fp4`` (:248-263), ``dequantize``
(:277-297); the expert GEMM is ``halo/kernels/expert_gemm.py:33-38``.  The e8m0 helpers are those of ``oracle.mxfp8``
with the format maximum 6 in place of 448.

The block exponent ``ceil(log2(max(amax, tiny) / 6))`` is evaluated in integer arithmetic on the operand's exponent and
mantissa (6 = 0.75 * 2^3), which is what the reference's fp32 ``log2`` gives for every bf16 amax; for fp32 inputs whose
amax / 6 lies within an ulp of a power of two the reference's result depends on its ``log2`` rounding, and such inputs
are outside what this oracle pins.
"""

from __future__ import annotations

import numpy as np
import torch

from oracle.mxfp8 import AMAX_FLOOR, E8M0_BIAS, E8M0_NAN, _round_to_bf16, e8m0_to_float, scale_down

BLOCK = 32
E2M1_MAX = 6.0
E2M1_LEVELS = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)  # magnitudes of codes 0..7


def e8m0_exponent(amax: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """``(exponent int64, biased uint8)`` per block (``quantization.py:154-160`` at format maximum 6): the smallest
    ``e`` with ``2^e >= max(amax, tiny) / 6``, clamped to [-127, 127]; a NaN block takes the code 0xFF."""
    amax = np.asarray(amax, dtype=np.float32)
    nan = np.isnan(amax)
    inf = np.isinf(amax)
    finite = np.where(nan | inf, np.float32(1.0), np.maximum(amax, AMAX_FLOOR))
    mantissa, exponent = np.frexp(finite.astype(np.float64))  # finite = mantissa * 2^exponent, mantissa in [0.5, 1)
    e = exponent.astype(np.int64) - 3 + (mantissa > 0.75)
    e = np.where(inf, E8M0_BIAS, np.clip(e, -E8M0_BIAS, E8M0_BIAS))
    biased = np.where(nan, E8M0_NAN, e + E8M0_BIAS).astype(np.uint8)
    return e, biased


def e2m1_round(scaled: np.ndarray) -> np.ndarray:
    """uint8 codes ``sign << 3 | level`` of values already brought to e2m1's range (``quantization.py:191-198``): the
    number of level midpoints strictly below the clamped magnitude (``bucketize``, which sends a value on a midpoint
    down and a NaN past the last one), plus one on the midpoints 0.75, 1.75 and 3.5, whose upper neighbour has the even
    code."""
    scaled = np.asarray(scaled, dtype=np.float32)
    with np.errstate(invalid="ignore"):
        sign = (scaled < 0).astype(np.uint8)
        mag = np.minimum(np.abs(scaled), np.float32(E2M1_MAX))  # NaN stays NaN, as torch's clamp keeps it
    midpoints = (E2M1_LEVELS[:-1] + E2M1_LEVELS[1:]) / 2
    with np.errstate(invalid="ignore"):
        below = (midpoints[None, :] < mag.reshape(-1, 1)).sum(axis=1).reshape(mag.shape)
    level = np.where(np.isnan(mag), len(midpoints), below).astype(np.uint8)
    ties_up = np.isin(mag, midpoints[1::2]).astype(np.uint8)
    return ((level + ties_up) | (sign << 3)).astype(np.uint8)


def quantize_mxfp4(t: np.ndarray, axis: int = -1) -> tuple[np.ndarray, np.ndarray]:
    """``(data uint8 with the axis halved, two codes per byte, the even element in the low nibble; scales uint8 with the
    axis divided by 32)`` (``quantization.py:208-211, 248-263``)."""
    t = np.asarray(t, dtype=np.float32)
    axis = axis % t.ndim
    if t.shape[axis] % BLOCK:
        raise ValueError(f"axis {axis} size {t.shape[axis]} not divisible by block_size {BLOCK}")
    work = np.moveaxis(t, axis, -1)
    blocks = work.reshape(*work.shape[:-1], work.shape[-1] // BLOCK, BLOCK)
    with np.errstate(invalid="ignore"):
        amax = np.abs(blocks).max(axis=-1)
    e, biased = e8m0_exponent(amax)
    scaled = scale_down(blocks, e[..., None])
    scaled = np.where((biased == E8M0_NAN)[..., None], np.float32(np.nan), scaled)  # exp2(-NaN) poisons the block
    code = e2m1_round(scaled).reshape(work.shape)
    packed = (code[..., 0::2] | (code[..., 1::2] << 4)).astype(np.uint8)
    return np.ascontiguousarray(np.moveaxis(packed, -1, axis)), np.ascontiguousarray(np.moveaxis(biased, -1, axis))


def unpack_codes(data: np.ndarray, axis: int = -1) -> np.ndarray:
    """The 4-bit codes of packed ``data``, the axis doubled."""
    work = np.moveaxis(np.asarray(data, dtype=np.uint8), axis % data.ndim, -1)
    codes = np.stack([work & 0x0F, work >> 4], axis=-1).reshape(*work.shape[:-1], work.shape[-1] * 2)
    return np.ascontiguousarray(np.moveaxis(codes, -1, axis % data.ndim))


def dequantize_mxfp4(data: np.ndarray, scales: np.ndarray, axis: int = -1) -> np.ndarray:
    """``level * sign * 2^(s - 127)`` in fp32, rounded to bf16 as the reference returns it (``quantization.py:277-297``);
    returned as fp32 holding bf16 values."""
    axis = axis % data.ndim
    codes = np.moveaxis(unpack_codes(data, axis), axis, -1)
    elems = E2M1_LEVELS[codes & 7] * (1 - 2 * (codes >> 3).astype(np.float32))
    s = e8m0_to_float(np.moveaxis(scales, axis, -1))
    with np.errstate(invalid="ignore", over="ignore"):
        out = (elems.reshape(*elems.shape[:-1], elems.shape[-1] // BLOCK, BLOCK) * s[..., None]).reshape(elems.shape)
    return np.ascontiguousarray(np.moveaxis(_round_to_bf16(out.astype(np.float32)), -1, axis))


def fake_quant_mxfp4(t: np.ndarray, axis: int = -1) -> np.ndarray:
    """Quantise then dequantise (``quantization.py:307-311``): fp32 holding bf16 values."""
    data, scales = quantize_mxfp4(t, axis)
    return dequantize_mxfp4(data, scales, axis)


def expert_gemm_mxfp4(a: np.ndarray, b: np.ndarray, offs, acc_dtype=np.float64) -> np.ndarray:
    """``grouped_mm(fake_quant(a, axis=-1), fake_quant(b, axis=1))`` (``expert_gemm.py:33-38``) accumulated in
    ``acc_dtype``.  ``a [R, K]``, ``b [G, K, N]``, ``offs`` the inclusive group ends."""
    aq = fake_quant_mxfp4(a, -1).astype(acc_dtype)
    bq = fake_quant_mxfp4(b, 1).astype(acc_dtype)
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
        out = fake_quant_mxfp4(t.detach().float().numpy(), axis)
        return torch.from_numpy(out).to(t.dtype)

    @staticmethod
    def backward(ctx, grad):
        return grad, None


def fake_quant_ste(t: torch.Tensor, axis: int = -1) -> torch.Tensor:
    """``fake_quant(t, "mxfp4", axis)`` for CPU tensors inside an autograd graph."""
    return _FakeQuantSTE.apply(t, axis)
