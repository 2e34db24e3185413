"""Oracle (test infrastructure): MXFP8 block-scaled quantisation (e4m3 elements, one e8m0 power-of-two scale per 32
values along the contraction axis), its dequantiser, the fake-quant round trip and the fake-quantised expert GEMM, in
numpy.

Follows the eager CPU path of ``halo/kernels/lowp/quantization.py``: ``_e8m0_scale`` (:154-160), ``_e8m0_to_float``
(:163-164), ``_e8m0_scale_down`` (:167-180), ``_mxfp8_core`` (:183-188), ``quantize_mxfp8`` (:236-245), ``dequantize``
(:277-297) and ``_block_round_trip`` / ``fake_quant`` (:307-311, :363-365); the expert GEMM is
``halo/kernels/expert_gemm.py:33-38`` (activations quantised along their last axis, ``[E, K, N]`` weights along axis
1, then the bf16 grouped product).  The e4m3 codec is the explicit one of ``oracle.block_fp8``.

The block exponent ``ceil(log2(max(amax, tiny) / 448))`` is evaluated here in integer arithmetic on the operand's
exponent and mantissa, which is what the reference's fp32 ``log2`` gives for every bf16 amax (the nearest bf16
neighbours of a power-of-two multiple of 448 lie 0.4 % away, far outside ``log2``'s rounding).  For fp32 inputs whose
amax / 448 lies within an ulp of a power of two the reference's result depends on its ``log2`` and divider rounding and
may be one higher or lower; such inputs are outside what this oracle pins.
"""

from __future__ import annotations

import numpy as np
import torch

from oracle.block_fp8 import decode_e4m3fn, encode_e4m3fn

BLOCK = 32
E4M3_MAX = 448.0
E8M0_BIAS = 127
E8M0_NAN = 255
AMAX_FLOOR = np.finfo(np.float32).tiny


def e8m0_exponent(amax: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """``(exponent int64, biased uint8)`` per block (``quantization.py:154-160``): the smallest ``e`` with
    ``2^e >= max(amax, tiny) / 448``, clamped to [-127, 127]; a NaN block takes the code 0xFF."""
    amax = np.asarray(amax, dtype=np.float32)
    nan = np.isnan(amax)
    inf = np.isinf(amax)
    finite = np.where(nan | inf, np.float32(1.0), np.maximum(amax, AMAX_FLOOR))
    mantissa, exponent = np.frexp(finite.astype(np.float64))  # finite = mantissa * 2^exponent, mantissa in [0.5, 1)
    # 448 = 0.875 * 2^9: finite / 448 = (mantissa / 0.875) * 2^(exponent - 9), whose log2 rounds up to exponent - 9 when
    # the mantissa is at most 0.875 and to one more above
    e = exponent.astype(np.int64) - 9 + (mantissa > 0.875)
    e = np.where(inf, E8M0_BIAS, np.clip(e, -E8M0_BIAS, E8M0_BIAS))
    biased = np.where(nan, E8M0_NAN, e + E8M0_BIAS).astype(np.uint8)
    return e, biased


def e8m0_to_float(scales: np.ndarray) -> np.ndarray:
    """``2^(s - 127)`` in fp32, NaN for 0xFF (``quantization.py:163-164``)."""
    scales = np.asarray(scales)
    exponent = np.where(scales == E8M0_NAN, 0, scales.astype(np.int64) - E8M0_BIAS)
    out = np.ldexp(np.float32(1.0), exponent).astype(np.float32)
    return np.where(scales == E8M0_NAN, np.float32(np.nan), out)


def scale_down(blocks: np.ndarray, e: np.ndarray) -> np.ndarray:
    """``blocks * 2^-e`` rounded once to fp32 (``quantization.py:167-180``); a block at exponent 127 is halved first and
    scaled by 2^-126, so that no subnormal scale enters."""
    top = e == E8M0_BIAS
    factor = np.ldexp(np.float32(1.0), (np.where(top, 1, 0) - e).astype(np.int64)).astype(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        return (blocks.astype(np.float32) * np.where(top, np.float32(0.5), np.float32(1.0))).astype(np.float32) * factor


def _encode_with_nan(scaled: np.ndarray) -> np.ndarray:
    """e4m3fn codes of clamped values; NaN keeps its sign and takes the format's only NaN pattern (0x7F)."""
    nan = np.isnan(scaled)
    codes = encode_e4m3fn(np.where(nan, np.float32(0.0), scaled))
    return np.where(nan, (np.signbit(scaled).astype(np.uint8) << 7) | 0x7F, codes).astype(np.uint8)


def quantize_mxfp8(t: np.ndarray, axis: int = -1) -> tuple[np.ndarray, np.ndarray]:
    """``(data uint8 e4m3fn codes of t's shape, scales uint8 with the axis divided by 32)`` (``quantization.py:183-188,
    236-245``)."""
    t = np.asarray(t, dtype=np.float32)
    axis = axis % t.ndim
    if t.shape[axis] % BLOCK:
        raise ValueError(f"axis {axis} size {t.shape[axis]} not divisible by block_size {BLOCK}")
    work = np.moveaxis(t, axis, -1)
    blocks = work.reshape(*work.shape[:-1], work.shape[-1] // BLOCK, BLOCK)
    with np.errstate(invalid="ignore"):
        amax = np.abs(blocks).max(axis=-1)  # numpy's max propagates NaN, as torch.amax does
    e, biased = e8m0_exponent(amax)
    scaled = scale_down(blocks, e[..., None])
    # a NaN amax makes the reference's exponent NaN and with it every element of the block (``exp2(-NaN)``)
    scaled = np.where((biased == E8M0_NAN)[..., None], np.float32(np.nan), scaled)
    with np.errstate(invalid="ignore"):
        clamped = np.where(np.isnan(scaled), scaled, np.clip(scaled, -E4M3_MAX, E4M3_MAX)).astype(np.float32)
    data = _encode_with_nan(clamped).reshape(work.shape)
    return np.ascontiguousarray(np.moveaxis(data, -1, axis)), np.ascontiguousarray(np.moveaxis(biased, -1, axis))


def _round_to_bf16(x: np.ndarray) -> np.ndarray:
    """fp32 values rounded to bf16 (nearest even), returned as fp32."""
    bits = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    out = rounded.view(np.float32)
    return np.where(np.isnan(x), np.float32(np.nan), out)


def dequantize_mxfp8(data: np.ndarray, scales: np.ndarray, axis: int = -1) -> np.ndarray:
    """``code * 2^(s - 127)`` in fp32, rounded to bf16 as the reference returns it (``quantization.py:277-297``);
    returned as fp32 holding bf16 values."""
    axis = axis % data.ndim
    elems = decode_e4m3fn(np.moveaxis(data, axis, -1))
    elems = np.where((np.moveaxis(data, axis, -1) & 0x7F) == 0x7F, np.float32(np.nan), elems)
    s = e8m0_to_float(np.moveaxis(scales, axis, -1))
    with np.errstate(invalid="ignore", over="ignore"):
        out = (elems.reshape(*elems.shape[:-1], elems.shape[-1] // BLOCK, BLOCK) * s[..., None]).reshape(elems.shape)
    return np.ascontiguousarray(np.moveaxis(_round_to_bf16(out.astype(np.float32)), -1, axis))


def fake_quant_mxfp8(t: np.ndarray, axis: int = -1) -> np.ndarray:
    """Quantise then dequantise (``quantization.py:307-311``): fp32 holding bf16 values."""
    data, scales = quantize_mxfp8(t, axis)
    return dequantize_mxfp8(data, scales, axis)


def expert_gemm_mxfp8(a: np.ndarray, b: np.ndarray, offs, acc_dtype=np.float64) -> np.ndarray:
    """``grouped_mm(fake_quant(a, axis=-1), fake_quant(b, axis=1))`` (``expert_gemm.py:33-38``) accumulated in
    ``acc_dtype``: every product of two dequantised values is exact in float64, so with float64 this is the value any
    accumulation order approximates.  ``a [R, K]``, ``b [G, K, N]``, ``offs`` the inclusive group ends."""
    aq = fake_quant_mxfp8(a, -1).astype(acc_dtype)
    bq = fake_quant_mxfp8(b, 1).astype(acc_dtype)
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
        out = fake_quant_mxfp8(t.detach().float().numpy(), axis)
        return torch.from_numpy(out).to(t.dtype)

    @staticmethod
    def backward(ctx, grad):
        return grad, None


def fake_quant_ste(t: torch.Tensor, axis: int = -1) -> torch.Tensor:
    """``fake_quant(t, "mxfp8", axis)`` for CPU tensors inside an autograd graph."""
    return _FakeQuantSTE.apply(t, axis)
