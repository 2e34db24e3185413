"""Oracle (test infrastructure): 128x128-block e4m3 weight quantiser and its dequantiser, in numpy.

Follows ``halo/kernels/lowp/block_fp8.py:16-34`` (quantise: per block ``scale = 2^ceil(log2(max(amax,1e-12)/448))``
read off the exponent bits, ``q = clamp(x/scale, +-448)`` rounded to float8_e4m3fn) and
``halo/checkpoint/tools/fp8_dequant.py:153-170`` (dequantise: ``q * scale`` in fp32, rounded once to bf16).
The e4m3fn encoder is explicit (round to nearest, ties to even; 4 exponent bits with bias 7, 3 mantissa bits,
subnormals at 2^-9 steps, maximum 448, no infinities).
"""

from __future__ import annotations

import numpy as np

BLOCK = 128
E4M3_MAX = 448.0
AMAX_FLOOR = 1e-12


def pow2_ceil(x: np.ndarray) -> np.ndarray:
    """Smallest power of two >= each positive fp32 ``x`` (``block_fp8.py:16-20``)."""
    mantissa, exponent = np.frexp(x.astype(np.float32))
    return np.ldexp(np.float32(1.0), exponent - (mantissa == 0.5)).astype(np.float32)


def encode_e4m3fn(x: np.ndarray) -> np.ndarray:
    """fp32 values with ``|x| <= 448`` to float8_e4m3fn bit patterns (uint8), round to nearest even."""
    x = x.astype(np.float32)
    sign = (np.signbit(x)).astype(np.uint8) << 7
    mag = np.abs(x).astype(np.float64)
    # exponent of the value's binade, clamped to the subnormal binade 2^-6
    _, e = np.frexp(mag)  # mag = m * 2^e, m in [0.5, 1)
    binade = np.maximum(e - 1, -6)
    step = np.ldexp(1.0, binade - 3)  # spacing of representable values in this binade
    quanta = np.rint(mag / step)  # numpy rint rounds half to even
    value = quanta * step
    # re-derive fields from the rounded value (rounding may carry into the next binade)
    _, e2 = np.frexp(value)
    binade2 = np.maximum(e2 - 1, -6)
    mant = np.rint(value / np.ldexp(1.0, binade2 - 3)).astype(np.int64)  # 0..15
    is_normal = mant >= 8
    exp_field = np.where(is_normal, binade2 + 7, 0).astype(np.int64)
    mant_field = np.where(is_normal, mant - 8, mant).astype(np.int64)
    bits = (exp_field << 3) | mant_field
    bits = np.where(value == 0, 0, bits)
    return (sign | bits.astype(np.uint8)).astype(np.uint8)


def decode_e4m3fn(bits: np.ndarray) -> np.ndarray:
    bits = bits.astype(np.uint8)
    sign = np.where(bits & 0x80, -1.0, 1.0)
    exp_field = ((bits >> 3) & 0xF).astype(np.int64)
    mant = (bits & 0x7).astype(np.float64)
    normal = np.ldexp(1.0 + mant / 8.0, exp_field - 7)
    subnormal = np.ldexp(mant / 8.0, -6)
    return (sign * np.where(exp_field == 0, subnormal, normal)).astype(np.float32)


def quantize_block_fp8(weight: np.ndarray):
    """``(q uint8 e4m3fn bits [..., N, K], scale fp32 [..., ceil(N/128), ceil(K/128)])``."""
    w = weight.astype(np.float32)
    n, k = w.shape[-2:]
    pad = [(0, 0)] * (w.ndim - 2) + [(0, -n % BLOCK), (0, -k % BLOCK)]
    padded = np.pad(w, pad)
    lead = padded.shape[:-2]
    blocks = padded.reshape(*lead, padded.shape[-2] // BLOCK, BLOCK, padded.shape[-1] // BLOCK, BLOCK)
    amax = np.maximum(np.abs(blocks).max(axis=(-3, -1), keepdims=True), np.float32(AMAX_FLOOR)).astype(np.float32)
    scale = pow2_ceil(amax / np.float32(E4M3_MAX))
    scaled = np.clip((blocks / scale).astype(np.float32), -E4M3_MAX, E4M3_MAX)
    q = encode_e4m3fn(scaled).reshape(padded.shape)[..., :n, :k]
    return np.ascontiguousarray(q), np.ascontiguousarray(scale[..., 0, :, 0])


def dequantize_block_fp8(q_bits: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """fp32 ``q * scale`` (the caller rounds to bf16 where the reference does)."""
    n, k = q_bits.shape[-2:]
    s = np.repeat(np.repeat(scale, BLOCK, axis=-2)[..., :n, :], BLOCK, axis=-1)[..., :k]
    return decode_e4m3fn(q_bits) * s.astype(np.float32)
