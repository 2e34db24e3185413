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


# ------------------------------------------------------------------------------- activations, one row and 128 values
# The "dynamic" activation scheme that block_fp8_quantization_config (``block_fp8.py:37-46``) names for the serving
# engine, which the reference itself holds no code for; the restatement below is the published recipe (one scale per
# token and 128 channels, amax / 448 rounded up to a power of two), pinned by its own properties in the tests: the
# scale is the smallest power of two that keeps the block inside e4m3's range, and q * scale is x to e4m3 precision.

def row_scale_exponents(x: np.ndarray) -> np.ndarray:
    """Biased exponents ``e + 127`` (uint8 ``[R, K/128]``) of the smallest power of two ``2^e`` with
    ``amax * 2^-e <= 448`` per row and 128 values; clamped at 0, which is also what an all-zero block gets."""
    rows, k = x.shape
    amax = np.abs(x.astype(np.float32)).reshape(rows, k // BLOCK, BLOCK).max(axis=2)
    mantissa, exponent = np.frexp(amax)  # amax = mantissa * 2^exponent, mantissa in [0.5, 1)
    # 448 = 0.875 * 2^9: e = exponent - 9, one more where the mantissa is above 0.875
    e = exponent.astype(np.int64) - 9 + (mantissa > 0.875)
    biased = np.where(amax == 0, 0, np.clip(e + 127, 0, 254))
    return biased.astype(np.uint8)


def quantize_rows_fp8(x: np.ndarray):
    """``(q uint8 e4m3fn bits [R, K], biased exponents uint8 [K/128, R])`` for fp32 ``x`` holding bf16 values."""
    rows, k = x.shape
    biased = row_scale_exponents(x)
    inv = np.ldexp(np.float64(1.0), 127 - biased.astype(np.int64))  # [R, K/128], exact
    scaled = x.astype(np.float64).reshape(rows, k // BLOCK, BLOCK) * inv[:, :, None]
    return encode_e4m3fn(scaled.reshape(rows, k).astype(np.float32)), np.ascontiguousarray(biased.T)


def dequantize_rows_fp8(q_bits: np.ndarray, biased_t: np.ndarray) -> np.ndarray:
    """float64 ``q * 2^e`` for the pair :func:`quantize_rows_fp8` returns."""
    rows, k = q_bits.shape
    scale = np.ldexp(np.float64(1.0), biased_t.T.astype(np.int64) - 127)  # [R, K/128]
    return (decode_e4m3fn(q_bits).astype(np.float64).reshape(rows, k // BLOCK, BLOCK) * scale[:, :, None]).reshape(rows, k)


def fp8_grouped_mm(q_bits: np.ndarray, biased_t: np.ndarray, w_bits: np.ndarray, w_scale: np.ndarray,
                   offs: np.ndarray) -> np.ndarray:
    """float64 ``[R, N]``: per group ``(q * 2^e)[s:e] @ (w * w_scale)[g]`` with ``w_bits [G, K, N]`` and
    ``w_scale [G, ceil(K/128), ceil(N/128)]``.  Every product of two e4m3 values and two scales is exact in
    float64, so this is the value the fp8 kernel's fp32 accumulation approximates."""
    a = dequantize_rows_fp8(q_bits, biased_t)
    w = dequantize_block_fp8(w_bits, w_scale).astype(np.float64)
    out = np.zeros((a.shape[0], w.shape[2]))
    start = 0
    for g, end in enumerate(np.asarray(offs).tolist()):
        out[start:end] = a[start:end] @ w[g]
        start = end
    return out
