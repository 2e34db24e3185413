// The tail shared by the kernels that write e4m3 activation panels: sixteen lanes hold one row's block of 128 values,
// eight each; the block's power-of-two scale is found and the values are written as e4m3 with their exponent byte.
#pragma once
#include "common.h"

namespace hmoe {

// v: this lane's eight values of row `row`, columns [8 chunk, 8 chunk + 8).  With amax = m 2^x (1 <= m < 2) the
// smallest e for which amax 2^-e <= 448 = 1.75 2^8 is x - 8, one more where m > 1.75; stored biased (e + 127),
// clamped at 0 (an all-zero block gets 0).  q = v 2^-e rounded to nearest even, into panels of 64 values: values
// [64 p, 64 p + 64) of row r at q[(p * out_rows + r) * 64]; the scale of block b at scale[b * out_rows + r].
// Every lane of a group of sixteen must call this together.
__device__ __forceinline__ void quantize_block_of_row(const float (&v)[8], int64_t row, int chunk, uint8_t* __restrict__ q,
                                                      uint8_t* __restrict__ scale, int64_t out_rows) {
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
#pragma unroll
  for (int off = 1; off < 16; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 16));
  const uint32_t bits = __float_as_uint(amax);
  int biased = static_cast<int>(bits >> 23) - 8 + ((bits & 0x007fffffu) > 0x00600000u ? 1 : 0);
  biased = biased < 0 ? 0 : biased;
  const float inv = __uint_as_float(static_cast<uint32_t>(254 - biased) << 23);  // 2^-(biased - 127), exact
  uint2 packed;
  int word = 0;
  word = __builtin_amdgcn_cvt_pk_fp8_f32(v[0] * inv, v[1] * inv, word, false);
  word = __builtin_amdgcn_cvt_pk_fp8_f32(v[2] * inv, v[3] * inv, word, true);
  packed.x = static_cast<uint32_t>(word);
  word = 0;
  word = __builtin_amdgcn_cvt_pk_fp8_f32(v[4] * inv, v[5] * inv, word, false);
  word = __builtin_amdgcn_cvt_pk_fp8_f32(v[6] * inv, v[7] * inv, word, true);
  packed.y = static_cast<uint32_t>(word);
  const int64_t slot = static_cast<int64_t>(chunk >> 3) * out_rows + row;
  *reinterpret_cast<uint2*>(q + slot * 64 + ((chunk & 7) << 3)) = packed;
  if ((chunk & 15) == 0) scale[static_cast<int64_t>(chunk >> 4) * out_rows + row] = static_cast<uint8_t>(biased);
}

// MXFP8: two lanes hold one row's block of 32 values, sixteen each.  The block's e8m0 code is the biased exponent of the
// smallest power of two 2^e >= amax / 448 with e clamped to [-127, 127] (an all-zero block gets 0, one holding an inf
// 254 and one holding a NaN 0xFF, the format's NaN), as quantize_mxfp8 of the reference computes it
// (halo/kernels/lowp/quantization.py:154-188).  q = clamp(v 2^-e, +-448) rounded to nearest even; a block at e = 127
// is halved and scaled by 2^-126, so that no subnormal factor enters (:167-180); every element of a NaN block is NaN.
// Panels as above; the scale of 32-block b at scale[b * out_rows + row].
__device__ __forceinline__ uint32_t mx_block_code(float amax, bool any_nan) {
  const uint32_t bits = __float_as_uint(amax);
  int biased = static_cast<int>(bits >> 23) - 8 + ((bits & 0x007fffffu) > 0x00600000u ? 1 : 0);
  biased = biased < 0 ? 0 : biased;
  if (bits >= 0x7f800000u) biased = 254;
  return any_nan ? 255u : static_cast<uint32_t>(biased);
}

// The factor pair that brings a block at code `biased` (0..254) to e4m3's range: v * pre * inv.
__device__ __forceinline__ void mx_scale_down(uint32_t biased, float& pre, float& inv) {
  const bool top = biased >= 254u;
  pre = top ? 0.5f : 1.0f;
  inv = __uint_as_float((top ? 1u : 254u - biased) << 23);  // 2^(127 - biased), 2^-126 at the top
}

__device__ __forceinline__ float mx_clamp(float v) { return fminf(fmaxf(v, -448.0f), 448.0f); }

// v: this lane's sixteen values of row `row`, values [16 sub, 16 sub + 16) of panel `panel`; the lane pair (sub, sub ^ 1)
// holds one block of 32.  Writes the lane's 16 codes into the panel (q[(panel * out_rows + row) * 64 + 16 sub]) and, from
// the even lane, the block's exponent (scale[(2 panel + sub / 2) * out_rows + row]).  Both lanes of a pair must call
// this together.
__device__ __forceinline__ void quantize_mx_half_block(const float (&v)[16], int64_t row, int panel, int sub,
                                                       uint8_t* __restrict__ q, uint8_t* __restrict__ scale,
                                                       int64_t out_rows) {
  float amax = 0.f;
  int nan = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    amax = fmaxf(amax, fabsf(v[i]));
    nan |= v[i] != v[i];
  }
  amax = fmaxf(amax, __shfl_xor(amax, 1, 2));
  nan |= __shfl_xor(nan, 1, 2);
  const uint32_t biased = mx_block_code(amax, nan != 0);
  float pre, inv;
  mx_scale_down(biased, pre, inv);
  uint32_t words[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    int word = 0;
    word = __builtin_amdgcn_cvt_pk_fp8_f32(mx_clamp(v[4 * w] * pre * inv), mx_clamp(v[4 * w + 1] * pre * inv), word, false);
    word = __builtin_amdgcn_cvt_pk_fp8_f32(mx_clamp(v[4 * w + 2] * pre * inv), mx_clamp(v[4 * w + 3] * pre * inv), word, true);
    words[w] = nan ? 0x7f7f7f7fu : static_cast<uint32_t>(word);
  }
  *reinterpret_cast<uint4*>(q + (static_cast<int64_t>(panel) * out_rows + row) * 64 + sub * 16) =
      make_uint4(words[0], words[1], words[2], words[3]);
  if ((sub & 1) == 0) scale[static_cast<int64_t>(2 * panel + (sub >> 1)) * out_rows + row] = static_cast<uint8_t>(biased);
}

}  // namespace hmoe
