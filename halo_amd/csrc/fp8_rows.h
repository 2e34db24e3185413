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

}  // namespace hmoe
