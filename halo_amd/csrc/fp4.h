// e2m1 (fp4) element conversion shared by the MXFP4 and NVFP4 kernels: codes by the conversion instruction, and the
// 16-value row piece both kernels' lanes load.
#pragma once

#include "common.h"

namespace hmoe {

// Two scaled values to two e2m1 codes (sign << 3 | level) in byte `kByte` of `word`, by the conversion instruction:
// the nearest level, a tie to the level with the even code, magnitudes above 6 (an inf too) to 6.  That is the
// reference's rule (quantization.py:191-198: bucketize sends a value on a boundary down, the ties-up table lifts 0.75,
// 1.75 and 3.5; the even code is the even significand, so it is IEEE round-to-nearest-even at e2m1's precision): the
// instruction gives the reference's code for every multiple of 1/64 in [-7, 7], for infinities and for a positive NaN
// (code 7, where bucketize puts it).  The sign bit is set for a value below zero and not for -0.0, as `scaled < 0` has
// it: adding +0.0 turns -0.0 into +0.0 and changes nothing else.  The addition must stay an operation of its own
// (contraction off): fused into the multiplication that scaled the value it would see the exact product, and a negative
// value that the fp32 product rounds to -0.0 (a block holding an inf, or one spanning more than 150 binades) would
// keep its sign where the reference's two operations drop it.
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float without_negative_zero(float x) {
#pragma clang fp contract(off)
  return x + 0.0f;
}
template <int kByte>
__device__ __forceinline__ uint32_t e2m1_pack2(uint32_t word, float lo, float hi) {
  return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(word, without_negative_zero(lo), without_negative_zero(hi), 1.0f,
                                                  kByte);
}
__device__ __forceinline__ uint32_t e2m1_pack8(const float* v) {
  uint32_t word = 0u;
  word = e2m1_pack2<0>(word, v[0], v[1]);
  word = e2m1_pack2<1>(word, v[2], v[3]);
  word = e2m1_pack2<2>(word, v[4], v[5]);
  word = e2m1_pack2<3>(word, v[6], v[7]);
  return word;
}
// the values of the eight codes of a word: levels 0, 0.5, 1, 1.5, 2, 3, 4, 6 under the sign bit
__device__ __forceinline__ void e2m1_unpack8(uint32_t word, float* v) {
  const f32x2_t a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 0);
  const f32x2_t b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 1);
  const f32x2_t c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 2);
  const f32x2_t d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 3);
  v[0] = a.x; v[1] = a.y; v[2] = b.x; v[3] = b.y; v[4] = c.x; v[5] = c.y; v[6] = d.x; v[7] = d.y;
}

template <typename T>
__device__ __forceinline__ void load16(const T* p, float (&v)[16]);
template <>
__device__ __forceinline__ void load16<bf16_t>(const bf16_t* p, float (&v)[16]) {
  Vec16<bf16_t> lo, hi;
  lo.load(p);
  hi.load(p + 8);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    v[i] = lo.v[i];
    v[8 + i] = hi.v[i];
  }
}
template <>
__device__ __forceinline__ void load16<float>(const float* p, float (&v)[16]) {
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const float4 t = *reinterpret_cast<const float4*>(p + 4 * c);
    v[4 * c] = t.x; v[4 * c + 1] = t.y; v[4 * c + 2] = t.z; v[4 * c + 3] = t.w;
  }
}

}  // namespace hmoe
