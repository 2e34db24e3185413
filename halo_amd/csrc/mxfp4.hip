// MXFP4 for gfx950: e2m1 elements (magnitudes 0, 0.5, 1, 1.5, 2, 3, 4, 6) with one e8m0 power-of-two scale per 32
// values along the contraction axis (OCP Microscaling).
//
// Replaces quantize_mxfp4 / dequantize / the fake-quant round trip of the reference for this format
// (halo/kernels/lowp/quantization.py:154-180, 191-198, 208-211, 248-269, 277-297, 307-311).  The reference's
// expert_gemm(quant_format="mxfp4") multiplies the two round-tripped operands with the bf16 grouped GEMM
// (halo/kernels/expert_gemm.py:33-38); that is what this build does too, so the kernels here produce the round trip's
// bf16 result in one pass (and, for the quantiser API, the packed codes and exponents in the reference's layout: two
// codes per byte along the quantised axis, low nibble first).
#include "common.h"
#include "fp8_rows.h"

namespace hmoe {
namespace {

// The block's e8m0 code: the biased exponent of the smallest power of two 2^e >= amax / 6, e clamped to [-127, 127];
// 254 for a block holding an inf, 0xFF for one holding a NaN.  6 = 1.5 * 2^2: with amax = (1 + f) 2^E the quotient is
// (1 + f) / 1.5 * 2^(E - 2), whose log2 rounds up to E - 2 while 1 + f <= 1.5 and to E - 1 above.
__device__ __forceinline__ uint32_t mx4_block_code(float amax, bool any_nan) {
  const uint32_t bits = __float_as_uint(amax);
  int biased = static_cast<int>(bits >> 23) - 2 + ((bits & 0x007fffffu) > 0x00400000u ? 1 : 0);
  biased = biased < 0 ? 0 : (biased > 254 ? 254 : biased);
  if (bits >= 0x7f800000u) biased = 254;
  return any_nan ? 255u : static_cast<uint32_t>(biased);
}

// |scaled| (clamped to 6) rounded to the nearest e2m1 magnitude, a tie going to the level with the even code
// (quantization.py:191-198: bucketize sends a value on a boundary down, the ties-up table lifts 0.75, 1.75 and 3.5).
// The even code is the even significand, so this is IEEE round-to-nearest-even at e2m1's precision: below 1 the levels
// are the multiples of 0.5, which adding 2^22 rounds to; from 1 up they keep one mantissa bit.  A NaN clamps to 6, the
// level bucketize gives it.
__device__ __forceinline__ float e2m1_round_mag(float scaled) {
  const float mag = fminf(fabsf(scaled), 6.0f);
  const uint32_t bits = __float_as_uint(mag);
  const float one_bit = __uint_as_float((bits + 0x001fffffu + ((bits >> 22) & 1u)) & 0xffc00000u);
  const float halves = (mag + 4194304.0f) - 4194304.0f;
  return mag < 1.0f ? halves : one_bit;
}

// the level's code: 0.5, 1, 1.5, 2, 3, 4, 6 have the top bits 252, 254, 255 .. 259 (exponent and first mantissa bit)
__device__ __forceinline__ uint32_t e2m1_level(float rounded_mag) {
  const int from_bits = static_cast<int>(__float_as_uint(rounded_mag) >> 22) - 252;
  return static_cast<uint32_t>(max(from_bits, rounded_mag > 0.0f ? 1 : 0));
}

// e2m1 code (sign << 3 | level) of a scaled value; the sign bit is set for a value below zero (not for -0.0)
__device__ __forceinline__ uint32_t e2m1_code(float scaled) {
  return e2m1_level(e2m1_round_mag(scaled)) | (scaled < 0.0f ? 8u : 0u);
}

// the round trip of a scaled value before the block's scale is put back: the rounded magnitude under that sign
__device__ __forceinline__ float e2m1_round(float scaled) {
  const float mag = e2m1_round_mag(scaled);
  return scaled < 0.0f ? -mag : mag;
}

// the value of a code: levels 0, 0.5, 1, 1.5, 2, 3, 4, 6 with the sign bit
__device__ __forceinline__ float e2m1_value(uint32_t code) {
  const uint32_t level = code & 7u;
  // level >= 2: (1 + (level & 1) / 2) * 2^((level >> 1) - 1), assembled as fp32 bits
  const float mag = level < 2u ? 0.5f * static_cast<float>(level)
                               : __uint_as_float(((126u + (level >> 1)) << 23) | ((level & 1u) << 22));
  return (code & 8u) ? -mag : mag;
}

__device__ __forceinline__ float e8m0_to_f32(uint32_t code) {
  return __uint_as_float(code == 255u ? 0x7fc00000u : (code == 0u ? 0x00400000u : code << 23));
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

// Rows [R, K] along their last axis; row r is x[row_index[r]] (zeros for an index outside [0, x_rows)) or x[r] without
// an index.  Two lanes hold a block of 32 values, sixteen each.  Outputs, each optional: packed [R, K / 2] (two codes
// per byte, the even element in the low nibble), scale [R, K / 32], and round_trip bf16 [R, K] (row stride ldo): code
// value times 2^(scale - 127).
template <typename T>
__global__ void __launch_bounds__(256)
mxfp4_rows_kernel(const T* __restrict__ x, int64_t ldx, const int64_t* __restrict__ row_index, int64_t x_rows,
                  int64_t rows, int k, uint8_t* __restrict__ packed, uint8_t* __restrict__ scale,
                  bf16_t* __restrict__ round_trip, int64_t ldo) {
  const int pieces = k >> 4;  // 16-value pieces per row
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t row = unit / pieces;
  const int piece = static_cast<int>(unit - row * pieces);
  if (row >= rows) return;  // lane pairs leave together (pieces is even)
  float v[16];
  const int64_t from = row_index != nullptr ? row_index[row] : row;
  if (from >= 0 && from < x_rows) {
    load16<T>(x + from * ldx + (piece << 4), v);
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = 0.f;
  }
  float amax = 0.f;
  int nan = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    amax = fmaxf(amax, fabsf(v[i]));
    nan |= v[i] != v[i];
  }
  amax = fmaxf(amax, __shfl_xor(amax, 1, 2));
  nan |= __shfl_xor(nan, 1, 2);
  const uint32_t biased = mx4_block_code(amax, nan != 0);
  float pre, inv;
  mx_scale_down(biased, pre, inv);
#pragma unroll
  for (int i = 0; i < 16; ++i) v[i] = nan ? 6.0f : v[i] * pre * inv;  // a NaN block: every code 7, the scale NaN
  if (packed != nullptr) {
    uint32_t words[2] = {0u, 0u};
#pragma unroll
    for (int i = 0; i < 16; ++i) words[i >> 3] |= e2m1_code(v[i]) << ((i & 7) * 4);
    *reinterpret_cast<uint2*>(packed + row * (k >> 1) + (piece << 3)) = make_uint2(words[0], words[1]);
  }
  if (scale != nullptr && (piece & 1) == 0) scale[row * (k >> 5) + (piece >> 1)] = static_cast<uint8_t>(biased);
  if (round_trip != nullptr) {
    const float s = e8m0_to_f32(biased);
    Vec16<bf16_t> o[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) o[i >> 3].v[i & 7] = e2m1_round(v[i]) * s;
    o[0].store(round_trip + row * ldo + (piece << 4));
    o[1].store(round_trip + row * ldo + (piece << 4) + 8);
  }
}

// Weights [G, K, N] along K (axis 1).  A workgroup takes 64 contraction values of 128 columns through LDS (fp32, pitch
// 129); thread (column, half) owns the block of 32 down its column.  Outputs, each optional: packed [G, K / 2, N]
// (rows 2 i and 2 i + 1 of K in one byte, the even one low), scale [G, K / 32, N], round_trip bf16 [G, K, N].
constexpr int kTileK = 64, kTileN = 128, kPitch = kTileN + 1;

template <typename T>
__global__ void __launch_bounds__(256)
mxfp4_weight_kernel(const T* __restrict__ w, int64_t k, int64_t n, uint8_t* __restrict__ packed,
                    uint8_t* __restrict__ scale, bf16_t* __restrict__ round_trip) {
  __shared__ float tile[kTileK * kPitch];
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * kTileN;
  const int64_t k0 = static_cast<int64_t>(blockIdx.y) * kTileK, g = blockIdx.z;
  const T* src = w + g * k * n;
  constexpr int kVec = Elem<T>::kVec;
  if (n % kVec == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0) {
    constexpr int kPerRow = kTileN / kVec;
    for (int i = threadIdx.x; i < kTileK * kPerRow; i += 256) {
      const int kk = i / kPerRow, cc = (i % kPerRow) * kVec;
      Vec16<T> in;
      if (k0 + kk < k && n0 + cc < n) {
        in.load(src + (k0 + kk) * n + n0 + cc);
      } else {
#pragma unroll
        for (int j = 0; j < kVec; ++j) in.v[j] = 0.f;
      }
#pragma unroll
      for (int j = 0; j < kVec; ++j) tile[kk * kPitch + cc + j] = in.v[j];
    }
  } else {
    for (int i = threadIdx.x; i < kTileK * kTileN; i += 256) {
      const int kk = i / kTileN, cc = i % kTileN;
      tile[kk * kPitch + cc] = (k0 + kk < k && n0 + cc < n) ? Elem<T>::load(src + (k0 + kk) * n + n0 + cc) : 0.f;
    }
  }
  __syncthreads();
  const int c = threadIdx.x & (kTileN - 1), h = threadIdx.x >> 7;
  const int64_t col = n0 + c, kb = blockIdx.y * 2 + h;
  if (col >= n || kb * 32 >= k) return;
  float v[32];
  float amax = 0.f;
  bool nan = false;
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    v[i] = tile[(h * 32 + i) * kPitch + c];
    amax = fmaxf(amax, fabsf(v[i]));
    nan |= v[i] != v[i];
  }
  const uint32_t biased = mx4_block_code(amax, nan);
  float pre, inv;
  mx_scale_down(biased, pre, inv);
  const float s = e8m0_to_f32(biased);
  if (scale != nullptr) scale[(g * (k / 32) + kb) * n + col] = static_cast<uint8_t>(biased);
#pragma unroll
  for (int i = 0; i < 32; ++i) v[i] = nan ? 6.0f : v[i] * pre * inv;
  if (packed != nullptr) {
#pragma unroll
    for (int i = 0; i < 32; i += 2)
      packed[(g * (k / 2) + kb * 16 + (i >> 1)) * n + col] =
          static_cast<uint8_t>(e2m1_code(v[i]) | (e2m1_code(v[i + 1]) << 4));
  }
  if (round_trip != nullptr) {
    bf16_t* out = round_trip + (g * k + kb * 32) * n + col;
#pragma unroll
    for (int i = 0; i < 32; ++i) out[i * n] = f32_to_bf16(e2m1_round(v[i]) * s);
  }
}

// packed codes and exponents back to bf16, rows along the last axis (the quantiser API's dequantize)
__global__ void __launch_bounds__(256)
mxfp4_dequantize_rows_kernel(const uint8_t* __restrict__ packed, const uint8_t* __restrict__ scale, int64_t rows, int k,
                             bf16_t* __restrict__ out, int64_t ldo) {
  const int pieces = k >> 4;
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t row = unit / pieces;
  const int piece = static_cast<int>(unit - row * pieces);
  if (row >= rows) return;
  const uint2 words = *reinterpret_cast<const uint2*>(packed + row * (k >> 1) + (piece << 3));
  const float s = e8m0_to_f32(scale[row * (k >> 5) + (piece >> 1)]);
  const uint32_t w[2] = {words.x, words.y};
  Vec16<bf16_t> o[2];
#pragma unroll
  for (int i = 0; i < 16; ++i) o[i >> 3].v[i & 7] = e2m1_value((w[i >> 3] >> ((i & 7) * 4)) & 15u) * s;
  o[0].store(out + row * ldo + (piece << 4));
  o[1].store(out + row * ldo + (piece << 4) + 8);
}

}  // namespace
}  // namespace hmoe

extern "C" {

int hmoe_mxfp4_rows(const void* x, int dtype, int64_t ldx, const int64_t* row_index, int64_t x_rows, int64_t rows,
                    int64_t k, uint8_t* packed, uint8_t* scale, void* round_trip, int64_t ldo, void* stream) {
  using namespace hmoe;
  if (rows < 0 || k < 0 || x_rows < 0) return HMOE_INVALID_ARGUMENT;
  if (!row_index && x_rows != rows) return HMOE_INVALID_ARGUMENT;
  if (dtype != HMOE_BF16 && dtype != HMOE_F32) return HMOE_UNSUPPORTED;
  if (k % 32 || ldx < k || ldx % 8) return HMOE_UNSUPPORTED;
  if (round_trip && (ldo < k || ldo % 8)) return HMOE_UNSUPPORTED;
  if (rows == 0 || k == 0) return HMOE_OK;
  if ((!x && x_rows > 0) || (!packed && !round_trip) || (packed && !scale)) return HMOE_INVALID_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(packed) % 8 ||
      reinterpret_cast<uintptr_t>(round_trip) % 16)
    return HMOE_UNSUPPORTED;
  const int64_t blocks = (rows * (k / 16) + 255) / 256;
  if (blocks >= (int64_t(1) << 31) || k >= (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(blocks));
  if (dtype == HMOE_BF16)
    mxfp4_rows_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(static_cast<const bf16_t*>(x), ldx, row_index, x_rows, rows,
                                                        static_cast<int>(k), packed, scale,
                                                        static_cast<bf16_t*>(round_trip), ldo);
  else
    mxfp4_rows_kernel<float><<<grid, dim3(256), 0, s>>>(static_cast<const float*>(x), ldx, row_index, x_rows, rows,
                                                       static_cast<int>(k), packed, scale,
                                                       static_cast<bf16_t*>(round_trip), ldo);
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

int hmoe_mxfp4_weight(const void* w, int dtype, int64_t groups, int64_t k, int64_t n, uint8_t* packed, uint8_t* scale,
                      void* round_trip, void* stream) {
  using namespace hmoe;
  if (groups < 0 || k < 0 || n < 0) return HMOE_INVALID_ARGUMENT;
  if (dtype != HMOE_BF16 && dtype != HMOE_F32) return HMOE_UNSUPPORTED;
  if (k % 32) return HMOE_UNSUPPORTED;
  if (groups == 0 || k == 0 || n == 0) return HMOE_OK;
  if (!w || (!packed && !round_trip) || (packed && !scale)) return HMOE_INVALID_ARGUMENT;
  const int64_t k_tiles = (k + kTileK - 1) / kTileK, col_tiles = (n + kTileN - 1) / kTileN;
  if (k_tiles > 65535 || groups > 65535 || col_tiles >= (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  const dim3 grid(static_cast<unsigned>(col_tiles), static_cast<unsigned>(k_tiles), static_cast<unsigned>(groups));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == HMOE_BF16)
    mxfp4_weight_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(static_cast<const bf16_t*>(w), k, n, packed, scale,
                                                          static_cast<bf16_t*>(round_trip));
  else
    mxfp4_weight_kernel<float><<<grid, dim3(256), 0, s>>>(static_cast<const float*>(w), k, n, packed, scale,
                                                         static_cast<bf16_t*>(round_trip));
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

int hmoe_mxfp4_dequantize_rows(const uint8_t* packed, const uint8_t* scale, int64_t rows, int64_t k, void* out,
                               int64_t ldo, void* stream) {
  using namespace hmoe;
  if (rows < 0 || k < 0) return HMOE_INVALID_ARGUMENT;
  if (k % 32 || ldo < k || ldo % 8) return HMOE_UNSUPPORTED;
  if (rows == 0 || k == 0) return HMOE_OK;
  if (!packed || !scale || !out) return HMOE_INVALID_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(packed) % 8 || reinterpret_cast<uintptr_t>(out) % 16) return HMOE_UNSUPPORTED;
  const int64_t blocks = (rows * (k / 16) + 255) / 256;
  if (blocks >= (int64_t(1) << 31) || k >= (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  mxfp4_dequantize_rows_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      packed, scale, rows, static_cast<int>(k), static_cast<bf16_t*>(out), ldo);
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

}  // extern "C"
