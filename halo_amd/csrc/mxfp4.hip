// MXFP4 for gfx950: e2m1 elements (magnitudes 0, 0.5, 1, 1.5, 2, 3, 4, 6) with one e8m0 power-of-two scale per 32
// values along the contraction axis (OCP Microscaling).
//
// Replaces quantize_mxfp4 / dequantize / the fake-quant round trip of the reference for this format
// (halo/kernels/lowp/quantization.py:154-180, 191-198, 208-211, 248-269, 277-297, 307-311).  The reference's
// expert_gemm(quant_format="mxfp4") multiplies the two round-tripped operands with the bf16 grouped GEMM
// (halo/kernels/expert_gemm.py:33-38).  Here the quantised operands go to the scaled matrix instruction (the e2m1
// variant of grouped_gemm_fp8_kernel), which sums the same products in fp32; the kernels of this file write its
// operands (codes and exponents in panels of 128 contraction values), the reference's logical layout for the quantiser
// API (two codes per byte along the quantised axis, low nibble first), and the round trip's bf16 result in one pass
// (the straight-through backward's operands, and the forward's for fp32 inputs).
#include "common.h"
#include "fp4.h"
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

__device__ __forceinline__ float e8m0_to_f32(uint32_t code) {
  return __uint_as_float(code == 255u ? 0x7fc00000u : (code == 0u ? 0x00400000u : code << 23));
}

// Rows [R, K] along their last axis; row r is x[row_index[r]] (zeros for an index outside [0, x_rows)) or x[r] without
// an index.  Two lanes hold a block of 32 values, sixteen each.  Outputs, each optional: packed [R, K / 2] (two codes
// per byte, the even element in the low nibble), scale [R, K / 32], and round_trip bf16 [R, K] (row stride ldo): code
// value times 2^(scale - 127).
//
// kPanels: the layout the e2m1 matrix kernel loads instead.  packed [ceil(K / 128)][out_rows][64]: the 128 values of
// panel p of row r in the 64 bytes at (p * out_rows + r) * 64, value 2 b in the low nibble of byte b; scale
// [ceil(K / 128)][out_rows][4]: the exponents of the panel's four blocks side by side.  Values past K are zeros (code
// 0, exponent 0).  Consecutive lanes run along a row (whole lines in); a panel's 64 bytes of a row go out together.
template <typename T, bool kPanels>
__global__ void __launch_bounds__(256)
mxfp4_rows_kernel(const T* __restrict__ x, int64_t ldx, const int64_t* __restrict__ row_index, int64_t x_rows,
                  int64_t rows, int k, uint8_t* __restrict__ packed, uint8_t* __restrict__ scale,
                  bf16_t* __restrict__ round_trip, int64_t ldo, int64_t out_rows) {
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  int64_t row;
  int piece;  // 16-value piece of the row
  {
    const int pieces = kPanels ? ((k + 127) >> 7) * 8 : k >> 4;  // whole panels: the last one's tail is written as zeros
    row = unit / pieces;
    piece = static_cast<int>(unit - row * pieces);
    if (row >= rows) return;  // lane pairs leave together (pieces is even)
  }
  float v[16];
  const int64_t from = row_index != nullptr ? row_index[row] : row;
  if (from >= 0 && from < x_rows && (piece << 4) < k) {
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
  const uint32_t words[2] = {e2m1_pack8(v), e2m1_pack8(v + 8)};
  if (packed != nullptr) {
    const int64_t at = kPanels ? ((piece >> 3) * out_rows + row) * 64 + ((piece & 7) << 3)
                               : row * (k >> 1) + (piece << 3);
    *reinterpret_cast<uint2*>(packed + at) = make_uint2(words[0], words[1]);
  }
  if (scale != nullptr && (piece & 1) == 0) {
    const int64_t at = kPanels ? ((piece >> 3) * out_rows + row) * 4 + ((piece & 7) >> 1) : row * (k >> 5) + (piece >> 1);
    scale[at] = static_cast<uint8_t>(biased);
  }
  if (round_trip != nullptr) {
    const float s = e8m0_to_f32(biased);
    Vec16<bf16_t> o[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      e2m1_unpack8(words[h], o[h].v);
#pragma unroll
      for (int i = 0; i < 8; ++i) o[h].v[i] *= s;
    }
    o[0].store(round_trip + row * ldo + (piece << 4));
    o[1].store(round_trip + row * ldo + (piece << 4) + 8);
  }
}

// Weights [G, K, N] along K (axis 1).  A workgroup takes 64 contraction values of 128 columns through LDS (fp32, pitch
// 129); thread (column, half) owns the block of 32 down its column.  Outputs, each optional: packed [G, K / 2, N]
// (rows 2 i and 2 i + 1 of K in one byte, the even one low), scale [G, K / 32, N], round_trip bf16 [G, K, N].
//
// kPanels: packed [G][ceil(K / 128)][N][64] (the 128 values of panel p down column c in the 64 bytes at
// ((g P + p) N + c) * 64) and scale [G][ceil(K / 128)][N][4], as the e2m1 matrix kernel loads them; the grid then covers
// whole panels, and values past K are zeros (code 0, exponent 0).
constexpr int kTileK = 64, kTileN = 128, kPitch = kTileN + 1;

template <typename T, bool kPanels>
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
  if (col >= n || (!kPanels && kb * 32 >= k)) return;
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
#pragma unroll
  for (int i = 0; i < 32; ++i) v[i] = nan ? 6.0f : v[i] * pre * inv;
  const uint32_t words[4] = {e2m1_pack8(v), e2m1_pack8(v + 8), e2m1_pack8(v + 16), e2m1_pack8(v + 24)};
  if constexpr (kPanels) {
    const int64_t at = (g * ((k + 127) >> 7) + (kb >> 2)) * n + col;  // the column's panel
    scale[at * 4 + (kb & 3)] = static_cast<uint8_t>(biased);
    *reinterpret_cast<uint4*>(packed + at * 64 + ((kb & 3) << 4)) = make_uint4(words[0], words[1], words[2], words[3]);
  } else {
    if (scale != nullptr) scale[(g * (k / 32) + kb) * n + col] = static_cast<uint8_t>(biased);
    if (packed != nullptr) {
#pragma unroll
      for (int i = 0; i < 16; ++i)
        packed[(g * (k / 2) + kb * 16 + i) * n + col] = static_cast<uint8_t>(words[i >> 2] >> ((i & 3) * 8));
    }
  }
  if (round_trip != nullptr && kb * 32 < k) {
    bf16_t* out = round_trip + (g * k + kb * 32) * n + col;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      float back[8];
      e2m1_unpack8(words[q], back);
#pragma unroll
      for (int i = 0; i < 8; ++i) out[(q * 8 + i) * n] = f32_to_bf16(back[i] * s);
    }
  }
}

// packed codes and exponents back to bf16, rows along the last axis (the quantiser API's dequantize); kPanels: from
// the matrix kernel's layout (q_rows rows per panel)
template <bool kPanels>
__global__ void __launch_bounds__(256)
mxfp4_dequantize_rows_kernel(const uint8_t* __restrict__ packed, const uint8_t* __restrict__ scale, int64_t rows, int k,
                             bf16_t* __restrict__ out, int64_t ldo, int64_t q_rows) {
  const int pieces = k >> 4;
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t row = unit / pieces;
  const int piece = static_cast<int>(unit - row * pieces);
  if (row >= rows) return;
  const int64_t at = kPanels ? ((piece >> 3) * q_rows + row) * 64 + ((piece & 7) << 3) : row * (k >> 1) + (piece << 3);
  const int64_t s_at = kPanels ? ((piece >> 3) * q_rows + row) * 4 + ((piece & 7) >> 1) : row * (k >> 5) + (piece >> 1);
  const uint2 words = *reinterpret_cast<const uint2*>(packed + at);
  const float s = e8m0_to_f32(scale[s_at]);
  Vec16<bf16_t> o[2];
  e2m1_unpack8(words.x, o[0].v);
  e2m1_unpack8(words.y, o[1].v);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    o[0].v[i] *= s;
    o[1].v[i] *= s;
  }
  o[0].store(out + row * ldo + (piece << 4));
  o[1].store(out + row * ldo + (piece << 4) + 8);
}

}  // namespace
}  // namespace hmoe

namespace hmoe {
namespace {

int launch_rows(const void* x, int dtype, int64_t ldx, const int64_t* row_index, int64_t x_rows, int64_t rows, int64_t k,
                uint8_t* packed, uint8_t* scale, void* round_trip, int64_t ldo, int64_t out_rows, bool panels,
                void* stream) {
  if (rows < 0 || k < 0 || x_rows < 0) return HMOE_INVALID_ARGUMENT;
  if (!row_index && x_rows != rows) return HMOE_INVALID_ARGUMENT;
  if (dtype != HMOE_BF16 && dtype != HMOE_F32) return HMOE_UNSUPPORTED;
  if (k % 32 || ldx < k || ldx % 8) return HMOE_UNSUPPORTED;
  if (round_trip && (ldo < k || ldo % 8)) return HMOE_UNSUPPORTED;
  if (panels && out_rows < rows) return HMOE_UNSUPPORTED;
  if (rows == 0 || k == 0) return HMOE_OK;
  if ((!x && x_rows > 0) || (!packed && !round_trip) || (packed && !scale)) return HMOE_INVALID_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(packed) % 8 ||
      reinterpret_cast<uintptr_t>(round_trip) % 16)
    return HMOE_UNSUPPORTED;
  const int64_t pieces = panels ? (k + 127) / 128 * 8 : k / 16;
  const int64_t blocks = (rows * pieces + 255) / 256;
  if (blocks >= (int64_t(1) << 31) || k >= (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(blocks));
  auto launch = [&](auto kernel, auto* typed) {
    kernel<<<grid, dim3(256), 0, s>>>(typed, ldx, row_index, x_rows, rows, static_cast<int>(k), packed, scale,
                                      static_cast<bf16_t*>(round_trip), ldo, out_rows);
  };
  if (dtype == HMOE_BF16) {
    if (panels) launch(mxfp4_rows_kernel<bf16_t, true>, static_cast<const bf16_t*>(x));
    else launch(mxfp4_rows_kernel<bf16_t, false>, static_cast<const bf16_t*>(x));
  } else {
    if (panels) launch(mxfp4_rows_kernel<float, true>, static_cast<const float*>(x));
    else launch(mxfp4_rows_kernel<float, false>, static_cast<const float*>(x));
  }
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

int launch_weight(const void* w, int dtype, int64_t groups, int64_t k, int64_t n, uint8_t* packed, uint8_t* scale,
                  void* round_trip, bool panels, void* stream) {
  if (groups < 0 || k < 0 || n < 0) return HMOE_INVALID_ARGUMENT;
  if (dtype != HMOE_BF16 && dtype != HMOE_F32) return HMOE_UNSUPPORTED;
  if (k % 32) return HMOE_UNSUPPORTED;
  if (groups == 0 || k == 0 || n == 0) return HMOE_OK;
  if (!w || (!packed && !round_trip) || (packed && !scale) || (panels && !packed)) return HMOE_INVALID_ARGUMENT;
  if (panels && reinterpret_cast<uintptr_t>(packed) % 16) return HMOE_UNSUPPORTED;
  const int64_t k_tiles = panels ? (k + 127) / 128 * 2 : (k + kTileK - 1) / kTileK;
  const int64_t col_tiles = (n + kTileN - 1) / kTileN;
  if (k_tiles > 65535 || groups > 65535 || col_tiles >= (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  const dim3 grid(static_cast<unsigned>(col_tiles), static_cast<unsigned>(k_tiles), static_cast<unsigned>(groups));
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto launch = [&](auto kernel, auto* typed) {
    kernel<<<grid, dim3(256), 0, s>>>(typed, k, n, packed, scale, static_cast<bf16_t*>(round_trip));
  };
  if (dtype == HMOE_BF16) {
    if (panels) launch(mxfp4_weight_kernel<bf16_t, true>, static_cast<const bf16_t*>(w));
    else launch(mxfp4_weight_kernel<bf16_t, false>, static_cast<const bf16_t*>(w));
  } else {
    if (panels) launch(mxfp4_weight_kernel<float, true>, static_cast<const float*>(w));
    else launch(mxfp4_weight_kernel<float, false>, static_cast<const float*>(w));
  }
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

int launch_dequantize(const uint8_t* packed, const uint8_t* scale, int64_t q_rows, int64_t rows, int64_t k, void* out,
                      int64_t ldo, bool panels, void* stream) {
  if (rows < 0 || k < 0) return HMOE_INVALID_ARGUMENT;
  if (k % 32 || ldo < k || ldo % 8) return HMOE_UNSUPPORTED;
  if (panels && q_rows < rows) return HMOE_INVALID_ARGUMENT;
  if (rows == 0 || k == 0) return HMOE_OK;
  if (!packed || !scale || !out) return HMOE_INVALID_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(packed) % 8 || reinterpret_cast<uintptr_t>(out) % 16) return HMOE_UNSUPPORTED;
  const int64_t blocks = (rows * (k / 16) + 255) / 256;
  if (blocks >= (int64_t(1) << 31) || k >= (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  const dim3 grid(static_cast<unsigned>(blocks));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (panels)
    mxfp4_dequantize_rows_kernel<true><<<grid, dim3(256), 0, s>>>(packed, scale, rows, static_cast<int>(k),
                                                                 static_cast<bf16_t*>(out), ldo, q_rows);
  else
    mxfp4_dequantize_rows_kernel<false><<<grid, dim3(256), 0, s>>>(packed, scale, rows, static_cast<int>(k),
                                                                  static_cast<bf16_t*>(out), ldo, q_rows);
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

}  // namespace
}  // namespace hmoe

extern "C" {

int hmoe_mxfp4_rows(const void* x, int dtype, int64_t ldx, const int64_t* row_index, int64_t x_rows, int64_t rows,
                    int64_t k, uint8_t* packed, uint8_t* scale, void* round_trip, int64_t ldo, void* stream) {
  return hmoe::launch_rows(x, dtype, ldx, row_index, x_rows, rows, k, packed, scale, round_trip, ldo, rows, false, stream);
}

int hmoe_mxfp4_weight(const void* w, int dtype, int64_t groups, int64_t k, int64_t n, uint8_t* packed, uint8_t* scale,
                      void* round_trip, void* stream) {
  return hmoe::launch_weight(w, dtype, groups, k, n, packed, scale, round_trip, false, stream);
}

int hmoe_mxfp4_dequantize_rows(const uint8_t* packed, const uint8_t* scale, int64_t rows, int64_t k, void* out,
                               int64_t ldo, void* stream) {
  return hmoe::launch_dequantize(packed, scale, rows, rows, k, out, ldo, false, stream);
}

int hmoe_mxfp4_rows_panels(const void* x, int dtype, int64_t ldx, const int64_t* row_index, int64_t x_rows, int64_t rows,
                           int64_t k, uint8_t* q, uint8_t* scale, int64_t out_rows, void* stream) {
  if (rows > 0 && k > 0 && !q) return HMOE_INVALID_ARGUMENT;
  return hmoe::launch_rows(x, dtype, ldx, row_index, x_rows, rows, k, q, scale, nullptr, 0, out_rows, true, stream);
}

int hmoe_mxfp4_weight_panels(const void* w, int dtype, int64_t groups, int64_t k, int64_t n, uint8_t* q, uint8_t* scale,
                             void* round_trip, void* stream) {
  return hmoe::launch_weight(w, dtype, groups, k, n, q, scale, round_trip, true, stream);
}

int hmoe_mxfp4_dequantize_panels(const uint8_t* q, const uint8_t* scale, int64_t q_rows, int64_t rows, int64_t k,
                                 void* out, int64_t ldo, void* stream) {
  return hmoe::launch_dequantize(q, scale, q_rows, rows, k, out, ldo, true, stream);
}

}  // extern "C"
