// NVFP4 for gfx950: e2m1 elements (two per byte) with one e4m3 scale per 16 values along the contraction axis and one
// fp32 power-of-two scale per tensor.
//
// Replaces quantize_nvfp4 / dequantize / the fake-quant round trip of the reference for this format
// (halo/kernels/lowp/quantization.py:209-226, 191-205, 248-270, 277-297, 307-311).  The reference's
// expert_gemm(quant_format="nvfp4") multiplies the two round-tripped operands with the bf16 grouped GEMM
// (halo/kernels/expert_gemm.py:33-38), and so does this build: the scaled matrix instruction takes power-of-two (e8m0)
// scales only, an e4m3 scale per 16 values has no place in it.  The kernels here write the reference's layout (packed
// codes, e4m3 scale bytes, the tensor's scale) and the round trip's bf16 result in one pass.
//
// The tensor's largest magnitude comes in as a device scalar (the caller reduces it: one more pass over the tensor,
// which the format demands before any block can be scaled).  Every fp32 operation is the reference's, in its order:
// scale = e4m3(min(amax_block / 6 / global, 448)), divisor = f32(scale) * global (1 where that is 0), code =
// e2m1(value / divisor); the divisions are IEEE divisions.
#include "common.h"
#include "fp4.h"

namespace hmoe {
namespace {

// The smallest power of two >= max(amax, tiny) / 2688 (2688 = 448 * 6 = 1.3125 * 2^11), from the amax's bits: with
// amax = (1 + f) 2^E the quotient is (1 + f) / 1.3125 * 2^(E - 11), whose log2 rounds up to E - 11 while 1 + f <=
// 1.3125 and to E - 10 above.  Down to 2^-137, a subnormal.  NaN for a NaN amax, inf for an infinite one.
__device__ __forceinline__ float nv_global_scale(float amax) {
  if (amax != amax) return amax;
  uint32_t bits = __float_as_uint(fabsf(amax));
  if (bits >= 0x7f800000u) return __uint_as_float(0x7f800000u);
  if (bits < 0x00800000u) bits = 0x00800000u;  // the floor: the smallest normal
  const int e = static_cast<int>(bits >> 23) - 127 - 11 + ((bits & 0x007fffffu) > 0x00280000u ? 1 : 0);
  return e >= -126 ? __uint_as_float(static_cast<uint32_t>(e + 127) << 23) : __uint_as_float(1u << (e + 149));
}

// One block of 16 values: its e4m3 scale byte, and the values divided by scale * global (6 for every value of a block
// whose divisor is NaN: the code bucketize gives a NaN, under the sign `NaN < 0` gives).
__device__ __forceinline__ uint32_t nv_block(float (&v)[16], float global, float& divisor) {
  float amax = 0.f;
  bool nan = false;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    amax = fmaxf(amax, fabsf(v[i]));
    nan |= v[i] != v[i];
  }
  float ratio = (amax / 6.0f) / global;
  nan |= ratio != ratio;
  ratio = fminf(ratio, 448.0f);
  uint32_t bits = static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(ratio, ratio, 0, false)) & 0xffu;
  if (nan) bits = 0x7fu;
  const float scale = nan ? __uint_as_float(0x7fc00000u) : __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(bits), 0);
  divisor = scale * global;
  const bool poisoned = divisor != divisor;
  const float by = divisor == 0.f ? 1.0f : divisor;
#pragma unroll
  for (int i = 0; i < 16; ++i) v[i] = poisoned ? 6.0f : v[i] / by;
  return bits;
}

// Rows [R, K] along their last axis; row r is x[row_index[r]] (zeros for an index outside [0, x_rows)) or x[r] without
// an index.  One lane per block of 16 values.  Outputs, each optional: packed [R, K / 2] (two codes per byte, the even
// element in the low nibble), scale [R, K / 16] (e4m3 bytes), round_trip bf16 [R, K] (row stride ldo) = code value
// times (scale * global); global_out (one float) = the tensor's scale.
template <typename T>
__global__ void __launch_bounds__(256)
nvfp4_rows_kernel(const T* __restrict__ x, int64_t ldx, const int64_t* __restrict__ row_index, int64_t x_rows,
                  int64_t rows, int k, const float* __restrict__ tensor_amax, uint8_t* __restrict__ packed,
                  uint8_t* __restrict__ scale, bf16_t* __restrict__ round_trip, int64_t ldo,
                  float* __restrict__ global_out) {
  const float global = nv_global_scale(*tensor_amax);
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (unit == 0 && global_out != nullptr) *global_out = global;
  const int pieces = k >> 4;
  const int64_t row = unit / pieces;
  const int piece = static_cast<int>(unit - row * pieces);
  if (row >= rows) return;
  float v[16];
  const int64_t from = row_index != nullptr ? row_index[row] : row;
  if (from >= 0 && from < x_rows) {
    load16<T>(x + from * ldx + (piece << 4), v);
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = 0.f;
  }
  float divisor;
  const uint32_t bits = nv_block(v, global, divisor);
  const uint32_t words[2] = {e2m1_pack8(v), e2m1_pack8(v + 8)};
  if (packed != nullptr) *reinterpret_cast<uint2*>(packed + row * (k >> 1) + (piece << 3)) = make_uint2(words[0], words[1]);
  if (scale != nullptr) scale[row * pieces + piece] = static_cast<uint8_t>(bits);
  if (round_trip != nullptr) {
    Vec16<bf16_t> o[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      e2m1_unpack8(words[h], o[h].v);
#pragma unroll
      for (int i = 0; i < 8; ++i) o[h].v[i] *= divisor;
    }
    o[0].store(round_trip + row * ldo + (piece << 4));
    o[1].store(round_trip + row * ldo + (piece << 4) + 8);
  }
}

// Weights [G, K, N] along K (axis 1), one global scale for the whole bank.  A workgroup takes 64 contraction values of
// 128 columns through LDS (fp32, pitch 129); thread (column, half) owns the two blocks of 16 down its column.
// Outputs, each optional: packed [G, K / 2, N], scale [G, K / 16, N], round_trip bf16 [G, K, N], global_out.
constexpr int kTileK = 64, kTileN = 128, kPitch = kTileN + 1;

template <typename T>
__global__ void __launch_bounds__(256)
nvfp4_weight_kernel(const T* __restrict__ w, int64_t k, int64_t n, const float* __restrict__ tensor_amax,
                    uint8_t* __restrict__ packed, uint8_t* __restrict__ scale, bf16_t* __restrict__ round_trip,
                    float* __restrict__ global_out) {
  __shared__ float tile[kTileK * kPitch];
  const float global = nv_global_scale(*tensor_amax);
  if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0 && global_out != nullptr)
    *global_out = global;
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
  const int64_t col = n0 + c;
  if (col >= n) return;
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int64_t kb = blockIdx.y * 4 + h * 2 + half;  // the block of 16 along K
    if (kb * 16 >= k) return;
    float v[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = tile[(h * 32 + half * 16 + i) * kPitch + c];
    float divisor;
    const uint32_t bits = nv_block(v, global, divisor);
    const uint32_t words[2] = {e2m1_pack8(v), e2m1_pack8(v + 8)};
    if (scale != nullptr) scale[(g * (k / 16) + kb) * n + col] = static_cast<uint8_t>(bits);
    if (packed != nullptr) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        packed[(g * (k / 2) + kb * 8 + i) * n + col] = static_cast<uint8_t>(words[i >> 2] >> ((i & 3) * 8));
    }
    if (round_trip != nullptr) {
      bf16_t* out = round_trip + (g * k + kb * 16) * n + col;
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        float back[8];
        e2m1_unpack8(words[q], back);
#pragma unroll
        for (int i = 0; i < 8; ++i) out[(q * 8 + i) * n] = f32_to_bf16(back[i] * divisor);
      }
    }
  }
}

// packed codes, e4m3 scales and the tensor's scale back to bf16, rows along the last axis
__global__ void __launch_bounds__(256)
nvfp4_dequantize_rows_kernel(const uint8_t* __restrict__ packed, const uint8_t* __restrict__ scale,
                             const float* __restrict__ global_scale, int64_t rows, int k, bf16_t* __restrict__ out,
                             int64_t ldo) {
  const int pieces = k >> 4;
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t row = unit / pieces;
  const int piece = static_cast<int>(unit - row * pieces);
  if (row >= rows) return;
  const uint2 words = *reinterpret_cast<const uint2*>(packed + row * (k >> 1) + (piece << 3));
  const uint32_t bits = scale[row * pieces + piece];
  const float s = ((bits & 0x7fu) == 0x7fu ? __uint_as_float(0x7fc00000u)
                                           : __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(bits), 0)) * *global_scale;
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

extern "C" {

int hmoe_nvfp4_rows(const void* x, int dtype, int64_t ldx, const int64_t* row_index, int64_t x_rows, int64_t rows,
                    int64_t k, const float* tensor_amax, uint8_t* packed, uint8_t* scale, void* round_trip, int64_t ldo,
                    float* global_out, void* stream) {
  using namespace hmoe;
  if (rows < 0 || k < 0 || x_rows < 0) return HMOE_INVALID_ARGUMENT;
  if (!row_index && x_rows != rows) return HMOE_INVALID_ARGUMENT;
  if (dtype != HMOE_BF16 && dtype != HMOE_F32) return HMOE_UNSUPPORTED;
  if (k % 16 || ldx < k || ldx % 8) return HMOE_UNSUPPORTED;
  if (round_trip && (ldo < k || ldo % 8)) return HMOE_UNSUPPORTED;
  if (rows == 0 || k == 0) return HMOE_OK;
  if ((!x && x_rows > 0) || !tensor_amax || (!packed && !round_trip) || (packed && !scale)) return HMOE_INVALID_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(packed) % 8 ||
      reinterpret_cast<uintptr_t>(round_trip) % 16 || reinterpret_cast<uintptr_t>(tensor_amax) % 4 ||
      reinterpret_cast<uintptr_t>(global_out) % 4)
    return HMOE_UNSUPPORTED;
  const int64_t blocks = (rows * (k / 16) + 255) / 256;
  if (blocks >= (int64_t(1) << 31) || k >= (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(blocks));
  if (dtype == HMOE_BF16)
    nvfp4_rows_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(static_cast<const bf16_t*>(x), ldx, row_index, x_rows, rows,
                                                        static_cast<int>(k), tensor_amax, packed, scale,
                                                        static_cast<bf16_t*>(round_trip), ldo, global_out);
  else
    nvfp4_rows_kernel<float><<<grid, dim3(256), 0, s>>>(static_cast<const float*>(x), ldx, row_index, x_rows, rows,
                                                       static_cast<int>(k), tensor_amax, packed, scale,
                                                       static_cast<bf16_t*>(round_trip), ldo, global_out);
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

int hmoe_nvfp4_weight(const void* w, int dtype, int64_t groups, int64_t k, int64_t n, const float* tensor_amax,
                      uint8_t* packed, uint8_t* scale, void* round_trip, float* global_out, void* stream) {
  using namespace hmoe;
  if (groups < 0 || k < 0 || n < 0) return HMOE_INVALID_ARGUMENT;
  if (dtype != HMOE_BF16 && dtype != HMOE_F32) return HMOE_UNSUPPORTED;
  if (k % 16) return HMOE_UNSUPPORTED;
  if (groups == 0 || k == 0 || n == 0) return HMOE_OK;
  if (!w || !tensor_amax || (!packed && !round_trip) || (packed && !scale)) return HMOE_INVALID_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(tensor_amax) % 4 || reinterpret_cast<uintptr_t>(global_out) % 4) return HMOE_UNSUPPORTED;
  const int64_t k_tiles = (k + kTileK - 1) / kTileK, col_tiles = (n + kTileN - 1) / kTileN;
  if (k_tiles > 65535 || groups > 65535 || col_tiles >= (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  const dim3 grid(static_cast<unsigned>(col_tiles), static_cast<unsigned>(k_tiles), static_cast<unsigned>(groups));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == HMOE_BF16)
    nvfp4_weight_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(static_cast<const bf16_t*>(w), k, n, tensor_amax, packed,
                                                          scale, static_cast<bf16_t*>(round_trip), global_out);
  else
    nvfp4_weight_kernel<float><<<grid, dim3(256), 0, s>>>(static_cast<const float*>(w), k, n, tensor_amax, packed,
                                                         scale, static_cast<bf16_t*>(round_trip), global_out);
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

int hmoe_nvfp4_dequantize_rows(const uint8_t* packed, const uint8_t* scale, const float* global_scale, int64_t rows,
                               int64_t k, void* out, int64_t ldo, void* stream) {
  using namespace hmoe;
  if (rows < 0 || k < 0) return HMOE_INVALID_ARGUMENT;
  if (k % 16 || ldo < k || ldo % 8) return HMOE_UNSUPPORTED;
  if (rows == 0 || k == 0) return HMOE_OK;
  if (!packed || !scale || !global_scale || !out) return HMOE_INVALID_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(packed) % 8 || reinterpret_cast<uintptr_t>(out) % 16 ||
      reinterpret_cast<uintptr_t>(global_scale) % 4)
    return HMOE_UNSUPPORTED;
  const int64_t blocks = (rows * (k / 16) + 255) / 256;
  if (blocks >= (int64_t(1) << 31) || k >= (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  nvfp4_dequantize_rows_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      packed, scale, global_scale, rows, static_cast<int>(k), static_cast<bf16_t*>(out), ldo);
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

}  // extern "C"
