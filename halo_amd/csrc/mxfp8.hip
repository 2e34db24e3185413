// MXFP8 operands for the expert GEMM on gfx950: e4m3 elements with one e8m0 power-of-two scale per 32 values along the
// contraction axis (OCP Microscaling), which is the granularity v_mfma_scale_f32_32x32x64_f8f6f4 applies by itself.
//
// Replaces quantize_mxfp8 / dequantize / the fake-quant round trip of the reference
// (halo/kernels/lowp/quantization.py:154-188, 236-245, 277-297, 307-311) for the two operand shapes of the expert GEMM
// (halo/kernels/expert_gemm.py:33-38): activation rows [R, K] quantised along their last axis and expert weights
// [G, K, N] along axis 1.  Both come out in the layout the GEMM kernel loads: panels of 64 contraction values
// (activations [K/64][R][64], weights [G][K/64][N][64]) with the exponents beside them ([K/32][R], [G][K/32][N]).
#include "common.h"
#include "fp8_rows.h"

namespace hmoe {
namespace {

typedef float f32x2 __attribute__((ext_vector_type(2)));

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

// Rows to MXFP8.  grid.y walks the panels of 64 contraction values, a workgroup takes 64 rows of one panel: four lanes
// per row, sixteen values each, so that a wavefront reads 16 rows x 128 bytes (whole lines) and writes 1 KB of the
// panel in one piece.  With row_index, output row r is x[row_index[r]] (zeros where the index is outside
// [0, x_rows)): the permute by expert taken on the way.
template <typename T>
__global__ void __launch_bounds__(256)
quantize_rows_mx_kernel(const T* __restrict__ x, int64_t ldx, const int64_t* __restrict__ row_index, int64_t x_rows,
                        int64_t rows, int k, uint8_t* __restrict__ q, uint8_t* __restrict__ scale, int64_t out_rows) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 64 + (threadIdx.x >> 2);
  const int panel = blockIdx.y, sub = threadIdx.x & 3;
  const int first = panel * 64 + sub * 16;
  if (row >= rows || first >= k) return;  // lane pairs leave together (k is a multiple of 32)
  float v[16];
  const int64_t from = row_index ? row_index[row] : row;
  if (from >= 0 && from < x_rows) {
    load16<T>(x + from * ldx + first, v);
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = 0.f;
  }
  quantize_mx_half_block(v, row, panel, sub, q, scale, out_rows);
}

// e8m0 code to its fp32 value: 2^(code - 127), with 2^-127 (a subnormal) for code 0 and NaN for 0xFF.
__device__ __forceinline__ float e8m0_value(uint32_t code) {
  return __uint_as_float(code == 255u ? 0x7fc00000u : (code == 0u ? 0x00400000u : code << 23));
}

// The rows back as bf16 [R, K]: code value times the block's power of two, rounded to bf16 (exact for every normal
// result).  The same thread layout as the quantiser: 1 KB of the panel read in one piece per wavefront, whole lines
// written.
__global__ void __launch_bounds__(256)
dequantize_rows_mx_kernel(const uint8_t* __restrict__ q, const uint8_t* __restrict__ scale, int64_t q_rows,
                          int64_t rows, int k, bf16_t* __restrict__ out, int64_t ldo) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 64 + (threadIdx.x >> 2);
  const int panel = blockIdx.y, sub = threadIdx.x & 3;
  const int first = panel * 64 + sub * 16;
  if (row >= rows || first >= k) return;
  const uint4 packed = *reinterpret_cast<const uint4*>(q + (static_cast<int64_t>(panel) * q_rows + row) * 64 + sub * 16);
  const float s = e8m0_value(scale[static_cast<int64_t>(2 * panel + (sub >> 1)) * q_rows + row]);
  const uint32_t words[4] = {packed.x, packed.y, packed.z, packed.w};
  Vec16<bf16_t> o[2];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(words[w]), false);
    const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(words[w]), true);
    o[w >> 1].v[4 * (w & 1) + 0] = lo.x * s;
    o[w >> 1].v[4 * (w & 1) + 1] = lo.y * s;
    o[w >> 1].v[4 * (w & 1) + 2] = hi.x * s;
    o[w >> 1].v[4 * (w & 1) + 3] = hi.y * s;
  }
  o[0].store(out + row * ldo + first);
  o[1].store(out + row * ldo + first + 8);
}

// Expert weights [G, K, N] to MXFP8 along K.  A workgroup takes one panel (64 contraction values) of 128 columns:
// the 64 x 128 values go through LDS as fp32 (rows K, pitch 129 so that a column walk is conflict-free), then thread
// (column c, half h) owns the 32 values of column c's block h: block maximum, exponent, 32 e4m3 bytes written as two
// 16-byte stores into the panel, and optionally the 32 dequantised values as bf16 into a [G, K, N] copy (what the
// fake-quant round trip returns, kept for the backward products).
constexpr int kWTileK = 64, kWTileN = 128, kWPitch = kWTileN + 1;

template <typename T>
__global__ void __launch_bounds__(256)
quantize_weight_mx_kernel(const T* __restrict__ w, int64_t k, int64_t n, uint8_t* __restrict__ q,
                          uint8_t* __restrict__ scale, bf16_t* __restrict__ dequant) {
  __shared__ float tile[kWTileK * kWPitch];
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * kWTileN;
  const int64_t panel = blockIdx.y, g = blockIdx.z;
  const int64_t k0 = panel * kWTileK;
  const int64_t panels = (k + kWTileK - 1) / kWTileK;
  const T* src = w + g * k * n;
  constexpr int kVec = Elem<T>::kVec;
  const bool vector_ok = n % kVec == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
  if (vector_ok) {
    constexpr int kPerRow = kWTileN / kVec;
    for (int i = threadIdx.x; i < kWTileK * kPerRow; i += 256) {
      const int kk = i / kPerRow, cc = (i % kPerRow) * kVec;
      Vec16<T> in;
      if (k0 + kk < k && n0 + cc < n) {
        in.load(src + (k0 + kk) * n + n0 + cc);
      } else {
#pragma unroll
        for (int j = 0; j < kVec; ++j) in.v[j] = 0.f;
      }
#pragma unroll
      for (int j = 0; j < kVec; ++j) tile[kk * kWPitch + cc + j] = in.v[j];
    }
  } else {
    for (int i = threadIdx.x; i < kWTileK * kWTileN; i += 256) {
      const int kk = i / kWTileN, cc = i % kWTileN;
      tile[kk * kWPitch + cc] = (k0 + kk < k && n0 + cc < n) ? Elem<T>::load(src + (k0 + kk) * n + n0 + cc) : 0.f;
    }
  }
  __syncthreads();
  const int c = threadIdx.x & (kWTileN - 1), h = threadIdx.x >> 7;
  const int64_t col = n0 + c, kb = panel * 2 + h;
  if (col >= n || kb * 32 >= k) return;
  float v[32];
  float amax = 0.f;
  bool nan = false;
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    v[i] = tile[(h * 32 + i) * kWPitch + c];
    amax = fmaxf(amax, fabsf(v[i]));
    nan |= v[i] != v[i];
  }
  const uint32_t biased = mx_block_code(amax, nan);
  float pre, inv;
  mx_scale_down(biased, pre, inv);
  scale[(g * (k / 32) + kb) * n + col] = static_cast<uint8_t>(biased);
  uint32_t words[8];
#pragma unroll
  for (int wd = 0; wd < 8; ++wd) {
    int word = 0;
    word = __builtin_amdgcn_cvt_pk_fp8_f32(mx_clamp(v[4 * wd] * pre * inv), mx_clamp(v[4 * wd + 1] * pre * inv), word, false);
    word = __builtin_amdgcn_cvt_pk_fp8_f32(mx_clamp(v[4 * wd + 2] * pre * inv), mx_clamp(v[4 * wd + 3] * pre * inv), word, true);
    words[wd] = nan ? 0x7f7f7f7fu : static_cast<uint32_t>(word);
  }
  uint8_t* dst = q + ((g * panels + panel) * n + col) * 64 + h * 32;
  *reinterpret_cast<uint4*>(dst) = make_uint4(words[0], words[1], words[2], words[3]);
  *reinterpret_cast<uint4*>(dst + 16) = make_uint4(words[4], words[5], words[6], words[7]);
  if (dequant != nullptr) {
    const float s = e8m0_value(biased);
    bf16_t* out = dequant + g * k * n + kb * 32 * n + col;
#pragma unroll
    for (int wd = 0; wd < 8; ++wd) {
      const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(words[wd]), false);
      const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(words[wd]), true);
      out[(4 * wd + 0) * n] = f32_to_bf16(lo.x * s);
      out[(4 * wd + 1) * n] = f32_to_bf16(lo.y * s);
      out[(4 * wd + 2) * n] = f32_to_bf16(hi.x * s);
      out[(4 * wd + 3) * n] = f32_to_bf16(hi.y * s);
    }
  }
}

}  // namespace
}  // namespace hmoe

extern "C" {

int hmoe_quantize_rows_mxfp8(const void* x, int dtype, int64_t ldx, const int64_t* row_index, int64_t x_rows,
                             int64_t rows, int64_t k, uint8_t* q, uint8_t* scale, int64_t out_rows, void* stream) {
  using namespace hmoe;
  if (rows < 0 || k < 0 || x_rows < 0) return HMOE_INVALID_ARGUMENT;
  if (!row_index && x_rows != rows) return HMOE_INVALID_ARGUMENT;
  if (dtype != HMOE_BF16 && dtype != HMOE_F32) return HMOE_UNSUPPORTED;
  if (k % 32 || ldx < k || ldx % 8 || out_rows < rows) return HMOE_UNSUPPORTED;
  if (rows == 0 || k == 0) return HMOE_OK;
  if (!q || !scale || (!x && x_rows > 0)) return HMOE_INVALID_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(q) % 16) return HMOE_UNSUPPORTED;
  const int64_t row_blocks = (rows + 63) / 64, panels = (k + 63) / 64;
  if (row_blocks >= (int64_t(1) << 31) || panels > 65535) return HMOE_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(row_blocks), static_cast<unsigned>(panels));
  if (dtype == HMOE_BF16)
    quantize_rows_mx_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(static_cast<const bf16_t*>(x), ldx, row_index, x_rows,
                                                              rows, static_cast<int>(k), q, scale, out_rows);
  else
    quantize_rows_mx_kernel<float><<<grid, dim3(256), 0, s>>>(static_cast<const float*>(x), ldx, row_index, x_rows,
                                                             rows, static_cast<int>(k), q, scale, out_rows);
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

int hmoe_dequantize_rows_mxfp8(const uint8_t* q, const uint8_t* scale, int64_t q_rows, int64_t rows, int64_t k,
                               void* out, int64_t ldo, void* stream) {
  using namespace hmoe;
  if (rows < 0 || k < 0 || q_rows < rows) return HMOE_INVALID_ARGUMENT;
  if (k % 32 || ldo < k || ldo % 8) return HMOE_UNSUPPORTED;
  if (rows == 0 || k == 0) return HMOE_OK;
  if (!q || !scale || !out) return HMOE_INVALID_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(out) % 16 || reinterpret_cast<uintptr_t>(q) % 16) return HMOE_UNSUPPORTED;
  const int64_t row_blocks = (rows + 63) / 64, panels = (k + 63) / 64;
  if (row_blocks >= (int64_t(1) << 31) || panels > 65535) return HMOE_UNSUPPORTED;
  dequantize_rows_mx_kernel<<<dim3(static_cast<unsigned>(row_blocks), static_cast<unsigned>(panels)), dim3(256), 0,
                              static_cast<hipStream_t>(stream)>>>(
      q, scale, q_rows, rows, static_cast<int>(k), static_cast<bf16_t*>(out), ldo);
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

int hmoe_quantize_weight_mxfp8(const void* w, int dtype, int64_t groups, int64_t k, int64_t n, uint8_t* q,
                               uint8_t* scale, void* dequant, void* stream) {
  using namespace hmoe;
  if (groups < 0 || k < 0 || n < 0) return HMOE_INVALID_ARGUMENT;
  if (dtype != HMOE_BF16 && dtype != HMOE_F32) return HMOE_UNSUPPORTED;
  if (k % 32) return HMOE_UNSUPPORTED;
  if (groups == 0 || k == 0 || n == 0) return HMOE_OK;
  if (!w || !q || !scale) return HMOE_INVALID_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(q) % 16) return HMOE_UNSUPPORTED;
  const int64_t panels = (k + kWTileK - 1) / kWTileK, col_tiles = (n + kWTileN - 1) / kWTileN;
  if (panels > 65535 || groups > 65535 || col_tiles >= (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  const dim3 grid(static_cast<unsigned>(col_tiles), static_cast<unsigned>(panels), static_cast<unsigned>(groups));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == HMOE_BF16)
    quantize_weight_mx_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(static_cast<const bf16_t*>(w), k, n, q, scale,
                                                                static_cast<bf16_t*>(dequant));
  else
    quantize_weight_mx_kernel<float><<<grid, dim3(256), 0, s>>>(static_cast<const float*>(w), k, n, q, scale,
                                                               static_cast<bf16_t*>(dequant));
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

}  // extern "C"
