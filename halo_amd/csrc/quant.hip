// 128x128-block e4m3 weight quantiser and dequantiser for gfx950 (OCP float8_e4m3fn, as torch.float8_e4m3fn).
//
// Replaces quantize_block_fp8 (halo/kernels/lowp/block_fp8.py:23-34) and dequantize_block_fp8
// (halo/checkpoint/tools/fp8_dequant.py:153-170) of the reference.  One workgroup per 128x128 block: a block-wide
// absolute maximum, scale = the smallest power of two >= max(amax, 1e-12) / 448 read off the exponent bits, then
// q = clamp(x / scale, +-448) rounded to e4m3 (nearest even).  Division by a power of two is exact, so the result
// does not depend on the device's divider.
#include "common.h"
#include "fp8_rows.h"

namespace hmoe {
namespace {

constexpr int kBlock = 128;
constexpr float kE4m3Max = 448.0f;
constexpr float kAmaxFloor = 1e-12f;

// Smallest power of two >= x for a positive finite fp32 x, from the exponent bits.
__device__ __forceinline__ float pow2_ceil(float x) {
  int e;
  const float m = frexpf(x, &e);  // x = m * 2^e, m in [0.5, 1)
  return ldexpf(1.0f, e - (m == 0.5f ? 1 : 0));
}

// fp32 (|x| <= 448) -> e4m3fn bits, round to nearest even.
__device__ __forceinline__ uint8_t encode_e4m3(float x) {
  // v_cvt_pk_fp8_f32 rounds to nearest even and saturates; on gfx950 it produces OCP e4m3fn
  const int packed = __builtin_amdgcn_cvt_pk_fp8_f32(x, x, 0, false);
  return static_cast<uint8_t>(packed & 0xff);
}

template <typename T>
__global__ void __launch_bounds__(256)
quantize_kernel(const T* __restrict__ w, uint8_t* __restrict__ q, float* __restrict__ scale, int64_t rows,
                int64_t cols, int row_blocks, int col_blocks) {
  __shared__ float wave_max_s[4];
  const int cb = blockIdx.x, rb = blockIdx.y;
  const int64_t batch = blockIdx.z;
  const T* src = w + batch * rows * cols;
  uint8_t* dst = q + batch * rows * cols;
  const int64_t r0 = static_cast<int64_t>(rb) * kBlock, c0 = static_cast<int64_t>(cb) * kBlock;
  float amax = 0.f;
  for (int i = threadIdx.x; i < kBlock * kBlock; i += 256) {
    const int64_t r = r0 + i / kBlock, c = c0 + i % kBlock;
    if (r < rows && c < cols) amax = fmaxf(amax, fabsf(Elem<T>::load(src + r * cols + c)));
  }
  amax = wave_max(amax);
  if (lane_id() == 0) wave_max_s[threadIdx.x / HMOE_WAVE] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(wave_max_s[0], wave_max_s[1]), fmaxf(wave_max_s[2], wave_max_s[3]));
  const float s = pow2_ceil(fmaxf(amax, kAmaxFloor) / kE4m3Max);
  if (threadIdx.x == 0) scale[(batch * row_blocks + rb) * col_blocks + cb] = s;
  const float inv = 1.0f / s;  // exact: s is a power of two
  for (int i = threadIdx.x; i < kBlock * kBlock; i += 256) {
    const int64_t r = r0 + i / kBlock, c = c0 + i % kBlock;
    if (r < rows && c < cols) {
      const float v = fminf(fmaxf(Elem<T>::load(src + r * cols + c) * inv, -kE4m3Max), kE4m3Max);
      dst[r * cols + c] = encode_e4m3(v);
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
dequantize_kernel(const uint8_t* __restrict__ q, const float* __restrict__ scale, T* __restrict__ out, int64_t rows,
                  int64_t cols, int row_blocks, int col_blocks) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  const int cb = blockIdx.x, rb = blockIdx.y;
  const int64_t batch = blockIdx.z;
  const float s = scale[(batch * row_blocks + rb) * col_blocks + cb];
  const int64_t r0 = static_cast<int64_t>(rb) * kBlock, c0 = static_cast<int64_t>(cb) * kBlock;
  for (int i = threadIdx.x; i < kBlock * kBlock; i += 256) {
    const int64_t r = r0 + i / kBlock, c = c0 + i % kBlock;
    if (r < rows && c < cols) {
      const int64_t at = (batch * rows + r) * cols + c;
      const f32x2 v = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(q[at]), false);
      Elem<T>::store(out + at, v.x * s);
    }
  }
}

// Activation rows to e4m3 with one power-of-two scale per row and 128 values, for the fp8 MFMA product (which takes
// an operand's scale as an e8m0 exponent byte).  Sixteen lanes share a block: each loads 8 values and hands them to
// quantize_block_of_row.  With row_index, output row r is x[row_index[r]] (the permute by
// expert taken on the way: the permuted bf16 copy is never written), zeros where the index is outside [0, x_rows).
__global__ void __launch_bounds__(256)
quantize_rows_kernel(const bf16_t* __restrict__ x, int64_t ldx, const int64_t* __restrict__ row_index, int64_t x_rows,
                     int64_t rows, int k, uint8_t* __restrict__ q, uint8_t* __restrict__ scale, int64_t out_rows) {
  // A workgroup takes sixteen consecutive rows of one scale block (128 values, two panels): a row's sixteen lanes read
  // its 256 bytes (two whole lines) and the sixteen rows' halves land side by side in each panel, 1 KB in one piece.
  // (With a workgroup walking along one row, every row's 64 bytes of a panel were a write of their own.)
  const int row_in = threadIdx.x >> 4, lane16 = threadIdx.x & 15;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 16 + row_in;
  const int chunk = static_cast<int>(blockIdx.y) * 16 + lane16;
  if (row >= rows) return;  // whole groups of sixteen lanes leave together
  Vec16<bf16_t> in;
  const int64_t from = row_index ? row_index[row] : row;
  if (from >= 0 && from < x_rows) {
    in.load(x + from * ldx + (chunk << 3));
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) in.v[i] = 0.f;
  }
  quantize_block_of_row(in.v, row, chunk, q, scale, out_rows);
}

}  // namespace
}  // namespace hmoe

extern "C" {

int hmoe_quantize_rows_fp8(const void* x, int64_t ldx, const int64_t* row_index, int64_t x_rows, int64_t rows, int64_t k,
                           uint8_t* q, uint8_t* scale, int64_t out_rows, void* stream) {
  using namespace hmoe;
  if (rows < 0 || k < 0 || x_rows < 0) return HMOE_INVALID_ARGUMENT;
  if (!row_index && x_rows != rows) return HMOE_INVALID_ARGUMENT;
  if (k % kBlock || ldx < k || ldx % 8 || out_rows < rows) return HMOE_UNSUPPORTED;
  if (rows == 0 || k == 0) return HMOE_OK;
  if (!q || !scale || (!x && x_rows > 0)) return HMOE_INVALID_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(q) % 8) return HMOE_UNSUPPORTED;
  const int64_t row_groups = (rows + 15) / 16, col_blocks = k / kBlock;
  if (row_groups >= (int64_t(1) << 31) || col_blocks > 65535) return HMOE_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  quantize_rows_kernel<<<dim3(static_cast<unsigned>(row_groups), static_cast<unsigned>(col_blocks)), dim3(256), 0, s>>>(
      static_cast<const bf16_t*>(x), ldx, row_index, x_rows, rows, static_cast<int>(k), q, scale, out_rows);
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

int hmoe_quantize_block_fp8(const void* w, int dtype, int64_t batch, int64_t rows, int64_t cols, uint8_t* q,
                            float* scale, void* stream) {
  using namespace hmoe;
  if (batch < 0 || rows < 0 || cols < 0) return HMOE_INVALID_ARGUMENT;
  if (batch == 0 || rows == 0 || cols == 0) return HMOE_OK;
  if (!w || !q || !scale) return HMOE_INVALID_ARGUMENT;
  const int64_t rb = (rows + kBlock - 1) / kBlock, cb = (cols + kBlock - 1) / kBlock;
  if (rb > 65535 || batch > 65535) return HMOE_UNSUPPORTED;
  const dim3 grid(static_cast<unsigned>(cb), static_cast<unsigned>(rb), static_cast<unsigned>(batch));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == HMOE_BF16)
    quantize_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(static_cast<const bf16_t*>(w), q, scale, rows, cols,
                                                      static_cast<int>(rb), static_cast<int>(cb));
  else if (dtype == HMOE_F32)
    quantize_kernel<float><<<grid, dim3(256), 0, s>>>(static_cast<const float*>(w), q, scale, rows, cols,
                                                     static_cast<int>(rb), static_cast<int>(cb));
  else
    return HMOE_UNSUPPORTED;
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

int hmoe_dequantize_block_fp8(const uint8_t* q, const float* scale, int64_t batch, int64_t rows, int64_t cols,
                              int dtype, void* out, void* stream) {
  using namespace hmoe;
  if (batch < 0 || rows < 0 || cols < 0) return HMOE_INVALID_ARGUMENT;
  if (batch == 0 || rows == 0 || cols == 0) return HMOE_OK;
  if (!q || !scale || !out) return HMOE_INVALID_ARGUMENT;
  const int64_t rb = (rows + kBlock - 1) / kBlock, cb = (cols + kBlock - 1) / kBlock;
  if (rb > 65535 || batch > 65535) return HMOE_UNSUPPORTED;
  const dim3 grid(static_cast<unsigned>(cb), static_cast<unsigned>(rb), static_cast<unsigned>(batch));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == HMOE_BF16)
    dequantize_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(q, scale, static_cast<bf16_t*>(out), rows, cols,
                                                        static_cast<int>(rb), static_cast<int>(cb));
  else if (dtype == HMOE_F32)
    dequantize_kernel<float><<<grid, dim3(256), 0, s>>>(q, scale, static_cast<float*>(out), rows, cols,
                                                       static_cast<int>(rb), static_cast<int>(cb));
  else
    return HMOE_UNSUPPORTED;
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

}  // extern "C"
