// What the matrix pipe of this device sustains with nothing else to do: a loop of independent bf16 MFMAs on register
// operands, two wavefronts per SIMD on every compute unit (the occupancy of the grouped GEMM kernels).  Two shapes
// (v_mfma_f32_32x32x16_bf16, the one the GEMM kernels use, and v_mfma_f32_16x16x32_bf16) and two kinds of operands:
// small integers, which toggle few bits, and pseudo-random values with random signs, which load the multipliers the
// way real activations and weights do -- the clock this part holds depends on the power the pipe draws.  A measuring
// stick for the benchmark's roofline figures; no counterpart in the reference.
#include "common.h"

namespace hmoe {
namespace {

typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));
typedef float probe_f32x4 __attribute__((ext_vector_type(4)));

constexpr int kProbeChains = 8;  // independent accumulators per wavefront: no MFMA waits for the one before it

// operand values of one lane: kRandom false = integers 0..3 and 0..1; true = a hash of (lane, element) mapped to
// [-2, 2) with 8 significant bits, signs mixed so that the accumulators random-walk instead of growing
template <bool kRandom>
__device__ __forceinline__ void probe_operands(probe_bf16x8& a, probe_bf16x8& b) {
#pragma unroll
  for (int v = 0; v < 8; ++v) {
    if (kRandom) {
      uint32_t h = (threadIdx.x * 8u + v + blockIdx.x * 4099u) * 2654435761u;
      h ^= h >> 15;
      h *= 2246822519u;
      h ^= h >> 13;
      a[v] = static_cast<__bf16>((static_cast<int>(h & 0x1ff) - 256) * (1.0f / 128));
      b[v] = static_cast<__bf16>((static_cast<int>(h >> 16 & 0x1ff) - 256) * (1.0f / 128));
    } else {
      a[v] = static_cast<__bf16>(static_cast<float>((threadIdx.x + v) & 3));
      b[v] = static_cast<__bf16>(static_cast<float>((threadIdx.x ^ v) & 1));
    }
  }
}

template <bool kSmallShape, bool kRandom>
__global__ void __launch_bounds__(512) mfma_probe_kernel(int64_t iterations, float* sink) {
  probe_bf16x8 a, b;
  probe_operands<kRandom>(a, b);
  float total = 0.f;
  if (kSmallShape) {  // 16x16x32: four accumulator registers per chain, half the flops per instruction
    probe_f32x4 acc[kProbeChains];
#pragma unroll
    for (int c = 0; c < kProbeChains; ++c) acc[c] = probe_f32x4{0.f, 0.f, 0.f, 0.f};
    for (int64_t i = 0; i < iterations; ++i) {
#pragma unroll
      for (int c = 0; c < kProbeChains; ++c) acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[c], 0, 0, 0);
    }
#pragma unroll
    for (int c = 0; c < kProbeChains; ++c)
#pragma unroll
      for (int v = 0; v < 4; ++v) total += acc[c][v];
  } else {
    probe_f32x16 acc[kProbeChains];
#pragma unroll
    for (int c = 0; c < kProbeChains; ++c)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[c][v] = 0.f;
    for (int64_t i = 0; i < iterations; ++i) {
#pragma unroll
      for (int c = 0; c < kProbeChains; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
    }
#pragma unroll
    for (int c = 0; c < kProbeChains; ++c)
#pragma unroll
      for (int v = 0; v < 16; ++v) total += acc[c][v];
  }
  // never true for the integer operands (their sums are non-negative) and as good as never for the random ones: the
  // store keeps the loop alive
  if (total == -1.25f) sink[blockIdx.x] = total;
}

// A read-only stream: every 16 bytes of `src` fetched once (non-temporal, eight fetches in flight per lane), folded
// into a value that is never stored.  What the memory system delivers to a kernel that only reads.
typedef unsigned int probe_u32x4 __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256) hbm_read_probe_kernel(const probe_u32x4* __restrict__ src, int64_t n16,
                                                             probe_u32x4* sink) {
  probe_u32x4 acc = {0u, 0u, 0u, 0u};
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  for (; i + 7 * stride < n16; i += 8 * stride) {
    probe_u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u];
  }
  for (; i < n16; i += stride) acc ^= __builtin_nontemporal_load(src + i);
  if (acc[0] == 0x12345678u && acc[1] == 77u && acc[2] == 5u) sink[0] = acc;  // keeps the loads alive
}

}  // namespace
}  // namespace hmoe

extern "C" {

int64_t hmoe_probe_hbm_read(const void* src, int64_t bytes, void* sink, void* stream) {
  if (bytes < 0 || bytes % 16 || (bytes > 0 && (!src || !sink))) return HMOE_INVALID_ARGUMENT;
  if (!hmoe::aligned16(src) || !hmoe::aligned16(sink)) return HMOE_UNSUPPORTED;
  if (bytes == 0) return 0;
  hmoe::hbm_read_probe_kernel<<<dim3(8192), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const hmoe::probe_u32x4*>(src), bytes / 16, static_cast<hmoe::probe_u32x4*>(sink));
  if (hipGetLastError() != hipSuccess) return HMOE_LAUNCH_FAILED;
  return bytes;
}

int64_t hmoe_probe_mfma_bf16(int64_t iterations, int shape, int operands, void* sink, void* stream) {
  if (iterations <= 0 || sink == nullptr || shape < 0 || shape > 1 || operands < 0 || operands > 1)
    return HMOE_INVALID_ARGUMENT;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return HMOE_LAUNCH_FAILED;
  const dim3 grid(cus), block(512);
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* out = static_cast<float*>(sink);
  if (shape == 0 && operands == 0) hmoe::mfma_probe_kernel<false, false><<<grid, block, 0, s>>>(iterations, out);
  if (shape == 0 && operands == 1) hmoe::mfma_probe_kernel<false, true><<<grid, block, 0, s>>>(iterations, out);
  if (shape == 1 && operands == 0) hmoe::mfma_probe_kernel<true, false><<<grid, block, 0, s>>>(iterations, out);
  if (shape == 1 && operands == 1) hmoe::mfma_probe_kernel<true, true><<<grid, block, 0, s>>>(iterations, out);
  if (hipGetLastError() != hipSuccess) return HMOE_LAUNCH_FAILED;
  // multiply-adds counted twice: workgroups x wavefronts x iterations x chains x (32 x 32 x 16 x 2 or 16 x 16 x 32 x 2)
  return static_cast<int64_t>(cus) * 8 * iterations * hmoe::kProbeChains * (shape == 0 ? 32768 : 16384);
}

}  // extern "C"
