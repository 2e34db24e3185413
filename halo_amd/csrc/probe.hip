// What the matrix pipe of this device sustains with nothing else to do: a loop of independent
// v_mfma_f32_32x32x16_bf16 on register operands, two wavefronts per SIMD on every compute unit (the occupancy of the
// grouped GEMM kernels).  A measuring stick for the benchmark's roofline figures; no counterpart in the reference.
#include "common.h"

namespace hmoe {
namespace {

typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));

constexpr int kProbeChains = 8;  // independent accumulators per wavefront: no MFMA waits for the one before it

__global__ void __launch_bounds__(512) mfma_probe_kernel(int64_t iterations, float* sink) {
  probe_f32x16 acc[kProbeChains];
#pragma unroll
  for (int c = 0; c < kProbeChains; ++c)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[c][v] = 0.f;
  probe_bf16x8 a, b;
#pragma unroll
  for (int v = 0; v < 8; ++v) {
    a[v] = static_cast<__bf16>(static_cast<float>((threadIdx.x + v) & 3));
    b[v] = static_cast<__bf16>(static_cast<float>((threadIdx.x ^ v) & 1));
  }
  for (int64_t i = 0; i < iterations; ++i) {
#pragma unroll
    for (int c = 0; c < kProbeChains; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
  }
  float total = 0.f;
#pragma unroll
  for (int c = 0; c < kProbeChains; ++c)
#pragma unroll
    for (int v = 0; v < 16; ++v) total += acc[c][v];
  if (total == -1.f) sink[blockIdx.x] = total;  // never true (the sums are non-negative): keeps the loop alive
}

}  // namespace
}  // namespace hmoe

extern "C" {

int64_t hmoe_probe_mfma_bf16(int64_t iterations, void* sink, void* stream) {
  if (iterations <= 0 || sink == nullptr) return HMOE_INVALID_ARGUMENT;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return HMOE_LAUNCH_FAILED;
  hmoe::mfma_probe_kernel<<<dim3(cus), dim3(512), 0, static_cast<hipStream_t>(stream)>>>(
      iterations, static_cast<float*>(sink));
  if (hipGetLastError() != hipSuccess) return HMOE_LAUNCH_FAILED;
  // multiply-adds counted twice: workgroups x wavefronts x iterations x chains x (32 x 32 x 16 x 2)
  return static_cast<int64_t>(cus) * 8 * iterations * hmoe::kProbeChains * 32768;
}

}  // extern "C"
