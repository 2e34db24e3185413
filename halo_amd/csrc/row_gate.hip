// The per-token output gate of a shared expert: gate[t] = sigmoid(<x[t], w>), a [T, H] x [H] matrix-vector product
// with a sigmoid behind it, and its backward.  Replaces the three tensor operations of
// halo/distributed/expert_parallel/families/qwen3_5.py:41-42 (shared_expert_gate = nn.Linear(H, 1), torch.sigmoid) and
// their autograd: a [T, 1] projection is below the grouped GEMM kernels' 16-byte row granularity, and as library calls
// it is three launches forward and four backward for 2 x T x H bytes of traffic.
//
// Roundings are those of the tensor operations: the dot product is accumulated in fp32 and rounded to the operands'
// dtype (the linear's output), the sigmoid is computed in fp32 from that and rounded again; backward rounds
// grad * (1 - gate) * gate (sigmoid's backward, fp32) to the dtype, grad_x[t] = that times w rounded once (a single
// product per element, the bits of the outer product), and grad_w = sum over tokens of that times x[t], accumulated in
// fp32 in a fixed order (a partial row per workgroup, then the partial rows in order) and rounded once: deterministic.
// HBM-bound: forward reads x once (H x e bytes per token), backward reads x and writes grad_x (2 x H x e per token).
#include "common.h"

namespace hmoe {
namespace {

constexpr int kGateThreads = 256;
constexpr int kGateMaxBlocks = 1024;  // partial rows of the weight gradient

template <typename T>
__global__ void __launch_bounds__(kGateThreads) row_gate_fwd_kernel(const T* __restrict__ x, int64_t ldx,
                                                                    const T* __restrict__ w, int64_t n_rows,
                                                                    int hidden, T* __restrict__ gate) {
  constexpr int N = Vec16<T>::N;
  const int lane = lane_id();
  const int64_t row = static_cast<int64_t>(blockIdx.x) * (kGateThreads / HMOE_WAVE) + (threadIdx.x / HMOE_WAVE);
  if (row >= n_rows) return;
  const T* xr = x + row * ldx;
  float sum = 0.f;
  for (int c = lane * N; c < hidden; c += HMOE_WAVE * N) {
    Vec16<T> xv, wv;
    xv.load(xr + c);
    wv.load(w + c);
#pragma unroll
    for (int i = 0; i < N; ++i) sum = fmaf(xv.v[i], wv.v[i], sum);
  }
  sum = wave_sum(sum);
  if (lane == 0) {
    const float logit = Elem<T>::round(sum);
    Elem<T>::store(gate + row, 1.0f / (1.0f + expf(-logit)));
  }
}

// grad_x[t] = gs[t] * w and a partial row of grad_w = sum_t gs[t] * x[t] over this workgroup's tokens, where
// gs[t] = round(grad_gate[t] * (1 - gate[t]) * gate[t]).  A thread owns 16-byte column chunks (chunk = thread, thread +
// 256, ...) and walks the workgroup's rows with four row loads in flight.
template <typename T, bool kGradX, bool kGradW>
__global__ void __launch_bounds__(kGateThreads) row_gate_bwd_kernel(const T* __restrict__ x, int64_t ldx,
                                                                    const T* __restrict__ w, const T* __restrict__ gate,
                                                                    const T* __restrict__ grad_gate, int64_t n_rows,
                                                                    int hidden, int64_t rows_per_block,
                                                                    T* __restrict__ grad_x, int64_t ld_grad_x,
                                                                    float* __restrict__ partial) {
  constexpr int N = Vec16<T>::N;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * rows_per_block;
  const int64_t row1 = row0 + rows_per_block < n_rows ? row0 + rows_per_block : n_rows;
  auto scaled_grad = [&](int64_t r) {
    const float g = Elem<T>::load(gate + r);
    return Elem<T>::round(Elem<T>::load(grad_gate + r) * (1.0f - g) * g);
  };
  for (int c = threadIdx.x * N; c < hidden; c += kGateThreads * N) {
    Vec16<T> wv;
    wv.load(w + c);
    float acc[N];
#pragma unroll
    for (int i = 0; i < N; ++i) acc[i] = 0.f;
    int64_t r = row0;
    for (; r + 4 <= row1; r += 4) {
      Vec16<T> xv[4];
      float gs[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if constexpr (kGradW) xv[u].load(x + (r + u) * ldx + c);
        gs[u] = scaled_grad(r + u);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if constexpr (kGradW) {
#pragma unroll
          for (int i = 0; i < N; ++i) acc[i] = fmaf(gs[u], xv[u].v[i], acc[i]);
        }
        if constexpr (kGradX) {
          Vec16<T> out;
#pragma unroll
          for (int i = 0; i < N; ++i) out.v[i] = gs[u] * wv.v[i];
          out.store(grad_x + (r + u) * ld_grad_x + c);
        }
      }
    }
    for (; r < row1; ++r) {
      const float gs = scaled_grad(r);
      if constexpr (kGradW) {
        Vec16<T> xv;
        xv.load(x + r * ldx + c);
#pragma unroll
        for (int i = 0; i < N; ++i) acc[i] = fmaf(gs, xv.v[i], acc[i]);
      }
      if constexpr (kGradX) {
        Vec16<T> out;
#pragma unroll
        for (int i = 0; i < N; ++i) out.v[i] = gs * wv.v[i];
        out.store(grad_x + r * ld_grad_x + c);
      }
    }
    if constexpr (kGradW) {
      float* dst = partial + static_cast<int64_t>(blockIdx.x) * hidden + c;
#pragma unroll
      for (int i = 0; i < N; ++i) dst[i] = acc[i];
    }
  }
}

// grad_w[c] = the partial rows' column c, rounded once.  Sixteen threads share a column: thread s adds the partial rows
// s, s + 16, ... in that order and the sixteen sums are added in the order of s, so the result does not depend on
// timing (one thread per column walking every partial row took 64 us for 256 rows: a chain of dependent loads).
constexpr int kFinalCols = 16, kFinalSlices = kGateThreads / kFinalCols;
template <typename T>
__global__ void __launch_bounds__(kGateThreads) row_gate_bwd_final_kernel(const float* __restrict__ partial, int blocks,
                                                                          int hidden, T* __restrict__ grad_w) {
  __shared__ float sums[kFinalSlices][kFinalCols];
  const int col_in = threadIdx.x % kFinalCols, slice = threadIdx.x / kFinalCols;
  const int c = blockIdx.x * kFinalCols + col_in;
  float sum = 0.f;
  if (c < hidden) {
#pragma unroll 4
    for (int b = slice; b < blocks; b += kFinalSlices) sum += partial[static_cast<int64_t>(b) * hidden + c];
  }
  sums[slice][col_in] = sum;
  __syncthreads();
  if (slice == 0 && c < hidden) {
    float total = 0.f;
#pragma unroll
    for (int s = 0; s < kFinalSlices; ++s) total += sums[s][col_in];
    Elem<T>::store(grad_w + c, total);
  }
}

inline int64_t gate_rows_per_block(int64_t n_rows) {
  const int64_t rows = (n_rows + kGateMaxBlocks - 1) / kGateMaxBlocks;
  return rows < 32 ? 32 : rows;
}
inline int gate_blocks(int64_t n_rows) {
  const int64_t per = gate_rows_per_block(n_rows);
  return static_cast<int>((n_rows + per - 1) / per);
}

template <typename T>
int launch_fwd(const void* x, int64_t ldx, const void* w, int64_t n_rows, int hidden, void* gate, hipStream_t s) {
  const int rows_per_block = kGateThreads / HMOE_WAVE;
  const int64_t blocks = (n_rows + rows_per_block - 1) / rows_per_block;
  row_gate_fwd_kernel<T><<<dim3(static_cast<unsigned>(blocks)), dim3(kGateThreads), 0, s>>>(
      static_cast<const T*>(x), ldx, static_cast<const T*>(w), n_rows, hidden, static_cast<T*>(gate));
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

template <typename T>
int launch_bwd(const void* x, int64_t ldx, const void* w, const void* gate, const void* grad_gate, int64_t n_rows,
               int hidden, void* grad_x, int64_t ld_grad_x, void* grad_w, void* workspace, hipStream_t s) {
  const int64_t per = gate_rows_per_block(n_rows);
  const int blocks = gate_blocks(n_rows);
  const dim3 grid(blocks), block(kGateThreads);
  auto* part = static_cast<float*>(workspace);
#define HMOE_GATE_BWD(GX, GW)                                                                                     \
  row_gate_bwd_kernel<T, GX, GW><<<grid, block, 0, s>>>(                                                          \
      static_cast<const T*>(x), ldx, static_cast<const T*>(w), static_cast<const T*>(gate),                       \
      static_cast<const T*>(grad_gate), n_rows, hidden, per, static_cast<T*>(grad_x), ld_grad_x, part)
  if (grad_x && grad_w) HMOE_GATE_BWD(true, true);
  else if (grad_x) HMOE_GATE_BWD(true, false);
  else HMOE_GATE_BWD(false, true);
#undef HMOE_GATE_BWD
  HMOE_CHECK_LAUNCH();
  if (grad_w) {
    row_gate_bwd_final_kernel<T><<<dim3((hidden + kFinalCols - 1) / kFinalCols), block, 0, s>>>(
        part, blocks, hidden, static_cast<T*>(grad_w));
    HMOE_CHECK_LAUNCH();
  }
  return HMOE_OK;
}

inline bool gate_shape_ok(int64_t ld, int hidden, int dtype, const void* a, const void* b) {
  const int n = dtype == HMOE_BF16 ? 8 : 4;
  return hidden % n == 0 && ld % n == 0 && aligned16(a) && aligned16(b);
}

}  // namespace
}  // namespace hmoe

extern "C" {

int hmoe_row_gate_fwd(const void* x, int64_t ldx, const void* w, int64_t n_rows, int hidden, int dtype, void* gate,
                      void* stream) {
  if (n_rows < 0 || hidden <= 0 || (dtype != HMOE_BF16 && dtype != HMOE_F32)) return HMOE_INVALID_ARGUMENT;
  if (n_rows == 0) return HMOE_OK;
  if (!x || !w || !gate) return HMOE_INVALID_ARGUMENT;
  if (!hmoe::gate_shape_ok(ldx, hidden, dtype, x, w)) return HMOE_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dtype == HMOE_BF16 ? hmoe::launch_fwd<hmoe::bf16_t>(x, ldx, w, n_rows, hidden, gate, s)
                            : hmoe::launch_fwd<float>(x, ldx, w, n_rows, hidden, gate, s);
}

int64_t hmoe_row_gate_bwd_workspace_bytes(int64_t n_rows, int hidden) {
  if (n_rows < 0 || hidden <= 0) return HMOE_INVALID_ARGUMENT;
  return static_cast<int64_t>(hmoe::gate_blocks(n_rows)) * hidden * static_cast<int64_t>(sizeof(float));
}

int hmoe_row_gate_bwd(const void* x, int64_t ldx, const void* w, const void* gate, const void* grad_gate,
                      int64_t n_rows, int hidden, int dtype, void* grad_x, int64_t ld_grad_x, void* grad_w,
                      void* workspace, void* stream) {
  if (n_rows < 0 || hidden <= 0 || (dtype != HMOE_BF16 && dtype != HMOE_F32)) return HMOE_INVALID_ARGUMENT;
  if (!grad_x && !grad_w) return HMOE_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (n_rows == 0) {  // no tokens: the weight gradient is zero (the sum over no partial rows)
    if (grad_w) {
      const dim3 grid((hidden + hmoe::kFinalCols - 1) / hmoe::kFinalCols), block(hmoe::kGateThreads);
      if (dtype == HMOE_BF16)
        hmoe::row_gate_bwd_final_kernel<hmoe::bf16_t><<<grid, block, 0, s>>>(nullptr, 0, hidden,
                                                                            static_cast<hmoe::bf16_t*>(grad_w));
      else
        hmoe::row_gate_bwd_final_kernel<float><<<grid, block, 0, s>>>(nullptr, 0, hidden, static_cast<float*>(grad_w));
      HMOE_CHECK_LAUNCH();
    }
    return HMOE_OK;
  }
  if (!x || !w || !gate || !grad_gate || (grad_w && !workspace)) return HMOE_INVALID_ARGUMENT;
  if (!hmoe::gate_shape_ok(ldx, hidden, dtype, x, w) ||
      (grad_x && !hmoe::gate_shape_ok(ld_grad_x, hidden, dtype, grad_x, grad_x)))
    return HMOE_UNSUPPORTED;
  return dtype == HMOE_BF16
             ? hmoe::launch_bwd<hmoe::bf16_t>(x, ldx, w, gate, grad_gate, n_rows, hidden, grad_x, ld_grad_x, grad_w,
                                              workspace, s)
             : hmoe::launch_bwd<float>(x, ldx, w, gate, grad_gate, n_rows, hidden, grad_x, ld_grad_x, grad_w,
                                       workspace, s);
}

}  // extern "C"
