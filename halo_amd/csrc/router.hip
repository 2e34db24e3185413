// Fused router gate: softmax / top-k / renormalise / cast in one kernel, one wavefront per token, and its gradient.
//
// Replaces the aten sequence softmax -> topk -> (renorm) -> cast the reference's family routers run after the logits
// projection (layer call sites halo/distributed/expert_parallel/moe_layer/shared_experts_layer.py:44-56 and
// families/gpt_oss.py:108; gate-weight rules routing.py:110-122 and families/gpt_oss.py:82-84).
//
// Selection: k rounds of a wave-wide arg-max on (logit descending, expert index ascending), so equal scores go to the
// lower expert index.  Softmax is monotone, so selecting on the logits equals selecting on the probabilities wherever
// those are distinct, and the comparison is exact on every device.
// Lane l holds experts l, l+64, l+128, ... (kPer per lane): loads are coalesced and the arg-max is a register scan
// followed by six xor-shuffles.
#include "common.h"

#include <math.h>

namespace hmoe {
namespace {

constexpr int kThreads = 256;
constexpr int kTokensPerBlock = kThreads / HMOE_WAVE;

struct Best {
  float v;
  int idx;
};

__device__ __forceinline__ Best better(Best a, Best b) {
  const bool take_b = (b.v > a.v) || (b.v == a.v && b.idx < a.idx);
  return take_b ? b : a;
}

__device__ __forceinline__ Best wave_best(Best x) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    Best o;
    o.v = __shfl_xor(x.v, off, HMOE_WAVE);
    o.idx = __shfl_xor(x.idx, off, HMOE_WAVE);
    x = better(x, o);
  }
  return x;
}

template <typename T>
__device__ __forceinline__ float round_to(float v);
template <>
__device__ __forceinline__ float round_to<float>(float v) { return v; }
template <>
__device__ __forceinline__ float round_to<bf16_t>(float v) { return bf16_to_f32(f32_to_bf16(v)); }

// Loads the token's logits, selects top_k; on return lane j < top_k holds the j-th pick (sel_idx, sel_val);
// row_max / row_sum describe the full softmax.
template <typename T, int kPer>
__device__ __forceinline__ void load_and_select(const T* __restrict__ row, int num_experts, int top_k,
                                                float (&x)[kPer], int& sel_idx, float& sel_val) {
  const int lane = lane_id();
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int e = i * HMOE_WAVE + lane;
    x[i] = e < num_experts ? Elem<T>::load(row + e) : -INFINITY;
  }
  uint32_t taken = 0;
  sel_idx = 0;
  sel_val = -INFINITY;
  for (int j = 0; j < top_k; ++j) {
    Best mine{-INFINITY, 0x7fffffff};
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      const int e = i * HMOE_WAVE + lane;
      if (e < num_experts && !((taken >> i) & 1u)) mine = better(mine, Best{x[i], e});
    }
    const Best win = wave_best(mine);
    if ((win.idx & (HMOE_WAVE - 1)) == lane && win.idx < num_experts) taken |= 1u << (win.idx / HMOE_WAVE);
    if (lane == j) {
      sel_idx = win.idx;
      sel_val = win.v;
    }
  }
}

template <typename T, int kPer>
__global__ void __launch_bounds__(kThreads)
router_fwd_kernel(const T* __restrict__ logits, int64_t n_tokens, int num_experts, int top_k, int mode,
                  int normalize, float eps, int64_t* __restrict__ indices, float* __restrict__ weights) {
  const int64_t token = static_cast<int64_t>(blockIdx.x) * kTokensPerBlock + threadIdx.x / HMOE_WAVE;
  if (token >= n_tokens) return;
  const int lane = lane_id();
  float x[kPer];
  int sel_idx;
  float sel_val;
  load_and_select<T, kPer>(logits + token * num_experts, num_experts, top_k, x, sel_idx, sel_val);
  const bool picked = lane < top_k;
  float w;
  if (mode == HMOE_ROUTER_SOFTMAX_ALL) {
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < kPer; ++i) m = fmaxf(m, x[i]);
    m = wave_max(m);
    float z = 0.f;
#pragma unroll
    for (int i = 0; i < kPer; ++i) z += (i * HMOE_WAVE + lane < num_experts) ? expf(x[i] - m) : 0.f;
    z = wave_sum(z);
    w = picked ? expf(sel_val - m) / z : 0.f;
    if (normalize) {
      const float s = wave_sum(w);
      w = w / (s + eps);
    }
  } else {
    const float m = __shfl(sel_val, 0, HMOE_WAVE);  // the first pick is the largest
    const float ex = picked ? expf(sel_val - m) : 0.f;
    const float s = wave_sum(ex);
    w = ex / s;
  }
  if (picked) {
    indices[token * top_k + lane] = sel_idx;
    weights[token * top_k + lane] = round_to<T>(w);
  }
}

template <typename T, int kPer>
__global__ void __launch_bounds__(kThreads)
router_bwd_kernel(const T* __restrict__ logits, const int64_t* __restrict__ indices,
                  const float* __restrict__ grad_weights, int64_t n_tokens, int num_experts, int top_k, int mode,
                  int normalize, float eps, T* __restrict__ grad_logits) {
  const int64_t token = static_cast<int64_t>(blockIdx.x) * kTokensPerBlock + threadIdx.x / HMOE_WAVE;
  if (token >= n_tokens) return;
  const int lane = lane_id();
  const T* row = logits + token * num_experts;
  float x[kPer], dl[kPer];
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int e = i * HMOE_WAVE + lane;
    x[i] = e < num_experts ? Elem<T>::load(row + e) : -INFINITY;
    dl[i] = 0.f;
  }
  const bool picked = lane < top_k;
  int sel_idx = 0;
  float g = 0.f, sel_val = -INFINITY;
  if (picked) {
    sel_idx = static_cast<int>(indices[token * top_k + lane]);
    g = grad_weights[token * top_k + lane];
    if (sel_idx >= 0 && sel_idx < num_experts) sel_val = Elem<T>::load(row + sel_idx);
  }
  float coeff;  // gradient w.r.t. the picked expert's probability (mode ALL) or logit (mode TOPK)
  float m = -INFINITY, z = 1.f;
  if (mode == HMOE_ROUTER_SOFTMAX_ALL) {
#pragma unroll
    for (int i = 0; i < kPer; ++i) m = fmaxf(m, x[i]);
    m = wave_max(m);
    z = 0.f;
#pragma unroll
    for (int i = 0; i < kPer; ++i) z += (i * HMOE_WAVE + lane < num_experts) ? expf(x[i] - m) : 0.f;
    z = wave_sum(z);
    const float p = picked ? expf(sel_val - m) / z : 0.f;
    float dp = g;
    if (normalize) {
      const float s = wave_sum(p) + eps;
      const float w = p / s;
      const float gw = wave_sum(g * w);
      dp = picked ? (g - gw) / s : 0.f;
    }
    const float d = wave_sum(dp * p);  // sum over the picks of dp * p
    // dl_i = p_i * (dp_i - d), dp_i = 0 for an expert that was not picked
#pragma unroll
    for (int i = 0; i < kPer; ++i) dl[i] = -d;
    coeff = dp;
  } else {
    float mx = picked ? sel_val : -INFINITY;
    mx = wave_max(mx);
    const float ex = picked ? expf(sel_val - mx) : 0.f;
    const float s = wave_sum(ex);
    const float w = ex / s;
    const float gw = wave_sum(g * w);
    coeff = picked ? w * (g - gw) : 0.f;
  }
  for (int j = 0; j < top_k; ++j) {
    const int idx = __shfl(sel_idx, j, HMOE_WAVE);
    const float c = __shfl(coeff, j, HMOE_WAVE);
#pragma unroll
    for (int i = 0; i < kPer; ++i)
      if (i * HMOE_WAVE + lane == idx) dl[i] += c;
  }
  T* out = grad_logits + token * num_experts;
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int e = i * HMOE_WAVE + lane;
    if (e < num_experts) {
      float v = dl[i];
      if (mode == HMOE_ROUTER_SOFTMAX_ALL) v *= expf(x[i] - m) / z;
      Elem<T>::store(out + e, v);
    }
  }
}

template <typename T, int kPer>
int launch(bool backward, const void* logits, int64_t n_tokens, int num_experts, int top_k, int mode, int normalize,
           float eps, int64_t* indices, float* weights, const float* grad_weights, void* grad_logits,
           hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>((n_tokens + kTokensPerBlock - 1) / kTokensPerBlock)), block(kThreads);
  if (!backward)
    router_fwd_kernel<T, kPer><<<grid, block, 0, stream>>>(static_cast<const T*>(logits), n_tokens, num_experts,
                                                          top_k, mode, normalize, eps, indices, weights);
  else
    router_bwd_kernel<T, kPer><<<grid, block, 0, stream>>>(static_cast<const T*>(logits), indices, grad_weights,
                                                          n_tokens, num_experts, top_k, mode, normalize, eps,
                                                          static_cast<T*>(grad_logits));
  if (hipGetLastError() != hipSuccess) return HMOE_LAUNCH_FAILED;
  return HMOE_OK;
}

template <typename T>
int dispatch(bool backward, const void* logits, int64_t n_tokens, int num_experts, int top_k, int mode,
             int normalize, float eps, int64_t* indices, float* weights, const float* grad_weights,
             void* grad_logits, hipStream_t stream) {
#define HMOE_ROUTER(P)                                                                                        \
  return launch<T, P>(backward, logits, n_tokens, num_experts, top_k, mode, normalize, eps, indices, weights, \
                      grad_weights, grad_logits, stream)
  if (num_experts <= 64) HMOE_ROUTER(1);
  if (num_experts <= 128) HMOE_ROUTER(2);
  if (num_experts <= 256) HMOE_ROUTER(4);
  if (num_experts <= 512) HMOE_ROUTER(8);
  if (num_experts <= 1024) HMOE_ROUTER(16);
#undef HMOE_ROUTER
  return HMOE_UNSUPPORTED;
}

int check(int64_t n_tokens, int num_experts, int top_k, int mode) {
  if (n_tokens < 0 || num_experts <= 0 || top_k <= 0) return HMOE_INVALID_ARGUMENT;
  if (mode != HMOE_ROUTER_SOFTMAX_ALL && mode != HMOE_ROUTER_SOFTMAX_TOPK) return HMOE_INVALID_ARGUMENT;
  if (top_k > num_experts) return HMOE_INVALID_ARGUMENT;
  if (top_k > HMOE_WAVE || num_experts > 1024) return HMOE_UNSUPPORTED;
  return HMOE_OK;
}

}  // namespace
}  // namespace hmoe

extern "C" {

int hmoe_router_topk_fwd(const void* logits, int dtype, int64_t n_tokens, int num_experts, int top_k, int mode,
                         int normalize, float eps, int64_t* indices, float* weights, void* stream) {
  using namespace hmoe;
  if (int rc = check(n_tokens, num_experts, top_k, mode)) return rc;
  if (n_tokens == 0) return HMOE_OK;
  if (!logits || !indices || !weights) return HMOE_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == HMOE_BF16)
    return dispatch<bf16_t>(false, logits, n_tokens, num_experts, top_k, mode, normalize, eps, indices, weights,
                            nullptr, nullptr, s);
  if (dtype == HMOE_F32)
    return dispatch<float>(false, logits, n_tokens, num_experts, top_k, mode, normalize, eps, indices, weights,
                           nullptr, nullptr, s);
  return HMOE_UNSUPPORTED;
}

int hmoe_router_topk_bwd(const void* logits, int dtype, const int64_t* indices, const float* grad_weights,
                         int64_t n_tokens, int num_experts, int top_k, int mode, int normalize, float eps,
                         void* grad_logits, void* stream) {
  using namespace hmoe;
  if (int rc = check(n_tokens, num_experts, top_k, mode)) return rc;
  if (n_tokens == 0) return HMOE_OK;
  if (!logits || !indices || !grad_weights || !grad_logits) return HMOE_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == HMOE_BF16)
    return dispatch<bf16_t>(true, logits, n_tokens, num_experts, top_k, mode, normalize, eps,
                            const_cast<int64_t*>(indices), nullptr, grad_weights, grad_logits, s);
  if (dtype == HMOE_F32)
    return dispatch<float>(true, logits, n_tokens, num_experts, top_k, mode, normalize, eps,
                           const_cast<int64_t*>(indices), nullptr, grad_weights, grad_logits, s);
  return HMOE_UNSUPPORTED;
}

}  // extern "C"
