// Fused GLU combines and their gradients for gfx950: SiLU, tanh-GELU and the clamped SwiGLU family, over row-strided
// gate / up operands so a packed [gate | up] projection is read in place and its gradient written as one buffer.
// fp32 math, 16-byte accesses, one thread per 16 bytes of output.
//
// Replaces _glu_fwd_kernel / _glu_bwd_kernel (halo/kernels/fused_glu.py:118-205) of the reference.
#include "common.h"
#include "fp8_rows.h"

#include <type_traits>

namespace hmoe {
namespace {

constexpr int kThreads = 256;

struct GluParams {
  float alpha;
  float limit;
};

__device__ __forceinline__ float fast_sigmoid(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }
__device__ __forceinline__ float fast_tanh(float x) { return 1.0f - 2.0f * __builtin_amdgcn_rcpf(__expf(2.0f * x) + 1.0f); }

constexpr float kSqrt2OverPi = 0.7978845608028654f;
constexpr float kGeluCoeff = 0.044715f;

// kAct: hmoe_glu_activation.  kClampAct / kPlusOne only matter for the clamped family.
template <int kAct, bool kClampAct, bool kPlusOne>
__device__ __forceinline__ float glu_value(float g, float u, GluParams p) {
  if constexpr (kAct == HMOE_GLU_SILU) {
    return g * fast_sigmoid(g) * u;
  } else if constexpr (kAct == HMOE_GLU_GELU_TANH) {
    const float t = fast_tanh(kSqrt2OverPi * (g + kGeluCoeff * g * g * g));
    return 0.5f * g * (1.0f + t) * u;
  } else {
    float ug = fminf(fmaxf(u, -p.limit), p.limit);
    if constexpr (kPlusOne) ug += 1.0f;
    const float ga = kClampAct ? g : fminf(g, p.limit);
    const float glu = ga * fast_sigmoid(ga * p.alpha);
    const float act = kClampAct ? fminf(glu, p.limit) : glu;
    return act * ug;
  }
}

template <int kAct, bool kClampAct, bool kPlusOne>
__device__ __forceinline__ void glu_grad(float g, float u, float d, GluParams p, float& dg, float& du) {
  if constexpr (kAct == HMOE_GLU_SILU) {
    const float s = fast_sigmoid(g);
    dg = d * u * (s * (1.0f + g * (1.0f - s)));
    du = d * (g * s);
  } else if constexpr (kAct == HMOE_GLU_GELU_TANH) {
    const float t = fast_tanh(kSqrt2OverPi * (g + kGeluCoeff * g * g * g));
    const float inner = kSqrt2OverPi * (1.0f + 3.0f * kGeluCoeff * (g * g));
    dg = d * u * (0.5f * (1.0f + t) + 0.5f * g * (1.0f - t * t) * inner);
    du = d * (0.5f * g * (1.0f + t));
  } else {
    float ug = fminf(fmaxf(u, -p.limit), p.limit);
    if constexpr (kPlusOne) ug += 1.0f;
    const float ga = kClampAct ? g : fminf(g, p.limit);
    const float s = fast_sigmoid(ga * p.alpha);
    const float glu = ga * s;
    const float act = kClampAct ? fminf(glu, p.limit) : glu;
    const float dglu = s + ga * p.alpha * s * (1.0f - s);
    // a clamp passes its gradient on the closed interval, the bound included
    const float up_in = (u >= -p.limit && u <= p.limit) ? 1.0f : 0.0f;
    const float gate_in = (kClampAct ? (glu <= p.limit) : (g <= p.limit)) ? 1.0f : 0.0f;
    dg = d * ug * dglu * gate_in;
    du = d * act * up_in;
  }
}

template <typename T, int W>
struct Chunk {
  float v[W];
  __device__ __forceinline__ void load(const T* p) {
    if constexpr (W == 1) {
      v[0] = Elem<T>::load(p);
    } else {
      Vec16<T> t;
      t.load(p);
#pragma unroll
      for (int i = 0; i < W; ++i) v[i] = t.v[i];
    }
  }
  __device__ __forceinline__ void store(T* p) const {
    if constexpr (W == 1) {
      Elem<T>::store(p, v[0]);
    } else {
      Vec16<T> t;
#pragma unroll
      for (int i = 0; i < W; ++i) t.v[i] = v[i];
      t.store(p);
    }
  }
};

template <typename T, int W, int kAct, bool kClampAct, bool kPlusOne>
__global__ void __launch_bounds__(kThreads)
glu_fwd_kernel(const T* __restrict__ gate, const T* __restrict__ up, T* __restrict__ out, int64_t stride_gate,
               int64_t stride_up, int64_t n_rows, int64_t chunks_per_row, int64_t width, GluParams p) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t row = i / chunks_per_row;
  if (row >= n_rows) return;
  const int64_t col = (i - row * chunks_per_row) * W;
  Chunk<T, W> g, u, o;
  g.load(gate + row * stride_gate + col);
  u.load(up + row * stride_up + col);
#pragma unroll
  for (int k = 0; k < W; ++k) o.v[k] = glu_value<kAct, kClampAct, kPlusOne>(g.v[k], u.v[k], p);
  o.store(out + row * width + col);
}

// The forward combine with its output written as e4m3 panels and scale exponents for the fp8 expert GEMM instead of
// as bf16: each value is rounded to bf16 first, so the result is what the row quantiser makes of glu_fwd_kernel's
// output, bit for bit, without the bf16 round trip through memory.  bf16, eight values per lane, width a multiple
// of 128 (sixteen lanes to a scale block).
template <int kAct, bool kClampAct, bool kPlusOne>
__global__ void __launch_bounds__(kThreads)
glu_fwd_quant_kernel(const bf16_t* __restrict__ gate, const bf16_t* __restrict__ up, uint8_t* __restrict__ q,
                     uint8_t* __restrict__ scale, int64_t out_rows, int64_t stride_gate, int64_t stride_up,
                     int64_t n_rows, int64_t chunks_per_row, GluParams p) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t row = i / chunks_per_row;
  if (row >= n_rows) return;  // whole groups of sixteen lanes leave together
  const int chunk = static_cast<int>(i - row * chunks_per_row);
  Chunk<bf16_t, 8> g, u;
  g.load(gate + row * stride_gate + chunk * 8);
  u.load(up + row * stride_up + chunk * 8);
  float v[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) v[k] = Elem<bf16_t>::round(glu_value<kAct, kClampAct, kPlusOne>(g.v[k], u.v[k], p));
  quantize_block_of_row(v, row, chunk, q, scale, out_rows);
}

template <typename T, int W, int kAct, bool kClampAct, bool kPlusOne>
__global__ void __launch_bounds__(kThreads)
glu_bwd_kernel(const T* __restrict__ gate, const T* __restrict__ up, const T* __restrict__ grad_out,
               T* __restrict__ dgate, T* __restrict__ dup, int64_t stride_gate, int64_t stride_up,
               int64_t stride_dgate, int64_t stride_dup, int64_t n_rows, int64_t chunks_per_row, int64_t width,
               GluParams p) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t row = i / chunks_per_row;
  if (row >= n_rows) return;
  const int64_t col = (i - row * chunks_per_row) * W;
  Chunk<T, W> g, u, d, dg, du;
  g.load(gate + row * stride_gate + col);
  u.load(up + row * stride_up + col);
  d.load(grad_out + row * width + col);
#pragma unroll
  for (int k = 0; k < W; ++k) glu_grad<kAct, kClampAct, kPlusOne>(g.v[k], u.v[k], d.v[k], p, dg.v[k], du.v[k]);
  dg.store(dgate + row * stride_dgate + col);
  du.store(dup + row * stride_dup + col);
}

// A row's gate weight: in the operands' dtype, or fp32 rounded to it here (what a cast of the weights would give,
// without the cast's launch).
template <typename T>
__device__ __forceinline__ float load_row_weight(const void* row_weight, bool weight_f32, int64_t row) {
  if (weight_f32) return Elem<T>::round(static_cast<const float*>(row_weight)[row]);
  return Elem<T>::load(static_cast<const T*>(row_weight) + row);
}

// The combine with the row's gate weight folded in: out[r] = round(w[r] * glu(gate[r], up[r])), the product taken in
// fp32, so the down projection runs on weighted rows and the combine behind it is a plain sum.
template <typename T, int W, int kAct, bool kClampAct, bool kPlusOne>
__global__ void __launch_bounds__(kThreads)
glu_fwd_weighted_kernel(const T* __restrict__ gate, const T* __restrict__ up, const void* __restrict__ row_weight,
                        bool weight_f32, T* __restrict__ out, int64_t stride_gate, int64_t stride_up, int64_t n_rows,
                        int64_t chunks_per_row, int64_t width, GluParams p) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t row = i / chunks_per_row;
  if (row >= n_rows) return;
  const int64_t col = (i - row * chunks_per_row) * W;
  const float w = load_row_weight<T>(row_weight, weight_f32, row);
  Chunk<T, W> g, u, o;
  g.load(gate + row * stride_gate + col);
  u.load(up + row * stride_up + col);
#pragma unroll
  for (int k = 0; k < W; ++k) o.v[k] = w * glu_value<kAct, kClampAct, kPlusOne>(g.v[k], u.v[k], p);
  o.store(out + row * width + col);
}

// Its gradient.  grad_out is the gradient of the weighted rows; with act = glu(gate, up) recomputed in fp32:
//   (dgate, dup) = glu_grad(gate, up, w[r] * grad_out[r]),   grad_weight[r] = <grad_out[r], act[r]>.
// kLanes lanes share a row (a power of two up to the wavefront), each taking every kLanes-th 16-byte chunk; the dot
// product is summed in fp32 in a fixed order (per lane in chunk order, then a butterfly over the lanes) and stored as
// fp32; with fp32 weights the stored value is rounded to the operands' dtype first (the gradient of weights that were
// cast to it arrives through that dtype).
template <typename T, int W, int kLanes, int kAct, bool kClampAct, bool kPlusOne>
__global__ void __launch_bounds__(kThreads)
glu_bwd_weighted_kernel(const T* __restrict__ gate, const T* __restrict__ up, const T* __restrict__ grad_out,
                        const void* __restrict__ row_weight, bool weight_f32, T* __restrict__ dgate,
                        T* __restrict__ dup, float* __restrict__ grad_weight, int64_t stride_gate, int64_t stride_up, int64_t stride_dgate,
                        int64_t stride_dup, int64_t n_rows, int chunks_per_row, int64_t width, GluParams p) {
  const int64_t thread = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t row = thread / kLanes;
  const int sub = static_cast<int>(thread % kLanes);
  float dot = 0.f;
  if (row < n_rows) {
    const float w = load_row_weight<T>(row_weight, weight_f32, row);
    // kPer chunks per pass, their loads issued together ahead of the arithmetic (a row of 768 values on 32 lanes is
    // one pass of three)
    constexpr int kPer = 3;
    for (int chunk0 = sub; chunk0 < chunks_per_row; chunk0 += kPer * kLanes) {
      Chunk<T, W> g[kPer], u[kPer], d[kPer];
#pragma unroll
      for (int q = 0; q < kPer; ++q) {
        const int chunk = chunk0 + q * kLanes;
        if (chunk < chunks_per_row) {
          const int64_t col = static_cast<int64_t>(chunk) * W;
          g[q].load(gate + row * stride_gate + col);
          u[q].load(up + row * stride_up + col);
          d[q].load(grad_out + row * width + col);
        }
      }
#pragma unroll
      for (int q = 0; q < kPer; ++q) {
        const int chunk = chunk0 + q * kLanes;
        if (chunk < chunks_per_row) {
          const int64_t col = static_cast<int64_t>(chunk) * W;
          Chunk<T, W> dg, du;
#pragma unroll
          for (int k = 0; k < W; ++k) {
            dot = fmaf(d[q].v[k], glu_value<kAct, kClampAct, kPlusOne>(g[q].v[k], u[q].v[k], p), dot);
            glu_grad<kAct, kClampAct, kPlusOne>(g[q].v[k], u[q].v[k], w * d[q].v[k], p, dg.v[k], du.v[k]);
          }
          dg.store(dgate + row * stride_dgate + col);
          du.store(dup + row * stride_dup + col);
        }
      }
    }
  }
#pragma unroll
  for (int off = kLanes / 2; off > 0; off >>= 1) dot += __shfl_xor(dot, off, HMOE_WAVE);
  if (row < n_rows && sub == 0) grad_weight[row] = weight_f32 ? Elem<T>::round(dot) : dot;
}

struct GluArgs {
  const void *gate, *up, *grad_out;
  void *out, *dgate, *dup;
  int64_t stride_gate, stride_up, stride_dgate, stride_dup, n_rows, width;
  GluParams p;
  bool backward;
  hipStream_t stream;
  uint8_t* q = nullptr;      // forward only: e4m3 panels and scale exponents instead of `out`
  uint8_t* scale = nullptr;
  int64_t out_rows = 0;
  const void* row_weight = nullptr;  // the weighted forms: one gate weight per row, in the operands' dtype
  bool weight_f32 = false;           // ... or fp32, rounded to the operands' dtype by the kernel
  float* grad_weight = nullptr;      // backward: its gradient, fp32 [n_rows]
};

template <typename T, int W, int kAct, bool kClampAct, bool kPlusOne>
void launch(const GluArgs& a) {
  const int64_t chunks = a.width / W;
  const int64_t total = chunks * a.n_rows;
  const dim3 grid(static_cast<unsigned>((total + kThreads - 1) / kThreads)), block(kThreads);
  if (a.q) {
    if constexpr (std::is_same<T, bf16_t>::value && W == 8)
      glu_fwd_quant_kernel<kAct, kClampAct, kPlusOne><<<grid, block, 0, a.stream>>>(
          static_cast<const bf16_t*>(a.gate), static_cast<const bf16_t*>(a.up), a.q, a.scale, a.out_rows,
          a.stride_gate, a.stride_up, a.n_rows, chunks, a.p);
  } else if (a.row_weight && !a.backward) {
    glu_fwd_weighted_kernel<T, W, kAct, kClampAct, kPlusOne><<<grid, block, 0, a.stream>>>(
        static_cast<const T*>(a.gate), static_cast<const T*>(a.up), a.row_weight, a.weight_f32,
        static_cast<T*>(a.out), a.stride_gate, a.stride_up, a.n_rows, chunks, a.width, a.p);
  } else if (a.row_weight) {
    // lanes per row: the power of two (16, 32 or 64) that leaves the fewest idle lane-iterations, larger on a tie
    int lanes = 64;
    int64_t waste = (chunks + 63) / 64 * 64 - chunks;
    for (int cand : {32, 16}) {
      const int64_t w = (chunks + cand - 1) / cand * cand - chunks;
      if (w < waste) lanes = cand, waste = w;
    }
    const int64_t threads = a.n_rows * lanes;
    const dim3 row_grid(static_cast<unsigned>((threads + kThreads - 1) / kThreads));
#define HMOE_GLU_BWD_W(L)                                                                                        \
  glu_bwd_weighted_kernel<T, W, L, kAct, kClampAct, kPlusOne><<<row_grid, block, 0, a.stream>>>(                 \
      static_cast<const T*>(a.gate), static_cast<const T*>(a.up), static_cast<const T*>(a.grad_out),             \
      a.row_weight, a.weight_f32, static_cast<T*>(a.dgate), static_cast<T*>(a.dup), a.grad_weight,               \
      a.stride_gate, a.stride_up, a.stride_dgate, a.stride_dup, a.n_rows, static_cast<int>(chunks), a.width, a.p)
    if (lanes == 64) HMOE_GLU_BWD_W(64);
    else if (lanes == 32) HMOE_GLU_BWD_W(32);
    else HMOE_GLU_BWD_W(16);
#undef HMOE_GLU_BWD_W
  } else if (!a.backward)
    glu_fwd_kernel<T, W, kAct, kClampAct, kPlusOne><<<grid, block, 0, a.stream>>>(
        static_cast<const T*>(a.gate), static_cast<const T*>(a.up), static_cast<T*>(a.out), a.stride_gate,
        a.stride_up, a.n_rows, chunks, a.width, a.p);
  else
    glu_bwd_kernel<T, W, kAct, kClampAct, kPlusOne><<<grid, block, 0, a.stream>>>(
        static_cast<const T*>(a.gate), static_cast<const T*>(a.up), static_cast<const T*>(a.grad_out),
        static_cast<T*>(a.dgate), static_cast<T*>(a.dup), a.stride_gate, a.stride_up, a.stride_dgate, a.stride_dup,
        a.n_rows, chunks, a.width, a.p);
}

template <typename T, int W>
int launch_activation(const GluArgs& a, int activation, int clamp_activated, int up_plus_one) {
  if (activation == HMOE_GLU_SILU) launch<T, W, HMOE_GLU_SILU, false, false>(a);
  else if (activation == HMOE_GLU_GELU_TANH) launch<T, W, HMOE_GLU_GELU_TANH, false, false>(a);
  else if (activation == HMOE_GLU_CLAMPED_SILU) {
    if (clamp_activated && up_plus_one) launch<T, W, HMOE_GLU_CLAMPED_SILU, true, true>(a);
    else if (clamp_activated) launch<T, W, HMOE_GLU_CLAMPED_SILU, true, false>(a);
    else if (up_plus_one) launch<T, W, HMOE_GLU_CLAMPED_SILU, false, true>(a);
    else launch<T, W, HMOE_GLU_CLAMPED_SILU, false, false>(a);
  } else {
    return HMOE_INVALID_ARGUMENT;
  }
  if (hipGetLastError() != hipSuccess) return HMOE_LAUNCH_FAILED;
  return HMOE_OK;
}

int run(const GluArgs& a, int dtype, int activation, int clamp_activated, int up_plus_one) {
  if (a.n_rows < 0 || a.width < 0) return HMOE_INVALID_ARGUMENT;
  if (a.n_rows == 0 || a.width == 0) return HMOE_OK;
  if (!a.gate || !a.up) return HMOE_INVALID_ARGUMENT;
  if (a.backward ? (!a.grad_out || !a.dgate || !a.dup) : (a.q ? !a.scale : !a.out)) return HMOE_INVALID_ARGUMENT;
  if (a.n_rows * a.width / 1 >= (int64_t(1) << 40)) return HMOE_UNSUPPORTED;
  if (a.row_weight && a.backward && !a.grad_weight) return HMOE_INVALID_ARGUMENT;
  if (a.row_weight && a.n_rows >= (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  const int64_t w = dtype == HMOE_BF16 ? 8 : 4;
  bool vec = a.width % w == 0 && a.stride_gate % w == 0 && a.stride_up % w == 0 && aligned16(a.gate) &&
             aligned16(a.up);
  if (a.backward)
    vec = vec && a.stride_dgate % w == 0 && a.stride_dup % w == 0 && aligned16(a.grad_out) && aligned16(a.dgate) &&
          aligned16(a.dup);
  else if (!a.q)
    vec = vec && aligned16(a.out);
  if (a.q) {
    // the quantising form has no scalar fallback: bf16, 16-byte operands, whole 128-value blocks
    if (dtype != HMOE_BF16 || !vec || a.width % 128 || a.out_rows < a.n_rows ||
        (reinterpret_cast<uintptr_t>(a.q) & 7u))
      return HMOE_UNSUPPORTED;
    return launch_activation<bf16_t, 8>(a, activation, clamp_activated, up_plus_one);
  }
  if (dtype == HMOE_BF16)
    return vec ? launch_activation<bf16_t, 8>(a, activation, clamp_activated, up_plus_one)
               : launch_activation<bf16_t, 1>(a, activation, clamp_activated, up_plus_one);
  if (dtype == HMOE_F32)
    return vec ? launch_activation<float, 4>(a, activation, clamp_activated, up_plus_one)
               : launch_activation<float, 1>(a, activation, clamp_activated, up_plus_one);
  return HMOE_UNSUPPORTED;
}

}  // namespace
}  // namespace hmoe

extern "C" {

int hmoe_glu_fwd(const void* gate, const void* up, int64_t stride_gate, int64_t stride_up, int64_t n_rows,
                 int64_t width, int dtype, int activation, float alpha, float limit, int clamp_activated,
                 int up_plus_one, void* out, void* stream) {
  hmoe::GluArgs a{};
  a.gate = gate; a.up = up; a.out = out;
  a.stride_gate = stride_gate; a.stride_up = stride_up; a.n_rows = n_rows; a.width = width;
  a.p = {alpha, limit};
  a.backward = false;
  a.stream = static_cast<hipStream_t>(stream);
  return hmoe::run(a, dtype, activation, clamp_activated, up_plus_one);
}

int hmoe_glu_fwd_quant_fp8(const void* gate, const void* up, int64_t stride_gate, int64_t stride_up, int64_t n_rows,
                           int64_t width, int activation, float alpha, float limit, int clamp_activated,
                           int up_plus_one, uint8_t* q, uint8_t* scale, int64_t out_rows, void* stream) {
  hmoe::GluArgs a{};
  a.gate = gate; a.up = up; a.q = q; a.scale = scale; a.out_rows = out_rows;
  a.stride_gate = stride_gate; a.stride_up = stride_up; a.n_rows = n_rows; a.width = width;
  a.p = {alpha, limit};
  a.backward = false;
  a.stream = static_cast<hipStream_t>(stream);
  if (n_rows > 0 && width > 0 && !q) return HMOE_INVALID_ARGUMENT;
  return hmoe::run(a, HMOE_BF16, activation, clamp_activated, up_plus_one);
}

int hmoe_glu_fwd_weighted(const void* gate, const void* up, int64_t stride_gate, int64_t stride_up,
                          const void* row_weight, int weight_dtype, int64_t n_rows, int64_t width, int dtype,
                          int activation, float alpha, float limit, int clamp_activated, int up_plus_one, void* out,
                          void* stream) {
  if (weight_dtype != dtype && weight_dtype != HMOE_F32) return HMOE_UNSUPPORTED;
  hmoe::GluArgs a{};
  a.gate = gate; a.up = up; a.out = out; a.row_weight = row_weight;
  a.weight_f32 = weight_dtype == HMOE_F32 && dtype != HMOE_F32;
  a.stride_gate = stride_gate; a.stride_up = stride_up; a.n_rows = n_rows; a.width = width;
  a.p = {alpha, limit};
  a.backward = false;
  a.stream = static_cast<hipStream_t>(stream);
  if (n_rows > 0 && width > 0 && !row_weight) return HMOE_INVALID_ARGUMENT;
  return hmoe::run(a, dtype, activation, clamp_activated, up_plus_one);
}

int hmoe_glu_bwd_weighted(const void* gate, const void* up, int64_t stride_gate, int64_t stride_up,
                          const void* grad_out, const void* row_weight, int weight_dtype, int64_t n_rows,
                          int64_t width, int dtype, int activation, float alpha, float limit, int clamp_activated,
                          int up_plus_one, void* dgate, void* dup, int64_t stride_dgate, int64_t stride_dup,
                          float* grad_weight, void* stream) {
  if (weight_dtype != dtype && weight_dtype != HMOE_F32) return HMOE_UNSUPPORTED;
  hmoe::GluArgs a{};
  a.weight_f32 = weight_dtype == HMOE_F32 && dtype != HMOE_F32;
  a.gate = gate; a.up = up; a.grad_out = grad_out; a.dgate = dgate; a.dup = dup;
  a.row_weight = row_weight; a.grad_weight = grad_weight;
  a.stride_gate = stride_gate; a.stride_up = stride_up; a.stride_dgate = stride_dgate; a.stride_dup = stride_dup;
  a.n_rows = n_rows; a.width = width;
  a.p = {alpha, limit};
  a.backward = true;
  a.stream = static_cast<hipStream_t>(stream);
  if (n_rows > 0 && width > 0 && (!row_weight || !grad_weight)) return HMOE_INVALID_ARGUMENT;
  return hmoe::run(a, dtype, activation, clamp_activated, up_plus_one);
}

int hmoe_glu_bwd(const void* gate, const void* up, int64_t stride_gate, int64_t stride_up, const void* grad_out,
                 int64_t n_rows, int64_t width, int dtype, int activation, float alpha, float limit,
                 int clamp_activated, int up_plus_one, void* dgate, void* dup, int64_t stride_dgate,
                 int64_t stride_dup, void* stream) {
  hmoe::GluArgs a{};
  a.gate = gate; a.up = up; a.grad_out = grad_out; a.dgate = dgate; a.dup = dup;
  a.stride_gate = stride_gate; a.stride_up = stride_up; a.stride_dgate = stride_dgate; a.stride_dup = stride_dup;
  a.n_rows = n_rows; a.width = width;
  a.p = {alpha, limit};
  a.backward = true;
  a.stream = static_cast<hipStream_t>(stream);
  return hmoe::run(a, dtype, activation, clamp_activated, up_plus_one);
}

}  // extern "C"
