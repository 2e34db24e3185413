// Token permute / weighted unpermute (combine) / expert-bias gradient for gfx950.  All four kernels stream rows:
// one wavefront per row, 16-byte accesses per lane, fp32 accumulation, one rounding.  No atomics.
//
// Replaces of the reference: tokens.index_select (halo/kernels/moe_permute.py:133-136), _gather_reduce_kernel
// (:17-41), _weighted_unpermute_bwd_kernel (:44-72) and MoEExpertBiasGather.backward's one-hot GEMM (:202-208).
#include "common.h"

#include <type_traits>

namespace hmoe {
namespace {

constexpr int kThreads = 256;
constexpr int kRowsPerBlock = kThreads / HMOE_WAVE;

// W consecutive elements of T held as floats; W is 16 bytes' worth when rows are 16-byte aligned, else 1.
template <typename T, int W>
struct Pack {
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
  // the same load with the non-temporal hint: for rows that are read once and never again
  __device__ __forceinline__ void load_once(const T* p) {
    if constexpr (W == 8 && sizeof(T) == 2) {
      typedef unsigned int word4 __attribute__((ext_vector_type(4)));
      const word4 t = __builtin_nontemporal_load(reinterpret_cast<const word4*>(p));
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(t[i] << 16);
        v[2 * i + 1] = __uint_as_float(t[i] & 0xffff0000u);
      }
    } else {
      load(p);
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

// Raw 16-byte (or one-element) copy chunk: a gather moves bits, it never converts.
template <typename T, int W>
struct Raw {
  using V = typename std::conditional<W == 1, T, uint4>::type;
  V bits;
  __device__ __forceinline__ void load(const T* p) { bits = *reinterpret_cast<const V*>(p); }
  __device__ __forceinline__ void store(T* p) const { *reinterpret_cast<V*>(p) = bits; }
};

// a chunk already in registers, as floats
template <typename T, int W>
__device__ __forceinline__ Pack<T, W> widen(const Raw<T, W>& raw) {
  Pack<T, W> x;
  x.load(reinterpret_cast<const T*>(&raw.bits));
  return x;
}

template <typename T, int W>
__global__ void __launch_bounds__(kThreads)
gather_rows_kernel(const T* __restrict__ src, int64_t src_stride, const int64_t* __restrict__ index,
                   T* __restrict__ out, int64_t n_out, int64_t hidden) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + threadIdx.x / HMOE_WAVE;
  if (row >= n_out) return;
  const T* from = src + index[row] * src_stride;
  T* to = out + row * hidden;
  const int64_t step = static_cast<int64_t>(HMOE_WAVE) * W;
  int64_t c = static_cast<int64_t>(lane_id()) * W;
  for (; c + 3 * step < hidden; c += 4 * step) {  // four loads in flight per lane
    Raw<T, W> a, b, d, e;
    a.load(from + c);
    b.load(from + c + step);
    d.load(from + c + 2 * step);
    e.load(from + c + 3 * step);
    a.store(to + c);
    b.store(to + c + step);
    d.store(to + c + 2 * step);
    e.store(to + c + 3 * step);
  }
  for (; c < hidden; c += step) {
    Raw<T, W> a;
    a.load(from + c);
    a.store(to + c);
  }
}

// out[t] = sum over k of (weight[j] *) src[j], j = inv_map[t][k], in slot order; a slot outside [0, n_src) adds
// nothing.  One wavefront per output row.  kTopK > 0 fixes top_k at compile time: the row's slots and weights are
// read once, and for every 16-byte column chunk the kTopK row loads are issued together before the first is used, so
// a lane keeps kTopK loads in flight instead of one (with one in flight the kernel reached half of the HBM rate).  An
// invalid slot contributes +0.0f, which leaves the fp32 sum exactly as skipping it does: the accumulator starts at
// +0.0f and a sum that started there is never -0.0f.
// kAllValid: the launch is expected to hold valid slots only (there are as many sources as slots: the inverse of a
// permutation), so the kernel is built around the all-valid form, four column chunks per pass at two wavefronts per
// SIMD; a row with an invalid slot is still reduced correctly, one chunk at a time.  Without it such rows take the
// compacted form, and the register budget stays at four wavefronts per SIMD: they have few fetches in flight per
// lane and need the wavefronts.
template <typename T, int W, bool kWeighted, int kTopK, bool kAllValid>
__global__ void __launch_bounds__(kThreads)
gather_reduce_kernel(const T* __restrict__ src, const T* __restrict__ weight, const int64_t* __restrict__ inv_map,
                     T* __restrict__ out, int64_t n_out, int top_k, int64_t n_src, int64_t hidden,
                     const T* __restrict__ addend, int64_t addend_stride, const T* __restrict__ addend_scale) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock +
                      __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / HMOE_WAVE);
  if (row >= n_out) return;
  const int64_t* map = inv_map + row * top_k;
  T* to = out + row * hidden;
  const int64_t step = static_cast<int64_t>(HMOE_WAVE) * W;
  // Optional second term: out[r] = round(round(sum) + round(scale[r] * addend[r])), each rounding where the tensor
  // operations `sum + scale * addend` round (the shared expert's output added to the routed one).
  const T* extra = addend ? addend + row * addend_stride : nullptr;
  const float extra_scale = addend_scale ? Elem<T>::load(addend_scale + row) : 1.f;
  auto finish = [&](Pack<T, W>& acc, const Pack<T, W>& term) {
#pragma clang fp contract(off)  // fp32: the multiple and the sum round separately, as the tensor operations do
    if (extra) {
#pragma unroll
      for (int i = 0; i < W; ++i) {
        float t = term.v[i];
        if (addend_scale) t = Elem<T>::round(__fmul_rn(extra_scale, t));
        acc.v[i] = __fadd_rn(Elem<T>::round(acc.v[i]), t);
      }
    }
  };
  if constexpr (kTopK > 0) {
    const T* from[kTopK];
    float w[kTopK];
    bool valid[kTopK];
#pragma unroll
    for (int k = 0; k < kTopK; ++k) {
      const int64_t j = map[k];
      valid[k] = j >= 0 && j < n_src;
      from[k] = src + (valid[k] ? j : 0) * hidden;
      w[k] = 1.f;
      if constexpr (kWeighted) w[k] = Elem<T>::load(weight + (valid[k] ? j : 0));
    }
    // Two forms of the loop, chosen once per row (the slots are the same for the whole wavefront).  All slots valid:
    // the kTopK fetches go out back to back with nothing between them.  Otherwise an invalid slot is not fetched:
    // on one GPU's share of an expert-parallel layer most of a token's slots belong to other ranks, and eight
    // fetches of which seven are row 0 again cost seven times the useful traffic between the L2 and the CU.  (The
    // branches of the second form keep the compiler from batching the fetches, which costs the first 20 %.)
    bool all_valid = true;
#pragma unroll
    for (int k = 0; k < kTopK; ++k) all_valid = all_valid && valid[k];
    auto reduce_row = [&](auto dense_tag) __attribute__((always_inline)) {
      constexpr bool kDense = decltype(dense_tag)::value;
      int64_t c = static_cast<int64_t>(lane_id()) * W;
      if constexpr (kDense && kTopK <= 8) {
        // kAllValid: four column chunks per pass while the row has them (a whole row of 2048 bf16), then two: 4 * kTopK
        // row fetches in flight per lane at two wavefronts per SIMD (two chunks per pass at three wavefronts: 6 % slower)
        auto pass = [&](auto width_tag) __attribute__((always_inline)) {
          constexpr int kWide = decltype(width_tag)::value;
          Pack<T, W> x[kWide][kTopK], acc[kWide], extra_chunk[kWide];
#pragma unroll
          for (int h = 0; h < kWide; ++h)
#pragma unroll
            for (int k = 0; k < kTopK; ++k) x[h][k].load_once(from[k] + c + h * step);
#pragma unroll
          for (int h = 0; h < kWide; ++h) {
            if (extra) extra_chunk[h].load(extra + c + h * step);
#pragma unroll
            for (int i = 0; i < W; ++i) acc[h].v[i] = 0.f;
#pragma unroll
            for (int k = 0; k < kTopK; ++k) {
#pragma unroll
              for (int i = 0; i < W; ++i) acc[h].v[i] += kWeighted ? x[h][k].v[i] * w[k] : x[h][k].v[i];
            }
            finish(acc[h], extra_chunk[h]);
            acc[h].store(to + c + h * step);
          }
        };
        if constexpr (kAllValid) {
          for (; c + 3 * step < hidden; c += 4 * step) pass(std::integral_constant<int, 4>{});
        }
        for (; c + step < hidden; c += 2 * step) pass(std::integral_constant<int, 2>{});
      }
      for (; c < hidden; c += step) {
        Pack<T, W> x[kTopK], acc, extra_chunk;
#pragma unroll
        for (int k = 0; k < kTopK; ++k) {
          if (kDense || valid[k]) {
            x[k].load_once(from[k] + c);
          } else {
#pragma unroll
            for (int i = 0; i < W; ++i) x[k].v[i] = 0.f;
          }
        }
        if (extra) extra_chunk.load(extra + c);
#pragma unroll
        for (int i = 0; i < W; ++i) acc.v[i] = 0.f;
#pragma unroll
        for (int k = 0; k < kTopK; ++k) {
#pragma unroll
          for (int i = 0; i < W; ++i) {
            const float term = kWeighted ? x[k].v[i] * w[k] : x[k].v[i];
            acc.v[i] += (kDense || valid[k]) ? term : 0.f;
          }
        }
        finish(acc, extra_chunk);
        acc.store(to + c);
      }
    };
    if (all_valid) {
      reduce_row(std::true_type{});
      return;
    }
    if constexpr (kAllValid) {  // the launch was expected to hold valid slots only: a row that does not, the plain way
      reduce_row(std::false_type{});
      return;
    }
    // Some slots are not this rank's (most of them on one GPU's share of an expert-parallel layer).  The valid ones are
    // moved to the front, in slot order (the sum keeps its order; a slot left out adds the +0.0f it added before), and
    // the row is reduced by the loop written for that many sources: every fetch of a pass goes out before the first is
    // used, and a row with few sources takes more column chunks per pass (four for one to three sources, two from
    // four up), so that 4 to 14 fetches are in flight per lane.
    // Everything here is the same for the whole wavefront (scalar registers, one branch).
    const T* live_from[kTopK];
    float live_w[kTopK];
    int n_live = 0;
#pragma unroll
    for (int k = 0; k < kTopK; ++k) {
      live_from[k] = src;
      live_w[k] = 0.f;
    }
#pragma unroll
    for (int k = 0; k < kTopK; ++k) {
      if (valid[k]) {
#pragma unroll
        for (int i = 0; i <= k; ++i) {  // slot k lands at position n_live <= k
          if (i == n_live) {
            live_from[i] = from[k];
            live_w[i] = w[k];
          }
        }
        ++n_live;
      }
    }
    auto reduce_live = [&](auto count_tag, auto chunks_tag) __attribute__((always_inline)) {
      constexpr int kLive = decltype(count_tag)::value, kChunks = decltype(chunks_tag)::value;
      int64_t c = static_cast<int64_t>(lane_id()) * W;
      auto pass = [&](auto width_tag) __attribute__((always_inline)) {
        constexpr int kWide = decltype(width_tag)::value;
        Pack<T, W> x[kWide][kLive > 0 ? kLive : 1], acc[kWide], extra_chunk[kWide];
#pragma unroll
        for (int h = 0; h < kWide; ++h)
#pragma unroll
          for (int k = 0; k < kLive; ++k) x[h][k].load_once(live_from[k] + c + h * step);
#pragma unroll
        for (int h = 0; h < kWide; ++h) {
          if (extra) extra_chunk[h].load(extra + c + h * step);
#pragma unroll
          for (int i = 0; i < W; ++i) acc[h].v[i] = 0.f;
#pragma unroll
          for (int k = 0; k < kLive; ++k) {
#pragma unroll
            for (int i = 0; i < W; ++i) acc[h].v[i] += kWeighted ? x[h][k].v[i] * live_w[k] : x[h][k].v[i];
          }
          finish(acc[h], extra_chunk[h]);
          acc[h].store(to + c + h * step);
        }
      };
      for (; c + (kChunks - 1) * step < hidden; c += kChunks * step) pass(std::integral_constant<int, kChunks>{});
      if constexpr (kChunks > 2) {
        for (; c + step < hidden; c += 2 * step) pass(std::integral_constant<int, 2>{});
      }
      for (; c < hidden; c += step) pass(std::integral_constant<int, 1>{});
    };
    using std::integral_constant;
    switch (n_live) {
      case 0: reduce_live(integral_constant<int, 0>{}, integral_constant<int, 4>{}); break;
      case 1: reduce_live(integral_constant<int, 1>{}, integral_constant<int, 4>{}); break;
      case 2: reduce_live(integral_constant<int, 2>{}, integral_constant<int, 4>{}); break;
      case 3: reduce_live(integral_constant<int, (kTopK >= 3 ? 3 : 1)>{}, integral_constant<int, 4>{}); break;
      case 4: reduce_live(integral_constant<int, (kTopK >= 4 ? 4 : 1)>{}, integral_constant<int, 2>{}); break;
      case 5: reduce_live(integral_constant<int, (kTopK >= 5 ? 5 : 1)>{}, integral_constant<int, 2>{}); break;
      case 6: reduce_live(integral_constant<int, (kTopK >= 6 ? 6 : 1)>{}, integral_constant<int, 2>{}); break;
      case 7: reduce_live(integral_constant<int, (kTopK >= 7 ? 7 : 1)>{}, integral_constant<int, 2>{}); break;
      default: reduce_row(std::false_type{}); break;
    }
  } else {
    for (int64_t c = static_cast<int64_t>(lane_id()) * W; c < hidden; c += step) {
      Pack<T, W> acc, extra_chunk;
      if (extra) extra_chunk.load(extra + c);
#pragma unroll
      for (int i = 0; i < W; ++i) acc.v[i] = 0.f;
      for (int k = 0; k < top_k; ++k) {
        const int64_t j = map[k];
        if (j >= 0 && j < n_src) {
          Pack<T, W> x;
          x.load(src + j * hidden + c);
          if constexpr (kWeighted) {
            const float w = Elem<T>::load(weight + j);
#pragma unroll
            for (int i = 0; i < W; ++i) acc.v[i] += x.v[i] * w;
          } else {
#pragma unroll
            for (int i = 0; i < W; ++i) acc.v[i] += x.v[i];
          }
        }
      }
      finish(acc, extra_chunk);
      acc.store(to + c);
    }
  }
}

template <typename T, int W>
__global__ void __launch_bounds__(kThreads)
unpermute_bwd_kernel(const T* __restrict__ grad_out, int64_t grad_stride, const T* __restrict__ expert_out,
                     const T* __restrict__ weights, const int64_t* __restrict__ token_idx,
                     T* __restrict__ grad_expert, float* __restrict__ grad_weights, int64_t n_sorted,
                     int64_t hidden) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + threadIdx.x / HMOE_WAVE;
  if (row >= n_sorted) return;
  const T* g = grad_out + token_idx[row] * grad_stride;
  const float w = Elem<T>::load(weights + row);
  const bool want_dot = expert_out != nullptr && grad_weights != nullptr;
  const T* y = want_dot ? expert_out + row * hidden : nullptr;
  T* to = grad_expert + row * hidden;
  float dot = 0.f;
  const int64_t step = static_cast<int64_t>(HMOE_WAVE) * W;
  for (int64_t c = static_cast<int64_t>(lane_id()) * W; c < hidden; c += step) {
    Pack<T, W> gv, ov;
    gv.load(g + c);
    if (want_dot) {
      Pack<T, W> yv;
      yv.load(y + c);
#pragma unroll
      for (int i = 0; i < W; ++i) dot += gv.v[i] * yv.v[i];
    }
#pragma unroll
    for (int i = 0; i < W; ++i) ov.v[i] = gv.v[i] * w;
    ov.store(to + c);
  }
  if (want_dot) {
    dot = wave_sum(dot);
    if (lane_id() == 0) grad_weights[row] = dot;
  }
}

// grid (num_experts, column chunks of 8 W columns).  A workgroup of 16 wavefronts sums its expert's contiguous row
// range (found by bisection on the sorted ids) over its columns: eight lanes cover a row's 8 W columns with one 16-byte
// load each, a wavefront takes eight rows per load, four loads in flight, and the wavefronts stride the range.  The
// partial sums meet by lane exchange inside a wavefront and through LDS across wavefronts, in a fixed order.  Narrow
// column chunks and many wavefronts per expert because expert loads can be very uneven: with one 4-wavefront workgroup
// per (expert, 512 columns) an expert holding a quarter of 65536 rows took 1.7 ms on its own.
constexpr int kColsumThreads = 1024;
constexpr int kColsumWaves = kColsumThreads / HMOE_WAVE;
constexpr int kColsumLanesPerRow = 8;
constexpr int kColsumRowsPerLoad = HMOE_WAVE / kColsumLanesPerRow;

template <typename T, int W>
__global__ void __launch_bounds__(kColsumThreads)
expert_colsum_kernel(const T* __restrict__ grad_out, const int64_t* __restrict__ eids, T* __restrict__ grad_bias,
                     int64_t n_rows, int64_t width) {
  __shared__ float partial[kColsumWaves][kColsumLanesPerRow * W];
  const int e = blockIdx.x;
  auto lower_bound = [&](int64_t key) {
    int64_t lo = 0, hi = n_rows;
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      if (eids[mid] < key) lo = mid + 1; else hi = mid;
    }
    return lo;
  };
  const int64_t begin = lower_bound(e), end = lower_bound(static_cast<int64_t>(e) + 1);
  const int wave = threadIdx.x / HMOE_WAVE;
  const int sub = lane_id() / kColsumLanesPerRow, part = lane_id() % kColsumLanesPerRow;
  const int64_t c = (static_cast<int64_t>(blockIdx.y) * kColsumLanesPerRow + part) * W;
  Pack<T, W> acc;
#pragma unroll
  for (int i = 0; i < W; ++i) acc.v[i] = 0.f;
  if (c < width) {
    constexpr int64_t kStride = static_cast<int64_t>(kColsumWaves) * kColsumRowsPerLoad;
    const T* col = grad_out + c;
    int64_t r = begin + wave * kColsumRowsPerLoad + sub;
    for (; r + 3 * kStride < end; r += 4 * kStride) {
      Pack<T, W> x0, x1, x2, x3;
      x0.load(col + r * width);
      x1.load(col + (r + kStride) * width);
      x2.load(col + (r + 2 * kStride) * width);
      x3.load(col + (r + 3 * kStride) * width);
#pragma unroll
      for (int i = 0; i < W; ++i) acc.v[i] += (x0.v[i] + x1.v[i]) + (x2.v[i] + x3.v[i]);
    }
    for (; r < end; r += kStride) {
      Pack<T, W> x;
      x.load(col + r * width);
#pragma unroll
      for (int i = 0; i < W; ++i) acc.v[i] += x.v[i];
    }
  }
#pragma unroll
  for (int off = kColsumLanesPerRow; off < HMOE_WAVE; off <<= 1) {
#pragma unroll
    for (int i = 0; i < W; ++i) acc.v[i] += __shfl_xor(acc.v[i], off, HMOE_WAVE);
  }
  if (sub == 0) {
#pragma unroll
    for (int i = 0; i < W; ++i) partial[wave][part * W + i] = acc.v[i];
  }
  __syncthreads();
  if (wave == 0 && sub == 0 && c < width) {
    Pack<T, W> sum;
#pragma unroll
    for (int i = 0; i < W; ++i) {
      float total = 0.f;
#pragma unroll
      for (int w = 0; w < kColsumWaves; ++w) total += partial[w][part * W + i];
      sum.v[i] = total;
    }
    sum.store(grad_bias + static_cast<int64_t>(e) * width + c);
  }
}

// The same sums in two launches, for 16-byte-aligned rows.  Expert loads can be very uneven (one expert holding a
// quarter of the rows), and a workgroup per (expert, column chunk) then leaves most of the chip waiting for that
// expert's few workgroups; here the rows are cut into blocks of 128 whatever expert they belong to.
//   partial: grid (column chunks, row blocks).  A thread owns W columns and walks the block's rows, eight row loads in
//            flight; the threads of a workgroup read a row side by side, so nothing is exchanged between lanes.  A
//            row's expert id is the same for every thread (a scalar load); when it changes, the sum so far goes to
//            row b + e of the fp32 workspace [row blocks + experts, width]: along the sorted rows the pairs
//            (block, expert) form a staircase, so b + e names each pair once.
//   final:   grid (experts, column chunks): expert e's row range by a 64-way search of the sorted ids, then the
//            partial rows of the blocks it spans: four wavefronts add a quarter of them each in block order, the four
//            sums are added in wavefront order and rounded once.
// The order of every addition is fixed, so the result is reproducible bit for bit.
constexpr int kColsumBlockRows = 128;
constexpr int kPartialLoads = 8;
static_assert(kColsumBlockRows % kPartialLoads == 0, "a block's rows come in whole batches");

template <typename T, int W>
__global__ void __launch_bounds__(1024)
expert_colsum_partial_kernel(const T* __restrict__ grad_out, const int64_t* __restrict__ eids,
                             float* __restrict__ partial, int64_t n_rows, int64_t width, int num_experts) {
  const int64_t blk = blockIdx.y;
  const int64_t row0 = blk * kColsumBlockRows;
  const int64_t row_end = row0 + kColsumBlockRows < n_rows ? row0 + kColsumBlockRows : n_rows;
  const int64_t c = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * W;
  if (c >= width) return;
  const T* col = grad_out + c;
  float acc[W];
#pragma unroll
  for (int i = 0; i < W; ++i) acc[i] = 0.f;
  int64_t current = -1;
  auto flush = [&]() {
    if (current >= 0 && current < num_experts) {
      float4* to = reinterpret_cast<float4*>(partial + (blk + current) * width + c);  // W is 4 or 8: 16-byte aligned
#pragma unroll
      for (int i = 0; i < W / 4; ++i) to[i] = make_float4(acc[4 * i], acc[4 * i + 1], acc[4 * i + 2], acc[4 * i + 3]);
    }
  };
  for (int64_t r = row0; r < row_end; r += kPartialLoads) {
    // all the batch's loads go out before the first is used: past the block's end they repeat its last row, whose
    // values are then left out below
    Raw<T, W> raw[kPartialLoads];
    int64_t id[kPartialLoads];
#pragma unroll
    for (int t = 0; t < kPartialLoads; ++t) {
      const int64_t row = r + t < row_end ? r + t : row_end - 1;  // the same for every thread
      id[t] = eids[row];
      raw[t].load(col + row * width);
    }
#pragma unroll
    for (int t = 0; t < kPartialLoads; ++t) {
      if (r + t >= row_end) break;
      if (id[t] != current) {
        flush();
        current = id[t];
#pragma unroll
        for (int i = 0; i < W; ++i) acc[i] = 0.f;
      }
      const Pack<T, W> x = widen(raw[t]);
#pragma unroll
      for (int i = 0; i < W; ++i) acc[i] += x.v[i];
    }
  }
  flush();
}

// First index of the sorted ids that holds `key` or more, found by the wavefront together: 64 probes a round.
__device__ __forceinline__ int64_t wave_lower_bound(const int64_t* __restrict__ ids, int64_t n, int64_t key) {
  int64_t lo = 0, len = n;  // the answer lies in [lo, lo + len]
  while (len > 0) {
    const int64_t step = (len + HMOE_WAVE - 1) / HMOE_WAVE;
    int64_t last = (static_cast<int64_t>(lane_id()) + 1) * step;  // this lane's chunk ends before lo + last
    if (last > len) last = len;
    const bool below = ids[lo + last - 1] < key;
    const int chunks_below = __popcll(__ballot(below));
    if (chunks_below * step >= len) return lo + len;
    lo += chunks_below * step;
    const int64_t rest = len - chunks_below * step;
    len = (rest < step ? rest : step) - 1;  // the chunk's last id is `key` or more: the answer is it or before it
  }
  return lo;
}

// W is 4 or 8.  Four wavefronts share a column chunk of 64 W columns; each adds a quarter of the expert's blocks in
// block order, and the four sums are added in wavefront order.
template <typename T, int W>
__global__ void __launch_bounds__(256)
expert_colsum_final_kernel(const float* __restrict__ partial, const int64_t* __restrict__ eids,
                           T* __restrict__ grad_bias, int64_t n_rows, int64_t width) {
  __shared__ float quarter[4][HMOE_WAVE * W];
  const int e = blockIdx.x;
  const int wave = threadIdx.x / HMOE_WAVE;
  const int64_t begin = wave_lower_bound(eids, n_rows, e);
  const int64_t end = wave_lower_bound(eids, n_rows, static_cast<int64_t>(e) + 1);
  const int64_t c = (static_cast<int64_t>(blockIdx.y) * HMOE_WAVE + lane_id()) * W;
  float sum[W];
#pragma unroll
  for (int i = 0; i < W; ++i) sum[i] = 0.f;
  if (begin < end && c < width) {
    const int64_t b_first = begin / kColsumBlockRows, b_last = (end - 1) / kColsumBlockRows + 1;
    const int64_t per_wave = (b_last - b_first + 3) / 4;
    const int64_t b0 = b_first + wave * per_wave;
    const int64_t b_end = b0 + per_wave < b_last ? b0 + per_wave : b_last;
    for (int64_t b = b0; b < b_end; b += 8) {  // eight partial rows in flight
      float4 part[8][W / 4];
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const float4* from = reinterpret_cast<const float4*>(partial + (b + t + e) * width + c);
#pragma unroll
        for (int i = 0; i < W / 4; ++i) part[t][i] = b + t < b_end ? from[i] : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        if (b + t < b_end) {
#pragma unroll
          for (int i = 0; i < W / 4; ++i) {
            sum[4 * i] += part[t][i].x;
            sum[4 * i + 1] += part[t][i].y;
            sum[4 * i + 2] += part[t][i].z;
            sum[4 * i + 3] += part[t][i].w;
          }
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < W; ++i) quarter[wave][lane_id() * W + i] = sum[i];
  __syncthreads();
  if (wave == 0 && c < width) {
    Pack<T, W> total;
#pragma unroll
    for (int i = 0; i < W; ++i)
      total.v[i] = ((quarter[0][lane_id() * W + i] + quarter[1][lane_id() * W + i]) + quarter[2][lane_id() * W + i]) +
                   quarter[3][lane_id() * W + i];
    total.store(grad_bias + static_cast<int64_t>(e) * width + c);
  }
}

template <typename T>
bool rows_vectorizable(int64_t hidden, std::initializer_list<int64_t> strides, std::initializer_list<const void*> ptrs) {
  constexpr int W = 16 / sizeof(T);
  if (hidden % W) return false;
  for (int64_t s : strides)
    if (s % W) return false;
  for (const void* p : ptrs)
    if (p && !aligned16(p)) return false;
  return true;
}

dim3 row_grid(int64_t rows) { return dim3(static_cast<unsigned>((rows + kRowsPerBlock - 1) / kRowsPerBlock)); }

}  // namespace
}  // namespace hmoe

using namespace hmoe;

#define HMOE_DISPATCH_ROWS(DTYPE, VEC_OK, CALL)                      \
  if ((DTYPE) == HMOE_BF16) {                                        \
    using T = bf16_t;                                                \
    if (VEC_OK) { constexpr int W = 8; CALL; } else { constexpr int W = 1; CALL; } \
  } else if ((DTYPE) == HMOE_F32) {                                  \
    using T = float;                                                 \
    if (VEC_OK) { constexpr int W = 4; CALL; } else { constexpr int W = 1; CALL; } \
  } else {                                                           \
    return HMOE_UNSUPPORTED;                                         \
  }

extern "C" {

int hmoe_gather_rows(const void* src, int64_t src_row_stride, const int64_t* index, int64_t n_out, int64_t hidden,
                     int dtype, void* out, void* stream) {
  if (n_out < 0 || hidden < 0 || src_row_stride < 0) return HMOE_INVALID_ARGUMENT;
  if (n_out == 0 || hidden == 0) return HMOE_OK;
  if (!src || !index || !out) return HMOE_INVALID_ARGUMENT;
  if (n_out > (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool vec = dtype == HMOE_BF16 ? rows_vectorizable<bf16_t>(hidden, {src_row_stride}, {src, out})
                                      : rows_vectorizable<float>(hidden, {src_row_stride}, {src, out});
  HMOE_DISPATCH_ROWS(dtype, vec,
                     (gather_rows_kernel<T, W><<<row_grid(n_out), dim3(kThreads), 0, s>>>(
                         static_cast<const T*>(src), src_row_stride, index, static_cast<T*>(out), n_out, hidden)));
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

int hmoe_gather_reduce_add(const void* src, const void* weight, const int64_t* inv_map, int64_t n_out, int top_k,
                           int64_t n_src, int64_t hidden, int dtype, const void* addend, int64_t addend_row_stride,
                           const void* addend_scale, void* out, void* stream) {
  if (n_out < 0 || hidden < 0 || n_src < 0 || top_k < 0 || addend_row_stride < 0) return HMOE_INVALID_ARGUMENT;
  if (n_out == 0 || hidden == 0) return HMOE_OK;
  if (!out || (top_k > 0 && !inv_map) || (n_src > 0 && !src)) return HMOE_INVALID_ARGUMENT;
  if (addend_scale && !addend) return HMOE_INVALID_ARGUMENT;
  if (addend && addend_row_stride < hidden) return HMOE_INVALID_ARGUMENT;
  if (n_out > (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool vec = dtype == HMOE_BF16 ? rows_vectorizable<bf16_t>(hidden, {addend_row_stride}, {src, out, addend})
                                      : rows_vectorizable<float>(hidden, {addend_row_stride}, {src, out, addend});
  // n_src == 0: every slot is invalid and the rows come out as zeros; the generic kernel never touches src then
  const int fixed = n_src > 0 && (top_k == 8 || top_k == 4 || top_k == 2) ? top_k : 0;
  // as many sources as slots: the inverse of a permutation, every slot valid (a hint: either kernel is correct for
  // any inv_map)
  const bool wide = fixed > 0 && n_src == n_out * top_k;
#define HMOE_GATHER_REDUCE_AS(WEIGHTED, TOPK, WIDE)                                                               \
  HMOE_DISPATCH_ROWS(dtype, vec,                                                                                  \
                     (gather_reduce_kernel<T, W, WEIGHTED, TOPK, WIDE><<<row_grid(n_out), dim3(kThreads), 0, s>>>( \
                         static_cast<const T*>(src), static_cast<const T*>(weight), inv_map, static_cast<T*>(out), \
                         n_out, top_k, n_src, hidden, static_cast<const T*>(addend), addend_row_stride,           \
                         static_cast<const T*>(addend_scale))))
#define HMOE_GATHER_REDUCE(WEIGHTED, TOPK)                    \
  if (wide && TOPK > 0) {                                     \
    HMOE_GATHER_REDUCE_AS(WEIGHTED, TOPK, (TOPK > 0));        \
  } else {                                                    \
    HMOE_GATHER_REDUCE_AS(WEIGHTED, TOPK, false);             \
  }
  if (weight) {
    if (fixed == 8) { HMOE_GATHER_REDUCE(true, 8); }
    else if (fixed == 4) { HMOE_GATHER_REDUCE(true, 4); }
    else if (fixed == 2) { HMOE_GATHER_REDUCE(true, 2); }
    else { HMOE_GATHER_REDUCE(true, 0); }
  } else {
    if (fixed == 8) { HMOE_GATHER_REDUCE(false, 8); }
    else if (fixed == 4) { HMOE_GATHER_REDUCE(false, 4); }
    else if (fixed == 2) { HMOE_GATHER_REDUCE(false, 2); }
    else { HMOE_GATHER_REDUCE(false, 0); }
  }
#undef HMOE_GATHER_REDUCE
#undef HMOE_GATHER_REDUCE_AS
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

int hmoe_gather_reduce(const void* src, const void* weight, const int64_t* inv_map, int64_t n_out, int top_k,
                       int64_t n_src, int64_t hidden, int dtype, void* out, void* stream) {
  return hmoe_gather_reduce_add(src, weight, inv_map, n_out, top_k, n_src, hidden, dtype, nullptr, 0, nullptr, out,
                                stream);
}

int hmoe_unpermute_bwd(const void* grad_out, int64_t grad_out_row_stride, const void* expert_out,
                       const void* weights, const int64_t* token_idx, int64_t n_sorted, int64_t hidden, int dtype,
                       void* grad_expert, float* grad_weights, void* stream) {
  if (n_sorted < 0 || hidden < 0 || grad_out_row_stride < 0) return HMOE_INVALID_ARGUMENT;
  if (n_sorted == 0) return HMOE_OK;
  if (!grad_out || !weights || !token_idx || !grad_expert) return HMOE_INVALID_ARGUMENT;
  if ((expert_out == nullptr) != (grad_weights == nullptr)) return HMOE_INVALID_ARGUMENT;
  if (n_sorted > (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool vec = dtype == HMOE_BF16
                       ? rows_vectorizable<bf16_t>(hidden, {grad_out_row_stride}, {grad_out, expert_out, grad_expert})
                       : rows_vectorizable<float>(hidden, {grad_out_row_stride}, {grad_out, expert_out, grad_expert});
  HMOE_DISPATCH_ROWS(dtype, vec,
                     (unpermute_bwd_kernel<T, W><<<row_grid(n_sorted), dim3(kThreads), 0, s>>>(
                         static_cast<const T*>(grad_out), grad_out_row_stride, static_cast<const T*>(expert_out),
                         static_cast<const T*>(weights), token_idx, static_cast<T*>(grad_expert), grad_weights,
                         n_sorted, hidden)));
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

int64_t hmoe_expert_colsum_workspace_bytes(int64_t n_rows, int64_t width, int num_experts) {
  if (n_rows < 0 || width < 0 || num_experts < 0) return 0;
  const int64_t blocks = (n_rows + kColsumBlockRows - 1) / kColsumBlockRows;
  return (blocks + num_experts) * width * static_cast<int64_t>(sizeof(float));
}

int hmoe_expert_colsum(const void* grad_out, const int64_t* eids, int64_t n_rows, int64_t width, int num_experts,
                       int dtype, void* grad_bias, void* workspace, void* stream) {
  if (n_rows < 0 || width < 0 || num_experts < 0) return HMOE_INVALID_ARGUMENT;
  if (num_experts == 0 || width == 0) return HMOE_OK;
  if (!grad_bias || (n_rows > 0 && (!grad_out || !eids))) return HMOE_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool vec = dtype == HMOE_BF16 ? rows_vectorizable<bf16_t>(width, {}, {grad_out, grad_bias})
                                      : rows_vectorizable<float>(width, {}, {grad_out, grad_bias});
  if (vec && workspace != nullptr && aligned16(workspace)) {
    const unsigned blocks = static_cast<unsigned>((n_rows + kColsumBlockRows - 1) / kColsumBlockRows);
    float* partial = static_cast<float*>(workspace);
    if (dtype == HMOE_BF16) {
      using T = bf16_t;
      constexpr int W = 8;
      const int64_t packs = width / W;
      const unsigned threads = packs >= 1024 ? 1024u : static_cast<unsigned>((packs + HMOE_WAVE - 1) / HMOE_WAVE * HMOE_WAVE);
      if (blocks > 0)
        expert_colsum_partial_kernel<T, W><<<dim3(static_cast<unsigned>((packs + threads - 1) / threads), blocks),
                                             dim3(threads), 0, s>>>(
            static_cast<const T*>(grad_out), eids, partial, n_rows, width, num_experts);
      expert_colsum_final_kernel<T, W><<<dim3(num_experts, (width + HMOE_WAVE * W - 1) / (HMOE_WAVE * W)), dim3(256), 0, s>>>(
          partial, eids, static_cast<T*>(grad_bias), n_rows, width);
    } else if (dtype == HMOE_F32) {
      using T = float;
      constexpr int W = 4;
      const int64_t packs = width / W;
      const unsigned threads = packs >= 1024 ? 1024u : static_cast<unsigned>((packs + HMOE_WAVE - 1) / HMOE_WAVE * HMOE_WAVE);
      if (blocks > 0)
        expert_colsum_partial_kernel<T, W><<<dim3(static_cast<unsigned>((packs + threads - 1) / threads), blocks),
                                             dim3(threads), 0, s>>>(
            static_cast<const T*>(grad_out), eids, partial, n_rows, width, num_experts);
      expert_colsum_final_kernel<T, W><<<dim3(num_experts, (width + HMOE_WAVE * W - 1) / (HMOE_WAVE * W)), dim3(256), 0, s>>>(
          partial, eids, static_cast<T*>(grad_bias), n_rows, width);
    } else {
      return HMOE_UNSUPPORTED;
    }
    HMOE_CHECK_LAUNCH();
    return HMOE_OK;
  }
  // rows that are not 16-byte aligned, or no workspace: one workgroup per (expert, column chunk)
  HMOE_DISPATCH_ROWS(dtype, vec,
                     (expert_colsum_kernel<T, W><<<dim3(num_experts, (width + kColsumLanesPerRow * W - 1) /
                                                                         (kColsumLanesPerRow * W)),
                                                  dim3(kColsumThreads), 0, s>>>(
                         static_cast<const T*>(grad_out), eids, static_cast<T*>(grad_bias), n_rows, width)));
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

}  // extern "C"
