// Expert-sorted routing for the grouped-GEMM MoE compute on gfx950: a stable counting sort in three launches
// (per-block histogram, one-workgroup scan, placement), no atomics on global memory and no host readback.
//
// Replaces halo/kernels/moe_route_sort.py:40-125 (Triton histogram / scan / place) of the reference.
//
// Layout: the slots (slot = row * top_k + k) are cut into sort blocks of whole rows, at most kBlockSlots slots each.
//   hist[b][e]   (workspace, i32)  number of valid slots of block b routed to expert e; the scan overwrites it with
//   start[b][e]                    the sorted position of block b's first expert-e slot.
// Placement walks a block's slots in slot order, one wavefront of 64 slots at a time: lanes routed to the same expert
// find each other with one ballot per expert-id bit, rank themselves with a popcount of the lower lanes, and the
// lowest lane advances the expert's running position kept in LDS.  Order within an expert is slot order, so the sort
// is stable and bit-reproducible.
//
// Also here: the sync-free histogram behind hmoe_bincount (halo/kernels/histogram.py:9-18 of the reference), whose
// many-workgroup form adds per-workgroup counts with vector atomics (integer sums: exact in any order).
#include "common.h"

#include <atomic>

namespace hmoe {
namespace {

// Scratch of hmoe_route_sort_static: the per-block histogram / start table of the sort, held by the library instead of
// a caller's workspace.  Each GPU the library runs on holds its own copy until the process ends.  In host code the
// array's name is only a handle: its device address comes from hipGetSymbolAddress (static_scratch below).
constexpr int64_t kStaticScratchInts = int64_t(1) << 20;  // 4 MiB: n_blocks * num_local_experts entries at most
// (`used`: no kernel names the array, the sort's kernels take its address as an argument)
static __device__ __align__(256) __attribute__((used)) int32_t scratch[kStaticScratchInts];

constexpr int kMaxDevices = 64;
std::atomic<int32_t*> g_scratch_address[kMaxDevices];  // per device, resolved on the first call with that device current

// The address of the current device's copy of `scratch`, or null with `status` set.
int32_t* static_scratch(int& status) {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
    status = HMOE_UNSUPPORTED;
    return nullptr;
  }
  int32_t* address = g_scratch_address[device].load(std::memory_order_acquire);
  if (address == nullptr) {
    void* resolved = nullptr;
    if (hipGetSymbolAddress(&resolved, HIP_SYMBOL(scratch)) != hipSuccess || resolved == nullptr) {
      status = HMOE_LAUNCH_FAILED;
      return nullptr;
    }
    address = static_cast<int32_t*>(resolved);
    g_scratch_address[device].store(address, std::memory_order_release);  // two first callers resolve the same value
  }
  status = HMOE_OK;
  return address;
}

constexpr int kBlockSlots = 1024;   // slots per sort block (whole rows)
constexpr int kPlaceThreads = 256;  // 4 wavefronts
constexpr int kScanThreads = 1024;
constexpr int kMaxExperts = 1024;   // scan keeps one column per thread

template <typename IdT>
__global__ void __launch_bounds__(kPlaceThreads)
histogram_kernel(const IdT* __restrict__ experts, int32_t* __restrict__ hist, int64_t n_slots, int slots_per_block,
                 int n_local) {
  extern __shared__ int32_t counts[];
  for (int e = threadIdx.x; e < n_local; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  const int64_t base = static_cast<int64_t>(blockIdx.x) * slots_per_block;
  for (int i = threadIdx.x; i < slots_per_block; i += blockDim.x) {
    const int64_t slot = base + i;
    if (slot < n_slots) {
      const int64_t e = static_cast<int64_t>(experts[slot]);
      if (e >= 0 && e < n_local) atomicAdd(&counts[e], 1);  // LDS atomic: integer adds commute, result is exact
    }
  }
  __syncthreads();
  int32_t* row = hist + static_cast<int64_t>(blockIdx.x) * n_local;
  for (int e = threadIdx.x; e < n_local; e += blockDim.x) row[e] = counts[e];
}

// One workgroup.  Thread t owns expert column e = t % e_pad and the block segment seg = t / e_pad.
__global__ void __launch_bounds__(kScanThreads)
scan_kernel(int32_t* __restrict__ hist, int32_t* __restrict__ offs, int32_t* __restrict__ ok, int n_blocks,
            int n_local, int e_pad, int64_t n_valid) {
  __shared__ int32_t part[kScanThreads];  // [seg][e_pad]
  __shared__ int32_t incl[kMaxExperts];
  __shared__ int32_t total[kMaxExperts];
  const int t = threadIdx.x;
  const int e = t % e_pad;
  const int seg = t / e_pad;
  const int segs = kScanThreads / e_pad;
  const int seg_len = (n_blocks + segs - 1) / segs;
  const int b0 = min(seg * seg_len, n_blocks);
  const int b1 = min(b0 + seg_len, n_blocks);
  int32_t sum = 0;
  if (e < n_local)
    for (int b = b0; b < b1; ++b) sum += hist[static_cast<int64_t>(b) * n_local + e];
  part[seg * e_pad + e] = sum;
  __syncthreads();
  if (t < e_pad) {
    int32_t running = 0;
    for (int s = 0; s < segs; ++s) {
      const int32_t v = part[s * e_pad + t];
      part[s * e_pad + t] = running;
      running += v;
    }
    total[t] = running;
    incl[t] = running;
  }
  __syncthreads();
  // inclusive scan over the expert columns (e_pad <= 1024 entries)
  for (int off = 1; off < e_pad; off <<= 1) {
    int32_t v = 0;
    if (t < e_pad) v = incl[t] + (t >= off ? incl[t - off] : 0);
    __syncthreads();
    if (t < e_pad) incl[t] = v;
    __syncthreads();
  }
  if (t < n_local) offs[t] = incl[t];
  if (t == 0) ok[0] = (static_cast<int64_t>(incl[e_pad - 1]) == n_valid) ? 1 : 0;
  if (e < n_local) {
    int32_t running = incl[e] - total[e] + part[seg * e_pad + e];
    for (int b = b0; b < b1; ++b) {
      const int64_t at = static_cast<int64_t>(b) * n_local + e;
      const int32_t h = hist[at];
      hist[at] = running;
      running += h;
    }
  }
}

template <typename IdT, typename WT>
__global__ void __launch_bounds__(kPlaceThreads)
place_kernel(const IdT* __restrict__ experts, const WT* __restrict__ weights, const int32_t* __restrict__ start,
             const int32_t* __restrict__ ok, int64_t* __restrict__ sorted_token, WT* __restrict__ sorted_weight,
             IdT* __restrict__ sorted_expert, int64_t* __restrict__ inv_map, int32_t* __restrict__ dest,
             int64_t n_slots, int slots_per_block, int top_k, int n_local, int id_bits, int64_t n_valid) {
  extern __shared__ int32_t lds[];
  int32_t* position = lds;           // [n_local] running sorted position of each expert within this block
  int32_t* slot_dest = lds + n_local;  // [slots_per_block]
  if (ok[0] == 0) return;            // a wrong total would write past the outputs the host count sized
  const int64_t base = static_cast<int64_t>(blockIdx.x) * slots_per_block;
  const int32_t* my_start = start + static_cast<int64_t>(blockIdx.x) * n_local;
  for (int e = threadIdx.x; e < n_local; e += blockDim.x) position[e] = my_start[e];
  __syncthreads();
  const int lane = lane_id();
  const int wave = threadIdx.x / HMOE_WAVE;
  constexpr int kWaves = kPlaceThreads / HMOE_WAVE;
  const uint64_t lower = (1ull << lane) - 1ull;
  for (int chunk = 0; chunk < slots_per_block; chunk += kPlaceThreads) {
    const int local = chunk + threadIdx.x;
    const int64_t slot = base + local;
    const bool exists = local < slots_per_block && slot < n_slots;
    int64_t id = -1;
    if (exists) id = static_cast<int64_t>(experts[slot]);
    const bool valid = exists && id >= 0 && id < n_local;
    const int e = valid ? static_cast<int>(id) : 0;
    // lanes of this wavefront routed to the same expert
    uint64_t peers = __ballot(valid);
    for (int bit = 0; bit < id_bits; ++bit) {
      const bool set = (e >> bit) & 1;
      const uint64_t with_bit = __ballot(valid && set);
      peers &= set ? with_bit : ~with_bit;
    }
    const int rank = __popcll(peers & lower);
    const int count = __popcll(peers);
    int32_t pos = static_cast<int32_t>(n_valid);
    for (int w = 0; w < kWaves; ++w) {  // wavefronts in slot order
      if (w == wave && valid) {
        const int32_t first = position[e];
        pos = first + rank;
        if (rank == 0) position[e] = first + count;
      }
      __syncthreads();
    }
    if (valid) {
      sorted_token[pos] = slot / top_k;
      sorted_weight[pos] = weights[slot];
      sorted_expert[pos] = static_cast<IdT>(e);
    }
    if (local < slots_per_block) slot_dest[local] = pos;
  }
  __syncthreads();
  // each slot ranks its sorted position within its row: the row's positions ascending, dropped slots (== n_valid) last
  for (int local = threadIdx.x; local < slots_per_block; local += blockDim.x) {
    const int64_t slot = base + local;
    if (slot >= n_slots) continue;
    const int32_t mine = slot_dest[local];
    dest[slot] = mine;
    const int j = local % top_k;
    const int row0 = local - j;
    int rank = 0;
    for (int i = 0; i < top_k; ++i) {
      const int32_t other = slot_dest[row0 + i];
      rank += (other < mine || (other == mine && i < j)) ? 1 : 0;
    }
    inv_map[(slot - j) + rank] = mine;
  }
}

template <typename T>
__global__ void sort_bwd_kernel(const T* __restrict__ grad_sorted, const int32_t* __restrict__ dest,
                                T* __restrict__ grad, int64_t n_slots, int64_t n_valid) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n_slots) return;
  const int32_t d = dest[i];
  grad[i] = (d >= 0 && d < n_valid) ? grad_sorted[d] : T(0);
}

__global__ void __launch_bounds__(1024)
bincount_kernel(const int64_t* __restrict__ indices, const float* __restrict__ weights, int64_t n, int size,
                int out_is_i64, void* __restrict__ out) {
  extern __shared__ int32_t counts[];
  float* sums = reinterpret_cast<float*>(counts);
  for (int v = threadIdx.x; v < size; v += blockDim.x) counts[v] = 0;  // all-zero bits: 0 and 0.0f alike
  __syncthreads();
  for (int64_t i = threadIdx.x; i < n; i += blockDim.x) {
    const int64_t v = indices[i];
    if (v >= 0 && v < size) {
      if (weights) atomicAdd(&sums[v], weights[i]);  // LDS float add: the sum's order is not fixed
      else atomicAdd(&counts[v], 1);
    }
  }
  __syncthreads();
  for (int v = threadIdx.x; v < size; v += blockDim.x) {
    if (weights) static_cast<float*>(out)[v] = sums[v];
    else if (out_is_i64) static_cast<int64_t*>(out)[v] = counts[v];
    else static_cast<float*>(out)[v] = static_cast<float>(counts[v]);
  }
}

constexpr int64_t kBincountLdsBins = 8192;     // bins a workgroup can count in LDS
constexpr int64_t kBincountOneBlock = 1 << 16;  // up to this many indices one workgroup does it all
constexpr int64_t kBincountPerBlock = 1 << 14;  // indices per workgroup beyond that (grid-stride past 2048 workgroups)

__global__ void __launch_bounds__(1024) bincount_clear_kernel(uint32_t* __restrict__ out, int64_t words) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < words;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    out[i] = 0u;
}

// Each workgroup counts its share of the indices, in LDS first where the bins fit (kLds), and adds what it found to
// the cleared output.  The output adds are vector atomics on global memory: integer counts come out exact whatever
// their order; a weighted sum's order is not fixed (as the reference's scatter_add_).
template <bool kLds>
__global__ void __launch_bounds__(1024)
bincount_blocks_kernel(const int64_t* __restrict__ indices, const float* __restrict__ weights, int64_t n, int64_t size,
                       int out_is_i64, void* __restrict__ out) {
  extern __shared__ int32_t counts[];
  float* sums = reinterpret_cast<float*>(counts);
  if constexpr (kLds) {
    for (int v = threadIdx.x; v < size; v += blockDim.x) counts[v] = 0;
    __syncthreads();
  }
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int64_t v = indices[i];
    if (v < 0 || v >= size) continue;
    if constexpr (kLds) {
      if (weights) atomicAdd(&sums[v], weights[i]);
      else atomicAdd(&counts[v], 1);
    } else {
      if (weights) atomicAdd(static_cast<float*>(out) + v, weights[i]);
      else if (out_is_i64) atomicAdd(static_cast<unsigned long long*>(out) + v, 1ull);
      else atomicAdd(static_cast<float*>(out) + v, 1.0f);
    }
  }
  if constexpr (kLds) {
    __syncthreads();
    for (int v = threadIdx.x; v < size; v += blockDim.x) {
      if (weights) {
        if (sums[v] != 0.0f) atomicAdd(static_cast<float*>(out) + v, sums[v]);
      } else if (counts[v] != 0) {
        if (out_is_i64) atomicAdd(static_cast<unsigned long long*>(out) + v, static_cast<unsigned long long>(counts[v]));
        else atomicAdd(static_cast<float*>(out) + v, static_cast<float>(counts[v]));
      }
    }
  }
}

int rows_per_block(int top_k) { return kBlockSlots / top_k > 0 ? kBlockSlots / top_k : 1; }

template <typename IdT, typename WT>
int launch_sort(const void* experts, const void* weights, int64_t n_rows, int top_k, int n_local, int64_t n_valid,
                int64_t* sorted_token, void* sorted_weight, void* sorted_expert, int32_t* offs, int64_t* inv_map,
                int32_t* dest, int32_t* ok, int32_t* hist, hipStream_t stream) {
  const int rows = rows_per_block(top_k);
  const int slots_per_block = rows * top_k;
  const int64_t n_slots = n_rows * top_k;
  const int64_t n_blocks = (n_rows + rows - 1) / rows;
  int e_pad = 1;
  while (e_pad < n_local) e_pad <<= 1;
  int id_bits = 0;
  while ((1 << id_bits) < n_local) ++id_bits;
  if (n_blocks > 0) {
    histogram_kernel<IdT><<<dim3(n_blocks), dim3(kPlaceThreads), n_local * sizeof(int32_t), stream>>>(
        static_cast<const IdT*>(experts), hist, n_slots, slots_per_block, n_local);
    HMOE_CHECK_LAUNCH();
  }
  scan_kernel<<<dim3(1), dim3(kScanThreads), 0, stream>>>(hist, offs, ok, static_cast<int>(n_blocks), n_local, e_pad,
                                                        n_valid);
  HMOE_CHECK_LAUNCH();
  if (n_blocks > 0) {
    const size_t lds = (static_cast<size_t>(n_local) + slots_per_block) * sizeof(int32_t);
    place_kernel<IdT, WT><<<dim3(n_blocks), dim3(kPlaceThreads), lds, stream>>>(
        static_cast<const IdT*>(experts), static_cast<const WT*>(weights), hist, ok, sorted_token,
        static_cast<WT*>(sorted_weight), static_cast<IdT*>(sorted_expert), inv_map, dest, n_slots, slots_per_block,
        top_k, n_local, id_bits, n_valid);
    HMOE_CHECK_LAUNCH();
  }
  return HMOE_OK;
}

}  // namespace
}  // namespace hmoe

extern "C" {

int64_t hmoe_route_sort_workspace_bytes(int64_t n_rows, int top_k, int num_local_experts) {
  if (n_rows < 0 || top_k <= 0 || num_local_experts <= 0) return HMOE_INVALID_ARGUMENT;
  const int rows = hmoe::rows_per_block(top_k);
  const int64_t n_blocks = (n_rows + rows - 1) / rows;
  const int64_t bytes = (n_blocks > 0 ? n_blocks : 1) * num_local_experts * static_cast<int64_t>(sizeof(int32_t));
  return (bytes + 15) & ~static_cast<int64_t>(15);
}

int hmoe_route_sort(const void* experts, int experts_elem_bytes, const void* weights, int weight_elem_bytes,
                    int64_t n_rows, int top_k, int num_local_experts, int64_t n_valid, int64_t* sorted_token_idx,
                    void* sorted_weights, void* sorted_expert_ids, int32_t* offs, int64_t* inv_map, int32_t* dest,
                    int32_t* ok, void* workspace, void* stream) {
  using namespace hmoe;
  if (n_rows < 0 || top_k <= 0 || num_local_experts <= 0 || n_valid < 0) return HMOE_INVALID_ARGUMENT;
  if (!offs || !ok || !workspace) return HMOE_INVALID_ARGUMENT;
  if (n_rows > 0 && (!experts || !weights || !inv_map || !dest)) return HMOE_INVALID_ARGUMENT;
  if (n_valid > 0 && (!sorted_token_idx || !sorted_weights || !sorted_expert_ids)) return HMOE_INVALID_ARGUMENT;
  if (num_local_experts > kMaxExperts || top_k > kBlockSlots) return HMOE_UNSUPPORTED;
  if (n_rows * top_k >= (int64_t(1) << 31) || n_valid >= (int64_t(1) << 31)) return HMOE_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int32_t* hist = static_cast<int32_t*>(workspace);
#define HMOE_SORT(ID, W)                                                                                         \
  return launch_sort<ID, W>(experts, weights, n_rows, top_k, num_local_experts, n_valid, sorted_token_idx,       \
                            sorted_weights, sorted_expert_ids, offs, inv_map, dest, ok, hist, s)
  if (experts_elem_bytes == 8) {
    if (weight_elem_bytes == 4) HMOE_SORT(int64_t, uint32_t);
    if (weight_elem_bytes == 2) HMOE_SORT(int64_t, uint16_t);
    if (weight_elem_bytes == 8) HMOE_SORT(int64_t, uint64_t);
  } else if (experts_elem_bytes == 4) {
    if (weight_elem_bytes == 4) HMOE_SORT(int32_t, uint32_t);
    if (weight_elem_bytes == 2) HMOE_SORT(int32_t, uint16_t);
    if (weight_elem_bytes == 8) HMOE_SORT(int32_t, uint64_t);
  }
#undef HMOE_SORT
  return HMOE_UNSUPPORTED;
}

int hmoe_route_sort_static(const void* experts, int experts_elem_bytes, const void* weights, int weight_elem_bytes,
                           int64_t n_rows, int top_k, int num_local_experts, int64_t n_valid,
                           int64_t* sorted_token_idx, void* sorted_weights, void* sorted_expert_ids, int32_t* offs,
                           int64_t* inv_map, int32_t* dest, int32_t* ok, void* stream) {
  using namespace hmoe;
  if (n_rows < 0 || top_k <= 0 || num_local_experts <= 0 || n_valid < 0) return HMOE_INVALID_ARGUMENT;
  const int64_t needed = hmoe_route_sort_workspace_bytes(n_rows, top_k, num_local_experts);
  if (needed < 0) return HMOE_INVALID_ARGUMENT;
  // the table must fit the library's array: refused, never truncated
  if (needed > kStaticScratchInts * static_cast<int64_t>(sizeof(int32_t))) return HMOE_UNSUPPORTED;
  int status = HMOE_OK;
  int32_t* table = static_scratch(status);
  if (table == nullptr) return status;
  // Every entry the scan and the placement read is written by this call's histogram launch first (each sort block
  // writes its whole row of the table), so what the previous call left in the array is never seen.
  return hmoe_route_sort(experts, experts_elem_bytes, weights, weight_elem_bytes, n_rows, top_k, num_local_experts,
                         n_valid, sorted_token_idx, sorted_weights, sorted_expert_ids, offs, inv_map, dest, ok, table,
                         stream);
}

int hmoe_route_sort_bwd(const void* grad_sorted, const int32_t* dest, int64_t n_slots, int64_t n_valid,
                        int elem_bytes, void* grad_weights, void* stream) {
  using namespace hmoe;
  if (n_slots < 0 || n_valid < 0) return HMOE_INVALID_ARGUMENT;
  if (n_slots == 0) return HMOE_OK;
  if (!dest || !grad_weights || (n_valid > 0 && !grad_sorted)) return HMOE_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((n_slots + 255) / 256), block(256);
  if (elem_bytes == 4)
    sort_bwd_kernel<float><<<grid, block, 0, s>>>(static_cast<const float*>(grad_sorted), dest,
                                                 static_cast<float*>(grad_weights), n_slots, n_valid);
  else if (elem_bytes == 8)
    sort_bwd_kernel<double><<<grid, block, 0, s>>>(static_cast<const double*>(grad_sorted), dest,
                                                  static_cast<double*>(grad_weights), n_slots, n_valid);
  else if (elem_bytes == 2)  // bf16 / fp16 bits: zero is all-zero bits in both
    sort_bwd_kernel<uint16_t><<<grid, block, 0, s>>>(static_cast<const uint16_t*>(grad_sorted), dest,
                                                    static_cast<uint16_t*>(grad_weights), n_slots, n_valid);
  else
    return HMOE_UNSUPPORTED;
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

int hmoe_bincount(const int64_t* indices, const float* weights, int64_t n, int64_t size, int out_is_i64, void* out,
                  void* stream) {
  using namespace hmoe;
  if (n < 0 || size < 0) return HMOE_INVALID_ARGUMENT;
  if (size == 0) return HMOE_OK;
  if (!out || (n > 0 && !indices)) return HMOE_INVALID_ARGUMENT;
  if (weights && out_is_i64) return HMOE_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (size <= kBincountLdsBins && n <= kBincountOneBlock) {
    bincount_kernel<<<dim3(1), dim3(1024), size * sizeof(int32_t), s>>>(indices, weights, n, static_cast<int>(size),
                                                                       out_is_i64, out);
    HMOE_CHECK_LAUNCH();
    return HMOE_OK;
  }
  // many indices or many bins: the output is cleared by a fill kernel, then every workgroup adds its share
  const int64_t words = out_is_i64 ? 2 * size : size;
  bincount_clear_kernel<<<dim3(static_cast<unsigned>((words + 1023) / 1024 < 1024 ? (words + 1023) / 1024 : 1024)),
                          dim3(1024), 0, s>>>(static_cast<uint32_t*>(out), words);
  HMOE_CHECK_LAUNCH();
  if (n == 0) return HMOE_OK;
  int64_t blocks = (n + kBincountPerBlock - 1) / kBincountPerBlock;
  if (blocks > 2048) blocks = 2048;
  if (size <= kBincountLdsBins)
    bincount_blocks_kernel<true><<<dim3(static_cast<unsigned>(blocks)), dim3(1024), size * sizeof(int32_t), s>>>(
        indices, weights, n, size, out_is_i64, out);
  else
    bincount_blocks_kernel<false><<<dim3(static_cast<unsigned>(blocks)), dim3(1024), 0, s>>>(indices, weights, n, size,
                                                                                          out_is_i64, out);
  HMOE_CHECK_LAUNCH();
  return HMOE_OK;
}

}  // extern "C"
