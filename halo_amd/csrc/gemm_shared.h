// Pieces shared by the grouped GEMM kernels (grouped_gemm.hip, grouped_gemm_duo.hip): the argument block, buffer
// descriptors, the direct-to-LDS load, the tile walk over ragged groups.
#pragma once

#include "common.h"

namespace hmoe {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));


constexpr int kXcds = 8;
constexpr int kMaxGroups = 1024;

enum Mode { kFwd = 0, kDgrad = 1, kWgrad = 2, kFwdFp8W = 3, kFwdFp8 = 4 };

struct GemmArgs {
  const void* a;  // fwd: A, dgrad: dO, wgrad: A
  int64_t lda;
  const void* b;  // fwd/dgrad: B [G,K,N], wgrad: dO
  int64_t ldb;
  void* c;  // fwd: out, dgrad: dA, wgrad: dB [G,K,N]
  int64_t ldc;
  const int32_t* offs;
  int64_t total_rows;
  int groups;
  int64_t k, n;
  const float* b_scale;  // kFwdFp8W: [G, ceil(K/128), ceil(N/128)]
  // one operand given as (array, row index): logical row r of it is array[a_index[r]].  A in fwd, dgrad and wgrad;
  // with gather_b, wgrad's B (the output gradient) instead
  const int64_t* a_index = nullptr;
  int64_t a_rows = 0;                // rows of the array a_index points into
  bool gather_b = false;
  const void* bias = nullptr;        // fwd: [G, N] in the operands' dtype, added to group g's output rows
  // fwd, dgrad: out = addend + addend_scale * product, element by element with the roundings of those tensor
  // operations (an adapter's low-rank delta joining the base projection; the input gradient of a second projection
  // of the same rows joining the first's); rows ld_addend apart, may be the output itself
  const void* addend = nullptr;
  int64_t ld_addend = 0;
  float addend_scale = 1.f;
  // kFwdFp8: both operands are e4m3 bytes in panels of 64 contraction values (A [K/64][a_scale_rows][64],
  // B [G][K/64][N][64]); k counts values
  const uint8_t* a_scale = nullptr;  // [K / 128][a_scale_rows]: the e8m0 exponent of row r's block b at (b, r)
  int64_t a_scale_rows = 0;
  int k_blocks = 0, n_blocks = 0;     // the grid of b_scale [G, k_blocks, n_blocks]
  // kFwdFp8 with one e8m0 exponent per 32 contraction values on both sides (MXFP8): a_scale is [K / 32][a_scale_rows]
  // and the weights' exponents are bytes [G][K / 32][N]
  const uint8_t* b_scale_e8m0 = nullptr;
};

// Group g's [start, end) clamped into [0, total_rows].
__device__ __forceinline__ void group_bounds(const int32_t* offs, int g, int64_t total_rows, int64_t& start,
                                             int64_t& end) {
  if (offs == nullptr) {
    start = 0;
    end = total_rows;
    return;
  }
  int64_t s = g > 0 ? offs[g - 1] : 0, e = offs[g];
  s = s < 0 ? 0 : (s > total_rows ? total_rows : s);
  e = e < s ? s : (e > total_rows ? total_rows : e);
  start = s;
  end = e;
}

constexpr uint32_t kOutOfRange = 0x80000000u;  // a byte offset no operand reaches: the buffer load returns zeros

// s_barrier alone.  __syncthreads() also fences, and the fence drains every load in flight (vmcnt(0)), including
// the direct-to-LDS loads a kernel wants to keep in flight across the barrier; the callers wait for exactly the
// loads they need before they come here.
__device__ __forceinline__ void workgroup_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// s_waitcnt vmcnt(v) only: expcnt and lgkmcnt left at their maxima
#define HMOE_WAIT_VM(v) __builtin_amdgcn_s_waitcnt(((v) & 15) | (((v) >> 4) << 14) | (7 << 4) | (15 << 8))

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

// The same descriptor as four words, for the direct-to-LDS loads below.
__device__ __forceinline__ u32x4 make_rsrc_words(const void* base, uint32_t bytes) {
  const uint64_t address = reinterpret_cast<uint64_t>(base);
  return u32x4{static_cast<uint32_t>(address), static_cast<uint32_t>(address >> 32) & 0xffffu, bytes, 0x00020000u};
}

typedef __attribute__((address_space(3))) char* lds_bytes_ptr;

// The scalar operands of the loads below, pinned to scalar registers (the compiler does not move an inline
// assembly operand out of a vector register by itself); free where the value is already known to be uniform.
__device__ __forceinline__ uint32_t uniform(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ u32x4 uniform(u32x4 v) {
  return u32x4{uniform(v[0]), uniform(v[1]), uniform(v[2]), uniform(v[3])};
}

// Direct-to-LDS load of 16 bytes per lane: lane L's bytes land at lds_base + 16 L; an offset at or past the
// descriptor's size loads zeros.  Written through inline assembly on purpose.  The compiler tracks the builtin form
// as a pending LDS write and drains every load in flight (vmcnt(0)) before the next LDS store and before the next
// transposing LDS read, which it also takes for a store; in a loop that issues the next step's loads and then reads
// this step's fragments that serialises the two.  Issued this way the loads are invisible to it, and the kernel
// waits for them itself (wait_loads) where it needs them.
__device__ __forceinline__ void lds_load16(u32x4 rsrc, lds_bytes_ptr lds_base, uint32_t voffset, uint32_t soffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(uniform(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds_base)))), "v"(voffset),
                 "s"(uniform(rsrc)), "s"(uniform(soffset))
               : "memory", "m0");
}

// Eight bf16 values plus eight more, each sum rounded to bf16: what a bf16 tensor addition does element by element.
__device__ __forceinline__ u32x4 add_bf16x8(u32x4 a, u32x4 b) {
  u32x4 out;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const float lo = __uint_as_float(a[w] << 16) + __uint_as_float(b[w] << 16);
    const float hi = __uint_as_float(a[w] & 0xffff0000u) + __uint_as_float(b[w] & 0xffff0000u);
    out[w] = pack_bf16x2(lo, hi);
  }
  return out;
}

// base + round(scale * product) per bf16 value, each operation rounded to bf16: `base + scale * product` as two tensor
// operations compute it.
__device__ __forceinline__ u32x4 scale_add_bf16x8(u32x4 product, u32x4 base, float scale) {
  u32x4 out;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const float lo = bf16_to_f32(f32_to_bf16(__fmul_rn(scale, __uint_as_float(product[w] << 16))));
    const float hi = bf16_to_f32(f32_to_bf16(__fmul_rn(scale, __uint_as_float(product[w] & 0xffff0000u))));
    out[w] = pack_bf16x2(__fadd_rn(__uint_as_float(base[w] << 16), lo),
                         __fadd_rn(__uint_as_float(base[w] & 0xffff0000u), hi));
  }
  return out;
}

// every direct-to-LDS load of this wavefront has landed
__device__ __forceinline__ void wait_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// ---------------------------------------------------------------------------------------------- tile schedule
struct TileInfo {
  int g, a_out0, a_out_lim, b_out0, b_out_lim, con_lim, row_start;
};


// The tile walk of a fwd / dgrad workgroup without tables: the kernel's LDS is all operand stages there, so the group
// of a tile is found by walking offs itself (scalar loads) from the previous tile's group.  Same logical order and the
// same chunks per XCD as TileSchedule; everything uniform across the workgroup.
template <int kMode, int BM, int BN>
struct RowTileWalk {
  const int32_t* offs;
  int groups, nt, k, n;
  int64_t total_rows, first, last, stride;
  int g, ts, mt, s, rows;  // the current group: its index, the row tiles before it, its row tiles, first row, rows

  __device__ __forceinline__ void load_group(int gi) {
    int64_t s64 = 0, e64 = 0;
    if (gi < groups) group_bounds(offs, gi, total_rows, s64, e64);
    s = __builtin_amdgcn_readfirstlane(static_cast<int>(s64));
    rows = __builtin_amdgcn_readfirstlane(static_cast<int>(e64 - s64));
    mt = (rows + BM - 1) / BM;
  }
  // chunk bounds of this workgroup's XCD, given the number of row tiles over all groups
  static __device__ __forceinline__ void chunk_of(int64_t total, int64_t& first, int64_t& last) {
    const int xcd = blockIdx.x % kXcds;
    const int64_t chunk = (total + kXcds - 1) / kXcds;
    first = xcd * chunk + blockIdx.x / kXcds;
    last = xcd * chunk + chunk < total ? xcd * chunk + chunk : total;
  }
  __device__ __forceinline__ void init(const GemmArgs& p, int total_row_tiles, int g0, int ts0) {
    offs = p.offs;
    groups = p.groups;
    total_rows = p.total_rows;
    k = static_cast<int>(p.k);
    n = static_cast<int>(p.n);
    const int64_t out_cols = kMode == kDgrad ? p.k : p.n;
    nt = static_cast<int>((out_cols + BN - 1) / BN);
    chunk_of(static_cast<int64_t>(total_row_tiles) * nt, first, last);
    stride = (static_cast<int>(gridDim.x) - static_cast<int>(blockIdx.x % kXcds) + kXcds - 1) / kXcds;
    g = g0;
    ts = ts0;
    load_group(g);
  }
  __device__ __forceinline__ TileInfo decode(int64_t t, int& /*cursor*/) {
    while (g < groups && static_cast<int64_t>(ts + mt) * nt <= t) {  // groups without rows have no tiles
      ts += mt;
      ++g;
      load_group(g);
    }
    const int r = static_cast<int>(t - static_cast<int64_t>(ts) * nt);
    const int n_t = r / mt, m_t = r - n_t * mt;
    TileInfo tile;
    tile.g = g;
    tile.row_start = s;
    tile.a_out0 = m_t * BM;
    tile.a_out_lim = rows;
    tile.b_out0 = n_t * BN;
    tile.b_out_lim = kMode == kDgrad ? k : n;
    tile.con_lim = kMode == kDgrad ? n : k;
    return tile;
  }
};

// grouped_gemm_duo.hip: the kernel on several workgroups per compute unit (a 128 x 256 tile on two, or with small_tile
// a 128 x 128 tile on three), for the bf16 product `mode` (kFwd, kDgrad, kWgrad) whose arguments the caller has
// validated; the variant (gathered operand, bias, addend) is read off p
int launch_duo(int mode, const GemmArgs& p, bool small_tile, hipStream_t stream);

}  // namespace hmoe
