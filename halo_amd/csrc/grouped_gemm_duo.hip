// Grouped GEMM, bf16, two workgroups per compute unit: the second tile configuration of grouped_gemm.hip's products
//   fwd    out[s:e]  = A[s:e]  @ B[g]          A [R,K],  B [G,K,N]
//   dgrad  dA[s:e]   = dO[s:e] @ B[g]^T        dO [R,N]
//   wgrad  dB[g]     = A[s:e]^T @ dO[s:e]      ragged contraction, empty group -> exact zeros
// (halo/kernels/grouped_mm.py:16-47 of the reference), with the same operand variants: one operand fetched through a
// row index, an expert bias or a scaled addend in the epilogue.
//
// A workgroup is four wavefronts (one per SIMD) and owns a 128 x 256 output tile; a wavefront owns all 128 rows of 64
// columns, 4 x 2 accumulator blocks of 32 x 32 (v_mfma_f32_32x32x16_bf16, operands swapped so that a lane owns an
// output row).  The contraction moves in steps of 32 through three LDS stages of 24 KB (8 KB of operand A, 16 KB of
// B), 72 KB in all, so that two workgroups are resident on a compute unit and each SIMD holds one wavefront of each:
// while one workgroup stands at its barrier, waits for its tile loads or stores a finished tile, the other one's
// MFMAs have the matrix pipe.  (One 256 x 256 workgroup per compute unit moves a third fewer operand bytes per
// multiply-add but stalls as a whole: both wavefronts of a SIMD meet the same barrier.)
//  * Tile loads go from global memory straight into LDS (buffer_load ... lds, 16 bytes per lane, issued through inline
//    assembly and waited for by count); the loads of step s + 2 are issued at the top of step s, so two refills are in
//    flight.  Every wavefront issues a quarter of a step's loads: 2 of A and 4 of B.
//  * A contraction-contiguous operand lands as [rows][32 con], 64-byte rows, the 16-byte chunk index XOR-ed with
//    (row >> 1 & 3) ^ (row >> 3 & 1); a fragment is one ds_read_b128.
//  * An output-contiguous operand lands in panels of 64 output columns, [panel][32 con][64 out], 128-byte rows (a load
//    instruction fetches eight whole 128-byte lines), chunk index XOR-ed with (con & 3) << 1; a fragment is two
//    ds_read_b64_tr_b16.  A lane stays on one contraction row for all loads of a step, so an operand whose rows are
//    gathered through an index costs one index read per step and lane.
//  * The barrier of a step sits in the middle of its last MFMAs, the next step's first fragments are read behind it.
//  * Epilogue through the third stage, 32 rows per wavefront at a time, whole 128-byte lines out; the next tile's
//    first two steps are requested before it.
// Tile order and XCD chunks as in grouped_gemm.hip: group-major, column tile, row tile; one contiguous chunk per XCD.
#include "gemm_shared.h"

#include <type_traits>

namespace hmoe {
namespace {

constexpr int DK = 32;                       // contraction per step
constexpr int kDuoWaves = 4;
constexpr int kDuoStages = 3;
constexpr int kDuoIndexSlot = 256;           // one dword per lane: the row indices of eight steps of a wavefront
constexpr int kDuoIndexArea = kDuoWaves * 2 * kDuoIndexSlot;
constexpr int kWN = 2;                       // a wavefront's 32 x 32 blocks along operand B's output index

// A tile configuration: GM x (4 / GM) wavefronts, each WM x 2 blocks of 32 x 32.
//   DuoTile<1, 4>: 128 x 256, 72 KB of stages, two workgroups per compute unit (the expert products)
//   DuoTile<2, 2>: 128 x 128, 48 KB of stages, three workgroups per compute unit (products with few tiles: a dense
//                  projection of some thousand rows, a narrow output)
template <int GM_, int WM_>
struct DuoTile {
  static constexpr int GM = GM_, GN = kDuoWaves / GM_, WM = WM_;
  static constexpr int DM = GM * WM * 32;    // operand A's output index
  static constexpr int DN = GN * kWN * 32;   // operand B's output index
  static_assert(DM % 64 == 0 && DN % 64 == 0, "operand tiles are loaded in pieces of 64 output indices");
  static constexpr int kA = DM * DK * 2;     // bytes of A per stage
  static constexpr int kB = DN * DK * 2;
  static constexpr int kStage = kA + kB;
  static constexpr int kStepLoads = DM / 64 + DN / 64;  // tile loads per wavefront and step
  static constexpr int kEpiRegion = 32 * (kWN * 32 + 8) * 2;  // bytes of epilogue staging per wavefront
  static constexpr int kEpiBase = 2 * kStage;                 // behind the stages the next tile's first loads use
  static constexpr int kTiles = kDuoStages * kStage > kEpiBase + kDuoWaves * kEpiRegion
                                    ? kDuoStages * kStage
                                    : kEpiBase + kDuoWaves * kEpiRegion;
  static constexpr int kWavesPerSimd = 3 * (kTiles + kDuoIndexArea) <= 160 * 1024 && WM <= 2 ? 3 : 2;
};

// one dword per lane, direct to LDS: lane L's dword lands at lds_base + 4 L
__device__ __forceinline__ void duo_load4(u32x4 rsrc, lds_bytes_ptr lds_base, uint32_t voffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds"
               :
               : "s"(uniform(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds_base)))), "v"(voffset),
                 "s"(uniform(rsrc))
               : "memory", "m0");
}

// s_waitcnt vmcnt(n) for a uniform n known only at run time (the loads and stores of a wavefront complete in the
// order they were issued, so "all but the newest n" names exactly the operations that may stay in flight)
__device__ __forceinline__ void wait_all_but(int n) {
  switch (n) {
    case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
    case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
    case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
    case 10: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
    case 12: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
    case 14: asm volatile("s_waitcnt vmcnt(14)" ::: "memory"); break;
    case 16: asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); break;
    case 18: asm volatile("s_waitcnt vmcnt(18)" ::: "memory"); break;
    case 22: asm volatile("s_waitcnt vmcnt(22)" ::: "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
  }
}

__device__ __forceinline__ int swizzle64(int row) { return ((row >> 1) & 3) ^ ((row >> 3) & 1); }

// ---------------------------------------------------------------------------------------------------- loaders
// element(out, con) = base[out * ld + con]; LDS [kRows][32 con].  A load instruction moves 16 rows of 64 bytes: lane L
// takes row L >> 2 and the chunk that belongs in its slot under the swizzle.  With kGathered the rows are
// base[index[out]].
template <int kRows, bool kGathered>
struct DuoDirect {
  static constexpr int kI = kRows / (16 * kDuoWaves);  // loads per wavefront and step (16 rows each)
  u32x4 rsrc;
  uint32_t voff[kGathered ? kI : 1];
  uint32_t t_stride;
  int con0, con_lim;

  // rows in place: `base` is the tile's first row, `bytes` ends at its last
  __device__ __forceinline__ void init(const bf16_t* base, int64_t ld, int64_t bytes, int con_lim_, int wave,
                                       int lane) {
    rsrc = make_rsrc_words(base, static_cast<uint32_t>(bytes));
    con_lim = con_lim_;
    const int logical = (lane & 3) ^ swizzle64(lane >> 2);
    con0 = logical << 3;
    t_stride = 16u * static_cast<uint32_t>(ld) * 2u;
    voff[0] = static_cast<uint32_t>(wave * kI * 16 + (lane >> 2)) * static_cast<uint32_t>(ld) * 2u + (logical << 4);
  }
  // rows through an index: logical row r of the tile is base[index[out0 + r]]; an index outside [0, a_rows) and a
  // row at or past out_lim load zeros
  __device__ __forceinline__ void init_gathered(const bf16_t* base, int64_t ld, int64_t a_rows, const int64_t* index,
                                                int out0, int out_lim, int con_lim_, int wave, int lane) {
    rsrc = make_rsrc_words(base, static_cast<uint32_t>(a_rows * ld * 2));
    con_lim = con_lim_;
    const int logical = (lane & 3) ^ swizzle64(lane >> 2);
    con0 = logical << 3;
    t_stride = 0;
#pragma unroll
    for (int t = 0; t < (kGathered ? kI : 1); ++t) {
      const int out = out0 + (wave * kI + t) * 16 + (lane >> 2);
      const int64_t row = out < out_lim ? index[out] : -1;
      voff[t] = row >= 0 && row < a_rows ? static_cast<uint32_t>(row) * static_cast<uint32_t>(ld) * 2u + (logical << 4)
                                         : kOutOfRange;
    }
  }
  __device__ __forceinline__ void issue(lds_bytes_ptr tile, int step, int wave) const {
    const uint32_t soff = static_cast<uint32_t>(step) * (DK * 2);
    const bool in_range = step * DK + con0 < con_lim;
#pragma unroll
    for (int t = 0; t < kI; ++t) {
      uint32_t off;
      if constexpr (kGathered) off = in_range ? voff[t] : kOutOfRange;
      else off = in_range ? voff[0] + t * t_stride : kOutOfRange;
      lds_load16(rsrc, tile + (wave * kI + t) * 1024, off, soff);
    }
  }
  // per-lane byte address (within the operand's tile) of the fragment of sub-step 0, block 0 from row0
  static __device__ __forceinline__ int fragment_base(int row0, int lane) {
    const int row = row0 + (lane & 31);
    return row * (DK * 2) + ((((lane >> 5)) ^ swizzle64(row)) << 4);
  }
  static __device__ __forceinline__ bf16x8 fragment(const char* tile, int base, int block, int kk) {
    return *reinterpret_cast<const bf16x8*>(tile + (base ^ (kk << 5)) + block * (32 * DK * 2));
  }
};

// element(out, con) = base[con * ld + out]; LDS [kPanels][32 con][64 out].  A load instruction moves eight contraction
// rows of one panel, 128 bytes each: lane L takes row L >> 3 of the wavefront's eight and the chunk that belongs in
// its slot.  kRebase (wgrad, whose contraction walks every row of a group: more than 32 bits of bytes for a large
// one): the descriptor is rebased every step.
template <int kPanels, bool kRebase>
struct DuoTransposed {
  u32x4 rsrc;
  uint64_t base_address;
  int64_t extent;
  uint32_t voff, step_bytes;
  int p_lim;  // panels p < p_lim hold this lane's chunk
  int con, con_lim;

  __device__ __forceinline__ void init(const bf16_t* base, int64_t ld, int64_t bytes, int out0, int out_lim,
                                       int con_lim_, int wave, int lane) {
    con_lim = con_lim_;
    if constexpr (kRebase) {
      base_address = reinterpret_cast<uint64_t>(base);
      extent = bytes;
    } else {
      rsrc = make_rsrc_words(base, static_cast<uint32_t>(bytes));
    }
    step_bytes = DK * static_cast<uint32_t>(ld) * 2u;
    con = wave * 8 + (lane >> 3);
    const int logical = (lane & 7) ^ ((con & 3) << 1);
    const int out = out0 + (logical << 3);
    voff = static_cast<uint32_t>(con) * static_cast<uint32_t>(ld) * 2u + static_cast<uint32_t>(out) * 2u;
    p_lim = out < out_lim ? (out_lim - out + 63) >> 6 : 0;
  }
  __device__ __forceinline__ u32x4 step_rsrc(int step) const {
    if constexpr (!kRebase) return rsrc;
    const int64_t offset = static_cast<int64_t>(step) * step_bytes;
    int64_t left = extent - offset;
    left = left < 0 ? 0 : (left > 0x7fffffff ? 0x7fffffff : left);  // below kOutOfRange, which must stay out of range
    return make_rsrc_words(reinterpret_cast<const void*>(base_address + static_cast<uint64_t>(offset)),
                           static_cast<uint32_t>(left));
  }
  __device__ __forceinline__ void issue(lds_bytes_ptr tile, int step, int wave) const {
    const u32x4 r = step_rsrc(step);
    const uint32_t soff = kRebase ? 0u : static_cast<uint32_t>(step) * step_bytes;
    // the contraction's end is checked here: the step offset takes no part in the descriptor's bounds check
    const int panels = step * DK + con < con_lim ? p_lim : 0;
#pragma unroll
    for (int p = 0; p < kPanels; ++p)
      lds_load16(r, tile + p * 4096 + wave * 1024, p < panels ? voff + p * 128u : kOutOfRange, soff);
  }
  // per-lane byte address of the fragment of sub-step 0 for the 32-column block `block` of the tile
  static __device__ __forceinline__ int fragment_base(int block, int lane) {
    const int i = lane & 15, g = lane >> 4;
    const int con = ((g >> 1) << 3) + (i >> 2);
    const int chunk = ((block & 1) << 2) + ((g & 1) << 1) + ((i & 3) >> 1);
    return (block >> 1) * 4096 + con * 128 + ((chunk ^ ((con & 3) << 1)) << 4) + ((i & 1) << 3);
  }
  static __device__ __forceinline__ bf16x8 fragment(const char* tile, int base, int /*block*/, int kk) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4* lds_ptr;
    const char* ptr = tile + base + kk * (16 * 128);
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(ptr));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(ptr + 4 * 128));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(bf16x8, both);
  }
};

// Fetch the row indices (low words) of steps 8 * block .. 8 * block + 7 of a group, given by its index descriptor and
// its row count, into slot `slot` of a wavefront's index area: lane L holds the row of step 8 * block + (L >> 3),
// row (L & 7) of the wavefront's eight.
__device__ __forceinline__ void duo_load_rows(lds_bytes_ptr area, u32x4 group_index, int group_rows, int block,
                                              int slot, int wave, int lane) {
  const int row = (block * 8 + (lane >> 3)) * DK + wave * 8 + (lane & 7);
  duo_load4(group_index, area + slot * kDuoIndexSlot, row < group_rows ? static_cast<uint32_t>(row) * 8u : kOutOfRange);
}

// The same LDS layout for an operand whose contraction rows are gathered: row r of the group is base[index[r]]
// (wgrad: the tokens, or the output gradient by token).  The indices of eight steps of a wavefront (64 rows, low
// words) are fetched into LDS with one load, a block of eight steps ahead, into the wavefront's own two slots.
template <int kPanels>
struct DuoGatherTransposed {
  u32x4 rsrc, index_rsrc;
  uint32_t a_rows, col, row_bytes;
  int p_lim, con_lim;
  lds_bytes_ptr rows_area;  // this wavefront's two slots

  __device__ __forceinline__ void init(const bf16_t* base, int64_t ld, int64_t a_rows_, const int64_t* index, int out0,
                                       int out_lim, int con_lim_, int lane) {
    rsrc = make_rsrc_words(base, static_cast<uint32_t>(a_rows_ * ld * 2));
    index_rsrc = make_rsrc_words(index, static_cast<uint32_t>(con_lim_) * 8u);
    a_rows = static_cast<uint32_t>(a_rows_);
    row_bytes = static_cast<uint32_t>(ld) * 2u;
    con_lim = con_lim_;
    const int logical = (lane & 7) ^ (((lane >> 3) & 3) << 1);
    const int out = out0 + (logical << 3);
    col = static_cast<uint32_t>(out) * 2u;
    p_lim = out < out_lim ? (out_lim - out + 63) >> 6 : 0;
  }
  // the loads of `step`, whose indices sit in `slot` (and whose arrival the caller has waited for)
  __device__ __forceinline__ void issue(lds_bytes_ptr tile, int step, int slot, int wave) const {
    const int lane = threadIdx.x & 63;
    const int mine = lane >> 3;
    const uint32_t row = *reinterpret_cast<const __attribute__((address_space(3))) uint32_t*>(
        rows_area + slot * kDuoIndexSlot + (((step & 7) << 3) + mine) * 4);
    const bool valid = step * DK + wave * 8 + mine < con_lim && row < a_rows;
    const uint32_t base = valid ? row * row_bytes + col : kOutOfRange;
#pragma unroll
    for (int p = 0; p < kPanels; ++p)
      lds_load16(rsrc, tile + p * 4096 + wave * 1024, p < p_lim ? base + p * 128u : kOutOfRange, 0u);
  }
  static __device__ __forceinline__ int fragment_base(int block, int lane) {
    return DuoTransposed<kPanels, false>::fragment_base(block, lane);
  }
  static __device__ __forceinline__ bf16x8 fragment(const char* tile, int base, int block, int kk) {
    return DuoTransposed<kPanels, false>::fragment(tile, base, block, kk);
  }
};

// ------------------------------------------------------------------------------------------- wgrad's tile walk
// Tiles in (group, column tile, row tile) order, each costing its group's contraction steps plus a fixed part; the
// XCD chunks are cut at equal cost.  No tables: the cuts are found once by wavefront 0, a tile's group is a division
// and its bounds two scalar loads.
constexpr int kWgradTileOverhead = 2;  // a tile's fixed cost in contraction steps (first loads, epilogue)

template <int DM, int DN>
struct DuoWgradWalk {
  const int32_t* offs;
  int groups, mt, nt, k, n;
  int64_t total_rows, per_group, first, last, stride;

  __device__ __forceinline__ TileInfo decode(int64_t t, int& /*cursor*/) const {
    const int g = static_cast<int>(t / per_group);
    const int r = static_cast<int>(t - g * per_group);
    const int n_t = r / mt, m_t = r - n_t * mt;
    int64_t s, e;
    group_bounds(offs, g, total_rows, s, e);
    TileInfo tile;
    tile.g = g;
    tile.row_start = __builtin_amdgcn_readfirstlane(static_cast<int>(s));
    tile.con_lim = __builtin_amdgcn_readfirstlane(static_cast<int>(e - s));
    tile.a_out0 = m_t * DM;
    tile.a_out_lim = k;
    tile.b_out0 = n_t * DN;
    tile.b_out_lim = n;
    return tile;
  }
};

// The first tile whose predecessors cost `target` or more, found by the lanes of one wavefront: lane L holds the
// groups [g0, g0 + per) with `excl` the cost of one tile of each group before them summed, `sum` its own groups'.
__device__ __forceinline__ int64_t wgrad_cut(const GemmArgs& p, int64_t per_group, int64_t target, int g0, int per,
                                             int64_t excl, int64_t total_cost) {
  int64_t found = -1;
  if (target >= total_cost * per_group) found = per_group * p.groups;
  else {
    int64_t before = excl;
    for (int g = g0; g < g0 + per && g < p.groups; ++g) {
      int64_t s, e;
      group_bounds(p.offs, g, p.total_rows, s, e);
      const int64_t each = (e - s + DK - 1) / DK + kWgradTileOverhead;
      if (per_group * before <= target && target < per_group * (before + each)) {
        int64_t within = (target - per_group * before + each - 1) / each;
        if (within > per_group) within = per_group;
        found = g * per_group + within;
      }
      before += each;
    }
  }
  // exactly one lane found it (or all of them, past the end)
  int64_t result = 0;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const int64_t other = __shfl_xor(found, off, HMOE_WAVE);
    found = found > other ? found : other;
  }
  result = found;
  return result;
}

// Scheduling hint for a region of kReads LDS reads and kMfmas MFMAs: spread the reads evenly under the MFMAs.
template <int kReads, int kMfmas>
__device__ __forceinline__ void spread_reads_under_mfmas() {
  if constexpr (kReads <= kMfmas) {
    constexpr int per = kMfmas / kReads;
#pragma unroll
    for (int r = 0; r < kReads; ++r) {
      __builtin_amdgcn_sched_group_barrier(0x008, per, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    if constexpr (kMfmas - per * kReads > 0) __builtin_amdgcn_sched_group_barrier(0x008, kMfmas - per * kReads, 0);
  } else {
    constexpr int per = (kReads + kMfmas - 1) / kMfmas;
#pragma unroll
    for (int m = 0; m < kMfmas; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, per, 0);
    }
  }
}

template <int kMode, typename Tile, int kGather, bool kBias, bool kAddTo>
__global__ void __launch_bounds__(64 * kDuoWaves)
    __attribute__((amdgpu_waves_per_eu(Tile::kWavesPerSimd, Tile::kWavesPerSimd)))
grouped_gemm_duo_kernel(GemmArgs p) {
  static_assert(!kAddTo || ((kMode == kFwd || kMode == kDgrad) && !kBias && !kGather),
                "the scaled sum into an addend belongs to the plain forward and the plain input gradient");
  static_assert(!kBias || kMode == kFwd, "the expert bias belongs to the forward product");
  static_assert(kGather >= 0 && kGather <= 2 && (kGather != 2 || kMode == kWgrad), "B is gathered in wgrad only");
  constexpr bool kGatherA = kGather == 1, kGatherB = kGather == 2;
  constexpr bool kDirectA = kMode != kWgrad, kDirectB = kMode == kDgrad;
  constexpr int DM = Tile::DM, DN = Tile::DN, kWM = Tile::WM;
  constexpr int kDuoA = Tile::kA, kDuoStage = Tile::kStage, kDuoTiles = Tile::kTiles;
  constexpr int kPanelsA = DM / 64, kPanelsB = DN / 64;
  using LoaderA = typename std::conditional<
      kDirectA, DuoDirect<DM, kGatherA>,
      typename std::conditional<kGatherA, DuoGatherTransposed<kPanelsA>, DuoTransposed<kPanelsA, true>>::type>::type;
  using LoaderB = typename std::conditional<
      kDirectB, DuoDirect<DN, false>,
      typename std::conditional<kGatherB, DuoGatherTransposed<kPanelsB>,
                                DuoTransposed<kPanelsB, kMode == kWgrad>>::type>::type;
  // the gathered rows are contraction rows (wgrad): new ones every step
  constexpr bool kRowsPerStep = (kGatherA && !kDirectA) || kGatherB;
  constexpr int kStepLoads = Tile::kStepLoads;
  using Sched = typename std::conditional<kMode == kWgrad, DuoWgradWalk<DM, DN>, RowTileWalk<kMode, DM, DN>>::type;

  extern __shared__ __attribute__((aligned(16))) char lds_raw[];
  auto lds = (lds_bytes_ptr)lds_raw;
  auto a_off = [](int stage) { return stage * kDuoStage; };
  auto b_off = [](int stage) { return stage * kDuoStage + kDuoA; };
  constexpr int kEpiBase = Tile::kEpiBase;  // the epilogue stages through the third stage
  bf16_t* c = static_cast<bf16_t*>(p.c);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int gm = wave / Tile::GN, gn = wave % Tile::GN;
  const int row_a = gm * (kWM * 32);    // this wavefront's first row and
  const int col_b = gn * (kWN * 32);    // first column of the tile

  // ---- the workgroup's share of the tile order, found by wavefront 0 and handed over through the first words of the
  // (still unused) stages
  Sched sched;
  {
    int64_t* handoff = reinterpret_cast<int64_t*>(lds_raw);
    const int xcd = blockIdx.x % kXcds;
    if (wave == 0) {
      const int per = (p.groups + HMOE_WAVE - 1) / HMOE_WAVE;
      const int g0 = lane * per;
      if constexpr (kMode == kWgrad) {
        int64_t sum = 0;
        for (int g = g0; g < g0 + per && g < p.groups; ++g) {
          int64_t s, e;
          group_bounds(p.offs, g, p.total_rows, s, e);
          sum += (e - s + DK - 1) / DK + kWgradTileOverhead;
        }
        int64_t incl = sum;
#pragma unroll
        for (int off = 1; off < HMOE_WAVE; off <<= 1) {
          const int64_t up = __shfl_up(incl, off, HMOE_WAVE);
          if (lane >= off) incl += up;
        }
        const int64_t total_cost = __shfl(incl, HMOE_WAVE - 1, HMOE_WAVE);
        const int64_t per_group = ((p.k + DM - 1) / DM) * ((p.n + DN - 1) / DN);
        const int64_t cost = per_group * total_cost;
        const int64_t lo = xcd == 0 ? 0 : wgrad_cut(p, per_group, cost * xcd / kXcds, g0, per, incl - sum, total_cost);
        const int64_t hi = xcd + 1 == kXcds
                               ? per_group * p.groups
                               : wgrad_cut(p, per_group, cost * (xcd + 1) / kXcds, g0, per, incl - sum, total_cost);
        if (lane == 0) {
          handoff[0] = lo;
          handoff[1] = hi;
        }
      } else {
        int sum = 0;
        for (int g = g0; g < g0 + per && g < p.groups; ++g) {
          int64_t s, e;
          group_bounds(p.offs, g, p.total_rows, s, e);
          sum += static_cast<int>((e - s + DM - 1) / DM);
        }
        int incl = sum;
#pragma unroll
        for (int off = 1; off < HMOE_WAVE; off <<= 1) {
          const int up = __shfl_up(incl, off, HMOE_WAVE);
          if (lane >= off) incl += up;
        }
        const int total = __shfl(incl, HMOE_WAVE - 1, HMOE_WAVE);
        const int64_t out_cols = kMode == kDgrad ? p.k : p.n;
        const int nt = static_cast<int>((out_cols + DN - 1) / DN);
        int64_t first, last;
        RowTileWalk<kMode, DM, DN>::chunk_of(static_cast<int64_t>(total) * nt, first, last);
        const int64_t q = first / nt;  // the row tile (counted over all groups) this workgroup's first tile lies in
        if (lane == 0) {
          handoff[0] = total;
          handoff[1] = p.groups;  // no tile for this workgroup: a walk that starts past the last group
          handoff[2] = total;
        }
        if (q >= incl - sum && q < incl) {  // it lies in one of this lane's groups
          int running = incl - sum;
          for (int g = g0; g < g0 + per && g < p.groups; ++g) {
            int64_t s, e;
            group_bounds(p.offs, g, p.total_rows, s, e);
            const int mt = static_cast<int>((e - s + DM - 1) / DM);
            if (q < running + mt) {
              handoff[1] = g;
              handoff[2] = running;
              break;
            }
            running += mt;
          }
        }
      }
    }
    __syncthreads();
    if constexpr (kMode == kWgrad) {
      sched.offs = p.offs;
      sched.groups = p.groups;
      sched.total_rows = p.total_rows;
      sched.k = static_cast<int>(p.k);
      sched.n = static_cast<int>(p.n);
      sched.mt = static_cast<int>((p.k + DM - 1) / DM);
      sched.nt = static_cast<int>((p.n + DN - 1) / DN);
      sched.per_group = static_cast<int64_t>(sched.mt) * sched.nt;
      sched.stride = (static_cast<int>(gridDim.x) - xcd + kXcds - 1) / kXcds;
      const int lo_lo = __builtin_amdgcn_readfirstlane(static_cast<int>(handoff[0]));
      const int lo_hi = __builtin_amdgcn_readfirstlane(static_cast<int>(handoff[0] >> 32));
      const int hi_lo = __builtin_amdgcn_readfirstlane(static_cast<int>(handoff[1]));
      const int hi_hi = __builtin_amdgcn_readfirstlane(static_cast<int>(handoff[1] >> 32));
      sched.first = ((static_cast<int64_t>(lo_hi) << 32) | static_cast<uint32_t>(lo_lo)) + blockIdx.x / kXcds;
      sched.last = (static_cast<int64_t>(hi_hi) << 32) | static_cast<uint32_t>(hi_lo);
      __syncthreads();
    } else {
      const int total = __builtin_amdgcn_readfirstlane(static_cast<int>(handoff[0]));
      const int g_first = __builtin_amdgcn_readfirstlane(static_cast<int>(handoff[1]));
      const int ts_first = __builtin_amdgcn_readfirstlane(static_cast<int>(handoff[2]));
      __syncthreads();  // the words are read before the first tile loads land on them
      sched.init(p, total, g_first, ts_first);
    }
  }
  const int64_t w_elems = p.k * p.n;

  LoaderA la;
  LoaderB lb;
  auto& lg = *[&]() { if constexpr (kGatherB) return &lb; else return &la; }();  // the gathered operand's loader
  lds_bytes_ptr rows_area = lds + kDuoTiles + wave * (2 * kDuoIndexSlot);
  if constexpr (kRowsPerStep) lg.rows_area = rows_area;
  int slot0 = 0;  // gathered contraction rows: the index slot of the current tile's steps 0..7

  auto issue_step = [&](int step, int stage) __attribute__((always_inline)) {
    if constexpr (kGatherA && !kDirectA) la.issue(lds + a_off(stage), step, (slot0 + (step >> 3)) & 1, wave);
    else la.issue(lds + a_off(stage), step, wave);
    if constexpr (kGatherB) lb.issue(lds + b_off(stage), step, (slot0 + (step >> 3)) & 1, wave);
    else lb.issue(lds + b_off(stage), step, wave);
  };

  // describe tile `t`'s operands to the loaders and request its first two steps into stages 0 and 1
  // `rows0_loaded`: the gathered contraction rows of its first eight steps were fetched during the previous tile
  auto begin_tile = [&](const TileInfo& tile, bool rows0_loaded) __attribute__((always_inline)) {
    const bf16_t* a = static_cast<const bf16_t*>(p.a);
    const bf16_t* b = static_cast<const bf16_t*>(p.b);
    if constexpr (kMode == kWgrad) {
      const int64_t rows = tile.con_lim;
      if constexpr (kGatherA)
        la.init(a, p.lda, p.a_rows, p.a_index + tile.row_start, tile.a_out0, tile.a_out_lim, tile.con_lim, lane);
      else
        la.init(a + tile.row_start * p.lda, p.lda, rows * p.lda * 2, tile.a_out0, tile.a_out_lim, tile.con_lim, wave,
                lane);
      if constexpr (kGatherB)
        lb.init(b, p.ldb, p.a_rows, p.a_index + tile.row_start, tile.b_out0, tile.b_out_lim, tile.con_lim, lane);
      else
        lb.init(b + tile.row_start * p.ldb, p.ldb, rows * p.ldb * 2, tile.b_out0, tile.b_out_lim, tile.con_lim, wave,
                lane);
    } else {
      if constexpr (kGatherA) {
        la.init_gathered(a, p.lda, p.a_rows, p.a_index + tile.row_start, tile.a_out0, tile.a_out_lim, tile.con_lim,
                         wave, lane);
      } else {
        // the descriptor starts at the tile's first row and ends at its last, so its 32-bit offsets span one tile
        // whatever the operand's or the group's size
        const int rows_left = tile.a_out_lim - tile.a_out0;
        la.init(a + (tile.row_start + tile.a_out0) * p.lda, p.lda, (rows_left < DM ? rows_left : DM) * p.lda * 2,
                tile.con_lim, wave, lane);
      }
      if constexpr (kMode == kFwd) {
        lb.init(b + tile.g * w_elems, p.ldb, w_elems * 2, tile.b_out0, tile.b_out_lim, tile.con_lim, wave, lane);
      } else {
        const int rows_left = tile.b_out_lim - tile.b_out0;  // rows of the weight: the input gradient's columns
        lb.init(b + tile.g * w_elems + static_cast<int64_t>(tile.b_out0) * p.ldb, p.ldb,
                (rows_left < DN ? rows_left : DN) * p.ldb * 2, tile.con_lim, wave, lane);
      }
    }
    if constexpr (kRowsPerStep) {
      if (!rows0_loaded) {
        duo_load_rows(rows_area, lg.index_rsrc, tile.con_lim, 0, slot0, wave, lane);
        wait_loads();
      }
    }
    if (tile.con_lim > 0) issue_step(0, 0);
    if (tile.con_lim > DK) issue_step(1, 1);
  };

  // ---- fragment addresses
  int fa_base[kDirectA ? 1 : kWM], fb_base[kDirectB ? 1 : kWN];
  if constexpr (kDirectA) fa_base[0] = LoaderA::fragment_base(row_a, lane);
  else
#pragma unroll
    for (int i = 0; i < kWM; ++i) fa_base[i] = LoaderA::fragment_base(gm * kWM + i, lane);
  if constexpr (kDirectB) fb_base[0] = LoaderB::fragment_base(col_b, lane);
  else
#pragma unroll
    for (int j = 0; j < kWN; ++j) fb_base[j] = LoaderB::fragment_base(gn * kWN + j, lane);
  bf16x8 fa[2][kWM], fb[2][kWN];
  auto read_fragments = [&](int stage, int kk, int buf, int rows_live) __attribute__((always_inline)) {
    const char* ta = lds_raw + a_off(stage);
    const char* tb = lds_raw + b_off(stage);
    if (rows_live > 0) {
#pragma unroll
      for (int j = 0; j < kWN; ++j) fb[buf][j] = LoaderB::fragment(tb, fb_base[kDirectB ? 0 : j], j, kk);
    }
#pragma unroll
    for (int i = 0; i < kWM; ++i)
      if (i < rows_live) fa[buf][i] = LoaderA::fragment(ta, fa_base[kDirectA ? 0 : i], i, kk);
  };
  constexpr int kReads = kWM * (kDirectA ? 1 : 2) + kWN * (kDirectB ? 1 : 2);  // LDS reads of one sub-step
  constexpr int kMfmas = kWM * kWN;
  constexpr int kEpiPitch = kWN * 32 + 8;
  constexpr int kEpiRegion = Tile::kEpiRegion / 2;  // elements per wavefront
  constexpr int kLanesPerRow = kWN * 4;
  constexpr int kRowsPerPass = 64 / kLanesPerRow;
  static_assert(kEpiRegion == 32 * kEpiPitch && kEpiBase + kEpiRegion * kDuoWaves * 2 <= kDuoTiles,
                "epilogue staging must fit behind the first two stages");
  const char* stage_rows = lds_raw + kEpiBase + wave * kEpiRegion * 2;
  const uint32_t stage_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + kEpiBase +
                              static_cast<uint32_t>((wave * kEpiRegion + (lane & 31) * kEpiPitch + ((lane >> 5) << 2)) * 2);

  int64_t t = sched.first;
  TileInfo tile, next;
  int cursor = 0;
  int stores_in_flight = 0;  // epilogue stores issued behind the current tile's first loads
  if (t < sched.last) {
    tile = sched.decode(t, cursor);
    begin_tile(tile, false);
  }
  while (t < sched.last) {
    const bool has_next = t + sched.stride < sched.last;
    if (has_next) next = sched.decode(t + sched.stride, cursor);
    bool next_rows0_loaded = false;
    f32x16 acc[kWM][kWN];
#pragma unroll
    for (int i = 0; i < kWM; ++i)
#pragma unroll
      for (int j = 0; j < kWN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    const int steps = (tile.con_lim + DK - 1) / DK;
    int live = (tile.a_out_lim - tile.a_out0 - row_a + 31) >> 5;  // this wavefront's 32-row blocks that hold rows
    live = live < 0 ? 0 : (live > kWM ? kWM : live);
    // The expert's bias for this lane's eight output columns, fetched where the tile's first loads are waited for
    // anyway and pinned as arrived right behind that wait.
    u32x4 bias_chunk = {0u, 0u, 0u, 0u};
    if constexpr (kBias) {
      const int col = tile.b_out0 + col_b + ((lane % kLanesPerRow) << 3);
      if (col < tile.b_out_lim)
        bias_chunk = *reinterpret_cast<const u32x4*>(static_cast<const bf16_t*>(p.bias) + tile.g * p.n + col);
    }
    // step 0 has landed: everything but step 1's loads and the previous epilogue's stores, which are younger
    wait_all_but((steps > 1 ? kStepLoads : 0) + stores_in_flight);
    if constexpr (kBias) asm volatile("" : "+v"(bias_chunk));
    workgroup_barrier();
    if (steps > 0) read_fragments(0, 0, 0, live);

    auto run = [&](auto full_tag) __attribute__((always_inline)) {
      constexpr bool kFull = decltype(full_tag)::value;
      auto mfmas = [&](int buf, int i0, int i1) __attribute__((always_inline)) {
#pragma unroll
        for (int i = i0; i < i1; ++i) {
          if (kFull || i < live) {
#pragma unroll
            for (int j = 0; j < kWN; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][j], fa[buf][i], acc[i][j], 0, 0, 0);
          }
        }
      };
      int cur = 0;  // the stage of this step: step % 3
      for (int step = 0; step < steps; ++step) {
        const bool more = step + 1 < steps, more2 = step + 2 < steps;
        const int nxt = cur == 2 ? 0 : cur + 1;
        const int nxt2 = nxt == 2 ? 0 : nxt + 1;
        if constexpr (kRowsPerStep) {
          // the row indices of the block of eight steps after this one, or of the next tile's first block while this
          // tile's last block runs; first in the step's burst, so that the step's wait covers them
          if ((step & 7) == 0) {
            const int block = step >> 3;
            if ((block + 1) * 8 < steps) {
              duo_load_rows(rows_area, lg.index_rsrc, tile.con_lim, block + 1, (slot0 + block + 1) & 1, wave, lane);
            } else if (has_next) {
              duo_load_rows(rows_area,
                                 make_rsrc_words(p.a_index + next.row_start, static_cast<uint32_t>(next.con_lim) * 8u),
                                 next.con_lim, 0, (slot0 + block + 1) & 1, wave, lane);
              next_rows0_loaded = true;
            }
          }
        }
        // the stage the previous step read is free since the barrier inside that step
        if (more2) issue_step(step + 2, nxt2);
        read_fragments(cur, 1, 1, kFull ? kWM : live);
        mfmas(0, 0, kWM);
        if constexpr (kFull) spread_reads_under_mfmas<kReads, kMfmas>();
        mfmas(1, 0, kWM / 2);
        __builtin_amdgcn_sched_barrier(0);
        // lgkmcnt(0): this stage is read out; vmcnt: the next step has landed (the loads complete in the order they
        // were issued, so the burst just issued may stay in flight)
        if (more2) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kStepLoads) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        workgroup_barrier();
        if (more) read_fragments(nxt, 0, 0, kFull ? kWM : live);
        mfmas(1, kWM / 2, kWM);
        if constexpr (kFull) spread_reads_under_mfmas<kReads, kMfmas / 2>();
        cur = nxt;
      }
    };
    if (live == kWM) run(std::true_type{});
    else run(std::false_type{});

    // every stage is free: request the next tile's first two steps before this tile's epilogue
    const TileInfo done = tile;
    t += sched.stride;
    if constexpr (kRowsPerStep) slot0 = (slot0 + ((steps + 7) >> 3)) & 1;
    if (has_next) {
      tile = next;
      begin_tile(tile, next_rows0_loaded);
    }

    // fwd, dgrad: the output descriptor spans this tile's rows only (as the A descriptor does)
    const int c_row0 = kMode == kWgrad ? 0 : done.a_out0;
    const int c_row_lim = kMode == kWgrad ? static_cast<int>(p.k) : done.a_out_lim - done.a_out0;
    bf16_t* c_base = kMode == kWgrad ? c + done.g * w_elems : c + (done.row_start + c_row0) * p.ldc;
    const int64_t c_rows = kMode == kWgrad ? p.k : (c_row_lim < DM ? c_row_lim : DM);
    const __amdgpu_buffer_rsrc_t c_rsrc = make_rsrc(c_base, static_cast<uint32_t>(c_rows * p.ldc * 2));
    __amdgpu_buffer_rsrc_t addend_rsrc = c_rsrc;
    if constexpr (kAddTo)
      addend_rsrc = make_rsrc(static_cast<const bf16_t*>(p.addend) + (done.row_start + c_row0) * p.ld_addend,
                              static_cast<uint32_t>(c_rows * p.ld_addend * 2));
    stores_in_flight = 0;
#pragma unroll
    for (int i = 0; i < kWM; ++i) {
      if (i < live) {
#pragma unroll
        for (int j = 0; j < kWN; ++j) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            uint2 packed;
            packed.x = pack_bf16x2(acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1]);
            packed.y = pack_bf16x2(acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]);
            // through inline assembly, like the tile loads: an LDS store the compiler can see makes it drain every
            // load in flight first
            asm volatile("ds_write_b64 %0, %1 offset:%2"
                         :
                         : "v"(stage_addr), "v"(packed), "n"((j * 32 + q * 8) * 2)
                         : "memory");
          }
        }
        __builtin_amdgcn_wave_barrier();  // the rows are private to the wavefront, whose LDS accesses stay in order
#pragma unroll
        for (int pass = 0; pass < 32 / kRowsPerPass; ++pass) {
          const int rr = pass * kRowsPerPass + lane / kLanesPerRow;
          const int cc = (lane % kLanesPerRow) << 3;
          const int row = (kMode == kWgrad ? done.a_out0 : 0) + row_a + i * 32 + rr;  // from the descriptor's first row
          const int col = done.b_out0 + col_b + cc;
          u32x4 v = *reinterpret_cast<const u32x4*>(stage_rows + (rr * kEpiPitch + cc) * 2);
          if constexpr (kBias) v = add_bf16x8(v, bias_chunk);
          if constexpr (kAddTo) {
            const uint32_t from = row < c_row_lim && col < done.b_out_lim
                                      ? static_cast<uint32_t>(row) * static_cast<uint32_t>(p.ld_addend) * 2u + col * 2u
                                      : kOutOfRange;
            const u32x4 base = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(addend_rsrc, from, 0, 0));
            v = scale_add_bf16x8(v, base, p.addend_scale);
          }
          const uint32_t off = row < c_row_lim && col < done.b_out_lim
                                   ? static_cast<uint32_t>(row) * static_cast<uint32_t>(p.ldc) * 2u + col * 2u
                                   : kOutOfRange;
          // a weight gradient is not read again before the optimizer: stored non-temporally
          __builtin_amdgcn_raw_buffer_store_b128(v, c_rsrc, off, 0, kMode == kWgrad ? 2 : 0);
        }
        __builtin_amdgcn_wave_barrier();
        stores_in_flight += 32 / kRowsPerPass;
      }
    }
  }
  wait_loads();  // no load may land in LDS after the workgroup has given it back
}

int duo_cus() {
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
  }
  return cus;
}

template <int kMode, typename Tile, int kGather = 0, bool kBias = false, bool kAddTo = false>
int launch_duo_instance(const GemmArgs& p, hipStream_t stream) {
  constexpr int DM = Tile::DM, DN = Tile::DN;
  const int64_t out_cols = kMode == kDgrad ? p.k : p.n;
  const int64_t nt = (out_cols + DN - 1) / DN;
  int64_t bound;  // no more workgroups than tiles
  if (kMode == kWgrad) bound = ((p.k + DM - 1) / DM) * nt * p.groups;
  else bound = (p.total_rows / DM + p.groups) * nt;
  int64_t workers = Tile::kWavesPerSimd * static_cast<int64_t>(duo_cus());
  if (bound < workers) workers = bound;
  workers = (workers + kXcds - 1) / kXcds * kXcds;
  if (workers <= 0) return HMOE_OK;
  constexpr size_t lds_bytes = Tile::kTiles + ((kMode == kWgrad && kGather) ? kDuoIndexArea : 0);
  auto kernel = grouped_gemm_duo_kernel<kMode, Tile, kGather, kBias, kAddTo>;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                          static_cast<int>(lds_bytes)) != hipSuccess)
    return HMOE_LAUNCH_FAILED;
  kernel<<<dim3(static_cast<unsigned>(workers)), dim3(64 * kDuoWaves), lds_bytes, stream>>>(p);
  if (hipGetLastError() != hipSuccess) return HMOE_LAUNCH_FAILED;
  return HMOE_OK;
}

template <typename Tile>
int launch_duo_tile(int mode, const GemmArgs& p, hipStream_t stream) {
  if (mode == kFwd) {
    return p.a_index ? (p.bias ? launch_duo_instance<kFwd, Tile, 1, true>(p, stream)
                               : launch_duo_instance<kFwd, Tile, 1>(p, stream))
           : p.bias  ? launch_duo_instance<kFwd, Tile, 0, true>(p, stream)
           : p.addend ? launch_duo_instance<kFwd, Tile, 0, false, true>(p, stream)
                      : launch_duo_instance<kFwd, Tile>(p, stream);
  }
  if (mode == kWgrad) {
    return !p.a_index   ? launch_duo_instance<kWgrad, Tile>(p, stream)
           : p.gather_b ? launch_duo_instance<kWgrad, Tile, 2>(p, stream)
                        : launch_duo_instance<kWgrad, Tile, 1>(p, stream);
  }
  if (mode == kDgrad) {
    return p.a_index  ? launch_duo_instance<kDgrad, Tile, 1>(p, stream)
           : p.addend ? launch_duo_instance<kDgrad, Tile, 0, false, true>(p, stream)
                      : launch_duo_instance<kDgrad, Tile>(p, stream);
  }
  return HMOE_UNSUPPORTED;
}

}  // namespace

int launch_duo(int mode, const GemmArgs& p, bool small_tile, hipStream_t stream) {
  return small_tile ? launch_duo_tile<DuoTile<2, 2>>(mode, p, stream) : launch_duo_tile<DuoTile<1, 4>>(mode, p, stream);
}

}  // namespace hmoe
