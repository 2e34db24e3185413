// Grouped GEMM for the MoE expert FFN on gfx950: forward, dgrad and wgrad over rows stacked by expert.
//
// Replaces torch's F.grouped_mm as the reference calls it (halo/kernels/grouped_mm.py:25-26, 39):
//   fwd    out[s:e]  = A[s:e]  @ B[g]          A [R,K],  B [G,K,N]
//   dgrad  dA[s:e]   = dO[s:e] @ B[g]^T        dO [R,N]
//   wgrad  dB[g]     = A[s:e]^T @ dO[s:e]      ragged contraction, empty group -> exact zeros
// with offs[g] the inclusive end of group g.  bf16 operands, fp32 accumulation on MFMA, one rounding.
//
// bf16 kernel (grouped_gemm_bf16_kernel).  One persistent launch; a workgroup of 8 wavefronts owns a 256 x 256 output
// tile and walks the contraction in steps of 64; each wavefront owns 4 x 2 accumulator blocks of 32 x 32
// (v_mfma_f32_32x32x16_bf16).  The tile is as large as the accumulators allow: the operand bytes that have to reach a
// compute unit per multiply-add fall with the tile's size, and the rate at which they arrive is what bounds these
// kernels; per contraction element a wavefront reads (4 + 2) * 32 operand values from LDS for 4 * 2 * 1024
// multiply-adds.
//  * Operand tiles go from global memory straight into LDS (buffer_load ... lds, 16 bytes per lane): no staging
//    registers, no ds_write, no register transposes.  Rows past a group's end and columns past an operand's edge come
//    back as zeros from the buffer bounds check, with no branches in the loop.  The loads are issued through inline
//    assembly and waited for explicitly (see lds_load16: the compiler would drain them before every transposing LDS
//    read).
//  * A contraction-contiguous operand lands as [256 rows][64 con] with the 16-byte chunk index XOR-ed with row & 7
//    (each lane fetches the chunk that belongs in its LDS slot); an MFMA fragment is one ds_read_b128, and the
//    fragments of other row blocks and contraction sub-steps are immediate offsets or one XOR away.
//  * An output-contiguous operand (B in fwd, both operands in wgrad) lands as it lies in memory, [64 con][256 out],
//    chunks XOR-ed with (con & 3) << 2, and a fragment is two ds_read_b64_tr_b16, the gfx950 transposing LDS read:
//    within 16 lanes, lane i supplies the address of row (i >> 2), columns 4 (i & 3)..+3 of a 4 x 16 patch and receives
//    the four rows of column i.
//  * Two LDS stages of A; the A loads of step k+1 are in flight during step k.  B has two stages in wgrad and three in
//    fwd and dgrad, where it is the weights, which every launch streams from HBM once: there the B tile of step k+2
//    is requested near the end of step k, so a weight line has a step and a half to arrive and two B refills are in
//    flight.  The five stages take all 160 KB of the LDS, so fwd and dgrad keep no tables there (RowTileWalk).
//    The fragments of sub-step kk+1 are read under
//    the MFMAs of sub-step kk, and the step's barrier sits in the middle of the last sub-step's MFMAs: the first
//    fragments of the next step are read behind it, under the rest.  The barrier is a bare s_barrier after an explicit
//    s_waitcnt: __syncthreads() would fence and drain loads that are meant to stay in flight.
//  * The MFMA is issued with the operands swapped (B fragment as srcA) so that a lane owns one output row and four
//    consecutive columns per accumulator quad.  The epilogue stages 32 rows per wavefront through LDS and writes whole
//    16-byte chunks with buffer stores; the next tile's first loads are issued before it.
//
// Tile schedule.  Every workgroup derives the group bounds and the per-group prefix of row tiles from offs (wgrad: as
// tables in LDS; fwd and dgrad: walking offs as the tiles go by), with no host readback, so ragged and empty groups
// cost exactly their tiles.  The logical tile order is group-major, then
// column tile, then row tile; it is cut into 8 contiguous chunks, one per XCD (workgroup w runs on XCD w % 8), so the
// workgroups that share an L2 work on the same expert's weights at the same time, and the tile count per XCD is
// balanced whatever the skew of the expert loads.  wgrad walks (group, column tile, row tile) the same way: dealt
// round-robin over all workgroups, neighbouring tiles landed on different XCDs and every operand row was fetched from
// HBM once per tile that uses it (4x the algorithmic bytes, measured).
//
// Gathered operand (template parameter kGather: 1 = A, 2 = wgrad's B).  The operand may be given as (array, row
// index): logical row r is array[index[r]].  With A gathered in fwd and wgrad this folds the reference's permute by
// expert (halo/kernels/moe_permute.py:130-141) into the first expert projection and its weight gradient; with the
// output gradient gathered in dgrad (A) and wgrad (B) the down projection's two gradients read grad_out[token of row]
// directly, so the combine's backward (moe_permute.py:44-72) writes no [R, H] gradient.  The direct-to-LDS load takes a
// per-lane offset, so a gathered row costs what a contiguous one does; see GatherDirect and GatherTransposed.
//
// Weights in block-scaled fp8 (grouped_gemm_staged_kernel, forward only) take the register-staged variant of the same
// tiling: global -> registers (dequantised there) -> LDS as [output index][64 contraction], both operands read back
// with ds_read_b128.
//
// Both operands in e4m3 (grouped_gemm_fp8_kernel, forward only): activations quantised per row and 128 values with
// power-of-two scales, weights with their 128 x 128 block scales, on v_mfma_scale_f32_32x32x64_f8f6f4, which takes each
// operand's scale as an exponent byte per lane.  Same tile and schedule; operands in panels of 64 contraction values,
// four LDS stages of 32 KB with three refills in flight, waited for by count.  Described where it is defined.
//
// fp32 operands take a plain LDS-tiled FMA kernel (the CPU-sized plumbing configuration and tests).
#include "gemm_shared.h"

#include <atomic>
#include <cstdlib>
#include <type_traits>

namespace hmoe {
namespace {


constexpr int BK = 64;  // contraction per step


// Tile configuration: GM x GN wavefronts, each WM x WN blocks of 32x32.
template <int GM_, int GN_, int WM_, int WN_>
struct Config {
  static constexpr int GM = GM_, GN = GN_, WM = WM_, WN = WN_;
  static constexpr int kThreads = 64 * GM * GN;
  static constexpr int BM = GM * WM * 32;  // output rows per tile (operand A's output index)
  static constexpr int BN = GN * WN * 32;  // output cols per tile (operand B's output index)
  static constexpr int kStage = (BM + BN) * BK;  // elements of one LDS stage (A tile then B tile)
};

__device__ __forceinline__ int swizzle(int row) { return (row & 7) ^ ((row >> 3) & 7); }
__device__ __forceinline__ int lds_offset(int row, int chunk) { return row * BK + ((chunk ^ swizzle(row)) << 3); }

// One operand tile's global -> register -> LDS path.  A loader describes the operand (a buffer resource bounded at
// the operand's end, row stride, first output index of the tile, limits) and moves one contraction step.
// kTrans == false: element(out, con) = base[out * ld + con]  (contraction contiguous); every thread of the
//                  workgroup moves kRows * 8 / kThreads 16-byte chunks.
// kTrans == true : element(out, con) = base[con * ld + out]  (output index contiguous), transposed on the way in;
//                  the kRows 8x8 blocks of a step are dealt to threads kFirst, kFirst + 1, ...
template <bool kTrans, int kRows, int kThreads, int kFirst>
struct Bf16Loader {
  static constexpr int kServing = kRows < kThreads ? kRows : kThreads;           // threads with transposing work
  static constexpr int kBlocks = kTrans ? (kRows + kServing - 1) / kServing : 1;  // 8x8 blocks per serving thread
  static constexpr int kChunks = kTrans ? 8 * kBlocks : kRows * 8 / kThreads;     // 16-byte loads per thread
  static constexpr int kOffsets = kTrans ? kBlocks : kChunks;
  static_assert(kTrans || (kRows * 8) % kThreads == 0, "tile rows must spread evenly over the workgroup");
  static_assert(!kTrans || kRows % kServing == 0, "transposed tile must spread evenly over its threads");

  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t voff[kOffsets];  // per chunk (direct) or per block (transposed) byte offset at contraction index 0
  uint32_t step_bytes;      // byte distance of one contraction step
  uint32_t row_bytes;       // transposed: byte distance of one contraction index
  int con_lim;
  bool serving;

  // `bytes` bounds the operand (rows past the group's end fall outside it).
  __device__ __forceinline__ void init(const bf16_t* base, int64_t ld, int64_t bytes, int out0, int out_lim,
                                       int con_lim_, int tid) {
    rsrc = make_rsrc(base, static_cast<uint32_t>(bytes));
    con_lim = con_lim_;
    if constexpr (!kTrans) {
      serving = true;
      step_bytes = BK * 2;
      row_bytes = 0;
#pragma unroll
      for (int i = 0; i < kChunks; ++i) {
        const int cid = tid + kThreads * i;
        const int out = out0 + (cid >> 3);
        voff[i] = out < out_lim ? static_cast<uint32_t>(out) * static_cast<uint32_t>(ld) * 2u + ((cid & 7) << 4)
                                : kOutOfRange;
      }
    } else {
      const int t = tid - kFirst;
      serving = t >= 0 && t < kServing;
      row_bytes = static_cast<uint32_t>(ld) * 2u;
      step_bytes = BK * row_bytes;
#pragma unroll
      for (int i = 0; i < kBlocks; ++i) {
        const int blk = t + kServing * i;
        const int ob = blk % (kRows / 8), cb = blk / (kRows / 8);
        const int out = out0 + (ob << 3);
        voff[i] = (serving && out < out_lim)
                      ? static_cast<uint32_t>(cb * 8) * row_bytes + static_cast<uint32_t>(out) * 2u
                      : kOutOfRange;
      }
    }
  }

  __device__ __forceinline__ void load(u32x4 (&reg)[kChunks], int step) const {
    const uint32_t soff = static_cast<uint32_t>(step) * step_bytes;
    if constexpr (!kTrans) {
#pragma unroll
      for (int i = 0; i < kChunks; ++i) {
        // only the last step can run past the contraction's end (con_lim is a multiple of 8)
        const int con = step * BK + (((threadIdx.x + kThreads * i) & 7) << 3);
        const uint32_t off = con < con_lim ? voff[i] : kOutOfRange;
        reg[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, soff, 0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < kBlocks; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j)  // rows past the contraction's end lie past the buffer's end
          reg[i * 8 + j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff[i] + j * row_bytes, soff, 0);
    }
  }

  // `tile` is the element offset of this operand's tile inside the workgroup's LDS array `smem` (an integer, so
  // every access stays an LDS instruction)
  __device__ __forceinline__ void store(const u32x4 (&reg)[kChunks], bf16_t* smem, int tile, int tid) const {
    if constexpr (!kTrans) {
#pragma unroll
      for (int i = 0; i < kChunks; ++i) {
        const int cid = tid + kThreads * i;
        *reinterpret_cast<u32x4*>(smem + tile + lds_offset(cid >> 3, cid & 7)) = reg[i];
      }
    } else {
      if (!serving) return;
      const int t = tid - kFirst;
#pragma unroll
      for (int i = 0; i < kBlocks; ++i) {
        const int blk = t + kServing * i;
        const int row0 = (blk % (kRows / 8)) << 3, chunk = blk / (kRows / 8);
        // reg[8i + c] holds contraction index c, output indices 0..7 (two per dword).  Row o of the 8x8 block
        // gathers output index o: dword w of the result packs contraction 2w (low half) and 2w+1 (high half).
#pragma unroll
        for (int o = 0; o < 8; ++o) {
          const uint32_t sel = (o & 1) ? 0x07060302u : 0x05040100u;
          u32x4 v;
          v.x = __builtin_amdgcn_perm(reg[8 * i + 1][o >> 1], reg[8 * i + 0][o >> 1], sel);
          v.y = __builtin_amdgcn_perm(reg[8 * i + 3][o >> 1], reg[8 * i + 2][o >> 1], sel);
          v.z = __builtin_amdgcn_perm(reg[8 * i + 5][o >> 1], reg[8 * i + 4][o >> 1], sel);
          v.w = __builtin_amdgcn_perm(reg[8 * i + 7][o >> 1], reg[8 * i + 6][o >> 1], sel);
          *reinterpret_cast<u32x4*>(smem + tile + lds_offset(row0 + o, chunk)) = v;
        }
      }
    }
  }
};

// e4m3fn weights [contraction, output] (output contiguous) with one power-of-two fp32 scale per 128x128 block,
// dequantised to bf16 (exactly: an e4m3 value times a power of two is a bf16 value) and transposed on the way into
// LDS.  Each 8-column block lies inside one scale column; a step spans one scale row (128 % BK == 0).
template <int kRows, int kThreads, int kFirst>
struct Fp8BlockLoader {
  static constexpr int kServing = kRows < kThreads ? kRows : kThreads;
  static constexpr int kBlocks = (kRows + kServing - 1) / kServing;
  static constexpr int kChunks = 4 * kBlocks;  // eight 8-byte loads per block, two per staging register
  static_assert(kRows % kServing == 0, "transposed tile must spread evenly over its threads");

  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t voff[kBlocks];
  uint32_t step_bytes, row_bytes;
  const float* scale[kBlocks];  // this block's scale column, at contraction block 0
  int scale_ld;
  float step_scale[kBlocks];
  bool serving;

  __device__ __forceinline__ void init(const uint8_t* base, int64_t ld, int64_t bytes, int out0, int out_lim,
                                       const float* group_scale, int scale_ld_, int tid) {
    rsrc = make_rsrc(base, static_cast<uint32_t>(bytes));
    const int t = tid - kFirst;
    serving = t >= 0 && t < kServing;
    row_bytes = static_cast<uint32_t>(ld);
    step_bytes = BK * row_bytes;
    scale_ld = scale_ld_;
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
      const int blk = t + kServing * i;
      const int ob = blk % (kRows / 8), cb = blk / (kRows / 8);
      const int out = out0 + (ob << 3);
      const bool ok = serving && out < out_lim;
      voff[i] = ok ? static_cast<uint32_t>(cb * 8) * row_bytes + static_cast<uint32_t>(out) : kOutOfRange;
      scale[i] = group_scale + (ok ? (out >> 7) : 0);
    }
  }

  __device__ __forceinline__ void load(u32x4 (&reg)[kChunks], int step) {
    const uint32_t soff = static_cast<uint32_t>(step) * step_bytes;
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
      step_scale[i] = serving ? scale[i][static_cast<int64_t>((step * BK) >> 7) * scale_ld] : 1.0f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const u32x2 lo = __builtin_amdgcn_raw_buffer_load_b64(rsrc, voff[i] + (2 * j) * row_bytes, soff, 0);
        const u32x2 hi = __builtin_amdgcn_raw_buffer_load_b64(rsrc, voff[i] + (2 * j + 1) * row_bytes, soff, 0);
        reg[i * 4 + j] = u32x4{lo.x, lo.y, hi.x, hi.y};  // contraction 2j in .xy, 2j+1 in .zw
      }
    }
  }

  __device__ __forceinline__ void store(const u32x4 (&reg)[kChunks], bf16_t* smem, int tile, int tid) const {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    if (!serving) return;
    const int t = tid - kFirst;
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
      const int blk = t + kServing * i;
      const int row0 = (blk % (kRows / 8)) << 3, chunk = blk / (kRows / 8);
      const float s = step_scale[i];
      uint32_t packed[8][4];  // [output][contraction pair]
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        float lo[8], hi[8];  // contraction 2w and 2w+1, outputs 0..7
        const u32x4 src = reg[i * 4 + w];
        const f32x2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(src.x, s, false);
        const f32x2 b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(src.x, s, true);
        const f32x2 c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(src.y, s, false);
        const f32x2 d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(src.y, s, true);
        lo[0] = a.x; lo[1] = a.y; lo[2] = b.x; lo[3] = b.y; lo[4] = c.x; lo[5] = c.y; lo[6] = d.x; lo[7] = d.y;
        const f32x2 e = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(src.z, s, false);
        const f32x2 f = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(src.z, s, true);
        const f32x2 g = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(src.w, s, false);
        const f32x2 h = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(src.w, s, true);
        hi[0] = e.x; hi[1] = e.y; hi[2] = f.x; hi[3] = f.y; hi[4] = g.x; hi[5] = g.y; hi[6] = h.x; hi[7] = h.y;
#pragma unroll
        for (int o = 0; o < 8; ++o)
          packed[o][w] =
              static_cast<uint32_t>(f32_to_bf16(lo[o])) | (static_cast<uint32_t>(f32_to_bf16(hi[o])) << 16);
      }
#pragma unroll
      for (int o = 0; o < 8; ++o)
        *reinterpret_cast<u32x4*>(smem + tile + lds_offset(row0 + o, chunk)) =
            u32x4{packed[o][0], packed[o][1], packed[o][2], packed[o][3]};
    }
  }
};

// C[a_out, b_out] = sum_con A(a_out, con) * B(b_out, con) over one BM x BN tile.
template <typename Cfg, typename LoaderA, typename LoaderB>
__device__ __forceinline__ void compute_tile(bf16_t* smem, LoaderA& la, LoaderB& lb, int a_out0,
                                             int a_out_lim, int b_out0, int b_out_lim, int con_lim,
                                             bf16_t* __restrict__ c_base, int64_t c_ld) {
  constexpr int WM = Cfg::WM, WN = Cfg::WN;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int gm = wave / Cfg::GN, gn = wave % Cfg::GN;
  constexpr int kTileB = Cfg::BM * BK;  // element offset of the B tile inside a stage
  constexpr int kStoreAfter = 1;        // contraction sub-step after which the staged tile is written to LDS

  u32x4 reg_a[LoaderA::kChunks];
  u32x4 reg_b[LoaderB::kChunks];
  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int steps = (con_lim + BK - 1) / BK;
  if (steps > 0) {
    la.load(reg_a, 0);
    lb.load(reg_b, 0);
    la.store(reg_a, smem, 0, tid);
    lb.store(reg_b, smem, kTileB, tid);
  }
  __syncthreads();
  const int row_a = gm * (WM * 32) + (lane & 31);
  const int row_b = gn * (WN * 32) + (lane & 31);
  // 32-row blocks of this wavefront that hold at least one valid output row: a group's last row tile is mostly empty,
  // and the blocks past its end are skipped (the wavefront still moves its share of the operand tiles)
  int live = (a_out_lim - (a_out0 + gm * (WM * 32)) + 31) >> 5;
  live = live < 0 ? 0 : (live > WM ? WM : live);

  auto run = [&](auto full_tag) {
    constexpr bool kFull = decltype(full_tag)::value;
    for (int step = 0; step < steps; ++step) {
      const int cur = step & 1;
      const bool more = step + 1 < steps;
      if (more) {
        la.load(reg_a, step + 1);
        lb.load(reg_b, step + 1);
      }
      const int ta = cur * Cfg::kStage;
      const int tb = ta + kTileB;
#pragma unroll
      for (int kk = 0; kk < BK / 16; ++kk) {
        const int chunk = kk * 2 + (lane >> 5);
        bf16x8 fa[WM], fb[WN];
#pragma unroll
        for (int j = 0; j < WN; ++j)
          fb[j] = *reinterpret_cast<const bf16x8*>(smem + tb + lds_offset(row_b + j * 32, chunk));
#pragma unroll
        for (int i = 0; i < WM; ++i) {
          if (kFull || i < live) {
            fa[i] = *reinterpret_cast<const bf16x8*>(smem + ta + lds_offset(row_a + i * 32, chunk));
#pragma unroll
            for (int j = 0; j < WN; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
          }
        }
        if (kk == kStoreAfter && more) {
          // the next stage's LDS writes go out between the MFMAs, not after them, so they overlap matrix work
          __builtin_amdgcn_sched_barrier(0);
          la.store(reg_a, smem, (cur ^ 1) * Cfg::kStage, tid);
          lb.store(reg_b, smem, (cur ^ 1) * Cfg::kStage + kTileB, tid);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      __syncthreads();
    }
  };
  if (live == WM) run(std::true_type{});
  else run(std::false_type{});
  // Epilogue.  After the swapped MFMA a lane owns output row (lane & 31) of each 32x32 block, and accumulator quad q
  // holds columns q*8 + (lane>>5)*4 .. +3: stored as they are, every store instruction would touch 32 different cache
  // lines with 16 bytes each.  Instead each wavefront passes its block through a private LDS region (the operand
  // stages are free after the last step's barrier), 64 rows at a time, and writes whole 16-byte chunks with the lanes
  // of a row segment contiguous: full lines per instruction.
  constexpr int kEpiPitch = WN * 32 + 8;               // elements per staged row (16 bytes of padding)
  constexpr int kEpiRegion = 64 * kEpiPitch;           // elements per wavefront
  constexpr int kLanesPerRow = WN * 4;                 // 16-byte chunks in a staged row
  constexpr int kRowsPerPass = 64 / kLanesPerRow;
  static_assert(kEpiRegion * Cfg::GM * Cfg::GN <= 2 * Cfg::kStage, "epilogue staging must fit in the operand stages");
  bf16_t* stage = smem + wave * kEpiRegion;
#pragma unroll
  for (int half = 0; half < (WM + 1) / 2; ++half) {
#pragma unroll
    for (int ii = 0; ii < 2; ++ii) {
      const int i = half * 2 + ii;
      if (i >= WM) break;
#pragma unroll
      for (int j = 0; j < WN; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          uint2 packed;
          packed.x = pack_bf16x2(acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1]);
          packed.y = pack_bf16x2(acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]);
          *reinterpret_cast<uint2*>(stage + (ii * 32 + (lane & 31)) * kEpiPitch + j * 32 + q * 8 + ((lane >> 5) << 2)) =
              packed;
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < 64 / kRowsPerPass; ++pass) {
      const int rr = pass * kRowsPerPass + lane / kLanesPerRow;
      const int cc = (lane % kLanesPerRow) << 3;
      const int row = a_out0 + gm * (WM * 32) + half * 64 + rr;
      const int col = b_out0 + gn * (WN * 32) + cc;
      if (half * 64 + rr < WM * 32 && row < a_out_lim && col < b_out_lim) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(stage + rr * kEpiPitch + cc);
        *reinterpret_cast<u32x4*>(c_base + static_cast<int64_t>(row) * c_ld + col) = v;
      }
    }
    __syncthreads();  // the region is rewritten by the next half, and by the next tile's first operand stage
  }
}

// Exclusive prefix of the per-group row-tile counts into LDS: tile_start[0..groups], by wavefront 0.
template <int BM>
__device__ __forceinline__ void build_tile_prefix(int32_t* tile_start, const int32_t* offs, int groups,
                                                  int64_t total_rows) {
  if (threadIdx.x < HMOE_WAVE) {
    const int lane = threadIdx.x;
    const int per = (groups + HMOE_WAVE - 1) / HMOE_WAVE;
    const int g0 = lane * per;
    int sum = 0;
    for (int g = g0; g < g0 + per && g < groups; ++g) {
      int64_t s, e;
      group_bounds(offs, g, total_rows, s, e);
      sum += static_cast<int>((e - s + BM - 1) / BM);
    }
    int incl = sum;
#pragma unroll
    for (int off = 1; off < HMOE_WAVE; off <<= 1) {
      const int up = __shfl_up(incl, off, HMOE_WAVE);
      if (lane >= off) incl += up;
    }
    int running = incl - sum;
    for (int g = g0; g < g0 + per && g < groups; ++g) {
      int64_t s, e;
      group_bounds(offs, g, total_rows, s, e);
      tile_start[g] = running;
      running += static_cast<int>((e - s + BM - 1) / BM);
    }
    if (lane == HMOE_WAVE - 1) tile_start[groups] = incl;
  }
  __syncthreads();
}

template <int kMode, typename Cfg>
__global__ void __launch_bounds__(Cfg::kThreads) grouped_gemm_staged_kernel(GemmArgs p) {
  extern __shared__ __attribute__((aligned(16))) bf16_t smem[];  // two stages of (A tile, B tile)
  __shared__ int32_t tile_start[kMode == kWgrad ? 1 : kMaxGroups + 1];
  constexpr int BM = Cfg::BM, BN = Cfg::BN, NT = Cfg::kThreads;
  const bf16_t* a = static_cast<const bf16_t*>(p.a);
  const bf16_t* b = static_cast<const bf16_t*>(p.b);
  bf16_t* c = static_cast<bf16_t*>(p.c);
  const int tid = threadIdx.x;

  const int workers = gridDim.x;
  const int xcd = blockIdx.x % kXcds;
  const int local = blockIdx.x / kXcds;
  const int workers_here = (workers - xcd + kXcds - 1) / kXcds;
  // the transposing loader of operand B takes the workgroup's last BN threads, so that in wgrad (both operands
  // transposed) the first threads move A's blocks and the last ones B's
  constexpr int kFirstB = BN < NT ? NT - BN : 0;

  if constexpr (kMode == kWgrad) {
    const int mt = static_cast<int>((p.k + BM - 1) / BM), nt = static_cast<int>((p.n + BN - 1) / BN);
    const int64_t per_group = static_cast<int64_t>(mt) * nt;
    const int64_t total = per_group * p.groups;
    for (int64_t t = blockIdx.x; t < total; t += workers) {  // interleaved: every worker sees every group size
      const int g = static_cast<int>(t / per_group);
      const int r = static_cast<int>(t - g * per_group);
      const int n_t = r / mt, m_t = r - n_t * mt;
      int64_t s, e;
      group_bounds(p.offs, g, p.total_rows, s, e);
      const int rows = static_cast<int>(e - s);
      Bf16Loader<true, BM, NT, 0> la;
      Bf16Loader<true, BN, NT, kFirstB> lb;
      la.init(a + s * p.lda, p.lda, rows * p.lda * 2, m_t * BM, static_cast<int>(p.k), rows, tid);
      lb.init(b + s * p.ldb, p.ldb, rows * p.ldb * 2, n_t * BN, static_cast<int>(p.n), rows, tid);
      compute_tile<Cfg>(smem, la, lb, m_t * BM, static_cast<int>(p.k), n_t * BN, static_cast<int>(p.n), rows,
                        c + static_cast<int64_t>(g) * p.k * p.n, p.ldc);
    }
  } else {
    build_tile_prefix<BM>(tile_start, p.offs, p.groups, p.total_rows);
    const int64_t out_cols = kMode == kDgrad ? p.k : p.n;
    const int con = static_cast<int>(kMode == kDgrad ? p.n : p.k);
    const int nt = static_cast<int>((out_cols + BN - 1) / BN);
    const int64_t total = static_cast<int64_t>(tile_start[p.groups]) * nt;
    const int64_t chunk = (total + kXcds - 1) / kXcds;
    const int64_t first = xcd * chunk;
    const int64_t last = first + chunk < total ? first + chunk : total;
    for (int64_t t = first + local; t < last; t += workers_here) {
      int lo = 0, hi = p.groups;  // largest g with tile_start[g] * nt <= t
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (static_cast<int64_t>(tile_start[mid]) * nt <= t) lo = mid; else hi = mid;
      }
      const int g = lo;
      const int mt = tile_start[g + 1] - tile_start[g];
      const int r = static_cast<int>(t - static_cast<int64_t>(tile_start[g]) * nt);
      const int n_t = r / mt, m_t = r - n_t * mt;
      int64_t s, e;
      group_bounds(p.offs, g, p.total_rows, s, e);
      const int rows = static_cast<int>(e - s);
      Bf16Loader<false, BM, NT, 0> la;
      la.init(a + s * p.lda, p.lda, rows * p.lda * 2, m_t * BM, rows, con, tid);
      const int64_t w_elems = p.k * p.n;
      if constexpr (kMode == kFwd) {
        Bf16Loader<true, BN, NT, kFirstB> lb;
        lb.init(b + g * w_elems, p.ldb, w_elems * 2, n_t * BN, static_cast<int>(p.n), con, tid);
        compute_tile<Cfg>(smem, la, lb, m_t * BM, rows, n_t * BN, static_cast<int>(p.n), con, c + s * p.ldc, p.ldc);
      } else if constexpr (kMode == kDgrad) {
        Bf16Loader<false, BN, NT, 0> lb;
        lb.init(b + g * w_elems, p.ldb, w_elems * 2, n_t * BN, static_cast<int>(p.k), con, tid);
        compute_tile<Cfg>(smem, la, lb, m_t * BM, rows, n_t * BN, static_cast<int>(p.k), con, c + s * p.ldc, p.ldc);
      } else {  // kFwdFp8W
        const int scale_ld = static_cast<int>((p.n + 127) >> 7);
        const int64_t scale_blocks = ((p.k + 127) >> 7) * scale_ld;
        Fp8BlockLoader<BN, NT, kFirstB> lb;
        lb.init(static_cast<const uint8_t*>(p.b) + g * w_elems, p.ldb, w_elems, n_t * BN, static_cast<int>(p.n),
                p.b_scale + g * scale_blocks, scale_ld, tid);
        compute_tile<Cfg>(smem, la, lb, m_t * BM, rows, n_t * BN, static_cast<int>(p.n), con, c + s * p.ldc, p.ldc);
      }
    }
  }
}

// The tile walk of one workgroup.  Tile ids only grow along the walk, so the group of a tile is found by scanning on
// from the previous tile's group.  Everything here is uniform across the workgroup and kept in scalar registers.
template <int kMode, int BM, int BN>
struct TileSchedule {
  const int32_t* grp_s;
  const int32_t* grp_e;
  const int32_t* tile_start;
  int nt, mt_w;
  int64_t per_group, first, last, stride;
  int k, n;

  __device__ __forceinline__ void init(const GemmArgs& p, const int32_t* s, const int32_t* e, const int32_t* ts) {
    grp_s = s;
    grp_e = e;
    tile_start = ts;
    k = static_cast<int>(p.k);
    n = static_cast<int>(p.n);
    mt_w = 1;
    per_group = 1;
    const int workers = gridDim.x;
    int64_t total;
    if constexpr (kMode == kWgrad) {
      mt_w = static_cast<int>((p.k + BM - 1) / BM);
      nt = static_cast<int>((p.n + BN - 1) / BN);
      per_group = static_cast<int64_t>(mt_w) * nt;
      total = per_group * p.groups;
    } else {
      const int64_t out_cols = kMode == kDgrad ? p.k : p.n;
      nt = static_cast<int>((out_cols + BN - 1) / BN);
      total = static_cast<int64_t>(__builtin_amdgcn_readfirstlane(tile_start[p.groups])) * nt;
    }
    // one contiguous chunk of the tile order per XCD (workgroup w runs on XCD w % 8): the workgroups that share an
    // L2 work on neighbouring tiles, which share operand rows
    const int xcd = blockIdx.x % kXcds;
    stride = (workers - xcd + kXcds - 1) / kXcds;
    if constexpr (kMode == kWgrad) {
      // A wgrad tile walks its group's rows, so tiles cost what their group holds: the chunks are cut at equal cost,
      // not at equal tile counts (with one expert holding a quarter of the rows, equal counts left one XCD with
      // twice the work of the others).
      const int64_t cost = per_group * static_cast<int64_t>(__builtin_amdgcn_readfirstlane(tile_start[p.groups]));
      first = p.groups > 0 ? cut(cost * xcd / kXcds, p.groups) + blockIdx.x / kXcds : 0;
      last = xcd + 1 == kXcds || p.groups == 0 ? total : cut(cost * (xcd + 1) / kXcds, p.groups);
    } else {
      const int64_t chunk = (total + kXcds - 1) / kXcds;
      first = xcd * chunk + blockIdx.x / kXcds;
      last = xcd * chunk + chunk < total ? xcd * chunk + chunk : total;
    }
  }

  // wgrad: the first tile whose predecessors cost `target` or more (tiles in order, a tile of group g costing
  // tile_start[g + 1] - tile_start[g])
  __device__ __forceinline__ int64_t cut(int64_t target, int groups) const {
    int lo = 0, hi = groups;  // the group the cut falls into: per_group * tile_start[g] <= target, largest such g
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (per_group * static_cast<int64_t>(__builtin_amdgcn_readfirstlane(tile_start[mid])) <= target) lo = mid;
      else hi = mid;
    }
    const int64_t before = per_group * static_cast<int64_t>(__builtin_amdgcn_readfirstlane(tile_start[lo]));
    const int64_t each = __builtin_amdgcn_readfirstlane(tile_start[lo + 1]) - __builtin_amdgcn_readfirstlane(tile_start[lo]);
    int64_t within = (target - before + each - 1) / each;
    if (within > per_group) within = per_group;
    return lo * per_group + within;
  }

  __device__ __forceinline__ TileInfo decode(int64_t t, int& cursor) const {
    int g, m_t, n_t;
    if constexpr (kMode == kWgrad) {
      g = static_cast<int>(t / per_group);
      const int r = static_cast<int>(t - g * per_group);
      n_t = r / mt_w;
      m_t = r - n_t * mt_w;
    } else {
      g = cursor;
      while (static_cast<int64_t>(__builtin_amdgcn_readfirstlane(tile_start[g + 1])) * nt <= t) ++g;
      cursor = g;
      const int ts = __builtin_amdgcn_readfirstlane(tile_start[g]);
      const int mt = __builtin_amdgcn_readfirstlane(tile_start[g + 1]) - ts;
      const int r = static_cast<int>(t - static_cast<int64_t>(ts) * nt);
      n_t = r / mt;
      m_t = r - n_t * mt;
    }
    const int s = __builtin_amdgcn_readfirstlane(grp_s[g]);
    const int rows = __builtin_amdgcn_readfirstlane(grp_e[g]) - s;
    TileInfo tile;
    tile.g = g;
    tile.row_start = s;
    tile.a_out0 = m_t * BM;
    tile.b_out0 = n_t * BN;
    if constexpr (kMode == kWgrad) {
      tile.a_out_lim = k;
      tile.b_out_lim = n;
      tile.con_lim = rows;
    } else {
      tile.a_out_lim = rows;
      tile.b_out_lim = kMode == kDgrad ? k : n;
      tile.con_lim = kMode == kDgrad ? n : k;
    }
    return tile;
  }
};

// ------------------------------------------------------------------------------- bf16 kernel, direct to LDS

template <int kI>
struct SlimDirect {  // element(out, con) = base[out * ld + con]; LDS [256 out][64 con], chunk ^= row & 7
  u32x4 rsrc;  // bounded at the operand's last output row: rows past it load as zeros
  uint32_t voff;                // this lane's chunk for the wavefront's first load of a step, at step 0
  uint32_t t_stride;            // bytes between the rows of consecutive loads (8 rows)
  int con0, con_lim;
  int t_lim;                    // loads t >= t_lim of this wavefront lie wholly past the operand's last row

  __device__ __forceinline__ void init(const bf16_t* base, int64_t ld, int64_t bytes, int out0, int out_lim,
                                       int con_lim_, int wave, int lane) {
    rsrc = make_rsrc_words(base, static_cast<uint32_t>(bytes));
    con_lim = con_lim_;
    t_lim = (out_lim - out0 - wave * kI * 8 + 7) >> 3;
    const int logical = (lane & 7) ^ (lane >> 3);  // row & 7 == lane >> 3 for every load
    con0 = logical << 3;
    t_stride = 8u * static_cast<uint32_t>(ld) * 2u;
    voff = static_cast<uint32_t>(out0 + wave * kI * 8 + (lane >> 3)) * static_cast<uint32_t>(ld) * 2u + (logical << 4);
  }
  // `live` false: the step lies past the contraction; the loads still issue (the schedule of the loop does not
  // change) but every offset is out of range, and the step offset stays below the buffer's size
  __device__ __forceinline__ void issue(__attribute__((address_space(3))) char* tile, int step, int wave,
                                        bool live = true) const {
    const uint32_t soff = live ? static_cast<uint32_t>(step) * (BK * 2) : 0u;
    const uint32_t base = live && step * BK + con0 < con_lim ? voff : kOutOfRange;
    // A load whose eight rows all lie past the operand's end is left out: nothing reads those rows of the tile
    // for a result that is kept (an output row takes its values from its own operand row only), and in a group's
    // last, short row tile most loads are of that kind.
    if (t_lim >= kI) {
#pragma unroll
      for (int t = 0; t < kI; ++t) lds_load16(rsrc, tile + (wave * kI + t) * 1024, base + t * t_stride, soff);
    } else {
#pragma unroll
      for (int t = 0; t < kI; ++t)
        if (t < t_lim) lds_load16(rsrc, tile + (wave * kI + t) * 1024, base + t * t_stride, soff);
    }
  }
  // every load of the step, absent rows included (they land as zeros): the same number of loads whatever the tile,
  // for a loop that waits for its loads by count
  __device__ __forceinline__ void issue_all(__attribute__((address_space(3))) char* tile, int step, int wave) const {
    const uint32_t soff = static_cast<uint32_t>(step) * (BK * 2);
    const uint32_t base = step * BK + con0 < con_lim ? voff : kOutOfRange;
#pragma unroll
    for (int t = 0; t < kI; ++t) lds_load16(rsrc, tile + (wave * kI + t) * 1024, base + t * t_stride, soff);
  }
  // per-lane byte address (within the operand tile) of the fragment of sub-step 0, block 0 of the wavefront
  static __device__ __forceinline__ int fragment_base(int row0, int lane) {
    return (row0 + (lane & 31)) * (BK * 2) + (((lane >> 5) ^ (lane & 7)) << 4);
  }
  // block b (32 rows further) and sub-step kk from there
  static __device__ __forceinline__ bf16x8 fragment(const char* tile, int base, int block, int kk) {
    return *reinterpret_cast<const bf16x8*>(tile + (base ^ (kk << 5)) + block * (32 * BK * 2));
  }
};

template <int kI, bool kRebase = false>
struct SlimTransposed {  // element(out, con) = base[con * ld + out]; LDS [64 con][256 out], chunk ^= (con & 3) << 2
  // With kRebase (wgrad, whose contraction walks every row of a group: more than 32 bits of bytes for a large one)
  // the descriptor is rebased every step: base + step * step_bytes in 64 bits, bounded at what is left of the operand
  // (or 2 GiB - 1), so that the per-lane offsets stay inside one step.  Without it (an expert's weight, below 2 GiB)
  // the descriptor is fixed and the step is a 32-bit offset.
  u32x4 rsrc;                   // !kRebase: bounded at the operand's last contraction row
  uint64_t base_address;        // kRebase
  int64_t extent;               // kRebase: bytes from the base to the operand's last contraction row
  uint32_t voff[2];             // even and odd loads of a step differ in (con & 3); pairs are 4 contraction rows apart
  uint32_t pair_stride, step_bytes;

  __device__ __forceinline__ void init(const bf16_t* base, int64_t ld, int64_t bytes, int out0, int out_lim,
                                       int /*con_lim*/, int wave, int lane) {
    static_assert(kI % 2 == 0, "loads come in even/odd pairs");
    if constexpr (kRebase) {
      base_address = reinterpret_cast<uint64_t>(base);
      extent = bytes;
    } else {
      rsrc = make_rsrc_words(base, static_cast<uint32_t>(bytes));
    }
    step_bytes = BK * static_cast<uint32_t>(ld) * 2u;
    pair_stride = 4u * static_cast<uint32_t>(ld) * 2u;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int con = (wave * kI + t) * 2 + (lane >> 5);
      const int logical = (lane & 31) ^ ((con & 3) << 2);
      const int out = out0 + (logical << 3);
      voff[t] = out < out_lim
                    ? static_cast<uint32_t>(con) * static_cast<uint32_t>(ld) * 2u + static_cast<uint32_t>(out) * 2u
                    : kOutOfRange;
    }
  }
  // the descriptor of one step
  __device__ __forceinline__ u32x4 step_rsrc(int step) const {
    if constexpr (!kRebase) return rsrc;
    const int64_t offset = static_cast<int64_t>(step) * step_bytes;
    int64_t left = extent - offset;
    left = left < 0 ? 0 : (left > 0x7fffffff ? 0x7fffffff : left);  // below kOutOfRange, which must stay out of range
    return make_rsrc_words(reinterpret_cast<const void*>(base_address + static_cast<uint64_t>(offset)),
                           static_cast<uint32_t>(left));
  }
  __device__ __forceinline__ void issue(__attribute__((address_space(3))) char* tile, int step, int wave,
                                        bool live = true) const {
    const u32x4 r = step_rsrc(live ? step : 0);
    const uint32_t soff = !kRebase && live ? static_cast<uint32_t>(step) * step_bytes : 0u;
    const uint32_t v0 = live ? voff[0] : kOutOfRange, v1 = live ? voff[1] : kOutOfRange;
#pragma unroll
    for (int t = 0; t < kI; ++t)
      lds_load16(r, tile + (wave * kI + t) * 1024, ((t & 1) ? v1 : v0) + (t >> 1) * pair_stride, soff);
  }
  __device__ __forceinline__ void issue_all(__attribute__((address_space(3))) char* tile, int step, int wave) const {
    issue(tile, step, wave, true);
  }
  // per-lane byte address of the fragment of sub-step 0 for block `block` of the wavefront (blocks do not reduce to
  // an immediate: the XOR reaches the bits the block index occupies)
  static __device__ __forceinline__ int fragment_base(int row0, int lane) {
    const int i = lane & 15, g = lane >> 4;
    const int out = row0 + ((g & 1) << 4) + ((i & 3) << 2);
    const int con = ((g >> 1) << 3) + (i >> 2);
    return (con * 256 + ((((out >> 3) ^ ((con & 3) << 2)) << 3) + (out & 7))) * 2;
  }
  static __device__ __forceinline__ bf16x8 fragment(const char* tile, int base, int /*block*/, int kk) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4* lds_ptr;
    const char* ptr = tile + base + kk * (16 * 256 * 2);
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(ptr));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(ptr + 4 * 256 * 2));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(bf16x8, both);
  }
};

// The two loaders again for an operand A whose rows are gathered: logical row r is base[index[r]] (the permute by
// expert folded into the GEMM: the direct-to-LDS load takes a per-lane offset, so a gathered row costs what a
// contiguous one does).  An index outside [0, a_rows) loads zeros.
template <int kI>
struct GatherDirect {  // LDS layout and fragments as SlimDirect
  u32x4 rsrc;
  uint32_t voff[kI];  // per load: this lane's chunk of its row at step 0, or out of range
  int con0, con_lim;
  int t_lim;          // as in SlimDirect

  __device__ __forceinline__ void init(const bf16_t* base, int64_t ld, int64_t a_rows, const int64_t* index, int out0,
                                       int out_lim, int con_lim_, int slot, int lane) {
    rsrc = make_rsrc_words(base, static_cast<uint32_t>(a_rows * ld * 2));
    con_lim = con_lim_;
    t_lim = (out_lim - out0 - slot * kI * 8 + 7) >> 3;
    const int logical = (lane & 7) ^ (lane >> 3);
    con0 = logical << 3;
#pragma unroll
    for (int t = 0; t < kI; ++t) {
      const int out = out0 + (slot * kI + t) * 8 + (lane >> 3);
      const int64_t row = out < out_lim ? index[out] : -1;
      voff[t] = row >= 0 && row < a_rows ? static_cast<uint32_t>(row) * static_cast<uint32_t>(ld) * 2u + (logical << 4)
                                         : kOutOfRange;
    }
  }
  __device__ __forceinline__ void issue(__attribute__((address_space(3))) char* tile, int step, int slot,
                                        bool live = true) const {
    const uint32_t soff = live ? static_cast<uint32_t>(step) * (BK * 2) : 0u;
    const bool in_range = live && step * BK + con0 < con_lim;
    if (t_lim >= kI) {
#pragma unroll
      for (int t = 0; t < kI; ++t)
        lds_load16(rsrc, tile + (slot * kI + t) * 1024, in_range ? voff[t] : kOutOfRange, soff);
    } else {
#pragma unroll
      for (int t = 0; t < kI; ++t)
        if (t < t_lim) lds_load16(rsrc, tile + (slot * kI + t) * 1024, in_range ? voff[t] : kOutOfRange, soff);
    }
  }
  static __device__ __forceinline__ int fragment_base(int row0, int lane) {
    return SlimDirect<kI>::fragment_base(row0, lane);
  }
  static __device__ __forceinline__ bf16x8 fragment(const char* tile, int base, int block, int kk) {
    return SlimDirect<kI>::fragment(tile, base, block, kk);
  }
};

// Gathered rows as contraction rows (wgrad): new rows every step.  The LDS tile is kept as eight panels of 32 output
// columns, [panel][64 con][32 out] with 64-byte rows, instead of SlimTransposed's [64 con][256 out]: a lane then
// stays on ONE contraction row for all of a step's loads (lane L: row L / 4 of the wavefront's 16, 16-byte chunk
// L % 4 of panel t in load t), so a step costs a lane one row index, one multiply and one add per load.  (With a
// load spanning two whole rows, as in SlimTransposed, every load needs its own pair of indices broadcast to the two
// half-wavefronts: 16 lane reads and 8 selects per step, which made this kernel 12 % slower than the plain one.)
// A load moves 16 rows x 64 bytes; loads t and t + 1 of a pair cover the two halves of the same 128-byte lines back
// to back.  The transposing read of a 32-column block touches 4 rows x 64 bytes per 32 lanes: every bank once,
// no swizzle.
template <int kI>
struct GatherTransposed {
  static_assert(kI == 8, "eight panels of 32 columns, one load per panel");
  u32x4 rsrc;
  u32x4 index_rsrc;  // the group's row indices, bounded at its last row
  uint32_t a_rows;
  uint32_t col;       // byte offset within a row of this lane's chunk in panel 0
  int t_lim;          // loads t < t_lim have this lane's chunk inside the operand
  uint32_t row_bytes;
  int con_lim;
  // The indices of a wavefront's 16 rows of a step (low words) are themselves fetched straight into LDS, one step
  // ahead, into the wavefront's own 2 x 1 KB (by step parity): a load into a register would have to be waited for,
  // and the compiler places that wait right behind the tile loads just issued.
  lds_bytes_ptr rows_area;
  int rows_valid0, rows_valid1;  // how many of the 16 rows exist, per parity

  __device__ __forceinline__ void init(const bf16_t* base, int64_t ld, int64_t a_rows_, const int64_t* index, int out0,
                                       int out_lim, int con_lim_, int /*slot*/, int lane) {
    rsrc = make_rsrc_words(base, static_cast<uint32_t>(a_rows_ * ld * 2));
    index_rsrc = make_rsrc_words(index, static_cast<uint32_t>(con_lim_) * 8u);
    a_rows = static_cast<uint32_t>(a_rows_);
    row_bytes = static_cast<uint32_t>(ld) * 2u;
    con_lim = con_lim_;
    const int chunk = lane & 3;
    col = static_cast<uint32_t>(out0) * 2u + chunk * 16u;
    const int chunks = (out_lim - out0 + 7) >> 3;  // 16-byte chunks of the operand from out0 on
    t_lim = (chunks - chunk + 3) >> 2;
  }
  // fetch the row indices of `step`
  __device__ __forceinline__ void load_rows(int step, int slot, int lane) {
    load_rows_of(index_rsrc, con_lim, step, slot, lane);
  }
  // the same for a group given by its index buffer and its row count (the next tile's, fetched ahead)
  __device__ __forceinline__ void load_rows_of(u32x4 group_index, int group_rows, int step, int slot, int lane) {
    const int first = step * BK + slot * 16;
    if (step & 1) rows_valid1 = group_rows - first;
    else rows_valid0 = group_rows - first;
    // lane l < 8 fetches indices first + 2l and first + 2l + 1; rows past the group's end read as 0 and are masked
    // on use
    lds_load16(group_index, rows_area + (step & 1) * 1024,
               first < group_rows && lane < 8 ? static_cast<uint32_t>(first + 2 * lane) * 8u : kOutOfRange, 0u);
  }
  // the loads of `step`, whose rows load_rows() fetched (and whose arrival the caller has waited for)
  __device__ __forceinline__ void issue(lds_bytes_ptr tile, int step, int slot, bool live = true) const {
    const int lane = threadIdx.x & 63;
    const int mine = lane >> 2;  // this lane's row among the wavefront's 16
    const uint32_t row = *reinterpret_cast<const __attribute__((address_space(3))) uint32_t*>(
        rows_area + (step & 1) * 1024 + mine * 8);  // the index's low word
    const int valid = (step & 1) ? rows_valid1 : rows_valid0;
    const uint32_t base = live && mine < valid && row < a_rows ? row * row_bytes + col : kOutOfRange;
#pragma unroll
    for (int t = 0; t < kI; ++t)  // an out-of-range base stays out of range with the panel's offset added
      lds_load16(rsrc, tile + t * 4096 + slot * 1024, t < t_lim ? base + t * 64 : kOutOfRange, 0u);
  }
  // per-lane byte address of the fragment of sub-step 0 for the 32-column block at row0 (a multiple of 32)
  static __device__ __forceinline__ int fragment_base(int row0, int lane) {
    const int i = lane & 15, g = lane >> 4;
    const int out = row0 + ((g & 1) << 4) + ((i & 3) << 2);
    const int con = ((g >> 1) << 3) + (i >> 2);
    return (out >> 5) * 4096 + con * 64 + (out & 31) * 2;
  }
  static __device__ __forceinline__ bf16x8 fragment(const char* tile, int base, int /*block*/, int kk) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4* lds_ptr;
    const char* ptr = tile + base + kk * (16 * 64);
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(ptr));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(ptr + 4 * 64));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(bf16x8, both);
  }
};

// Scheduling hint for a region of kReads LDS reads and kMfmas MFMAs: spread the reads evenly under the MFMAs.
template <int kReads, int kMfmas, int kLoads = 0>
__device__ __forceinline__ void interleave_reads_under_mfmas() {
  if constexpr (kLoads > 0 && kLoads <= kMfmas && kReads <= kMfmas) {
    // one global->LDS load behind each of the first MFMAs, LDS reads behind every (kMfmas / kReads)-th
    constexpr int every = kMfmas / kReads;
#pragma unroll
    for (int m = 0; m < kMfmas; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (m < kLoads) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      if (m % every == every - 1 && m / every < kReads) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
  } else if constexpr (kReads <= kMfmas) {
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


template <int kMode, typename Cfg, int kGather = 0, bool kBias = false, bool kAddTo = false>
__global__ void __launch_bounds__(Cfg::kThreads) grouped_gemm_bf16_kernel(GemmArgs p) {
  static_assert(!kAddTo || ((kMode == kFwd || kMode == kDgrad) && !kBias && !kGather),
                "the scaled sum into an addend belongs to the plain forward and the plain input gradient");
  static_assert(Cfg::BM == 256 && Cfg::BN == 256, "the direct-to-LDS loaders move 256-row tiles");
  static_assert(!kBias || kMode == kFwd, "the expert bias belongs to the forward product");
  static_assert(kGather >= 0 && kGather <= 2 && (kGather != 2 || kMode == kWgrad), "B is gathered in wgrad only");
  constexpr bool kGatherA = kGather == 1, kGatherB = kGather == 2;
  constexpr int WM = Cfg::WM, WN = Cfg::WN, BM = Cfg::BM, BN = Cfg::BN;
  constexpr int kWaves = Cfg::GM * Cfg::GN;
  // Wavefronts 0-3 issue all the tile loads and wait for them (16 loads of 1 KB each per step, measured slightly
  // ahead of dealing them to every wavefront); every wavefront runs the MFMAs.
  constexpr int kLoadWaves = 4;
  constexpr int kI = 32 / kLoadWaves;
  constexpr bool kDirectA = kMode != kWgrad, kDirectB = kMode == kDgrad;
  using PlainA = typename std::conditional<kDirectA, SlimDirect<kI>, SlimTransposed<kI, true>>::type;
  using GatheredA = typename std::conditional<kDirectA, GatherDirect<kI>, GatherTransposed<kI>>::type;
  using LoaderA = typename std::conditional<kGatherA, GatheredA, PlainA>::type;
  using PlainB = typename std::conditional<kDirectB, SlimDirect<kI>, SlimTransposed<kI, kMode == kWgrad>>::type;
  using LoaderB = typename std::conditional<kGatherB, GatherTransposed<kI>, PlainB>::type;
  // the gathered rows are contraction rows (wgrad): new ones every step
  constexpr bool kRowsPerStep = (kGatherA && !kDirectA) || kGatherB;
  // fwd and dgrad keep operand B (the weights, which every launch streams from HBM once) on THREE stages and A on
  // two: the B tile of step s + 2 is requested while step s runs, so two B refills are in flight and a weight line has
  // two steps to arrive instead of one.  That takes all 160 KB of the LDS (A0 | B0 | B1 | A1 | B2, 32 KB each), so
  // these modes hold no tables there: the tile walk reads offs itself.  wgrad keeps two stages of (A, B) and its tables.
  constexpr bool kRingB = kMode != kWgrad;
  using Sched = typename std::conditional<kRingB, RowTileWalk<kMode, BM, BN>, TileSchedule<kMode, BM, BN>>::type;
  extern __shared__ __attribute__((aligned(16))) char lds_raw[];
  auto lds = (__attribute__((address_space(3))) char*)lds_raw;
  constexpr int kTileBytes = 256 * BK * 2, kStageBytes = 2 * kTileBytes;
  // byte offsets of A stage i (0, 1) and B stage j (0, 1; 2 with the ring)
  auto a_off = [](int i) { return kRingB ? i * (3 * kTileBytes) : i * kStageBytes; };
  auto b_off = [](int j) { return kRingB ? (j == 2 ? 4 * kTileBytes : (j + 1) * kTileBytes) : j * kStageBytes + kTileBytes; };
  constexpr int kEpiBase = kRingB ? 3 * kTileBytes : kStageBytes;  // the epilogue stages through A1 (and B2)
  bf16_t* c = static_cast<bf16_t*>(p.c);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int gm = wave / Cfg::GN, gn = wave % Cfg::GN;
  const int row_a = gm * (WM * 32), row_b = gn * (WN * 32);
  const bool load_wave = wave < kLoadWaves;
  const int load_slot = wave & (kLoadWaves - 1);

  Sched sched;
  if constexpr (!kRingB) {
    // tile_start: per group, the prefix of its tiles' cost (contraction steps + 1 per tile, the same for every tile
    // of a group)
    __shared__ int32_t grp_s[kMaxGroups], grp_e[kMaxGroups], tile_start[kMaxGroups + 1];
    // ---- group bounds and the cost prefix, by wavefront 0
    if (wave == 0) {
      const int per = (p.groups + HMOE_WAVE - 1) / HMOE_WAVE;
      const int g0 = lane * per;
      int sum = 0;
      for (int g = g0; g < g0 + per && g < p.groups; ++g) {
        int64_t s, e;
        group_bounds(p.offs, g, p.total_rows, s, e);
        grp_s[g] = static_cast<int32_t>(s);
        grp_e[g] = static_cast<int32_t>(e);
        sum += static_cast<int>((e - s + BK - 1) / BK) + 1;
      }
      int incl = sum;
#pragma unroll
      for (int off = 1; off < HMOE_WAVE; off <<= 1) {
        const int up = __shfl_up(incl, off, HMOE_WAVE);
        if (lane >= off) incl += up;
      }
      int running = incl - sum;
      for (int g = g0; g < g0 + per && g < p.groups; ++g) {
        tile_start[g] = running;
        running += (grp_e[g] - grp_s[g] + BK - 1) / BK + 1;
      }
      if (lane == HMOE_WAVE - 1) tile_start[p.groups] = incl;
    }
    __syncthreads();
    sched.init(p, grp_s, grp_e, tile_start);
  } else {
    // ---- the number of row tiles over all groups and the group of this workgroup's first tile, by wavefront 0;
    // handed to the other wavefronts through the first words of the (still unused) operand stages
    int32_t* handoff = reinterpret_cast<int32_t*>(lds_raw);
    if (wave == 0) {
      const int per = (p.groups + HMOE_WAVE - 1) / HMOE_WAVE;
      const int g0 = lane * per;
      int sum = 0;
      for (int g = g0; g < g0 + per && g < p.groups; ++g) {
        int64_t s, e;
        group_bounds(p.offs, g, p.total_rows, s, e);
        sum += static_cast<int>((e - s + BM - 1) / BM);
      }
      int incl = sum;
#pragma unroll
      for (int off = 1; off < HMOE_WAVE; off <<= 1) {
        const int up = __shfl_up(incl, off, HMOE_WAVE);
        if (lane >= off) incl += up;
      }
      const int total = __shfl(incl, HMOE_WAVE - 1, HMOE_WAVE);
      const int64_t out_cols = kMode == kDgrad ? p.k : p.n;
      const int nt = static_cast<int>((out_cols + BN - 1) / BN);
      int64_t first, last;
      Sched::chunk_of(static_cast<int64_t>(total) * nt, first, last);
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
          const int mt = static_cast<int>((e - s + BM - 1) / BM);
          if (q < running + mt) {
            handoff[1] = g;
            handoff[2] = running;
            break;
          }
          running += mt;
        }
      }
    }
    __syncthreads();
    const int total = __builtin_amdgcn_readfirstlane(handoff[0]);
    const int g_first = __builtin_amdgcn_readfirstlane(handoff[1]);
    const int ts_first = __builtin_amdgcn_readfirstlane(handoff[2]);
    __syncthreads();  // the words are read before the first tile loads land on them
    sched.init(p, total, g_first, ts_first);
  }
  const int64_t w_elems = p.k * p.n;

  LoaderA la;
  LoaderB lb;
  auto& lg = *[&]() { if constexpr (kGatherB) return &lb; else return &la; }();  // the gathered operand's loader
  if constexpr (kRowsPerStep) lg.rows_area = lds + 2 * kStageBytes + load_slot * 2048;
  int cursor = 0;
  // describe tile `t`'s operands to the loaders and start its first step into stage 0
  // `rows0_loaded`: the gathered contraction rows of its step 0 were fetched during the previous tile's last step
  auto begin_tile = [&](const TileInfo& tile, bool rows0_loaded) __attribute__((always_inline)) {
    const bf16_t* a = static_cast<const bf16_t*>(p.a);
    const bf16_t* b = static_cast<const bf16_t*>(p.b);
    const int64_t rows = kMode == kWgrad ? tile.con_lim : tile.a_out_lim;
    if constexpr (kGatherA) {
      if (load_wave)  // the row indices are fetched by the lanes that use them
        la.init(a, p.lda, p.a_rows, p.a_index + tile.row_start, tile.a_out0, tile.a_out_lim, tile.con_lim, load_slot,
                lane);
    } else if constexpr (kMode == kWgrad) {
      la.init(a + tile.row_start * p.lda, p.lda, rows * p.lda * 2, tile.a_out0, tile.a_out_lim, tile.con_lim,
              load_slot, lane);
    } else {
      // the descriptor starts at the tile's first row and ends at its last, so its 32-bit offsets span one tile
      // whatever the operand's or the group's size
      const int rows_left = tile.a_out_lim - tile.a_out0;
      la.init(a + (tile.row_start + tile.a_out0) * p.lda, p.lda, (rows_left < BM ? rows_left : BM) * p.lda * 2, 0,
              rows_left, tile.con_lim, load_slot, lane);
    }
    if constexpr (kGatherB) {
      if (load_wave)
        lb.init(b, p.ldb, p.a_rows, p.a_index + tile.row_start, tile.b_out0, tile.b_out_lim, tile.con_lim, load_slot,
                lane);
    } else if constexpr (kMode == kWgrad)
      lb.init(b + tile.row_start * p.ldb, p.ldb, rows * p.ldb * 2, tile.b_out0, tile.b_out_lim, tile.con_lim,
              load_slot, lane);
    else
      lb.init(b + tile.g * w_elems, p.ldb, w_elems * 2, tile.b_out0, tile.b_out_lim, tile.con_lim, load_slot, lane);
    if (load_wave) {
      if constexpr (kRowsPerStep) {
        if (!rows0_loaded) {
          lg.load_rows(0, load_slot, lane);
          wait_loads();
        }
      }
      if (tile.con_lim > 0) {
        la.issue(lds + a_off(0), 0, load_slot);
        if constexpr (kRingB) {
          lb.issue_all(lds + b_off(0), 0, load_slot);
          if (tile.con_lim > BK) lb.issue_all(lds + b_off(1), 1, load_slot);
        } else {
          lb.issue(lds + b_off(0), 0, load_slot);
        }
      }
      if constexpr (kRowsPerStep) lg.load_rows(1, load_slot, lane);
    }
  };

  // ---- fragment addresses
  int fa_base[kDirectA ? 1 : WM], fb_base[kDirectB ? 1 : WN];
  if constexpr (kDirectA) fa_base[0] = LoaderA::fragment_base(row_a, lane);
  else
#pragma unroll
    for (int i = 0; i < WM; ++i) fa_base[i] = LoaderA::fragment_base(row_a + i * 32, lane);
  if constexpr (kDirectB) fb_base[0] = LoaderB::fragment_base(row_b, lane);
  else
#pragma unroll
    for (int j = 0; j < WN; ++j) fb_base[j] = LoaderB::fragment_base(row_b + j * 32, lane);
  bf16x8 fa[2][WM], fb[2][WN];
  auto read_fragments = [&](int a_stage, int b_stage, int kk, int buf) __attribute__((always_inline)) {
    const char* ta = lds_raw + a_off(a_stage);
    const char* tb = lds_raw + b_off(b_stage);
#pragma unroll
    for (int j = 0; j < WN; ++j) fb[buf][j] = LoaderB::fragment(tb, fb_base[kDirectB ? 0 : j], j, kk);
#pragma unroll
    for (int i = 0; i < WM; ++i) fa[buf][i] = LoaderA::fragment(ta, fa_base[kDirectA ? 0 : i], i, kk);
  };
  // the same for a tile whose last rows are missing: only the fragments of the `rows_live` row blocks that hold
  // rows (a short tile's steps are otherwise bound by these reads: 64 per sub-step and CU whatever the row count)
  auto read_live_fragments = [&](int a_stage, int b_stage, int kk, int buf, int rows_live)
                                 __attribute__((always_inline)) {
    const char* ta = lds_raw + a_off(a_stage);
    const char* tb = lds_raw + b_off(b_stage);
    if (rows_live > 0) {
#pragma unroll
      for (int j = 0; j < WN; ++j) fb[buf][j] = LoaderB::fragment(tb, fb_base[kDirectB ? 0 : j], j, kk);
    }
#pragma unroll
    for (int i = 0; i < WM; ++i)
      if (i < rows_live) fa[buf][i] = LoaderA::fragment(ta, fa_base[kDirectA ? 0 : i], i, kk);
  };
  // fp8: a fragment of the 32x32x64 MFMA is two 16-byte reads, the chunks sub-steps 2 h and 2 h + 1 of the bf16
  // geometry would take.  Which 32 of the 64 values a lane holds does not matter to the product as long as both
  // operands agree, and here it does not matter to the scales either: a step is one scale block.
  constexpr int kReads = WM * (kDirectA ? 1 : 2) + WN * (kDirectB ? 1 : 2);  // LDS reads of one sub-step
  constexpr int kMfmas = WM * WN;
  constexpr int kEpiPitch = WN * 32 + 8;
  constexpr int kEpiRegion = 32 * kEpiPitch;
  constexpr int kLanesPerRow = WN * 4;
  constexpr int kRowsPerPass = 64 / kLanesPerRow;
  static_assert(kEpiRegion * kWaves * 2 <= kStageBytes, "epilogue staging must fit in one stage");
  const char* stage_rows = lds_raw + kEpiBase + wave * kEpiRegion * 2;
  const uint32_t stage_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + kEpiBase +
                              static_cast<uint32_t>((wave * kEpiRegion + (lane & 31) * kEpiPitch + ((lane >> 5) << 2)) * 2);

  int64_t t = sched.first;
  TileInfo tile, next;
  if (t < sched.last) {
    tile = sched.decode(t, cursor);
    begin_tile(tile, false);
  }
  while (t < sched.last) {
    const bool has_next = t + sched.stride < sched.last;
    if (has_next) next = sched.decode(t + sched.stride, cursor);
    bool next_rows0_loaded = false;
    f32x16 acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    const int steps = (tile.con_lim + BK - 1) / BK;
    int live = (tile.a_out_lim - (tile.a_out0 + row_a) + 31) >> 5;
    live = live < 0 ? 0 : (live > WM ? WM : live);
    // a wavefront whose columns all lie past the operand's edge (the last column tile of a width that is no multiple
    // of 256) has nothing to multiply either: its blocks would be products with zeros that are never stored
    if (tile.b_out0 + row_b >= tile.b_out_lim) live = 0;
    // The expert's bias for this lane's eight output columns (the same columns in every store of the epilogue).  It
    // is fetched here, where the tile's first loads are waited for anyway, and pinned as arrived right behind that
    // wait: a wait placed by the compiler at its first use, in the epilogue, would be for every load in flight, the
    // next tile's first step among them.
    u32x4 bias_chunk = {0u, 0u, 0u, 0u};
    if constexpr (kBias) {
      const int col = tile.b_out0 + row_b + ((lane % kLanesPerRow) << 3);
      if (col < tile.b_out_lim)
        bias_chunk = *reinterpret_cast<const u32x4*>(static_cast<const bf16_t*>(p.bias) + tile.g * p.n + col);
    }
    if (load_wave) wait_loads();
    if constexpr (kBias) asm volatile("" : "+v"(bias_chunk));
    workgroup_barrier();  // step 0 of this tile has landed in stage 0
    if (steps > 0) read_live_fragments(0, 0, 0, 0, live);

    auto run = [&](auto full_tag) __attribute__((always_inline)) {
      constexpr bool kFull = decltype(full_tag)::value;
      auto mfmas = [&](int buf, int i0, int i1) __attribute__((always_inline)) {
#pragma unroll
        for (int i = i0; i < i1; ++i) {
          if (kFull || i < live) {
#pragma unroll
            for (int j = 0; j < WN; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][j], fa[buf][i], acc[i][j], 0, 0, 0);
          }
        }
      };
      int b_cur = 0;  // operand B's stage of this step: step % 3 with the ring, step & 1 without
      for (int step = 0; step < steps; ++step) {
        const int cur = step & 1;
        const bool more = step + 1 < steps;
        const int b_next = kRingB ? (b_cur == 2 ? 0 : b_cur + 1) : cur ^ 1;
        const bool more2 = kRingB && step + 2 < steps;
        // the other A stage is free since the barrier inside the previous step, and so is the B stage that step read;
        // past the last step the A loads are issued all the same, out of range, so that the loop has one shape
        if (load_wave) {
          la.issue(lds + a_off(cur ^ 1), step + 1, load_slot, more);
          if constexpr (!kRingB) lb.issue(lds + b_off(cur ^ 1), step + 1, load_slot, more);
          // the rows of the step after that: their indices arrive under this step, with its tile loads; in the
          // tile's last step that is the next tile's first
          if constexpr (kRowsPerStep) {
            if (more) lg.load_rows(step + 2, load_slot, lane);
            else if (has_next)
              lg.load_rows_of(make_rsrc_words(p.a_index + next.row_start, static_cast<uint32_t>(next.con_lim) * 8u),
                              next.con_lim, 0, load_slot, lane);
          }
        }
        if constexpr (kRowsPerStep) next_rows0_loaded = !more && has_next;
#pragma unroll
        for (int kk = 0; kk < 3; ++kk) {
          if constexpr (kFull) read_fragments(cur, b_cur, kk + 1, (kk + 1) & 1);
          else read_live_fragments(cur, b_cur, kk + 1, (kk + 1) & 1, live);
          mfmas(kk & 1, 0, WM);
          if constexpr (kFull) {
            interleave_reads_under_mfmas<kReads, kMfmas>();
          }
        }
        mfmas(1, 0, WM / 2);
        __builtin_amdgcn_sched_barrier(0);
        // With the ring, B of the step after next goes out here, into the stage the previous step read: behind this
        // wavefront's MFMAs rather than ahead of them (a loading wavefront sits in the address unit's queue for the
        // length of its burst; at the top of the step that delayed its first MFMA by as much, and this burst is
        // waited for by nobody before the next step's end).
        if constexpr (kRingB) {
          if (load_wave && more2) lb.issue_all(lds + b_off(b_next == 2 ? 0 : b_next + 1), step + 2, load_slot);
        }
        // lgkmcnt(0): this stage is read out; vmcnt where tile loads were issued: the next step has landed.  The
        // loads complete in the order they were issued, so with the ring the newest kI (the burst above) may stay
        // in flight.
        if (load_wave) {
          if (more2) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kI) : "memory");
          else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        } else {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
        workgroup_barrier();
        if (more) {
          if constexpr (kFull) read_fragments(cur ^ 1, b_next, 0, 0);
          else read_live_fragments(cur ^ 1, b_next, 0, 0, live);
        }
        mfmas(1, WM / 2, WM);
        if constexpr (kFull) interleave_reads_under_mfmas<kReads, kMfmas / 2>();
        b_cur = b_next;
      }
    };
    if (live == WM) run(std::true_type{});
    else run(std::false_type{});

    // both stages are free: start the next tile's first step into stage 0 before this tile's epilogue
    const TileInfo done = tile;
    t += sched.stride;
    if (has_next) {
      tile = next;
      begin_tile(tile, next_rows0_loaded);
    }

    // epilogue through the second stage: 32 rows at a time per wavefront, whole 16-byte chunks out
    // fwd, dgrad: the output descriptor spans this tile's rows only (as the A descriptor does)
    const int c_row0 = kMode == kWgrad ? 0 : done.a_out0;
    const int c_row_lim = kMode == kWgrad ? static_cast<int>(p.k) : done.a_out_lim - done.a_out0;
    bf16_t* c_base = kMode == kWgrad ? c + done.g * w_elems : c + (done.row_start + c_row0) * p.ldc;
    const int64_t c_rows = kMode == kWgrad ? p.k : (c_row_lim < BM ? c_row_lim : BM);
    const __amdgpu_buffer_rsrc_t c_rsrc = make_rsrc(c_base, static_cast<uint32_t>(c_rows * p.ldc * 2));
    __amdgpu_buffer_rsrc_t addend_rsrc = c_rsrc;
    if constexpr (kAddTo)
      addend_rsrc = make_rsrc(static_cast<const bf16_t*>(p.addend) + (done.row_start + c_row0) * p.ld_addend,
                              static_cast<uint32_t>(c_rows * p.ld_addend * 2));
#pragma unroll
    for (int i = 0; i < WM; ++i) {
      if (i < live) {
#pragma unroll
        for (int j = 0; j < WN; ++j) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            uint2 packed;
            packed.x = pack_bf16x2(acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1]);
            packed.y = pack_bf16x2(acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]);
            // Written through inline assembly on purpose: before an LDS store it can see, the compiler drains every
            // direct-to-LDS load in flight (it cannot tell that these rows are not their target), which here would
            // wait for the next tile's first step.
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
          const int col = done.b_out0 + row_b + cc;
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
          // a weight gradient is not read again before the optimizer: stored non-temporally, it leaves the L2's
          // lines to the operands (measured: the two weight-gradient launches of a step 3-4 % faster; the forward
          // and input-gradient outputs are read by the next kernel and keep the default policy)
          __builtin_amdgcn_raw_buffer_store_b128(v, c_rsrc, off, 0, kMode == kWgrad ? 2 : 0);
        }
        __builtin_amdgcn_wave_barrier();
      }
    }
  }
  wait_loads();  // no load may land in LDS after the workgroup has given it back
}

#define HMOE_BF16_INSTANCE(mode) \
  template __global__ void grouped_gemm_bf16_kernel<mode, Config<2, 4, 4, 2>>(GemmArgs);
HMOE_BF16_INSTANCE(kFwd)
HMOE_BF16_INSTANCE(kDgrad)
HMOE_BF16_INSTANCE(kWgrad)
#undef HMOE_BF16_INSTANCE
template __global__ void grouped_gemm_bf16_kernel<kFwd, Config<2, 4, 4, 2>, 1>(GemmArgs);
template __global__ void grouped_gemm_bf16_kernel<kFwd, Config<2, 4, 4, 2>, 0, true>(GemmArgs);
template __global__ void grouped_gemm_bf16_kernel<kFwd, Config<2, 4, 4, 2>, 0, false, true>(GemmArgs);
template __global__ void grouped_gemm_bf16_kernel<kFwd, Config<2, 4, 4, 2>, 1, true>(GemmArgs);
template __global__ void grouped_gemm_bf16_kernel<kDgrad, Config<2, 4, 4, 2>, 0, false, true>(GemmArgs);
template __global__ void grouped_gemm_bf16_kernel<kDgrad, Config<2, 4, 4, 2>, 1>(GemmArgs);
template __global__ void grouped_gemm_bf16_kernel<kWgrad, Config<2, 4, 4, 2>, 1>(GemmArgs);
template __global__ void grouped_gemm_bf16_kernel<kWgrad, Config<2, 4, 4, 2>, 2>(GemmArgs);

// ------------------------------------------------------------------------------------------------ fp32 path
// 64x64 tile, contraction step 16, 256 threads each owning a 4x4 block.  grid.x walks row tiles of every group
// (an upper bound of ceil(R/64)+G tiles; surplus workgroups exit), grid.y column tiles.
// ------------------------------------------------------------------- fp8 kernel, four stages of 64 contraction bytes
// Both operands e4m3 in panels of 64 contraction values (A [K/64][a_rows][64], B [G][K/64][N][64]); a stage is one
// panel's share of a 256 x 256 tile, 16 KB per operand, and four stages are resident, so that three refills are in
// flight while one stage is computed.  (With two stages of 64 KB one refill is in flight, and the step then takes as
// long as the slowest line of that refill: the latency of a miss under load, about 1.5 us, whatever the hit rate.)
// The scales travel with their stage: the rows' e8m0 bytes and the two weight scales of the tile's column blocks are
// loaded into LDS beside the tiles by the same wavefronts.
constexpr int kF8Stages = 4;
constexpr int kF8K = 64;                              // contraction values (bytes) per stage
constexpr int kF8Tile = 256 * kF8K;                   // one operand's share of a stage
constexpr int kF8Stage = 2 * kF8Tile;
constexpr int kF8ScaleBase = kF8Stages * kF8Stage;
// The scales of a stage.  Block scales (kMx false): a dword per tile row holding the row's exponent for the stage's
// 128-value block, and 64 dwords of weight scales.  MXFP8 (kMx true): an exponent per 32 values on both sides, so a
// stage (64 values) carries two planes of 256 dwords per operand, plane h for the stage's contraction half h.
// MXFP4 (kFmt 2): e2m1 elements, 128 values in a panel's 64 bytes, so a stage carries four blocks of 32; their four
// exponents lie side by side in one dword per tile row and per tile column (the quantisers write them so), one plane
// of 256 dwords per operand.
enum F8Format { kBlockFp8 = 0, kMxFp8 = 1, kMxFp4 = 2 };
template <int kFmt>
struct F8Scales {
  static constexpr int kA = kFmt == kMxFp8 ? 2 * 256 * 4 : 256 * 4;
  static constexpr int kB = kFmt == kMxFp8 ? 2 * 256 * 4 : (kFmt == kMxFp4 ? 256 * 4 : 64 * 4);
  static constexpr int kLds = kF8ScaleBase + kF8Stages * (kA + kB);
  // per loading wavefront and stage: 4 + 4 tile loads, then the scales
  static constexpr int kLoads = kFmt == kMxFp8 ? 12 : 10;
};

__device__ __forceinline__ void lds_load4(u32x4 rsrc, lds_bytes_ptr lds_base, uint32_t voffset, uint32_t soffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
               :
               : "s"(uniform(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds_base)))), "v"(voffset),
                 "s"(uniform(rsrc)), "s"(uniform(soffset))
               : "memory", "m0");
}
// one byte per lane, which lands zero-extended in the lane's dword
__device__ __forceinline__ void lds_load1(u32x4 rsrc, lds_bytes_ptr lds_base, uint32_t voffset, uint32_t soffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_ubyte %1, %2, %3 offen lds"
               :
               : "s"(uniform(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds_base)))), "v"(voffset),
                 "s"(uniform(rsrc)), "s"(uniform(soffset))
               : "memory", "m0");
}

template <int kFmt, bool kBias = false>
__global__ void __launch_bounds__(512) grouped_gemm_fp8_kernel(GemmArgs p) {
  constexpr bool kMx = kFmt != kBlockFp8;   // an e8m0 exponent per 32 values on both sides
  constexpr bool kMx8 = kFmt == kMxFp8, kFp4 = kFmt == kMxFp4;
  constexpr int WM = 4, WN = 2, BM = 256, BN = 256, kLoadWaves = 4;
  constexpr int kF8ScaleA = F8Scales<kFmt>::kA, kF8ScaleB = F8Scales<kFmt>::kB;
  using Sched = TileSchedule<kFwd, BM, BN>;
  extern __shared__ __attribute__((aligned(16))) char lds_raw[];
  __shared__ int32_t grp_s[kMaxGroups], grp_e[kMaxGroups], tile_start[kMaxGroups + 1];
  auto lds = (lds_bytes_ptr)lds_raw;
  bf16_t* c = static_cast<bf16_t*>(p.c);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int gm = wave >> 2, gn = wave & 3;
  const int row_a = gm * 128, row_b = gn * 64;
  const bool load_wave = wave < kLoadWaves;
  const int slot = wave & (kLoadWaves - 1);

  if (wave == 0) {
    const int per = (p.groups + HMOE_WAVE - 1) / HMOE_WAVE;
    const int g0 = lane * per;
    int sum = 0;
    for (int g = g0; g < g0 + per && g < p.groups; ++g) {
      int64_t s, e;
      group_bounds(p.offs, g, p.total_rows, s, e);
      grp_s[g] = static_cast<int32_t>(s);
      grp_e[g] = static_cast<int32_t>(e);
      sum += static_cast<int>((e - s + BM - 1) / BM);
    }
    int incl = sum;
#pragma unroll
    for (int off = 1; off < HMOE_WAVE; off <<= 1) {
      const int up = __shfl_up(incl, off, HMOE_WAVE);
      if (lane >= off) incl += up;
    }
    int running = incl - sum;
    for (int g = g0; g < g0 + per && g < p.groups; ++g) {
      tile_start[g] = running;
      running += (grp_e[g] - grp_s[g] + BM - 1) / BM;
    }
    if (lane == HMOE_WAVE - 1) tile_start[p.groups] = incl;
  }
  __syncthreads();
  Sched sched;
  sched.init(p, grp_s, grp_e, tile_start);
  // the same for every tile; an e2m1 panel holds 128 values, its last one zeros past K
  const int steps = kFp4 ? static_cast<int>((p.k + 127) / 128) : static_cast<int>(p.k / kF8K);
  const int64_t a_panel = p.a_scale_rows * kF8K;  // bytes of one panel of the activations
  const uint32_t b_panel = static_cast<uint32_t>(p.n) * kF8K;
  const int64_t w_bytes = static_cast<int64_t>(steps) * kF8K * p.n;

  // ---- the loading wavefronts' view of a tile
  // A load instruction moves 16 rows of 64 bytes: lane L takes row L >> 2, and the chunk that belongs at its place
  // under the swizzle: physical chunk = logical ^ ((row >> 1) & 3) ^ ((row >> 3) & 1), under which the fragment
  // reads (one chunk of each of 32 consecutive rows) fall on distinct 16-byte slots both within any 8 consecutive
  // rows modulo 128 bytes and within any 16 modulo 256.  Rows past the tile's last are whatever follows in the panel (another
  // expert's rows, or zeros past the array's end): they reach only output rows and columns that are not stored.
  const uint32_t lane_off =
      static_cast<uint32_t>(lane >> 2) * kF8K + (((lane & 3) ^ ((lane >> 3) & 3) ^ ((lane >> 5) & 1)) << 4);
  // The activations' descriptor is rebased every stage: it starts at the tile's first row in the stage's panel and
  // spans the tile's rows there (or what the panel holds past them), so the offsets inside it are a tile's 16 KB
  // whatever the number of rows or panels (the panels of a long batch exceed 32 bits of bytes).
  u32x4 rsrc_b, rsrc_sa, rsrc_sb;
  const uint8_t* a_tile = nullptr;  // the tile's first row in panel 0
  uint32_t a_extent = 0;            // bytes from there to the tile's last row, or to the panel's end
  const uint32_t voff_a = static_cast<uint32_t>(slot * 64) * kF8K + lane_off;
  uint32_t voff_b = 0, voff_sa = 0, voff_sb = 0;
  auto describe = [&](const TileInfo& tile) __attribute__((always_inline)) {
    if (load_wave) {
      const int64_t row0 = static_cast<int64_t>(tile.row_start) + tile.a_out0;
      a_tile = static_cast<const uint8_t*>(p.a) + row0 * kF8K;
      const int64_t rows_left = p.a_scale_rows - row0;
      a_extent = static_cast<uint32_t>(rows_left < BM ? rows_left : BM) * kF8K;
      rsrc_b = make_rsrc_words(static_cast<const uint8_t*>(p.b) + tile.g * w_bytes, static_cast<uint32_t>(w_bytes));
      rsrc_sa = make_rsrc_words(p.a_scale, static_cast<uint32_t>(p.k_blocks) * static_cast<uint32_t>(p.a_scale_rows));
      if constexpr (kMx)  // k_blocks counts the exponent bytes per row or column (MXFP4: four per panel)
        rsrc_sb = make_rsrc_words(p.b_scale_e8m0 + static_cast<int64_t>(tile.g) * p.k_blocks * p.n,
                                  static_cast<uint32_t>(p.k_blocks) * static_cast<uint32_t>(p.n));
      else
        rsrc_sb = make_rsrc_words(p.b_scale, static_cast<uint32_t>(p.groups) * p.k_blocks * p.n_blocks * 4u);
      voff_b = static_cast<uint32_t>(tile.b_out0 + slot * 64) * kF8K + lane_off;
      // the dword this lane's byte lands in is d = 64 slot + lane; it takes the scale of tile row
      // (d >> 7) * 128 + (d & 3) * 32 + ((d & 127) >> 2), so that the four row blocks of a wavefront's lane lie in
      // one 16-byte read
      const int d = slot * 64 + lane;
      voff_sa = static_cast<uint32_t>(tile.row_start + tile.a_out0 + (d >> 7) * 128 + (d & 3) * 32 + ((d & 127) >> 2));
      if constexpr (kFp4) voff_sa *= 4u;  // a dword of four exponents per row
      if constexpr (kMx) {
        // the weights' plane: dword d takes tile column (d >> 6) * 64 + (d & 1) * 32 + ((d & 63) >> 1), so that the two
        // column blocks of a wavefront's lane lie in one 8-byte read.  A column past N reads another column's
        // exponent (or zero past the group's end) and reaches only outputs that are not stored.
        voff_sb = static_cast<uint32_t>(tile.b_out0 + (d >> 6) * 64 + (d & 1) * 32 + ((d & 63) >> 1));
        if constexpr (kFp4) voff_sb *= 4u;
      } else {
        int nb = (tile.b_out0 >> 7) + (lane & 1);
        nb = nb < p.n_blocks ? nb : p.n_blocks - 1;
        voff_sb = (static_cast<uint32_t>(tile.g) * p.k_blocks * p.n_blocks + nb) * 4u;
      }
    }
  };
  // stage `step` of the described tile into buffer step & 3: always F8Scales<kMx>::kLoads loads, so that the waits below
  // can count them
  auto issue = [&](int step) __attribute__((always_inline)) {
    const int buf = step & (kF8Stages - 1);
    lds_bytes_ptr ta = lds + buf * kF8Stage + slot * 4096;
    const uint32_t soff_b = static_cast<uint32_t>(step) * b_panel;
    const u32x4 rsrc_a = make_rsrc_words(a_tile + static_cast<int64_t>(step) * a_panel, a_extent);
#pragma unroll
    for (int t = 0; t < 4; ++t) lds_load16(rsrc_a, ta + t * 1024, voff_a + t * 1024, 0u);
#pragma unroll
    for (int t = 0; t < 4; ++t) lds_load16(rsrc_b, ta + kF8Tile + t * 1024, voff_b + t * 1024, soff_b);
    lds_bytes_ptr sc = lds + kF8ScaleBase + buf * (kF8ScaleA + kF8ScaleB);
    if constexpr (kFp4) {
      lds_load4(rsrc_sa, sc + slot * 256, voff_sa, static_cast<uint32_t>(step) * static_cast<uint32_t>(p.a_scale_rows) * 4u);
      lds_load4(rsrc_sb, sc + kF8ScaleA + slot * 256, voff_sb, static_cast<uint32_t>(step) * static_cast<uint32_t>(p.n) * 4u);
    } else if constexpr (kMx) {
      const uint32_t rows_a = static_cast<uint32_t>(p.a_scale_rows), cols_b = static_cast<uint32_t>(p.n);
#pragma unroll
      for (int h = 0; h < 2; ++h)
        lds_load1(rsrc_sa, sc + h * 1024 + slot * 256, voff_sa, static_cast<uint32_t>(2 * step + h) * rows_a);
#pragma unroll
      for (int h = 0; h < 2; ++h)
        lds_load1(rsrc_sb, sc + kF8ScaleA + h * 1024 + slot * 256, voff_sb, static_cast<uint32_t>(2 * step + h) * cols_b);
    } else {
      lds_load1(rsrc_sa, sc + slot * 256, voff_sa, static_cast<uint32_t>(step >> 1) * static_cast<uint32_t>(p.a_scale_rows));
      lds_load4(rsrc_sb, sc + kF8ScaleA, voff_sb, static_cast<uint32_t>(step >> 1) * static_cast<uint32_t>(p.n_blocks) * 4u);
    }
  };

  // ---- the computing view
  // A lane of half h = lane >> 5 holds its row's contraction values [16 h, 16 h + 16) in its first four registers and
  // [32 + 16 h, 48 + 16 h) in the other four: logical chunks h and h ^ 2.  That is the instruction's own layout, which
  // shows once a scale differs between the two blocks of 32: registers 0-3 of either half are scaled by the exponent
  // that the row's lane of half 0 supplies and registers 4-7 by the one the lane of half 1 supplies, so lane
  // (row, h) must supply the exponent of block h, whatever values it holds itself.
  const int half = lane >> 5;
  const int frag_chunk = (half ^ ((lane >> 1) & 3) ^ ((lane >> 3) & 1)) << 4;
  constexpr int kPartner = 32;
  const int fa0 = (row_a + (lane & 31)) * kF8K + frag_chunk;
  const int fb0 = kF8Tile + (row_b + (lane & 31)) * kF8K + frag_chunk;
  const int sa_at = kF8ScaleBase + (kMx8 ? half * 1024 : 0) + (row_a + (lane & 31) * 4) * 4;
  const int sb_at = kMx ? kF8ScaleBase + kF8ScaleA + (kMx8 ? half * 1024 : 0) + (row_b + (lane & 31) * 2) * 4
                        : kF8ScaleBase + kF8ScaleA + (gn >> 1) * 4;
  // MXFP4: a stage is two instructions of 64 values; in instruction m the lane of half h holds block 2 m + h of the
  // stage (32 values, the 16 bytes of chunk 2 m + h) and supplies that block's exponent.  Byte selectors that pull
  // block c out of two neighbouring dwords of exponents (v_perm_b32: selector bytes 0-3 name the second operand's
  // bytes, 4-7 the first's):
  const uint32_t sel_a0 = static_cast<uint32_t>(half) * 0x0101u + 0x0400u;
  const uint32_t sel_a1 = static_cast<uint32_t>(2 + half) * 0x0101u + 0x0400u;
  const uint32_t sel_b = static_cast<uint32_t>(half) * 0x01010101u + 0x06020400u;
  i32x8 fa8[WM], fb8[WN];
  auto fragment = [&](int at) __attribute__((always_inline)) {
    const i32x4 lo = *reinterpret_cast<const i32x4*>(lds_raw + at);
    const i32x4 hi = *reinterpret_cast<const i32x4*>(lds_raw + (at ^ kPartner));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  // epilogue staging in buffer 3, one 32 x 32 block at a time per wavefront
  constexpr int kEpiPitch = 32 + 8, kEpiRegion = 32 * kEpiPitch * 2;
  static_assert(kEpiRegion * 8 <= kF8Stage, "epilogue staging must fit in one stage");
  const char* stage_rows = lds_raw + 3 * kF8Stage + wave * kEpiRegion;
  const uint32_t stage_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + 3 * kF8Stage + wave * kEpiRegion +
                              static_cast<uint32_t>(((lane & 31) * kEpiPitch + ((lane >> 5) << 2)) * 2);

  int cursor = 0;
  int stores_out = 0;  // stores this wavefront issued in the previous tile's epilogue
  int64_t t = sched.first;
  TileInfo tile, next;
  if (t < sched.last) {
    tile = sched.decode(t, cursor);
    describe(tile);
    if (load_wave)
      for (int st = 0; st < 3 && st < steps; ++st) issue(st);
  }
  while (t < sched.last) {
    const bool has_next = t + sched.stride < sched.last;
    if (has_next) next = sched.decode(t + sched.stride, cursor);
    f32x16 acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    int live = (tile.a_out_lim - (tile.a_out0 + row_a) + 31) >> 5;
    live = live < 0 ? 0 : (live > WM ? WM : live);
    if (tile.b_out0 + row_b >= tile.b_out_lim) live = 0;  // this wavefront's columns lie past the operand's edge
    // The tile's first three stages (issued before the previous tile's epilogue) must be in; that epilogue's stores,
    // issued after them, need not be (vector memory operations complete in issue order, so "all but the youngest n"
    // leaves exactly the stores out): they drain under this tile's first steps.
    if (stores_out >= 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else if (stores_out == 12) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    else if (stores_out == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else if (stores_out == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else wait_loads();
    workgroup_barrier();   // and every wavefront is through with that epilogue's use of buffer 3
    // The expert's bias for this lane's eight output columns in either column block (the same in every store of the
    // epilogue).  Fetched here and pinned as arrived right behind the main loop, where nothing else is in flight: a wait
    // placed by the compiler at the first use, in the epilogue, would be for the next tile's first stages as well.
    u32x4 bias_chunk[WN];
    if constexpr (kBias) {
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        const int col = tile.b_out0 + row_b + j * 32 + ((lane & 3) << 3);
        bias_chunk[j] = u32x4{0u, 0u, 0u, 0u};
        if (col < tile.b_out_lim)
          bias_chunk[j] = *reinterpret_cast<const u32x4*>(static_cast<const bf16_t*>(p.bias) + tile.g * p.n + col);
      }
    }
    if (load_wave && steps > 3) issue(3);
    // stage 0 into registers
    uint32_t sa_pack, sb_bits;
    uint32_t sa_pack1 = 0;  // MXFP4: the row blocks' exponents for the stage's second instruction
    auto read_scales = [&](int buf) __attribute__((always_inline)) {
      const char* sc = lds_raw + buf * (kF8ScaleA + kF8ScaleB);
      const u32x4 q = *reinterpret_cast<const u32x4*>(sc + sa_at);
      if constexpr (kFp4) {
        const u32x2 w = *reinterpret_cast<const u32x2*>(sc + sb_at);
        sa_pack = __builtin_amdgcn_perm(__builtin_amdgcn_perm(q[3], q[2], sel_a0),
                                        __builtin_amdgcn_perm(q[1], q[0], sel_a0), 0x05040100u);
        sa_pack1 = __builtin_amdgcn_perm(__builtin_amdgcn_perm(q[3], q[2], sel_a1),
                                         __builtin_amdgcn_perm(q[1], q[0], sel_a1), 0x05040100u);
        // bytes: (instruction 0, column block 0), (0, 1), (1, 0), (1, 1)
        sb_bits = __builtin_amdgcn_perm(w[1], w[0], sel_b);
        return;
      }
      sa_pack = (q[0] & 0xffu) | ((q[1] & 0xffu) << 8) | ((q[2] & 0xffu) << 16) | (q[3] << 24);
      if constexpr (kMx) {
        const u32x2 w = *reinterpret_cast<const u32x2*>(sc + sb_at);
        sb_bits = (w[0] & 0xffu) | ((w[1] & 0xffu) << 8);  // the lane's exponents for its two column blocks
      } else {
        sb_bits = *reinterpret_cast<const uint32_t*>(sc + sb_at);
      }
    };
    {
#pragma unroll
      for (int j = 0; j < WN; ++j) fb8[j] = fragment(fb0 + j * 2048);
#pragma unroll
      for (int i = 0; i < WM; ++i) fa8[i] = fragment(fa0 + i * 2048);
      read_scales(0);
    }
    float mant_last = 1.0f;

    auto run = [&](auto full_tag) __attribute__((always_inline)) {
      constexpr bool kFull = decltype(full_tag)::value;
      auto mfma = [&](auto row_block, auto col_block, int sa, int sb) __attribute__((always_inline)) {
        constexpr int i = decltype(row_block)::value, j = decltype(col_block)::value;
        if (kFull || i < live) {
          if constexpr (kFp4) {
            // cbsz = blgp = 4: e2m1 operands, of which the instruction reads the first four registers
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb8[j], fa8[i], acc[i][j], 4, 4, j, sb, i, sa);
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                __builtin_shufflevector(fb8[j], fb8[j], 4, 5, 6, 7, 4, 5, 6, 7),
                __builtin_shufflevector(fa8[i], fa8[i], 4, 5, 6, 7, 4, 5, 6, 7), acc[i][j], 4, 4, 2 + j, sb, i,
                static_cast<int>(sa_pack1));
          } else {
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb8[j], fa8[i], acc[i][j], 0, 0, kMx ? j : 0, sb, i, sa);
          }
        }
      };
      using std::integral_constant;
      const integral_constant<int, 0> b0;
      const integral_constant<int, 1> b1;
      const integral_constant<int, 2> b2;
      const integral_constant<int, 3> b3;
      for (int step = 0; step < steps; ++step) {
        const int buf = step & (kF8Stages - 1), nbuf = (step + 1) & (kF8Stages - 1);
        // the weight scale: exponent to the MFMA, mantissa carried by the accumulators (1 for power-of-two scales);
        // zero or subnormal goes in as 2^-127 with mantissa 1 and contributes nothing either way
        int sb;
        if constexpr (kMx) {
          sb = static_cast<int>(sb_bits);  // a byte per column block, picked by the instruction's operand select
        } else {
          const uint32_t bits = uniform(sb_bits);
          const uint32_t sb_exp = bits >> 23;
          const float mant = sb_exp ? __uint_as_float((bits & 0x007fffffu) | 0x3f800000u) : 1.0f;
          if (mant != mant_last) {
            const float ratio = mant_last / mant;
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
              for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] *= ratio;
            mant_last = mant;
          }
          sb = static_cast<int>(sb_exp);
        }
        const int sa = static_cast<int>(sa_pack);
        __builtin_amdgcn_sched_barrier(0);
        mfma(b0, b0, sa, sb);
        mfma(b1, b0, sa, sb);
        mfma(b2, b0, sa, sb);
        mfma(b3, b0, sa, sb);
        // Nothing reads these accumulators before the next stage, so the compiler would sink the four MFMAs below
        // the barrier (they are register operations: the barrier's memory clobber does not hold them), and the
        // matrix pipe would then stand still through the wait.  Naming them in an empty statement keeps them here.
        asm volatile("" : "+v"(acc[0][0]), "+v"(acc[1][0]), "+v"(acc[2][0]), "+v"(acc[3][0]));
        __builtin_amdgcn_sched_barrier(0);
        // stage step + 1 must be in: the loads of at most two younger stages may still be out
        const int younger = steps - 2 - step;
        if (load_wave) {
          constexpr int kLoads = F8Scales<kFmt>::kLoads;
          static_assert(kLoads == 10 || kLoads == 12, "the waits below count them");
          if (younger >= 2) {
            if constexpr (kLoads == 12) asm volatile("s_waitcnt vmcnt(24) lgkmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(20) lgkmcnt(0)" ::: "memory");
          } else if (younger == 1) {
            if constexpr (kLoads == 12) asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(10) lgkmcnt(0)" ::: "memory");
          } else {
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
          }
        } else {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
        workgroup_barrier();
        // this step's buffer is read out (its fragments were taken during the previous step): refill it
        if (load_wave && step + 4 < steps) issue(step + 4);
        // the second column of MFMAs, each followed by the refill of its fragment from the next stage (after a
        // tile's last step these read what nothing uses)
        const int na = nbuf * kF8Stage;
        if (kFull || live > 0) fb8[0] = fragment(na + fb0);
        __builtin_amdgcn_sched_barrier(0);
        mfma(b0, b1, sa, sb);
        if (kFull || 0 < live) fa8[0] = fragment(na + fa0);
        __builtin_amdgcn_sched_barrier(0);
        mfma(b1, b1, sa, sb);
        if (kFull || 1 < live) fa8[1] = fragment(na + fa0 + 2048);
        __builtin_amdgcn_sched_barrier(0);
        mfma(b2, b1, sa, sb);
        if (kFull || 2 < live) fa8[2] = fragment(na + fa0 + 2 * 2048);
        __builtin_amdgcn_sched_barrier(0);
        mfma(b3, b1, sa, sb);
        if (kFull || 3 < live) fa8[3] = fragment(na + fa0 + 3 * 2048);
        if (kFull || live > 0) fb8[1] = fragment(na + fb0 + 2048);
        read_scales(nbuf);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    if (live == WM) run(std::true_type{});
    else run(std::false_type{});
    if (!kMx && mant_last != 1.0f) {
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) acc[i][j][v] *= mant_last;
    }

    if constexpr (kBias) {
#pragma unroll
      for (int j = 0; j < WN; ++j) asm volatile("" : "+v"(bias_chunk[j]));
    }
    // buffers 0-2 are free since the last barrier: the next tile's first stages go out before this tile's epilogue
    const TileInfo done = tile;
    t += sched.stride;
    if (has_next) {
      tile = next;
      describe(tile);
      if (load_wave)
        for (int st = 0; st < 3 && st < steps; ++st) issue(st);
    }

    // the output descriptor spans this tile's rows only, so its 32-bit offsets hold whatever the batch's size
    const int c_row_lim = done.a_out_lim - done.a_out0;
    bf16_t* c_base = c + (static_cast<int64_t>(done.row_start) + done.a_out0) * p.ldc;
    const __amdgpu_buffer_rsrc_t c_rsrc =
        make_rsrc(c_base, static_cast<uint32_t>((c_row_lim < BM ? c_row_lim : BM) * p.ldc * 2));
    stores_out = 4 * live;
#pragma unroll
    for (int i = 0; i < WM; ++i) {
      if (i < live) {
#pragma unroll
        for (int j = 0; j < WN; ++j) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            uint2 packed;
            packed.x = pack_bf16x2(acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1]);
            packed.y = pack_bf16x2(acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]);
            // inline assembly: an LDS store the compiler can see makes it drain the loads in flight first
            asm volatile("ds_write_b64 %0, %1 offset:%2" : : "v"(stage_addr), "v"(packed), "n"(q * 8 * 2) : "memory");
          }
          __builtin_amdgcn_wave_barrier();  // the rows are private to the wavefront, whose LDS accesses stay in order
#pragma unroll
          for (int pass = 0; pass < 2; ++pass) {
            const int rr = pass * 16 + (lane >> 2);
            const int cc = (lane & 3) << 3;
            const int row = row_a + i * 32 + rr;  // from the descriptor's first row
            const int col = done.b_out0 + row_b + j * 32 + cc;
            u32x4 v = *reinterpret_cast<const u32x4*>(stage_rows + (rr * kEpiPitch + cc) * 2);
            if constexpr (kBias) v = add_bf16x8(v, bias_chunk[j]);
            const uint32_t off = row < c_row_lim && col < done.b_out_lim
                                     ? static_cast<uint32_t>(row) * static_cast<uint32_t>(p.ldc) * 2u + col * 2u
                                     : kOutOfRange;
            __builtin_amdgcn_raw_buffer_store_b128(v, c_rsrc, off, 0, 0);
          }
          __builtin_amdgcn_wave_barrier();
        }
      }
    }
  }
  wait_loads();  // no load may land in LDS after the workgroup has given it back
}


constexpr int FT = 64, FK = 16;

template <int kMode>
__global__ void __launch_bounds__(256) grouped_gemm_f32_kernel(GemmArgs p) {
  __shared__ float sa[FK][FT + 1];
  __shared__ float sb[FK][FT + 1];
  const float* a = static_cast<const float*>(p.a);
  const float* b = static_cast<const float*>(p.b);
  float* c = static_cast<float*>(p.c);
  int g;
  int64_t s = 0, e = 0;
  int row0, col0;
  int64_t rows_out, cols_out, con;
  if constexpr (kMode == kWgrad) {
    g = blockIdx.z;
    group_bounds(p.offs, g, p.total_rows, s, e);
    row0 = blockIdx.x * FT;
    col0 = blockIdx.y * FT;
    rows_out = p.k;
    cols_out = p.n;
    con = e - s;
  } else {
    int tile = blockIdx.x;
    bool found = false;
    for (g = 0; g < p.groups; ++g) {
      group_bounds(p.offs, g, p.total_rows, s, e);
      const int mt = static_cast<int>((e - s + FT - 1) / FT);
      if (tile < mt) { found = true; break; }
      tile -= mt;
    }
    if (!found) return;
    row0 = tile * FT;
    col0 = blockIdx.y * FT;
    rows_out = e - s;
    cols_out = kMode == kFwd ? p.n : p.k;
    con = kMode == kFwd ? p.k : p.n;
  }
  const float* w = b + static_cast<int64_t>(g) * p.k * p.n;
  auto a_at = [&](int64_t out, int64_t cc) -> float {
    if constexpr (kMode == kWgrad) return a[(s + cc) * p.lda + out];
    else return a[(s + out) * p.lda + cc];
  };
  auto b_at = [&](int64_t out, int64_t cc) -> float {
    if constexpr (kMode == kFwd) return w[cc * p.n + out];
    else if constexpr (kMode == kDgrad) return w[out * p.n + cc];
    else return b[(s + cc) * p.ldb + out];
  };
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  float acc[4][4] = {};
  for (int64_t k0 = 0; k0 < con; k0 += FK) {
    for (int i = threadIdx.x; i < FK * FT; i += 256) {
      const int kk = i / FT, o = i % FT;
      const int64_t cc = k0 + kk;
      sa[kk][o] = (cc < con && row0 + o < rows_out) ? a_at(row0 + o, cc) : 0.f;
      sb[kk][o] = (cc < con && col0 + o < cols_out) ? b_at(col0 + o, cc) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < FK; ++kk) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        av[i] = sa[kk][ty * 4 + i];
        bv[i] = sb[kk][tx * 4 + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }
  float* out = kMode == kWgrad ? c + static_cast<int64_t>(g) * p.k * p.n : c + s * p.ldc;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t r = row0 + ty * 4 + i, cc = col0 + tx * 4 + j;
      if (r < rows_out && cc < cols_out) {
        float v = acc[i][j];
        if (kMode == kFwd && p.bias != nullptr) v += static_cast<const float*>(p.bias)[static_cast<int64_t>(g) * p.n + cc];
        if ((kMode == kFwd || kMode == kDgrad) && p.addend != nullptr) {
          // two roundings, as the tensor operations have them: the multiply must not contract into the add
#pragma clang fp contract(off)
          const float scaled = p.addend_scale * v;
          v = static_cast<const float*>(p.addend)[(s + r) * p.ld_addend + cc] + scaled;
        }
        out[r * p.ldc + cc] = v;
      }
    }
}

int device_cus() {
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
  }
  return cus;
}

template <int kMode, typename Cfg>
int launch_staged(const GemmArgs& p, int workgroups_per_cu, hipStream_t stream) {
  // upper bound on the number of tiles, so no more workgroups start than can find work
  const int64_t out_cols = kMode == kDgrad ? p.k : p.n;
  const int64_t nt = (out_cols + Cfg::BN - 1) / Cfg::BN;
  int64_t bound;
  if (kMode == kWgrad) bound = ((p.k + Cfg::BM - 1) / Cfg::BM) * nt * p.groups;
  else bound = (p.total_rows / Cfg::BM + p.groups) * nt;
  int64_t workers = static_cast<int64_t>(device_cus()) * workgroups_per_cu;
  if (bound < workers) workers = bound;
  workers = (workers + kXcds - 1) / kXcds * kXcds;
  if (workers <= 0) return HMOE_OK;
  constexpr size_t lds_bytes = 2 * Cfg::kStage * sizeof(bf16_t);
  auto kernel = grouped_gemm_staged_kernel<kMode, Cfg>;
  if (lds_bytes > 48 * 1024) {
    // raising the dynamic LDS limit is idempotent: racing threads set the same value
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(lds_bytes)) != hipSuccess)
      return HMOE_LAUNCH_FAILED;
  }
  kernel<<<dim3(static_cast<unsigned>(workers)), dim3(Cfg::kThreads), lds_bytes, stream>>>(p);
  return HMOE_OK;
}

template <int kMode, typename Cfg, int kGather = 0, bool kBias = false, bool kAddTo = false>
int launch_direct(const GemmArgs& p, hipStream_t stream) {
  const int64_t out_cols = kMode == kDgrad ? p.k : p.n;
  const int64_t nt = (out_cols + Cfg::BN - 1) / Cfg::BN;
  int64_t bound;
  if (kMode == kWgrad) bound = ((p.k + Cfg::BM - 1) / Cfg::BM) * nt * p.groups;
  else bound = (p.total_rows / Cfg::BM + p.groups) * nt;
  int64_t workers = device_cus();
  if (bound < workers) workers = bound;
  workers = (workers + kXcds - 1) / kXcds * kXcds;
  if (workers <= 0) return HMOE_OK;
  // wgrad: two stages; gathered, 2 x 1 KB of row indices per loading wavefront behind them.  fwd, dgrad: two stages
  // of A and three of B
  constexpr size_t lds_bytes = kMode == kWgrad
                                   ? 2 * Cfg::kStage * sizeof(bf16_t) + (kGather ? 4 * 2048 : 0)
                                   : (2 * Cfg::BM + 3 * Cfg::BN) * BK * sizeof(bf16_t);
  auto kernel = grouped_gemm_bf16_kernel<kMode, Cfg, kGather, kBias, kAddTo>;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                          static_cast<int>(lds_bytes)) != hipSuccess)
    return HMOE_LAUNCH_FAILED;
  kernel<<<dim3(static_cast<unsigned>(workers)), dim3(Cfg::kThreads), lds_bytes, stream>>>(p);
  return HMOE_OK;
}

// Which of the three bf16 tile configurations a product takes: the 256 x 256 tile on one workgroup per compute unit
// (this file), or the 128 x 256 tile on two or the 128 x 128 tile on three (grouped_gemm_duo.hip).  All give the same
// bits (the contraction is summed in the same order).  Left to itself the choice goes by the tile count: the largest
// tile of which the product has at least one per compute unit, since a larger tile moves fewer operand bytes per
// multiply-add (the 256 x 256 tile is 10-25 % faster than the 128 x 256 one at the expert products of every benchmark
// configuration) and a launch with fewer tiles than compute units leaves some idle (a dense projection of a few
// thousand rows, a narrow output); an output of at most 128 columns takes the 128 x 128 tile whatever its tile count
// (the logits of 32 768 tokens over 128 experts: 39 against 53 us).  hmoe_set_gemm_tile() or
// HALO_GEMM_TILE=mono|duo|small forces one configuration for every product.
enum TilePolicy { kTileBySize = 0, kTileMono = 1, kTileDuo = 2, kTileSmall = 3 };
std::atomic<int> g_gemm_tile{-1};  // a TilePolicy; -1: not yet read from the environment

int gemm_tile_policy() {
  int v = g_gemm_tile.load(std::memory_order_relaxed);
  if (v < 0) {
    const char* e = std::getenv("HALO_GEMM_TILE");
    v = e == nullptr ? kTileBySize : (e[0] == 'm' ? kTileMono : (e[0] == 'd' ? kTileDuo : (e[0] == 's' ? kTileSmall : kTileBySize)));
    g_gemm_tile.store(v, std::memory_order_relaxed);
  }
  return v;
}

// an upper bound on the product's tiles of tile_m x tile_n
template <int kMode>
int64_t tile_bound(const GemmArgs& p, int tile_m, int tile_n) {
  const int64_t out_cols = kMode == kDgrad ? p.k : p.n;
  const int64_t column_tiles = (out_cols + tile_n - 1) / tile_n;
  return kMode == kWgrad ? ((p.k + tile_m - 1) / tile_m) * column_tiles * p.groups
                         : (p.total_rows / tile_m + p.groups) * column_tiles;
}

template <int kMode>
int tile_for(const GemmArgs& p) {
  const int forced = gemm_tile_policy();
  if (forced != kTileBySize) return forced;
  const int cus = device_cus();
  // an output of at most 128 columns (a router's logits) would leave half of every 256-wide tile empty
  if ((kMode == kDgrad ? p.k : p.n) <= 128) return kTileSmall;
  if (tile_bound<kMode>(p, 256, 256) >= cus) return kTileMono;
  if (tile_bound<kMode>(p, 128, 256) >= cus) return kTileDuo;
  return kTileSmall;
}

template <int kMode>
int launch(const GemmArgs& p, int dtype, hipStream_t stream) {
  if (dtype == HMOE_BF16) {
    using Tile = Config<2, 4, 4, 2>;  // 256 x 256 tile on 8 wavefronts of 4 x 2 blocks
    int rc;
    if constexpr (kMode == kFwd || kMode == kDgrad || kMode == kWgrad) {
      const int tile = tile_for<kMode>(p);
      if (tile != kTileMono) return launch_duo(kMode, p, tile == kTileSmall, stream);
    }
    if constexpr (kMode == kFwdFp8W) {
      rc = launch_staged<kMode, Tile>(p, 1, stream);
    } else if constexpr (kMode == kFwd) {
      rc = p.a_index  ? (p.bias ? launch_direct<kMode, Tile, 1, true>(p, stream) : launch_direct<kMode, Tile, 1>(p, stream))
           : p.bias   ? launch_direct<kMode, Tile, 0, true>(p, stream)
           : p.addend ? launch_direct<kMode, Tile, 0, false, true>(p, stream)
                      : launch_direct<kMode, Tile>(p, stream);
    } else if constexpr (kMode == kWgrad) {
      rc = !p.a_index ? launch_direct<kMode, Tile>(p, stream)
           : p.gather_b ? launch_direct<kMode, Tile, 2>(p, stream)
                        : launch_direct<kMode, Tile, 1>(p, stream);
    } else {
      rc = p.a_index  ? launch_direct<kMode, Tile, 1>(p, stream)
           : p.addend ? launch_direct<kMode, Tile, 0, false, true>(p, stream)
                      : launch_direct<kMode, Tile>(p, stream);
    }
    if (rc) return rc;
  } else if constexpr (kMode != kFwdFp8W) {
    if (kMode == kWgrad) {
      const dim3 grid((p.k + FT - 1) / FT, (p.n + FT - 1) / FT, p.groups);
      grouped_gemm_f32_kernel<kMode><<<grid, dim3(256), 0, stream>>>(p);
    } else {
      const int64_t out_cols = kMode == kFwd ? p.n : p.k;
      const dim3 grid(p.total_rows / FT + p.groups, (out_cols + FT - 1) / FT);
      grouped_gemm_f32_kernel<kMode><<<grid, dim3(256), 0, stream>>>(p);
    }
  }
  if (hipGetLastError() != hipSuccess) return HMOE_LAUNCH_FAILED;
  return HMOE_OK;
}

int validate(const GemmArgs& p, int dtype) {
  if (p.total_rows < 0 || p.groups <= 0 || p.k < 0 || p.n < 0) return HMOE_INVALID_ARGUMENT;
  if (dtype != HMOE_BF16 && dtype != HMOE_F32) return HMOE_UNSUPPORTED;
  if (p.offs == nullptr && p.groups != 1) return HMOE_INVALID_ARGUMENT;
  if (p.groups > kMaxGroups) return HMOE_UNSUPPORTED;
  if (p.total_rows >= (int64_t(1) << 31) || p.k >= (int64_t(1) << 31) || p.n >= (int64_t(1) << 31))
    return HMOE_UNSUPPORTED;
  if (dtype == HMOE_BF16) {
    // 16-byte rows: the alignment torch's grouped GEMM asks for as well
    if (p.k % 8 || p.n % 8 || p.lda % 8 || p.ldb % 8 || p.ldc % 8) return HMOE_UNSUPPORTED;
    if (!aligned16(p.a) || !aligned16(p.b) || !aligned16(p.c)) return HMOE_UNSUPPORTED;
    // Buffer loads address memory with 32-bit byte offsets from a descriptor's base.  The kernels base their
    // descriptors at a tile's first row (activations and outputs) or rebase them every contraction step (wgrad), so
    // the activation operands and the outputs may be of any size; what must stay below 2 GiB is one expert's weight,
    // one 256-row tile of any operand, and an array that is gathered from by row index.
    const int64_t lim = int64_t(1) << 31;
    const int64_t widest = p.lda > p.ldb ? (p.lda > p.ldc ? p.lda : p.ldc) : (p.ldb > p.ldc ? p.ldb : p.ldc);
    if (widest * 2 * 512 >= lim || p.k * p.n * 2 >= lim) return HMOE_UNSUPPORTED;
    if (p.a_index && p.a_rows * (p.gather_b ? p.ldb : p.lda) * 2 >= lim) return HMOE_UNSUPPORTED;
    if (p.b_scale && (p.total_rows * p.lda * 2 >= lim || p.total_rows * p.ldc * 2 >= lim))
      return HMOE_UNSUPPORTED;  // the register-staged fp8-weight kernel still spans a group per descriptor
  }
  return HMOE_OK;
}

template <int kFmt, bool kBias = false>
int launch_fp8(const GemmArgs& p, int64_t workers, void* stream) {
  constexpr int kLds = F8Scales<kFmt>::kLds;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(grouped_gemm_fp8_kernel<kFmt, kBias>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, kLds) != hipSuccess)
    return HMOE_LAUNCH_FAILED;
  grouped_gemm_fp8_kernel<kFmt, kBias><<<dim3(static_cast<unsigned>(workers)), dim3(512), kLds,
                                        static_cast<hipStream_t>(stream)>>>(p);
  if (hipGetLastError() != hipSuccess) return HMOE_LAUNCH_FAILED;
  return HMOE_OK;
}

// Whether the scaled-MFMA kernel can address the operands of an MX product.  The quantised activations and the output
// may be of any size (their descriptors are rebased per stage and per tile); what must stay below 2 GiB is one
// expert's weight panels, the rows' exponent bytes and a tile's 256 output rows.  A caller whose operands do not fit
// multiplies the round-tripped operands on the bf16 kernels.
bool mx_product_fits(int64_t a_rows, int64_t total_rows, int64_t k, int64_t n, int64_t ldo, int panel_values) {
  if (a_rows < 0 || total_rows < 0 || k < 0 || n < 0 || ldo < 0 || (panel_values != 64 && panel_values != 128)) return false;
  const int64_t lim = int64_t(1) << 31, panels = (k + panel_values - 1) / panel_values;
  // products of two values below 2^31 each stay inside int64
  if (a_rows >= lim || total_rows >= lim || panels >= lim || n >= lim || ldo >= lim) return false;
  // one expert's weight panels, the rows' exponent bytes (a dword per row and panel for e2m1) and 256 output rows
  return panels * n < lim / 64 && a_rows * panels * 4 < lim && 256 * ldo < lim / 2;
}

// The MX products' arguments, checked: `panel_values` contraction values lie in a panel's 64 bytes (64 for e4m3, 128 for
// e2m1) and `k_multiple` is what k must be a multiple of.
int mx_args(GemmArgs& p, const uint8_t* a_q, const uint8_t* a_scale, int64_t a_rows, const uint8_t* bq,
            const uint8_t* b_scale, const int32_t* offs, int64_t total_rows, int num_groups, int64_t k, int64_t n,
            const void* bias, bool with_bias, void* out, int64_t ldo, int panel_values, int k_multiple,
            int64_t& workers) {
  if (total_rows < 0 || num_groups <= 0 || k < 0 || n < 0) return HMOE_INVALID_ARGUMENT;
  if (offs == nullptr && num_groups != 1) return HMOE_INVALID_ARGUMENT;
  if (num_groups > kMaxGroups) return HMOE_UNSUPPORTED;
  if (k % k_multiple || n % 8 || ldo % 8 || ldo < n || a_rows < total_rows) return HMOE_UNSUPPORTED;
  if (total_rows == 0 || n == 0) return 1;  // nothing to do
  if (k == 0) return HMOE_UNSUPPORTED;
  if (!a_q || !a_scale || !bq || !b_scale || !out || (with_bias && !bias)) return HMOE_INVALID_ARGUMENT;
  if (!aligned16(a_q) || !aligned16(bq) || !aligned16(out) || (with_bias && !aligned16(bias))) return HMOE_UNSUPPORTED;
  if (panel_values == 128 && (reinterpret_cast<uintptr_t>(a_scale) % 4 || reinterpret_cast<uintptr_t>(b_scale) % 4))
    return HMOE_UNSUPPORTED;
  const int64_t panels = (k + panel_values - 1) / panel_values;
  if (!mx_product_fits(a_rows, total_rows, k, n, ldo, panel_values)) return HMOE_UNSUPPORTED;
  p.a = a_q;
  p.b = bq;
  p.c = out;
  p.ldc = ldo;
  p.offs = offs;
  p.total_rows = total_rows;
  p.groups = num_groups;
  p.k = k;
  p.n = n;
  p.b_scale_e8m0 = b_scale;
  p.a_scale = a_scale;
  p.a_scale_rows = a_rows;
  p.k_blocks = static_cast<int>(panels * (panel_values / 32));
  p.bias = bias;
  const int64_t bound = (total_rows / 256 + num_groups) * ((n + 255) / 256);
  workers = device_cus();
  if (bound < workers) workers = bound;
  workers = (workers + kXcds - 1) / kXcds * kXcds;
  return HMOE_OK;
}

}  // namespace
}  // namespace hmoe

extern "C" {

int hmoe_grouped_gemm_mx_fits(int64_t a_rows, int64_t total_rows, int64_t k, int64_t n, int64_t ldo,
                              int panel_values) {
  return hmoe::mx_product_fits(a_rows, total_rows, k, n, ldo, panel_values) ? 1 : 0;
}

int hmoe_set_gemm_tile(int tile) {
  if (tile < 0 || tile > 3) return HMOE_INVALID_ARGUMENT;
  const int before = hmoe::gemm_tile_policy();
  hmoe::g_gemm_tile.store(tile, std::memory_order_relaxed);
  return before;
}


int hmoe_grouped_gemm_fwd(const void* a, int64_t lda, const void* b, const int32_t* offs, int64_t total_rows,
                          int num_groups, int64_t k, int64_t n, int dtype, void* out, int64_t ldo, void* stream) {
  using namespace hmoe;
  GemmArgs p{a, lda, b, n, out, ldo, offs, total_rows, num_groups, k, n, nullptr};
  if (int rc = validate(p, dtype)) return rc;
  if (total_rows == 0 || n == 0) return HMOE_OK;
  if (!a || !b || !out) return HMOE_INVALID_ARGUMENT;
  if (lda < k || ldo < n) return HMOE_INVALID_ARGUMENT;
  return launch<kFwd>(p, dtype, static_cast<hipStream_t>(stream));
}

int hmoe_grouped_gemm_fwd_bias(const void* a, int64_t lda, const void* b, const void* bias, const int32_t* offs,
                               int64_t total_rows, int num_groups, int64_t k, int64_t n, int dtype, void* out,
                               int64_t ldo, void* stream) {
  using namespace hmoe;
  GemmArgs p{a, lda, b, n, out, ldo, offs, total_rows, num_groups, k, n, nullptr};
  p.bias = bias;
  if (int rc = validate(p, dtype)) return rc;
  if (total_rows == 0 || n == 0) return HMOE_OK;
  if (!a || !b || !out || !bias) return HMOE_INVALID_ARGUMENT;
  if (lda < k || ldo < n) return HMOE_INVALID_ARGUMENT;
  if (dtype == HMOE_BF16 && !aligned16(bias)) return HMOE_UNSUPPORTED;
  return launch<kFwd>(p, dtype, static_cast<hipStream_t>(stream));
}

int hmoe_grouped_gemm_fwd_addto(const void* a, int64_t lda, const void* b, const int32_t* offs, int64_t total_rows,
                                int num_groups, int64_t k, int64_t n, int dtype, const void* addend,
                                int64_t ld_addend, float scale, void* out, int64_t ldo, void* stream) {
  using namespace hmoe;
  GemmArgs p{a, lda, b, n, out, ldo, offs, total_rows, num_groups, k, n, nullptr};
  p.addend = addend;
  p.ld_addend = ld_addend;
  p.addend_scale = scale;
  if (int rc = validate(p, dtype)) return rc;
  if (total_rows == 0 || n == 0) return HMOE_OK;
  if (!a || !b || !out || !addend) return HMOE_INVALID_ARGUMENT;
  if (lda < k || ldo < n || ld_addend < n) return HMOE_INVALID_ARGUMENT;
  if (dtype == HMOE_BF16 && (!aligned16(addend) || ld_addend % 8 || ld_addend * 2 * 512 >= (int64_t(1) << 31)))
    return HMOE_UNSUPPORTED;
  return launch<kFwd>(p, dtype, static_cast<hipStream_t>(stream));
}

int hmoe_grouped_gemm_fwd_gather(const void* a, int64_t lda, int64_t a_rows, const int64_t* row_index, const void* b,
                                 const int32_t* offs, int64_t total_rows, int num_groups, int64_t k, int64_t n,
                                 int dtype, void* out, int64_t ldo, void* stream) {
  using namespace hmoe;
  if (dtype != HMOE_BF16) return HMOE_UNSUPPORTED;
  if (a_rows < 0) return HMOE_INVALID_ARGUMENT;
  GemmArgs p{a, lda, b, n, out, ldo, offs, total_rows, num_groups, k, n, nullptr, row_index, a_rows};
  if (int rc = validate(p, dtype)) return rc;
  if (total_rows == 0 || n == 0) return HMOE_OK;
  if (!a || !b || !out || !row_index) return HMOE_INVALID_ARGUMENT;
  if (lda < k || ldo < n) return HMOE_INVALID_ARGUMENT;
  return launch<kFwd>(p, dtype, static_cast<hipStream_t>(stream));
}

int hmoe_grouped_gemm_fwd_gather_bias(const void* a, int64_t lda, int64_t a_rows, const int64_t* row_index,
                                      const void* b, const void* bias, const int32_t* offs, int64_t total_rows,
                                      int num_groups, int64_t k, int64_t n, int dtype, void* out, int64_t ldo,
                                      void* stream) {
  using namespace hmoe;
  if (dtype != HMOE_BF16) return HMOE_UNSUPPORTED;
  if (a_rows < 0) return HMOE_INVALID_ARGUMENT;
  GemmArgs p{a, lda, b, n, out, ldo, offs, total_rows, num_groups, k, n, nullptr, row_index, a_rows};
  p.bias = bias;
  if (int rc = validate(p, dtype)) return rc;
  if (total_rows == 0 || n == 0) return HMOE_OK;
  if (!a || !b || !out || !row_index || !bias) return HMOE_INVALID_ARGUMENT;
  if (lda < k || ldo < n) return HMOE_INVALID_ARGUMENT;
  if (!aligned16(bias)) return HMOE_UNSUPPORTED;
  return launch<kFwd>(p, dtype, static_cast<hipStream_t>(stream));
}

int hmoe_grouped_gemm_wgrad_gather(const void* a, int64_t lda, int64_t a_rows, const int64_t* row_index,
                                   const void* grad_out, int64_t ldg, const int32_t* offs, int64_t total_rows,
                                   int num_groups, int64_t k, int64_t n, int dtype, void* grad_b, void* stream) {
  using namespace hmoe;
  if (dtype != HMOE_BF16) return HMOE_UNSUPPORTED;
  if (a_rows < 0) return HMOE_INVALID_ARGUMENT;
  GemmArgs p{a, lda, grad_out, ldg, grad_b, n, offs, total_rows, num_groups, k, n, nullptr, row_index, a_rows};
  if (int rc = validate(p, dtype)) return rc;
  if (k == 0 || n == 0) return HMOE_OK;
  if (!grad_b || (total_rows > 0 && (!a || !grad_out || !row_index))) return HMOE_INVALID_ARGUMENT;
  if (lda < k || ldg < n) return HMOE_INVALID_ARGUMENT;
  return launch<kWgrad>(p, dtype, static_cast<hipStream_t>(stream));
}

int hmoe_grouped_gemm_dgrad_gather(const void* grad_out, int64_t ldg, int64_t grad_rows, const int64_t* row_index,
                                   const void* b, const int32_t* offs, int64_t total_rows, int num_groups, int64_t k,
                                   int64_t n, int dtype, void* grad_a, int64_t lda, void* stream) {
  using namespace hmoe;
  if (dtype != HMOE_BF16) return HMOE_UNSUPPORTED;
  if (grad_rows < 0) return HMOE_INVALID_ARGUMENT;
  GemmArgs p{grad_out, ldg, b, n, grad_a, lda, offs, total_rows, num_groups, k, n, nullptr, row_index, grad_rows};
  if (int rc = validate(p, dtype)) return rc;
  if (total_rows == 0 || k == 0) return HMOE_OK;
  if (!grad_out || !b || !grad_a || !row_index) return HMOE_INVALID_ARGUMENT;
  if (ldg < n || lda < k) return HMOE_INVALID_ARGUMENT;
  return launch<kDgrad>(p, dtype, static_cast<hipStream_t>(stream));
}

int hmoe_grouped_gemm_wgrad_gather_grad(const void* a, int64_t lda, const void* grad_out, int64_t ldg,
                                        int64_t grad_rows, const int64_t* row_index, const int32_t* offs,
                                        int64_t total_rows, int num_groups, int64_t k, int64_t n, int dtype,
                                        void* grad_b, void* stream) {
  using namespace hmoe;
  if (dtype != HMOE_BF16) return HMOE_UNSUPPORTED;
  if (grad_rows < 0) return HMOE_INVALID_ARGUMENT;
  GemmArgs p{a, lda, grad_out, ldg, grad_b, n, offs, total_rows, num_groups, k, n, nullptr, row_index, grad_rows};
  p.gather_b = true;
  if (int rc = validate(p, dtype)) return rc;
  if (k == 0 || n == 0) return HMOE_OK;
  if (!grad_b || (total_rows > 0 && (!a || !grad_out || !row_index))) return HMOE_INVALID_ARGUMENT;
  if (lda < k || ldg < n) return HMOE_INVALID_ARGUMENT;
  return launch<kWgrad>(p, dtype, static_cast<hipStream_t>(stream));
}

int hmoe_grouped_gemm_fwd_fp8w(const void* a, int64_t lda, const uint8_t* bq, const float* b_scale,
                               const int32_t* offs, int64_t total_rows, int num_groups, int64_t k, int64_t n,
                               void* out, int64_t ldo, void* stream) {
  using namespace hmoe;
  GemmArgs p{a, lda, bq, n, out, ldo, offs, total_rows, num_groups, k, n, b_scale};
  if (int rc = validate(p, HMOE_BF16)) return rc;
  if (total_rows == 0 || n == 0) return HMOE_OK;
  if (!a || !bq || !b_scale || !out) return HMOE_INVALID_ARGUMENT;
  if (lda < k || ldo < n) return HMOE_INVALID_ARGUMENT;
  return launch<kFwdFp8W>(p, HMOE_BF16, static_cast<hipStream_t>(stream));
}

int hmoe_grouped_gemm_fwd_fp8(const uint8_t* a_q, const uint8_t* a_scale, int64_t a_rows, const uint8_t* bq,
                              const float* b_scale, const int32_t* offs, int64_t total_rows, int num_groups, int64_t k,
                              int64_t n, void* out, int64_t ldo, void* stream) {
  using namespace hmoe;
  if (total_rows < 0 || num_groups <= 0 || k < 0 || n < 0) return HMOE_INVALID_ARGUMENT;
  if (offs == nullptr && num_groups != 1) return HMOE_INVALID_ARGUMENT;
  if (num_groups > kMaxGroups) return HMOE_UNSUPPORTED;
  // whole scale blocks along the contraction; 16-byte rows on both sides
  if (k % 128 || n % 8 || ldo % 8 || ldo < n || a_rows < total_rows) return HMOE_UNSUPPORTED;
  if (total_rows == 0 || n == 0) return HMOE_OK;
  if (k == 0) return HMOE_UNSUPPORTED;  // an empty contraction has no scale block to speak of
  if (!a_q || !a_scale || !bq || !b_scale || !out) return HMOE_INVALID_ARGUMENT;
  if (!aligned16(a_q) || !aligned16(bq) || !aligned16(out) || reinterpret_cast<uintptr_t>(b_scale) % 4)
    return HMOE_UNSUPPORTED;
  const int64_t lim = int64_t(1) << 31;
  const int64_t k_blocks = k / 128, n_blocks = (n + 127) / 128;
  // activations and output of any size (descriptors rebased per stage and per tile); below 2 GiB: one expert's weight,
  // the rows' exponent bytes, the weight scales, a tile's 256 output rows
  if (a_rows >= lim || total_rows >= lim || a_rows * k_blocks >= lim || k * n >= lim || 256 * ldo * 2 >= lim ||
      num_groups * k_blocks * n_blocks * 4 >= lim)
    return HMOE_UNSUPPORTED;
  GemmArgs p{};
  p.a = a_q;
  p.b = bq;
  p.c = out;
  p.ldc = ldo;
  p.offs = offs;
  p.total_rows = total_rows;
  p.groups = num_groups;
  p.k = k;
  p.n = n;
  p.b_scale = b_scale;
  p.a_scale = a_scale;
  p.a_scale_rows = a_rows;
  p.k_blocks = static_cast<int>(k_blocks);
  p.n_blocks = static_cast<int>(n_blocks);
  const int64_t bound = (total_rows / 256 + num_groups) * ((n + 255) / 256);
  int64_t workers = device_cus();
  if (bound < workers) workers = bound;
  workers = (workers + kXcds - 1) / kXcds * kXcds;
  return launch_fp8<kBlockFp8>(p, workers, stream);
}

int hmoe_grouped_gemm_fwd_mxfp8(const uint8_t* a_q, const uint8_t* a_scale, int64_t a_rows, const uint8_t* bq,
                                const uint8_t* b_scale, const int32_t* offs, int64_t total_rows, int num_groups,
                                int64_t k, int64_t n, void* out, int64_t ldo, void* stream) {
  using namespace hmoe;
  GemmArgs p{};
  int64_t workers = 0;
  // whole panels of 64 values along the contraction; 16-byte rows on both sides
  const int rc = mx_args(p, a_q, a_scale, a_rows, bq, b_scale, offs, total_rows, num_groups, k, n, nullptr, false, out,
                         ldo, 64, 64, workers);
  if (rc) return rc > 0 ? HMOE_OK : rc;
  return launch_fp8<kMxFp8>(p, workers, stream);
}

int hmoe_grouped_gemm_fwd_mxfp8_bias(const uint8_t* a_q, const uint8_t* a_scale, int64_t a_rows, const uint8_t* bq,
                                     const uint8_t* b_scale, const void* bias, const int32_t* offs, int64_t total_rows,
                                     int num_groups, int64_t k, int64_t n, void* out, int64_t ldo, void* stream) {
  using namespace hmoe;
  GemmArgs p{};
  int64_t workers = 0;
  const int rc = mx_args(p, a_q, a_scale, a_rows, bq, b_scale, offs, total_rows, num_groups, k, n, bias, true, out, ldo,
                         64, 64, workers);
  if (rc) return rc > 0 ? HMOE_OK : rc;
  return launch_fp8<kMxFp8, true>(p, workers, stream);
}

int hmoe_grouped_gemm_fwd_mxfp4(const uint8_t* a_q, const uint8_t* a_scale, int64_t a_rows, const uint8_t* bq,
                                const uint8_t* b_scale, const int32_t* offs, int64_t total_rows, int num_groups,
                                int64_t k, int64_t n, void* out, int64_t ldo, void* stream) {
  using namespace hmoe;
  GemmArgs p{};
  int64_t workers = 0;
  // whole blocks of 32 values along the contraction (the operands' last panel is zeros past K); 16-byte rows
  const int rc = mx_args(p, a_q, a_scale, a_rows, bq, b_scale, offs, total_rows, num_groups, k, n, nullptr, false, out,
                         ldo, 128, 32, workers);
  if (rc) return rc > 0 ? HMOE_OK : rc;
  return launch_fp8<kMxFp4>(p, workers, stream);
}

int hmoe_grouped_gemm_fwd_mxfp4_bias(const uint8_t* a_q, const uint8_t* a_scale, int64_t a_rows, const uint8_t* bq,
                                     const uint8_t* b_scale, const void* bias, const int32_t* offs, int64_t total_rows,
                                     int num_groups, int64_t k, int64_t n, void* out, int64_t ldo, void* stream) {
  using namespace hmoe;
  GemmArgs p{};
  int64_t workers = 0;
  const int rc = mx_args(p, a_q, a_scale, a_rows, bq, b_scale, offs, total_rows, num_groups, k, n, bias, true, out, ldo,
                         128, 32, workers);
  if (rc) return rc > 0 ? HMOE_OK : rc;
  return launch_fp8<kMxFp4, true>(p, workers, stream);
}

int hmoe_grouped_gemm_dgrad(const void* grad_out, int64_t ldg, const void* b, const int32_t* offs,
                            int64_t total_rows, int num_groups, int64_t k, int64_t n, int dtype, void* grad_a,
                            int64_t lda, void* stream) {
  using namespace hmoe;
  GemmArgs p{grad_out, ldg, b, n, grad_a, lda, offs, total_rows, num_groups, k, n, nullptr};
  if (int rc = validate(p, dtype)) return rc;
  if (total_rows == 0 || k == 0) return HMOE_OK;
  if (!grad_out || !b || !grad_a) return HMOE_INVALID_ARGUMENT;
  if (ldg < n || lda < k) return HMOE_INVALID_ARGUMENT;
  return launch<kDgrad>(p, dtype, static_cast<hipStream_t>(stream));
}

int hmoe_grouped_gemm_dgrad_addto(const void* grad_out, int64_t ldg, const void* b, const int32_t* offs,
                                  int64_t total_rows, int num_groups, int64_t k, int64_t n, int dtype,
                                  const void* addend, int64_t ld_addend, void* grad_a, int64_t lda, void* stream) {
  using namespace hmoe;
  GemmArgs p{grad_out, ldg, b, n, grad_a, lda, offs, total_rows, num_groups, k, n, nullptr};
  p.addend = addend;
  p.ld_addend = ld_addend;
  p.addend_scale = 1.f;
  if (int rc = validate(p, dtype)) return rc;
  if (total_rows == 0 || k == 0) return HMOE_OK;
  if (!grad_out || !b || !grad_a || !addend) return HMOE_INVALID_ARGUMENT;
  if (ldg < n || lda < k || ld_addend < k) return HMOE_INVALID_ARGUMENT;
  if (dtype == HMOE_BF16 && (!aligned16(addend) || ld_addend % 8 || ld_addend * 2 * 512 >= (int64_t(1) << 31)))
    return HMOE_UNSUPPORTED;
  return launch<kDgrad>(p, dtype, static_cast<hipStream_t>(stream));
}

int hmoe_grouped_gemm_wgrad(const void* a, int64_t lda, const void* grad_out, int64_t ldg, const int32_t* offs,
                            int64_t total_rows, int num_groups, int64_t k, int64_t n, int dtype, void* grad_b,
                            void* stream) {
  using namespace hmoe;
  GemmArgs p{a, lda, grad_out, ldg, grad_b, n, offs, total_rows, num_groups, k, n, nullptr};
  if (int rc = validate(p, dtype)) return rc;
  if (k == 0 || n == 0) return HMOE_OK;
  if (!grad_b || (total_rows > 0 && (!a || !grad_out))) return HMOE_INVALID_ARGUMENT;
  if (lda < k || ldg < n) return HMOE_INVALID_ARGUMENT;
  return launch<kWgrad>(p, dtype, static_cast<hipStream_t>(stream));
}

}  // extern "C"
