// Grouped GEMM for the MoE expert FFN on gfx950: forward, dgrad and wgrad over rows stacked by expert.
//
// Replaces torch's F.grouped_mm as the reference calls it (halo/kernels/grouped_mm.py:25-26, 39):
//   fwd    out[s:e]  = A[s:e]  @ B[g]          A [R,K],  B [G,K,N]
//   dgrad  dA[s:e]   = dO[s:e] @ B[g]^T        dO [R,N]
//   wgrad  dB[g]     = A[s:e]^T @ dO[s:e]      ragged contraction, empty group -> exact zeros
// with offs[g] the inclusive end of group g.  bf16 operands, fp32 accumulation on MFMA, one rounding.
//
// bf16 kernel.  One persistent launch; a workgroup (4 wavefronts) owns a 128x128 output tile and walks the
// contraction in steps of 64.  Both operand tiles sit in LDS as [128 output index][64 contraction index] with the
// contraction contiguous, so every MFMA fragment is one 16-byte LDS read; the 16-byte chunk index is XOR-swizzled with
// the row so fragment reads, straight copies and transposed writes are all bank-conflict free.  An operand whose
// contraction index is the strided one in global memory (B in fwd, both operands in wgrad) is transposed in registers
// (8x8 blocks of bf16, v_perm_b32) on its way into LDS.  Wavefronts 0-1 load operand A, 2-3 operand B; global loads
// for step k+1 are issued before the MFMAs of step k (register prefetch, two LDS buffers, one barrier per step).
// MFMA v_mfma_f32_32x32x16_bf16 is issued with the operands swapped (B fragment as srcA) so that a lane owns one
// output row and four consecutive columns per accumulator quad: stores are 8 bytes per lane.
//
// Tile schedule.  Every workgroup builds the per-group prefix of row tiles from offs in LDS (no host readback), so
// ragged and empty groups cost exactly their tiles.  The logical tile order is group-major, then column tile, then
// row tile; it is cut into 8 contiguous chunks, one per XCD (workgroup w runs on XCD w % 8), so the workgroups that
// share an L2 work on the same expert's weights at the same time, and the tile count per XCD is balanced whatever
// the skew of the expert loads.
//
// fp32 operands take a plain LDS-tiled FMA kernel (the CPU-sized plumbing configuration and tests).
#include "common.h"

namespace hmoe {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128;  // output rows per tile (operand A's output index)
constexpr int BN = 128;  // output cols per tile (operand B's output index)
constexpr int BK = 64;   // contraction per step
constexpr int kThreads = 256;
constexpr int kTile = 128 * BK;  // elements of one operand tile
constexpr int kXcds = 8;
constexpr int kMaxGroups = 1024;

enum Mode { kFwd = 0, kDgrad = 1, kWgrad = 2, kFwdFp8W = 3 };

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
};

__device__ __forceinline__ int swizzle(int row) { return (row & 7) ^ ((row >> 3) & 7); }
__device__ __forceinline__ int lds_offset(int row, int chunk) { return row * BK + ((chunk ^ swizzle(row)) << 3); }

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

// One operand tile's global -> register -> LDS path for the 128 threads that serve it.  A loader describes the
// operand (base pointer, row stride, first output index of the tile, limits) and moves one contraction step.
// kTrans == false: element(out, con) = base[out * ld + con]  (contraction contiguous)
// kTrans == true : element(out, con) = base[con * ld + out]  (output index contiguous), transposed on the way in
template <bool kTrans>
struct Bf16Loader {
  const bf16_t* __restrict__ base;
  int64_t ld;
  int out0, out_lim, con_lim;

  __device__ __forceinline__ void load(uint4 (&reg)[8], int con0, int tt) {
    if constexpr (!kTrans) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int cid = tt + 128 * i;
        const int out = out0 + (cid >> 3), con = con0 + ((cid & 7) << 3);
        reg[i] = make_uint4(0, 0, 0, 0);
        if (out < out_lim && con < con_lim)
          reg[i] = *reinterpret_cast<const uint4*>(base + static_cast<int64_t>(out) * ld + con);
      }
    } else {
      const int out = out0 + ((tt & 15) << 3);
      const int con_first = con0 + ((tt >> 4) << 3);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int con = con_first + i;
        reg[i] = make_uint4(0, 0, 0, 0);
        if (out < out_lim && con < con_lim)
          reg[i] = *reinterpret_cast<const uint4*>(base + static_cast<int64_t>(con) * ld + out);
      }
    }
  }

  __device__ __forceinline__ void store(const uint4 (&reg)[8], bf16_t* __restrict__ tile, int tt) const {
    if constexpr (!kTrans) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int cid = tt + 128 * i;
        *reinterpret_cast<uint4*>(tile + lds_offset(cid >> 3, cid & 7)) = reg[i];
      }
    } else {
      // reg[i] holds contraction index i, output indices 0..7 (two per dword).  Row o of the 8x8 block gathers
      // output index o from the eight registers: dword w of the result packs contraction 2w (low) and 2w+1 (high).
      const int row0 = (tt & 15) << 3, chunk = tt >> 4;
      const uint32_t(*r)[4] = reinterpret_cast<const uint32_t(*)[4]>(reg);
#pragma unroll
      for (int o = 0; o < 8; ++o) {
        const uint32_t sel = (o & 1) ? 0x07060302u : 0x05040100u;
        uint4 v;
        v.x = __builtin_amdgcn_perm(r[1][o >> 1], r[0][o >> 1], sel);
        v.y = __builtin_amdgcn_perm(r[3][o >> 1], r[2][o >> 1], sel);
        v.z = __builtin_amdgcn_perm(r[5][o >> 1], r[4][o >> 1], sel);
        v.w = __builtin_amdgcn_perm(r[7][o >> 1], r[6][o >> 1], sel);
        *reinterpret_cast<uint4*>(tile + lds_offset(row0 + o, chunk)) = v;
      }
    }
  }
};

// e4m3fn weights [contraction, output] (output contiguous) with one power-of-two fp32 scale per 128x128 block,
// dequantised to bf16 (exactly: an e4m3 value times a power of two is a bf16 value) and transposed on the way into
// LDS.  A tile spans one scale block across the outputs and at most one along the contraction step (128 % BK == 0).
struct Fp8BlockLoader {
  const uint8_t* __restrict__ base;
  int64_t ld;
  int out0, out_lim, con_lim;
  const float* __restrict__ scale;  // this group's scale grid, at column block out0 / 128
  int scale_ld;                     // scale blocks per contraction block row
  float step_scale;

  __device__ __forceinline__ void load(uint4 (&reg)[8], int con0, int tt) {
    const int out = out0 + ((tt & 15) << 3);
    const int con_first = con0 + ((tt >> 4) << 3);
    step_scale = scale[static_cast<int64_t>(con0 >> 7) * scale_ld];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int con = con_first + i;
      uint2 v = make_uint2(0, 0);
      if (out < out_lim && con < con_lim)
        v = *reinterpret_cast<const uint2*>(base + static_cast<int64_t>(con) * ld + out);
      reg[i].x = v.x;
      reg[i].y = v.y;
    }
  }

  __device__ __forceinline__ void store(const uint4 (&reg)[8], bf16_t* __restrict__ tile, int tt) const {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    const int row0 = (tt & 15) << 3, chunk = tt >> 4;
    uint32_t packed[8][4];  // [output][contraction pair]
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      float lo[8], hi[8];  // contraction 2w and 2w+1, outputs 0..7
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uint4 src = reg[2 * w + h];
        float* f = h ? hi : lo;
        const f32x2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(src.x, step_scale, false);
        const f32x2 b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(src.x, step_scale, true);
        const f32x2 c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(src.y, step_scale, false);
        const f32x2 d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(src.y, step_scale, true);
        f[0] = a.x; f[1] = a.y; f[2] = b.x; f[3] = b.y; f[4] = c.x; f[5] = c.y; f[6] = d.x; f[7] = d.y;
      }
#pragma unroll
      for (int o = 0; o < 8; ++o)
        packed[o][w] = static_cast<uint32_t>(f32_to_bf16(lo[o])) | (static_cast<uint32_t>(f32_to_bf16(hi[o])) << 16);
    }
#pragma unroll
    for (int o = 0; o < 8; ++o)
      *reinterpret_cast<uint4*>(tile + lds_offset(row0 + o, chunk)) =
          make_uint4(packed[o][0], packed[o][1], packed[o][2], packed[o][3]);
  }
};

// C[a_out, b_out] = sum_con A(a_out, con) * B(b_out, con) over one 128x128 tile.
template <typename LoaderA, typename LoaderB>
__device__ __forceinline__ void compute_tile(bf16_t* __restrict__ smem, LoaderA la, LoaderB lb,
                                             bf16_t* __restrict__ c_base, int64_t c_ld) {
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const bool loads_a = tid < 128;
  const int tt = tid & 127;
  bf16_t* s_a = smem;               // [2][kTile]
  bf16_t* s_b = smem + 2 * kTile;   // [2][kTile]
  const int a_out0 = la.out0, a_out_lim = la.out_lim, b_out0 = lb.out0, b_out_lim = lb.out_lim;
  const int con_lim = la.con_lim;

  uint4 reg[8];  // the thread's share of the next operand tile (A for wavefronts 0-1, B for 2-3)
  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int steps = (con_lim + BK - 1) / BK;
  if (steps > 0) {
    if (loads_a) {
      la.load(reg, 0, tt);
      la.store(reg, s_a, tt);
    } else {
      lb.load(reg, 0, tt);
      lb.store(reg, s_b, tt);
    }
  }
  __syncthreads();
  for (int step = 0; step < steps; ++step) {
    const int cur = step & 1;
    const bool more = step + 1 < steps;
    if (more) {
      if (loads_a) la.load(reg, (step + 1) * BK, tt);
      else lb.load(reg, (step + 1) * BK, tt);
    }
    const bf16_t* ta = s_a + cur * kTile;
    const bf16_t* tb = s_b + cur * kTile;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      const int chunk = kk * 2 + (lane >> 5);
      bf16x8 fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int ra = wm * 64 + i * 32 + (lane & 31);
        const int rb = wn * 64 + i * 32 + (lane & 31);
        fa[i] = *reinterpret_cast<const bf16x8*>(ta + lds_offset(ra, chunk));
        fb[i] = *reinterpret_cast<const bf16x8*>(tb + lds_offset(rb, chunk));
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
    if (more) {
      if (loads_a) la.store(reg, s_a + (cur ^ 1) * kTile, tt);
      else lb.store(reg, s_b + (cur ^ 1) * kTile, tt);
    }
    __syncthreads();
  }
  // lane owns output row (lane & 31) of each 32x32 block; accumulator quad q holds columns q*8 + (lane>>5)*4 .. +3
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = a_out0 + wm * 64 + i * 32 + (lane & 31);
    if (row >= a_out_lim) continue;
    bf16_t* c_row = c_base + static_cast<int64_t>(row) * c_ld;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int col = b_out0 + wn * 64 + j * 32 + q * 8 + ((lane >> 5) << 2);
        if (col < b_out_lim) {
          uint2 packed;
          packed.x = static_cast<uint32_t>(f32_to_bf16(acc[i][j][q * 4 + 0])) |
                     (static_cast<uint32_t>(f32_to_bf16(acc[i][j][q * 4 + 1])) << 16);
          packed.y = static_cast<uint32_t>(f32_to_bf16(acc[i][j][q * 4 + 2])) |
                     (static_cast<uint32_t>(f32_to_bf16(acc[i][j][q * 4 + 3])) << 16);
          *reinterpret_cast<uint2*>(c_row + col) = packed;
        }
      }
    }
  }
}

// Exclusive prefix of the per-group row-tile counts into LDS: tile_start[0..groups], by wavefront 0.
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

template <int kMode>
__global__ void __launch_bounds__(kThreads, 2) grouped_gemm_bf16_kernel(GemmArgs p) {
  __shared__ __attribute__((aligned(16))) bf16_t smem[4 * kTile];
  __shared__ int32_t tile_start[kMode == kWgrad ? 1 : kMaxGroups + 1];
  const bf16_t* a = static_cast<const bf16_t*>(p.a);
  const bf16_t* b = static_cast<const bf16_t*>(p.b);
  bf16_t* c = static_cast<bf16_t*>(p.c);

  const int workers = gridDim.x;
  const int xcd = blockIdx.x % kXcds;
  const int local = blockIdx.x / kXcds;
  const int workers_here = (workers - xcd + kXcds - 1) / kXcds;

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
      compute_tile(smem, Bf16Loader<true>{a + s * p.lda, p.lda, m_t * BM, static_cast<int>(p.k), rows},
                   Bf16Loader<true>{b + s * p.ldb, p.ldb, n_t * BN, static_cast<int>(p.n), rows},
                   c + static_cast<int64_t>(g) * p.k * p.n, p.ldc);
    }
  } else {
    build_tile_prefix(tile_start, p.offs, p.groups, p.total_rows);
    const int64_t out_cols = kMode == kDgrad ? p.k : p.n;
    const int64_t con = kMode == kDgrad ? p.n : p.k;
    const int nt = static_cast<int>((out_cols + BN - 1) / BN);
    const int64_t total = static_cast<int64_t>(tile_start[p.groups]) * nt;
    const int64_t chunk = (total + kXcds - 1) / kXcds;
    const int64_t first = xcd * chunk;
    const int64_t last = first + chunk < total ? first + chunk : total;
    for (int64_t t = first + local; t < last; t += workers_here) {
      int lo = 0, hi = p.groups;        // largest g with tile_start[g] * nt <= t
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
      const Bf16Loader<false> la{a + s * p.lda, p.lda, m_t * BM, static_cast<int>(e - s), static_cast<int>(con)};
      if constexpr (kMode == kFwd) {
        const bf16_t* w = b + static_cast<int64_t>(g) * p.k * p.n;
        compute_tile(smem, la, Bf16Loader<true>{w, p.ldb, n_t * BN, static_cast<int>(p.n), static_cast<int>(con)},
                     c + s * p.ldc, p.ldc);
      } else if constexpr (kMode == kDgrad) {
        const bf16_t* w = b + static_cast<int64_t>(g) * p.k * p.n;
        compute_tile(smem, la, Bf16Loader<false>{w, p.ldb, n_t * BN, static_cast<int>(p.k), static_cast<int>(con)},
                     c + s * p.ldc, p.ldc);
      } else {  // kFwdFp8W
        const int scale_ld = static_cast<int>((p.n + 127) >> 7);
        const int64_t scale_blocks = ((p.k + 127) >> 7) * scale_ld;
        const uint8_t* w = static_cast<const uint8_t*>(p.b) + static_cast<int64_t>(g) * p.k * p.n;
        compute_tile(smem, la,
                     Fp8BlockLoader{w, p.ldb, n_t * BN, static_cast<int>(p.n), static_cast<int>(con),
                                    p.b_scale + g * scale_blocks + ((n_t * BN) >> 7), scale_ld, 1.0f},
                     c + s * p.ldc, p.ldc);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------ fp32 path
// 64x64 tile, contraction step 16, 256 threads each owning a 4x4 block.  grid.x walks row tiles of every group
// (an upper bound of ceil(R/64)+G tiles; surplus workgroups exit), grid.y column tiles.
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
      if (r < rows_out && cc < cols_out) out[r * p.ldc + cc] = acc[i][j];
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

template <int kMode>
int launch(const GemmArgs& p, int dtype, hipStream_t stream) {
  if (dtype == HMOE_BF16) {
    // upper bound on the number of tiles, so no more workgroups start than can find work
    const int64_t out_cols = kMode == kDgrad ? p.k : p.n;
    const int64_t nt = (out_cols + BN - 1) / BN;
    int64_t bound;
    if (kMode == kWgrad) bound = ((p.k + BM - 1) / BM) * nt * p.groups;
    else bound = (p.total_rows / BM + p.groups) * nt;
    int64_t workers = static_cast<int64_t>(device_cus()) * 2;
    if (bound < workers) workers = bound;
    workers = (workers + kXcds - 1) / kXcds * kXcds;
    if (workers <= 0) return HMOE_OK;
    grouped_gemm_bf16_kernel<kMode><<<dim3(static_cast<unsigned>(workers)), dim3(kThreads), 0, stream>>>(p);
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
  }
  return HMOE_OK;
}

}  // namespace
}  // namespace hmoe

extern "C" {

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
