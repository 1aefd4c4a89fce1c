// Large-M dequant-GEMM on the matrix cores: forward Y = X * W^T, input gradient dX = dY * W,
// and the same two over token-sorted expert segments (one launch for all experts).
//
// One kernel template covers all four.  Seen from the matrix core every case is
//     D[M, C] = A[M, R] * B[R, C]          A = activations (X or dY), row-major, R contiguous
// with B drawn from the stored weight W[N,K]:
//     forward : C = N, R = K, B[r][c] = W[c][r]   (a weight row is contiguous along R)
//     backward: C = K, R = N, B[r][c] = W[r][c]   (a weight row is contiguous along C)
// A workgroup of 512 threads owns a BM x 128 tile of D (BM = 256 when that still gives enough
// tiles to fill the chip, else 128) and walks R in steps of 64.  Its waves are specialised: waves
// 4..7 ("producers") stage operands, waves 0..3 ("consumers", laid out 2x2 over the tile) run the
// MFMAs, one of each per SIMD, so unpacking arithmetic and the matrix pipe overlap without any
// instruction-level interleaving.  Per step the producers move a BMx64 tile of A and the matching
// 64x128 piece of W from global memory into registers two steps ahead of their use, dequantise W
// there (code * scale in fp32, one rounding to the compute dtype: bit-identical to the reference's
// dequantise-then-cast weight) and write both tiles to the other half of a double-buffered LDS
// area, as [row][64 values along R] with the 16-byte chunks of a row XOR-swizzled by row bits so
// that the 128-bit operand reads of v_mfma_f32_32x32x16 and the transposed writes of the backward
// case spread over all banks.  For the backward case the weight piece is transposed on the way:
// a thread holds 4 weight rows x 8 columns and writes 8 runs of 4 values along R.
// A consumer wave accumulates a (BM/2) x 64 sub-tile (64 or 128 fp32 accumulators per lane) and
// keeps the operand fragments of the next 16-wide k step in flight while the MFMAs of the current
// one issue.  All eight waves meet at one barrier per step.
// No dense copy of W ever reaches HBM; the only HBM traffic is A, the packed W and D.
#pragma once

#include "caifx_internal.hpp"

#include <atomic>
#include <type_traits>

namespace caifx {
namespace gemm_tile {

// how the weight is stored: int8 codes, packed int4 codes, or values of the 16-bit compute type (no dequantisation)
enum { W_CODES8 = 0, W_CODES4 = 1, W_DENSE16 = 2 };

constexpr int BC = 128;      // columns of D per workgroup
constexpr int BR = 64;       // reduction extent per step
constexpr int kWStagers = 256;              // producer threads that stage the W piece (the first four producer waves)
constexpr int kBTileBytes = BC * BR * 2;   // weight tile in LDS (16 KiB)

enum { SM_SCALAR = 0, SM_VEC4 = 1, SM_ANY = 2 };   // how int8 scales are fetched
// What the store does besides rounding the accumulator v to the result type T:
//   EPI_SWIGLU_FWD  the launch is the up projection: d = v, d2 = T(T(silu(e1)) * v)             (e1 = gate)
//   EPI_SWIGLU_BWD  the launch is the input gradient of the down projection, v = grad of hidden:
//                   d = T(silu'(e1) * T(v * e2)), d2 = T(v * T(silu(e1)))                       (e1 = gate, e2 = up)
enum { EPI_NONE = 0, EPI_SWIGLU_FWD = 1, EPI_SWIGLU_BWD = 2 };

struct TileArgs {
  int64_t M, N, K;           // N = OutputDim, K = InputDim of the weight
  const void *a;             // activations [M, R]
  void *d;                   // result [M, C]
  int d_dtype;
  const void *addend;        // optional [M, C] of d_dtype: d = T(float(T(acc)) + float(addend))
  int vec_store;             // C % 8 == 0, 16-byte aligned pointers: the store goes through LDS in 16-byte pieces
  // gated-expert epilogues (16-bit results through the staged store only), see EPI_*
  int epilogue;
  const void *e1, *e2;       // [M, C] of d_dtype: gate (forward); gate, up (backward)
  void *d2;                  // second result [M, C]
  const void *wq;
  const void *scales;
  int group_shift;           // int4: log2(group_size)
  int scale_mode;            // int8
  int64_t period;            // int8
  uint32_t scale_step;       // int8, SM_VEC4: how far the scale index moves per 64-deep step, modulo period
  // grouped form
  const int32_t *offsets;
  const void *const *wq_ptrs;
  const void *const *scales_ptrs;
  int num_experts;
  // plain form with few tiles: ksplit workgroups share a tile, each takes split_steps 64-deep steps of the
  // reduction and writes its fp32 partial tile to d + split * M * C (d is then the caller's workspace)
  int ksplit;
  int split_steps;
  // grouped form, measurement only: per tile {expert, rows, start, end} in 100 MHz ticks (null: nothing is recorded)
  unsigned long long *stamps;
  long long stamps_capacity;
};

// byte offset of 16-byte chunk `chunk` (0..7) of LDS tile row `row`.  The chunk position is XORed
// with bits of the row so that (a) 8 consecutive rows at one chunk index and (b) rows 8 apart at one
// chunk index (the transposed weight writes of the backward case) land in different banks.
__device__ __forceinline__ int swz(int row, int chunk) { return row * 128 + ((chunk ^ ((row ^ (row >> 3)) & 7)) << 4); }

__device__ __forceinline__ float int8_scale_at(const float *scales, int mode, int64_t period, int64_t flat)
{
  if (mode == SM_SCALAR) return scales ? scales[0] : 1.0f;
  return scales[flat % period];
}

// BM: rows of D per workgroup (128 or 256); a wave owns (BM/2) x 64 of D.
// kSLds (int8 with a periodic scale vector that fits): the scale vector sits in LDS behind the
// tile buffers and is read when a weight piece is dequantised, instead of travelling through
// registers with the codes.
// kCW: consumer waves (4 or 8), laid out (kCW/2) x 2 over the tile; there are as many producer waves.
template <typename CT, typename XT, int kW, bool kSLds, bool kBackward, bool kGrouped, int BM, int kCW>
__global__ __launch_bounds__(2 * kCW * 64, (kCW == 8 || (BM == 128 && (kW == W_CODES4 || kSLds))) ? 4 : 2) void qgemm_kernel(TileArgs g)
{
  constexpr bool kInt4 = kW == W_CODES4;
  constexpr bool kDense = kW == W_DENSE16;       // the stored weight already is the compute type: producers only copy
  constexpr int kThreads = 2 * kCW * 64;
  constexpr int kStagers = kCW * 64;                         // producer threads
  constexpr int kWaveRows = BM / (kCW / 2);                  // rows of D per consumer wave
  typedef typename Mfma32<CT>::vec_t vec_t;
  constexpr int kATileBytes = BM * BR * 2;
  constexpr int kAStages = 2;
  constexpr int kBBase = kAStages * kATileBytes;             // LDS: A ring, then two B buffers
  constexpr int kSBase = kBBase + 2 * kBTileBytes;           // ... then the int8 scale vector (kSLds)
  constexpr int WR = kWaveRows / 32;                         // 32-row MFMA tiles per wave along M
  constexpr int kAChunks = BM * 8 / kStagers;                // 16-byte LDS chunks of A per thread per step
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];          // 2 x kStageBytes
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const bool producer = wave >= kCW;               // the upper half of the waves stages tiles, the lower half runs the MFMAs
  const int tid = threadIdx.x - kStagers;          // staging thread index (producers)
  const bool w_stager = tid < kWStagers;           // wave-uniform: the W piece is laid out for 256 threads
  const int wm = wave >> 1;        // consumer wave row: kWaveRows rows of D
  const int wc = wave & 1;         // consumer wave column (0..1): 64 columns of D

  const int64_t R = kBackward ? g.N : g.K;     // reduction length
  const int64_t C = kBackward ? g.K : g.N;     // columns of D

  // ---- which tile -----------------------------------------------------------------------
  int64_t row_lo, row_hi;        // rows of A / D this workgroup may touch: [row_lo, row_hi)
  int split = 0;                 // which part of the reduction (plain form with ksplit > 1)
  int64_t stamp_pos = -1;        // grouped form with a stamp buffer: thread 0 writes the tile's end time there
  int64_t col_tile = blockIdx.x;
  const uint8_t *wq = static_cast<const uint8_t *>(g.wq);
  const void *scales = g.scales;
  if constexpr (kGrouped) {
    // tiles are numbered expert by expert, row tile by row tile, column tile last, one contiguous eighth of the
    // list per XCD (grouped_tile); the grid is an upper bound padded to a multiple of 8
    const int64_t col_tiles = (C + BC - 1) / BC;
    GroupedTile gt;
    if (!grouped_tile<BM>(g.offsets, g.num_experts, g.M, col_tiles, g.wq_ptrs, g.scales_ptrs, lane, gt)) return;
    const int e = gt.e;
    const int64_t pos = gt.pos;
    col_tile = gt.col_tile;
    row_lo = gt.row0;
    row_hi = gt.row_end;
    wq = static_cast<const uint8_t *>(gt.wq);
    scales = gt.scales;
    if (g.stamps && threadIdx.x == 0 && pos < g.stamps_capacity) {
      const int64_t rows = row_hi - row_lo < BM ? row_hi - row_lo : BM;
      g.stamps[4 * pos] = static_cast<unsigned long long>(e);
      g.stamps[4 * pos + 1] = static_cast<unsigned long long>(rows);
      g.stamps[4 * pos + 2] = wall_clock64();
      stamp_pos = pos;
    }
  } else {
    // Workgroups are handed to the 8 XCDs in turn (linear id mod 8), and each XCD has its own L2.
    // The tiles are therefore numbered so that one XCD walks one contiguous eighth of the list, and
    // the list runs through bands of 512 rows column by column: the 32 tiles an XCD works on at any
    // time form a 512-row x 16-tile patch, which touches far fewer distinct rows of A than a
    // full-height stripe of the same area.  The grid is padded to a multiple of 8.
    constexpr int kBandTiles = 512 / BM;
    const int64_t col_tiles = (C + BC - 1) / BC;
    const int64_t row_tiles = (g.M + BM - 1) / BM;
    const unsigned bid = blockIdx.x / static_cast<unsigned>(g.ksplit);
    split = static_cast<int>(blockIdx.x - bid * static_cast<unsigned>(g.ksplit));
    const int64_t per_xcd = (gridDim.x / static_cast<unsigned>(g.ksplit)) >> 3;
    const int64_t pos = static_cast<int64_t>(bid & 7) * per_xcd + (bid >> 3);
    if (pos >= row_tiles * col_tiles) return;
    const int64_t band = pos / (kBandTiles * col_tiles);
    const int64_t within = pos - band * kBandTiles * col_tiles;
    const int64_t left = row_tiles - band * kBandTiles;
    const int64_t band_rows = left < kBandTiles ? left : kBandTiles;
    col_tile = within / band_rows;
    row_lo = (band * kBandTiles + within % band_rows) * BM;
    row_hi = g.M;
  }
  const int64_t col0 = col_tile * BC;
  const XT *ag = static_cast<const XT *>(g.a);
  float *slds = reinterpret_cast<float *>(smem + kSBase);
  if constexpr (kSLds) {
    const floatx4_t *src = static_cast<const floatx4_t *>(scales);
    for (int i = threadIdx.x; i < static_cast<int>(g.period >> 2); i += kThreads)
      reinterpret_cast<floatx4_t *>(slds)[i] = src[i];
    __syncthreads();
  }

  // ---- global -> register staging ---------------------------------------------------------
  // Two register sets: while the matrix cores work on the tile in LDS buffer (s & 1), set (s+1)&1
  // (loaded one step earlier) is dequantised into the other buffer and set s&1 receives tile s+2
  // from global memory.  (A third set, i.e. two steps of load latency, measured no faster.)  The store work is cut in four parts, one per 16-wide k step, so that it
  // can be interleaved with the MFMAs of that k step.
  // A tile: BM rows x 8 chunks (8 values each); producer thread handles chunks q = tid + 256*i
  constexpr int kAVecs = (sizeof(XT) == 4) ? 2 * kAChunks : kAChunks;     // 16-byte loads per thread per step
  u32x4_t areg[2][kAVecs];
  int a_off[kAChunks];            // LDS byte offset of each chunk inside the A tile
  const XT *a_ptr[kAChunks];
#pragma unroll
  for (int i = 0; i < kAChunks; ++i) {
    const int q = tid + kStagers * i;
    a_off[i] = swz(q >> 3, q & 7);
    int64_t m = row_lo + (q >> 3);
    if (m >= row_hi) m = row_hi - 1;                    // clamp: rows past the end are never stored
    a_ptr[i] = ag + m * R + (q & 7) * 8;
  }
  // part < 0: the whole tile; else the quarter of this thread's chunks that store_a(part) has just
  // written out, so that the requests spread over the step instead of queueing up at its end
  auto load_a = [&](auto set_, int64_t r0, int part = -1) {
    constexpr int set = decltype(set_)::value;
    constexpr int per = kAChunks / 4;
#pragma unroll
    for (int i = 0; i < kAChunks; ++i) {
      if (part >= 0 && i / per != part) continue;
      if constexpr (sizeof(XT) == 4) {
        areg[set][2 * i] = *reinterpret_cast<const u32x4_t *>(a_ptr[i] + r0);
        areg[set][2 * i + 1] = *reinterpret_cast<const u32x4_t *>(a_ptr[i] + r0 + 4);
      } else {
        areg[set][i] = *reinterpret_cast<const u32x4_t *>(a_ptr[i] + r0);
      }
    }
  };
  auto store_a = [&](auto set_, unsigned char *dst, int part) {
    constexpr int set = decltype(set_)::value;
    constexpr int per = kAChunks / 4;
#pragma unroll
    for (int ii = 0; ii < per; ++ii) {
      const int i = part * per + ii;
      u32x4_t v;
      if constexpr (sizeof(XT) == 4) {
        const float *f0 = reinterpret_cast<const float *>(&areg[set][2 * i]);
        const float *f1 = reinterpret_cast<const float *>(&areg[set][2 * i + 1]);
        v[0] = pack2<CT>(f0[0], f0[1]);
        v[1] = pack2<CT>(f0[2], f0[3]);
        v[2] = pack2<CT>(f1[0], f1[1]);
        v[3] = pack2<CT>(f1[2], f1[3]);
      } else {
        v = areg[set][i];
      }
      *reinterpret_cast<u32x4_t *>(dst + a_off[i]) = v;
    }
  };

  // W piece.  Registers hold raw codes (+ int4 scales); dequantisation happens at store time.
  //   forward  int4: row c = tid/2, 32 codes (16 B) at r = (tid%2)*32           -> 4 chunks
  //   forward  int8: rows c = tid/4 (+64), 16 codes (16 B) at r = (tid%4)*16    -> 2 x 2 chunks
  //   backward int4: rows r = (tid/16)*4 .. +3, 8 codes (4 B) at c = (tid%16)*8 -> 8 runs of 4
  //   backward int8: same rows, 8 codes (8 B)
  //   dense forward / backward: the int4 geometry with 2 bytes per value -> 4 x 16 bytes per thread and step
  uint32_t wreg[2][kDense ? 16 : 8];
  f16_t wscale[2][4];
  int64_t w_flat[4] = {0, 0, 0, 0};   // flat index n*K + k of each register row's first code at step 0
  const f16_t *s16 = static_cast<const f16_t *>(scales);
  const float *s32 = static_cast<const float *>(scales);
  int wf_c = 0, wf_r = 0;  // forward: tile-local column / first r;  backward: first r row / first c
  if constexpr (!kBackward) {
    if constexpr (kInt4 || kDense) {
      wf_c = tid >> 1;
      wf_r = (tid & 1) * 32;
      int64_t n = col0 + wf_c;
      if (n >= g.N) n = g.N - 1;
      w_flat[0] = n * g.K + wf_r;
    } else {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        int64_t n = col0 + (tid >> 2) + 64 * i;
        if (n >= g.N) n = g.N - 1;
        w_flat[i] = n * g.K + (tid & 3) * 16;
      }
      wf_c = tid >> 2;
      wf_r = (tid & 3) * 16;
    }
  } else {
    wf_r = (tid >> 4) * 4;
    wf_c = (tid & 15) * 8;
    int64_t k = col0 + wf_c;
    if (k + 8 > g.K) k = g.K - 8;                        // clamp: those columns are never stored
#pragma unroll
    for (int i = 0; i < 4; ++i) w_flat[i] = static_cast<int64_t>(wf_r + i) * g.K + k;
  }
  // int8 with a periodic scale vector (SM_VEC4): the four scales of every code dword travel with
  // the codes, fetched at position (flat index mod period).  That position is kept per register
  // row and moved by scale_step after each tile, so no division runs in the loop.
  floatx4_t wsc8[2][8];
  uint32_t sidx[4] = {0, 0, 0, 0};
  const uint32_t period32 = static_cast<uint32_t>(g.period);
  int steps = static_cast<int>(R / BR);
  if constexpr (!kGrouped) {
    if (g.ksplit > 1) {
      // this workgroup's part of the reduction: everything below counts steps from its first one
      const int first = split * g.split_steps;
      const int64_t r_begin = static_cast<int64_t>(first) * BR;
      steps = steps - first < g.split_steps ? steps - first : g.split_steps;
#pragma unroll
      for (int i = 0; i < kAChunks; ++i) a_ptr[i] += r_begin;
#pragma unroll
      for (int i = 0; i < 4; ++i) w_flat[i] += kBackward ? r_begin * g.K : r_begin;
    }
  }
  if constexpr (kW == W_CODES8) {
    if (g.scale_mode == SM_VEC4) {
#pragma unroll
      for (int i = 0; i < (kBackward ? 4 : 2); ++i) sidx[i] = static_cast<uint32_t>(w_flat[i] % g.period);
    }
  }
  const int last = steps - 1;
  auto tile_r0 = [&](int t) { return static_cast<int64_t>(t < last ? t : last) * BR; };   // clamped: reloading the last tile is harmless
  auto load_w = [&](auto set_, int t) {
    constexpr int set = decltype(set_)::value;
    const int64_t r0 = tile_r0(t);
    if constexpr (kW == W_CODES8 && !kSLds) {
      if (g.scale_mode == SM_VEC4) {
        constexpr int rows = kBackward ? 4 : 2;
        constexpr int quads = kBackward ? 2 : 4;
#pragma unroll
        for (int i = 0; i < rows; ++i) {
#pragma unroll
          for (int q = 0; q < quads; ++q) {
            uint32_t idx = sidx[i] + 4 * q;
            if (idx >= period32) idx -= period32;
            wsc8[set][quads * i + q] = *reinterpret_cast<const floatx4_t *>(s32 + idx);
          }
          if (t < last) {
            sidx[i] += g.scale_step;
            if (sidx[i] >= period32) sidx[i] -= period32;
          }
        }
      }
    }
    if constexpr (!kBackward) {
      if constexpr (kDense) {
        const int64_t f = w_flat[0] + r0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const u32x4_t v = *reinterpret_cast<const u32x4_t *>(wq + 2 * f + 16 * q);
#pragma unroll
          for (int j = 0; j < 4; ++j) wreg[set][4 * q + j] = v[j];
        }
      } else if constexpr (kInt4) {
        const int64_t f = w_flat[0] + r0;
        const u32x4_t v = *reinterpret_cast<const u32x4_t *>(wq + (f >> 1));
#pragma unroll
        for (int j = 0; j < 4; ++j) wreg[set][j] = v[j];
        wscale[set][0] = s16[f >> g.group_shift];
      } else {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const u32x4_t v = *reinterpret_cast<const u32x4_t *>(wq + w_flat[i] + r0);
#pragma unroll
          for (int j = 0; j < 4; ++j) wreg[set][4 * i + j] = v[j];
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t f = w_flat[i] + r0 * g.K;
        if constexpr (kDense) {
          const u32x4_t v = *reinterpret_cast<const u32x4_t *>(wq + 2 * f);
#pragma unroll
          for (int j = 0; j < 4; ++j) wreg[set][4 * i + j] = v[j];
        } else if constexpr (kInt4) {
          wreg[set][i] = *reinterpret_cast<const uint32_t *>(wq + (f >> 1));
          wscale[set][i] = s16[f >> g.group_shift];
        } else {
          const u32x2_t v = *reinterpret_cast<const u32x2_t *>(wq + f);
          wreg[set][2 * i] = v[0];
          wreg[set][2 * i + 1] = v[1];
        }
      }
    }
  };
  // int8: fp32 value of 4 codes of dword p whose first code has flat index f
  // the four scales of code dword `slot` of register row `row` (quads of a row are 4 apart)
  auto scale_quad = [&](auto set_, int row, int quad, int slot) {
    constexpr int set = decltype(set_)::value;
    if constexpr (kSLds) {
      uint32_t idx = sidx[row] + 4 * quad;
      if (idx >= period32) idx -= period32;
      return *reinterpret_cast<const floatx4_t *>(slds + idx);
    } else {
      return wsc8[set][slot];
    }
  };
  auto deq8 = [&](uint32_t p, const floatx4_t &s, int64_t f, float (&out)[4]) {
    float q[4];
    int8x4_to_f32(p, q);
    if (kSLds || g.scale_mode == SM_VEC4) {
#pragma unroll
      for (int j = 0; j < 4; ++j) out[j] = q[j] * s[j];
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) out[j] = q[j] * int8_scale_at(s32, g.scale_mode, g.period, f + j);
    }
  };
  // Backward keeps the dequantised 4 x 8 block between parts: parts 0..3 dequantise one weight row
  // each, part 3 then writes the 8 transposed runs.
  float et[4][8];
  auto store_w = [&](auto set_, unsigned char *dst, int64_t r0, int part) {
    constexpr int set = decltype(set_)::value;
    if constexpr (!kBackward) {
      if constexpr (kDense) {
        const int j = part;
        u32x4_t v;
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = wreg[set][4 * j + q];
        *reinterpret_cast<u32x4_t *>(dst + swz(wf_c, (wf_r >> 3) + j)) = v;
      } else if constexpr (kInt4) {
        const float s = to_f32(wscale[set][0]);
        const int j = part;
        float e[8];
        dequant_int4x8(wreg[set][j], s, e);
        u32x4_t v;
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = pack2<CT>(e[2 * q], e[2 * q + 1]);
        *reinterpret_cast<u32x4_t *>(dst + swz(wf_c, (wf_r >> 3) + j)) = v;
      } else {
        const int i = part >> 1;
        const int j = part & 1;
        float lo[4], hi[4];
        deq8(wreg[set][4 * i + 2 * j], scale_quad(set_, i, 2 * j, 4 * i + 2 * j), w_flat[i] + r0 + 8 * j, lo);
        deq8(wreg[set][4 * i + 2 * j + 1], scale_quad(set_, i, 2 * j + 1, 4 * i + 2 * j + 1), w_flat[i] + r0 + 8 * j + 4, hi);
        u32x4_t v;
        v[0] = pack2<CT>(lo[0], lo[1]);
        v[1] = pack2<CT>(lo[2], lo[3]);
        v[2] = pack2<CT>(hi[0], hi[1]);
        v[3] = pack2<CT>(hi[2], hi[3]);
        *reinterpret_cast<u32x4_t *>(dst + swz(wf_c + 64 * i, (wf_r >> 3) + j)) = v;
      }
    } else {
      const int i = part;      // et[i][j]: weight row (reduction index) wf_r + i, column wf_c + j
      if constexpr (kDense) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          typedef __attribute__((__vector_size__(2 * sizeof(CT)))) CT pair_t;
          const pair_t pr = __builtin_bit_cast(pair_t, wreg[set][4 * i + q]);
          et[i][2 * q] = to_f32<CT>(pr[0]);
          et[i][2 * q + 1] = to_f32<CT>(pr[1]);
        }
      } else if constexpr (kInt4) {
        dequant_int4x8(wreg[set][i], to_f32(wscale[set][i]), et[i]);
      } else {
        const int64_t f = w_flat[i] + r0 * g.K;
        float lo[4], hi[4];
        deq8(wreg[set][2 * i], scale_quad(set_, i, 0, 2 * i), f, lo);
        deq8(wreg[set][2 * i + 1], scale_quad(set_, i, 1, 2 * i + 1), f + 4, hi);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          et[i][j] = lo[j];
          et[i][4 + j] = hi[j];
        }
      }
      if (part == 3) {
        // transposed write: LDS row = column c, run of 4 values along R at r = wf_r .. wf_r+3
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          u32x2_t v;
          v[0] = pack2<CT>(et[0][j], et[1][j]);
          v[1] = pack2<CT>(et[2][j], et[3][j]);
          *reinterpret_cast<u32x2_t *>(dst + swz(wf_c + j, wf_r >> 3) + ((wf_r & 4) << 1)) = v;
        }
      }
    }
    if constexpr (kW == W_CODES8 && kSLds) {
      if (part == 3) {        // tiles are stored in order: move every row's scale position to the next tile
#pragma unroll
        for (int i = 0; i < (kBackward ? 4 : 2); ++i) {
          sidx[i] += g.scale_step;
          if (sidx[i] >= period32) sidx[i] -= period32;
        }
      }
    }
  };

  // ---- main loop ------------------------------------------------------------------------
  // Wave specialisation: the four producer waves move tile s+1 from their registers into LDS
  // buffer (s+1)&1 (dequantising W on the way) and fetch tile s+2 from global memory, while the
  // four consumer waves run the MFMAs of tile s out of buffer s&1.  One producer and one consumer
  // wave share each SIMD, so the VALU work of unpacking and the matrix pipe overlap without any
  // instruction-level interleaving; all eight waves meet at one barrier per step.
  typedef std::integral_constant<int, 0> I0;
  typedef std::integral_constant<int, 1> I1;

  if (producer) {
    load_a(I0{}, 0);
    if (w_stager) load_w(I0{}, 0);
#pragma unroll
    for (int part = 0; part < 4; ++part) {
      store_a(I0{}, smem, part);
      if (w_stager) store_w(I0{}, smem + kBBase, 0, part);
    }
    load_a(I1{}, tile_r0(1));
    if (w_stager) load_w(I1{}, 1);
    load_a(I0{}, tile_r0(2));
    if (w_stager) load_w(I0{}, 2);
    __syncthreads();
    // step s: register set (s+1)&1 holds tile s+1 -> LDS buffer (s+1)&1, then that set <- tile s+3
    // (set p always carries tiles of parity p; a load has two steps to arrive).  The A chunks are
    // requested again right after they have been written out, so that the requests spread over the
    // step instead of queueing up at its end.
    auto pstep = [&](auto buf_, int s) {
      constexpr int buf = decltype(buf_)::value;
      typedef std::integral_constant<int, 1 - buf> NxtSet;
      const int64_t r_next = tile_r0(s + 1);
      const int64_t r_load = tile_r0(s + 3);
#pragma unroll
      for (int part = 0; part < 4; ++part) {
        store_a(NxtSet{}, smem + (1 - buf) * kATileBytes, part);
        load_a(NxtSet{}, r_load, part);
        if (w_stager) store_w(NxtSet{}, smem + kBBase + (1 - buf) * kBTileBytes, r_next, part);
      }
      if (w_stager) load_w(NxtSet{}, s + 3);
      __syncthreads();
    };
    int s = 0;
    for (; s + 2 <= steps; s += 2) {
      pstep(I0{}, s);
      pstep(I1{}, s + 1);
    }
    if (s < steps) pstep(I0{}, s);
    return;
  }

  floatx16_t acc[WR][2];
#pragma unroll
  for (int i = 0; i < WR; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int frow = lane & 31;    // row of the operand tile this lane supplies
  const int fh = lane >> 5;      // which half of the 16-wide k step

  __syncthreads();               // tile 0 is in LDS
  auto cstep = [&](auto abuf_, auto bbuf_, int s) {
    constexpr int astage = decltype(abuf_)::value;
    constexpr int bstage = decltype(bbuf_)::value;
    const unsigned char *abuf = smem + astage * kATileBytes;
    const unsigned char *bbuf = smem + kBBase + bstage * kBTileBytes;
    // operand fragments are double buffered in registers: the reads of k step ks+1 are issued
    // before the MFMAs of k step ks
    vec_t af[2][WR], bf[2][2];
    auto read_frags = [&](int fb, int ks) {
#pragma unroll
      for (int i = 0; i < WR; ++i)
        af[fb][i] = *reinterpret_cast<const vec_t *>(abuf + swz(wm * kWaveRows + i * 32 + frow, ks * 2 + fh));
#pragma unroll
      for (int j = 0; j < 2; ++j)
        bf[fb][j] = *reinterpret_cast<const vec_t *>(bbuf + swz(wc * 64 + j * 32 + frow, ks * 2 + fh));
    };
    read_frags(0, 0);
#pragma unroll
    for (int ks = 0; ks < BR / 16; ++ks) {
      const int fsel = ks & 1;
      if (ks + 1 < BR / 16) read_frags((ks + 1) & 1, ks + 1);
#pragma unroll
      for (int i = 0; i < WR; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = Mfma32<CT>::run(af[fsel][i], bf[fsel][j], acc[i][j]);
    }
    __syncthreads();
  };
  {
    int s = 0;
    for (; s + 2 <= steps; s += 2) {
      cstep(I0{}, I0{}, s);
      cstep(I1{}, I1{}, s + 1);
    }
    if (s < steps) cstep(I0{}, I0{}, s);
  }

  // ---- epilogue: acc[i][j][r] = D[row][col], row = 8*(r/4) + 4*(lane/32) + r%4, col = lane%32
  const int64_t d_off = static_cast<int64_t>(split) * g.M * C;      // partial tiles of a shared reduction: one [M, C] slab per part
  // A lane's values sit in 16 different rows, one element each, so a direct store moves 64- or 128-byte pieces
  // with one instruction per element.  After the last barrier nobody reads the operand tiles any more, so each
  // consumer wave lays its (BM/2) x 64 sub-tile out in a private piece of LDS (row pitch = row + 16 bytes:
  // conflict free both ways; fp32 in two halves) and writes it, and reads the optional addend, as 16 bytes
  // per lane and whole 128- or 256-byte row pieces.
  if (g.vec_store) {
    auto staged = [&](auto tag) {
      typedef decltype(tag) T;
      constexpr int kPitch = 64 * sizeof(T) + 16;
      constexpr int kPasses = sizeof(T) == 4 ? 2 : 1;        // fp32: half of the sub-tile's rows at a time
      constexpr int kRowsPerPass = kWaveRows / kPasses;
      constexpr int kPer = 16 / sizeof(T);                   // elements per 16-byte piece
      constexpr int kLanesPerRow = 64 / kPer;
      unsigned char *stage = smem + wave * (kRowsPerPass * kPitch);
#pragma unroll
      for (int pass = 0; pass < kPasses; ++pass) {
        if (pass > 0) asm volatile("" ::: "memory");
#pragma unroll
        for (int ii = 0; ii < WR / kPasses; ++ii) {
          const int i = pass * (WR / kPasses) + ii;
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int lrow = ii * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
              *reinterpret_cast<T *>(stage + lrow * kPitch + (j * 32 + (lane & 31)) * sizeof(T)) = from_f32<T>(acc[i][j][r]);
            }
        }
        // same wave, LDS executes a wave's accesses in order: only the compiler must not move the reads up
        asm volatile("" ::: "memory");
        const int chunk = lane % kLanesPerRow;
        const int64_t gcol = col0 + wc * 64 + chunk * kPer;
#pragma unroll
        for (int it = 0; it < kRowsPerPass * kLanesPerRow / 64; ++it) {
          const int lrow = it * (64 / kLanesPerRow) + lane / kLanesPerRow;
          const int64_t grow = row_lo + wm * kWaveRows + pass * kRowsPerPass + lrow;
          if (grow < row_hi && gcol < C) {
            u32x4_t v = *reinterpret_cast<const u32x4_t *>(stage + lrow * kPitch + chunk * 16);
            const int64_t o = d_off + grow * C + gcol;
            if constexpr (sizeof(T) == 2 && kGrouped) {        // only the grouped launches carry these
              if (g.epilogue != EPI_NONE) {
                const u32x4_t gv = *reinterpret_cast<const u32x4_t *>(static_cast<const T *>(g.e1) + o);
                const T *vp = reinterpret_cast<const T *>(&v);
                const T *gp = reinterpret_cast<const T *>(&gv);
                u32x4_t w1 = v, w2;
                T *p1 = reinterpret_cast<T *>(&w1);
                T *p2 = reinterpret_cast<T *>(&w2);
                if (g.epilogue == EPI_SWIGLU_FWD) {
#pragma unroll
                  for (int e = 0; e < kPer; ++e) p2[e] = swiglu_fwd_one<T>(gp[e], vp[e]);
                } else {
                  const u32x4_t uv = *reinterpret_cast<const u32x4_t *>(static_cast<const T *>(g.e2) + o);
                  const T *up = reinterpret_cast<const T *>(&uv);
#pragma unroll
                  for (int e = 0; e < kPer; ++e) swiglu_bwd_one<T>(gp[e], up[e], vp[e], p1[e], p2[e]);
                }
                *reinterpret_cast<u32x4_t *>(static_cast<T *>(g.d) + o) = w1;
                *reinterpret_cast<u32x4_t *>(static_cast<T *>(g.d2) + o) = w2;
                continue;
              }
            }
            if (g.addend) {
              const u32x4_t av = *reinterpret_cast<const u32x4_t *>(static_cast<const T *>(g.addend) + o);
              const T *vp = reinterpret_cast<const T *>(&v);
              const T *ap = reinterpret_cast<const T *>(&av);
              u32x4_t w;
              T *wp = reinterpret_cast<T *>(&w);
#pragma unroll
              for (int e = 0; e < kPer; ++e) wp[e] = from_f32<T>(to_f32<T>(vp[e]) + to_f32<T>(ap[e]));
              v = w;
            }
            *reinterpret_cast<u32x4_t *>(static_cast<T *>(g.d) + o) = v;
          }
        }
      }
    };
    if (g.d_dtype == CAIFX_BF16) staged(bf16_t{});
    else if (g.d_dtype == CAIFX_F16) staged(f16_t{});
    else staged(float{});
    if constexpr (kGrouped) {
      if (stamp_pos >= 0) g.stamps[4 * stamp_pos + 3] = wall_clock64();      // thread 0 is in consumer wave 0
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < WR; ++i) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t col = col0 + wc * 64 + j * 32 + (lane & 31);
      if (col < C) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t row = row_lo + wm * kWaveRows + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          if (row < row_hi) {
            const int64_t o = d_off + row * C + col;
            float v = acc[i][j][r];
            if (g.addend) {
              // the caller's cast of this result to the tensor dtype followed by an element-wise Add, same roundings
              if (g.d_dtype == CAIFX_F32) v += static_cast<const float *>(g.addend)[o];
              else if (g.d_dtype == CAIFX_BF16) v = round_through<bf16_t>(v) + to_f32(static_cast<const bf16_t *>(g.addend)[o]);
              else v = round_through<f16_t>(v) + to_f32(static_cast<const f16_t *>(g.addend)[o]);
            }
            if (g.d_dtype == CAIFX_F32) static_cast<float *>(g.d)[o] = v;
            else if (g.d_dtype == CAIFX_BF16) static_cast<bf16_t *>(g.d)[o] = from_f32<bf16_t>(v);
            else static_cast<f16_t *>(g.d)[o] = from_f32<f16_t>(v);
          }
        }
      }
    }
  }
  if constexpr (kGrouped) {
    if (stamp_pos >= 0) g.stamps[4 * stamp_pos + 3] = wall_clock64();
  }
}

template <typename CT, typename XT, int kW, bool kSLds, bool kBackward, bool kGrouped, int BM, int kCW = 4>
int launch_one(const TileArgs &t, int64_t row_tiles, hipStream_t s)
{
  constexpr int kThreads = 2 * kCW * 64;
  const int64_t C = kBackward ? t.K : t.N;
  const size_t lds = 2 * (static_cast<size_t>(BM) * BR * 2 + kBTileBytes) + (kSLds ? static_cast<size_t>(t.period) * 4 : 0);
  auto kern = qgemm_kernel<CT, XT, kW, kSLds, kBackward, kGrouped, BM, kCW>;
  if (lds > 64 * 1024) {
    // largest dynamic LDS size this kernel has been enabled for (the attribute is per kernel and sticky;
    // two threads racing here both set it, which is harmless)
    static std::atomic<size_t> raised{0};
    if (lds > raised.load(std::memory_order_relaxed)) {
      if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(lds)) != hipSuccess)
        return CAIFX_ERR_LAUNCH_FAILED;
      size_t seen = raised.load(std::memory_order_relaxed);
      while (seen < lds && !raised.compare_exchange_weak(seen, lds, std::memory_order_relaxed)) {
      }
    }
  }
  const int64_t col_tiles = (C + BC - 1) / BC;
  dim3 grid(static_cast<unsigned>(col_tiles), static_cast<unsigned>(row_tiles));
  {
    const int64_t padded = (row_tiles * col_tiles + 7) / 8 * 8 * (kGrouped ? 1 : t.ksplit);      // linear grid, see the tile numbering in the kernel
    if (padded > 0x7fffffff) return CAIFX_ERR_UNSUPPORTED;
    grid = dim3(static_cast<unsigned>(padded), 1);
  }
  hipLaunchKernelGGL(kern, grid, dim3(kThreads), lds, s, t);
  return launch_status();
}

// int8 scale vectors up to this many entries are kept in LDS: 8 KiB next to the 64 KiB of a
// 128-row workgroup leaves room for two workgroups per compute unit, 56 KiB next to the 96 KiB of
// a 256-row workgroup fills the 160 KiB of one.
constexpr int64_t kSLdsMax128 = 2048;
constexpr int64_t kSLdsMax256 = 14336;

template <typename CT, typename XT, int kW, bool kBackward, bool kGrouped, int BM>
int launch_scales(const TileArgs &t, int64_t row_tiles, hipStream_t s)
{
  if constexpr (kW == W_CODES8) {
    if (t.scale_mode == SM_VEC4 && t.period <= (BM == 128 ? kSLdsMax128 : kSLdsMax256))
      return launch_one<CT, XT, W_CODES8, true, kBackward, kGrouped, BM>(t, row_tiles, s);
  }
  return launch_one<CT, XT, kW, false, kBackward, kGrouped, BM>(t, row_tiles, s);
}

// Tile height.  What a step costs is mostly the staging chain of the producers, and a 256-row
// tile stages the same 64x128 weight piece as a 128-row tile for twice the MFMA work; its consumer
// waves (128x64 each) also need only 0.75 operand-fragment reads per MFMA instead of 1.  So
// 256-row tiles are used whenever there are enough of them to fill the chip.
template <typename CT, typename XT, int kW, bool kBackward>
int launch_tile(const TileArgs &t, bool grouped, hipStream_t s)
{
  const int64_t C = kBackward ? t.K : t.N;
  const int64_t col_tiles = (C + BC - 1) / BC;
  if (grouped) {
    // Segment lengths live on the device; the host only knows their mean, so the grid is an upper
    // bound: every expert can add one partial tile.  128-row tiles throughout: two workgroups share a
    // compute unit and a segment's last tile wastes 64 rows on average instead of 128; with the
    // expert-by-expert tile numbering they measured 10-20 % faster than 256-row tiles for 8, 24 and
    // 64 experts over 24576 rows (int4 and int8, forward and input gradient).
    const int64_t row_tiles = (t.M + 127) / 128 + t.num_experts;
    return launch_scales<CT, XT, kW, kBackward, true, 128>(t, row_tiles, s);
  }
  const int64_t tall = (t.M + 255) / 256;
  // 256-row tiles when there are enough of them and the reduction is long; with 2048 steps of
  // reduction or fewer the tile prologue and store weigh more and two 128-row workgroups per compute
  // unit hide them behind each other (M=24576, N=1408, K=2048: 166 us against 191 us forward)
  const int64_t R = kBackward ? t.N : t.K;
  if (tall * col_tiles >= 200 && tall <= 65535 && R > 2048) return launch_scales<CT, XT, kW, kBackward, false, 256>(t, tall, s);
  const int64_t row_tiles = (t.M + 127) / 128;
  if (row_tiles > 65535) return CAIFX_ERR_UNSUPPORTED;
  return launch_scales<CT, XT, kW, kBackward, false, 128>(t, row_tiles, s);
}

// the W_DENSE16 instantiations (caifx_gemm_dense.hip): t is filled by the caller, compute type bf16 or fp16,
// activations in the compute type or fp32
int dense_launch(const TileArgs &t, int compute_dtype, int x_dtype, bool backward, bool grouped, hipStream_t s);

}  // namespace gemm_tile
}  // namespace caifx
