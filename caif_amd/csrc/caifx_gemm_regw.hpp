// Pieces shared by the forward kernels that keep the weight out of the shared operand tiles
// (caifx_gemm_regw.hip: packed int4; caifx_gemm_regw8.hip: int8): the LDS swizzle of 128-byte rows and the
// staged store of a workgroup's 128 x 256 tile.
#pragma once

#include "caifx_internal.hpp"

namespace caifx {
namespace regw {

constexpr int kBK = 64;        // reduction extent of a step
constexpr int kBN = 256;       // columns of Y per workgroup: 8 waves x 32
constexpr int kStages = 4;     // LDS ring of activation tiles

// byte offset of 16-byte chunk `chunk` (0..7) of row `row` in an LDS tile of 128-byte rows
__device__ __forceinline__ int swz(int row, int chunk) { return row * 128 + ((chunk ^ ((row ^ (row >> 3)) & 7)) << 4); }

// LDS bytes the staged store of a BM-row tile needs (fp32 results, the widest)
constexpr size_t store_bytes(int BM)
{
  const size_t pitch = kBN * 4 + 32;
  return (static_cast<size_t>(BM) * pitch <= 150 * 1024 ? BM : BM / 2) * pitch;
}

// Store of a workgroup's tile: acc[i][r] = Y[row0 + 32 i + 8 (r / 4) + 4 (lane / 32) + r % 4][col0 + 32 wave + lane % 32].
// The whole tile is laid out in LDS (row pitch = row + 32 bytes, so the two lane halves, four rows apart, use
// different halves of the banks), then every wave writes whole tile rows: 16 bytes per lane, 1 KiB (fp32) or two
// rows of 512 bytes (16-bit results) per instruction, and reads the optional addend the same way.  Tiles taller
// than the LDS holds go in passes.  Rows from row_end on and columns from N on are not written.  Every thread of
// the workgroup calls it; nobody may still be reading the LDS it overwrites.
// With gate and d2 (16-bit T, N % 8 == 0, no addend: the caller checks) the launch is the up projection of a gated
// expert: d = v and d2 = T(T(silu(gate)) * v), the bits of the separate SiLU-multiply pass.
template <typename T, int WR>
__device__ __forceinline__ void store_tile(unsigned char *smem, const floatx16_t (&acc)[WR], int wave, int lane, int64_t row0,
                                           int64_t row_end, int64_t col0, int64_t N, T *dp, const T *ap,
                                           const T *gate = nullptr, T *d2 = nullptr)
{
  constexpr int BM = 32 * WR;
  constexpr int kPitch = kBN * sizeof(T) + 32;
  constexpr int kPer16 = 16 / sizeof(T);                 // elements per 16-byte piece
  constexpr int kLanesPerRow = kBN / kPer16;             // 64 (fp32) or 32
  constexpr int kRowsPerInstr = 64 / kLanesPerRow;       // 1 or 2
  constexpr int kPassRows = (BM * kPitch <= 150 * 1024) ? BM : BM / 2;
  constexpr int kPassBlocks = kPassRows / 32;
  const int frow = lane & 31;
  const int fh = lane >> 5;
  const int chunk = lane % kLanesPerRow;
  const int64_t gcol = col0 + chunk * kPer16;
  const bool vec_ok = (N % kPer16 == 0);
#pragma unroll
  for (int pass = 0; pass < BM / kPassRows; ++pass) {
    if (pass > 0) __syncthreads();
#pragma unroll
    for (int ii = 0; ii < kPassBlocks; ++ii) {
      const int i = pass * kPassBlocks + ii;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int lrow = ii * 32 + 8 * (r >> 2) + 4 * fh + (r & 3);
        *reinterpret_cast<T *>(smem + lrow * kPitch + (wave * 32 + frow) * sizeof(T)) = from_f32<T>(acc[i][r]);
      }
    }
    __syncthreads();
    constexpr int kInstr = kPassRows / (8 * kRowsPerInstr);      // row pieces per wave
#pragma unroll
    for (int it = 0; it < kInstr; ++it) {
      const int lrow = (it * 8 + wave) * kRowsPerInstr + lane / kLanesPerRow;
      const int64_t grow = row0 + pass * kPassRows + lrow;
      if (grow >= row_end || gcol >= N) continue;
      u32x4_t v = *reinterpret_cast<const u32x4_t *>(smem + lrow * kPitch + chunk * 16);
      const int64_t o = grow * N + gcol;
      if (vec_ok) {
        if constexpr (sizeof(T) == 2) {
          if (gate) {
            const u32x4_t gv = *reinterpret_cast<const u32x4_t *>(gate + o);
            const T *vp = reinterpret_cast<const T *>(&v);
            const T *gp = reinterpret_cast<const T *>(&gv);
            u32x4_t w2;
            T *p2 = reinterpret_cast<T *>(&w2);
#pragma unroll
            for (int e = 0; e < kPer16; ++e) p2[e] = swiglu_fwd_one<T>(gp[e], vp[e]);
            *reinterpret_cast<u32x4_t *>(dp + o) = v;
            *reinterpret_cast<u32x4_t *>(d2 + o) = w2;
            continue;
          }
        }
        if (ap) {
          const u32x4_t av = *reinterpret_cast<const u32x4_t *>(ap + o);
          const T *vp = reinterpret_cast<const T *>(&v);
          const T *aq = reinterpret_cast<const T *>(&av);
          u32x4_t w;
          T *wp = reinterpret_cast<T *>(&w);
#pragma unroll
          for (int e = 0; e < kPer16; ++e) wp[e] = from_f32<T>(to_f32<T>(vp[e]) + to_f32<T>(aq[e]));
          v = w;
        }
        *reinterpret_cast<u32x4_t *>(dp + o) = v;
      } else {
        const T *vp = reinterpret_cast<const T *>(&v);
#pragma unroll
        for (int e = 0; e < kPer16; ++e) {
          if (gcol + e < N) {
            T val = vp[e];
            if (ap) val = from_f32<T>(to_f32<T>(val) + to_f32<T>(ap[o + e]));
            dp[o + e] = val;
          }
        }
      }
    }
  }
}

}  // namespace regw

// int8 counterpart of mfma_regw_forward, plain and grouped: scale vectors (or one scale, or none) whose table fits
// 16 KiB of LDS, K a multiple of 128.  CAIFX_ERR_UNSUPPORTED for everything else.
int mfma_regw8_forward(const GemmArgs &a, hipStream_t s);
// where grouped launches record their tiles (see mfma_grouped_tile_stamps); null when switched off
void mfma_grouped_stamp_target(unsigned long long **buf, long long *capacity);

}  // namespace caifx
