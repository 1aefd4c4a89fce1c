// Large-M dequant-GEMM on the matrix cores: forward Y = X * W^T, input gradient dX = dY * W,
// and the same two over token-sorted expert segments (one launch for all experts).
//
// One kernel template covers all four.  Seen from the matrix core every case is
//     D[M, C] = A[M, R] * B[R, C]          A = activations (X or dY), row-major, R contiguous
// with B drawn from the stored weight W[N,K]:
//     forward : C = N, R = K, B[r][c] = W[c][r]   (a weight row is contiguous along R)
//     backward: C = K, R = N, B[r][c] = W[r][c]   (a weight row is contiguous along C)
// A workgroup (256 threads, 2x2 waves) owns a 128 x 128 tile of D and walks R in steps of 64.
// Per step it moves a 128x64 tile of A and the matching 64x128 piece of W from global memory
// into registers while the matrix cores work on the previous step, then dequantises W in
// registers (code * scale in fp32, one rounding to the compute dtype: bit-identical to the
// reference's dequantise-then-cast weight) and writes both tiles to the other half of a
// double-buffered LDS area, as [row][64 values along R] with the 16-byte chunks of a row
// XOR-swizzled by (row & 7) so that the 128-bit operand reads of v_mfma_f32_32x32x16 spread
// over all banks.  For the backward case the weight piece is transposed on the way: a thread
// holds 4 weight rows x 8 columns and writes 8 runs of 4 values along R.
// Each wave accumulates a 64 x 64 sub-tile (2x2 MFMA tiles, 64 fp32 accumulators per lane).
// No dense copy of W ever reaches HBM; the only HBM traffic is A, the packed W and D.
#include "caifx_internal.hpp"

namespace caifx {
namespace {

constexpr int BM = 128;      // rows of D per workgroup
constexpr int BC = 128;      // columns of D per workgroup
constexpr int BR = 64;       // reduction extent per step
constexpr int kThreads = 256;
constexpr int kTileBytes = 128 * BR * 2;   // one operand tile in LDS (16 KiB)

template <typename CT> struct Mfma32;
template <> struct Mfma32<bf16_t> {
  typedef bf16x8_t vec_t;
  static __device__ __forceinline__ floatx16_t run(vec_t a, vec_t b, floatx16_t c)
  {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma32<f16_t> {
  typedef f16x8_t vec_t;
  static __device__ __forceinline__ floatx16_t run(vec_t a, vec_t b, floatx16_t c)
  {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

enum { SM_SCALAR = 0, SM_VEC4 = 1, SM_ANY = 2 };   // how int8 scales are fetched

struct TileArgs {
  int64_t M, N, K;           // N = OutputDim, K = InputDim of the weight
  const void *a;             // activations [M, R]
  void *d;                   // result [M, C]
  int d_dtype;
  const void *wq;
  const void *scales;
  int group_shift;           // int4: log2(group_size)
  int scale_mode;            // int8
  int64_t period;            // int8
  // grouped form
  const int32_t *offsets;
  const void *const *wq_ptrs;
  const void *const *scales_ptrs;
  int num_experts;
};

// byte offset of 16-byte chunk `chunk` (0..7) of LDS tile row `row`
__device__ __forceinline__ int swz(int row, int chunk) { return row * 128 + ((chunk ^ (row & 7)) << 4); }

template <typename CT> __device__ __forceinline__ uint32_t pack2(float lo, float hi)
{
  typedef __attribute__((__vector_size__(2 * sizeof(CT)))) CT pair_t;
  pair_t p;
  p[0] = from_f32<CT>(lo);
  p[1] = from_f32<CT>(hi);
  return __builtin_bit_cast(uint32_t, p);
}

__device__ __forceinline__ float int8_scale_at(const float *scales, int mode, int64_t period, int64_t flat)
{
  if (mode == SM_SCALAR) return scales ? scales[0] : 1.0f;
  return scales[flat % period];
}

template <typename CT, typename XT, bool kInt4, bool kBackward, bool kGrouped>
__global__ __launch_bounds__(kThreads) void qgemm_kernel(TileArgs g)
{
  typedef typename Mfma32<CT>::vec_t vec_t;
  __shared__ __attribute__((aligned(16))) unsigned char smem[4 * kTileBytes];   // A0 B0 A1 B1
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1;      // wave row (0..1): 64 rows of D
  const int wc = wave & 1;       // wave column (0..1): 64 columns of D

  const int64_t R = kBackward ? g.N : g.K;     // reduction length
  const int64_t C = kBackward ? g.K : g.N;     // columns of D

  // ---- which tile -----------------------------------------------------------------------
  int64_t row_lo, row_hi;        // rows of A / D this workgroup may touch: [row_lo, row_hi)
  const uint8_t *wq = static_cast<const uint8_t *>(g.wq);
  const void *scales = g.scales;
  if constexpr (kGrouped) {
    // blockIdx.y counts row tiles over all experts; find the expert by walking the offsets
    int t = blockIdx.y;
    int e = 0;
    int64_t lo = 0, hi = 0;
    bool found = false;
    for (; e < g.num_experts; ++e) {
      lo = g.offsets[e];
      hi = g.offsets[e + 1];
      const int tiles = static_cast<int>((hi - lo + BM - 1) / BM);
      if (t < tiles) {
        found = true;
        break;
      }
      t -= tiles;
    }
    if (!found) return;
    row_lo = lo + static_cast<int64_t>(t) * BM;
    row_hi = hi;
    wq = static_cast<const uint8_t *>(g.wq_ptrs[e]);
    scales = g.scales_ptrs ? g.scales_ptrs[e] : nullptr;
  } else {
    row_lo = static_cast<int64_t>(blockIdx.y) * BM;
    row_hi = g.M;
  }
  const int64_t col0 = static_cast<int64_t>(blockIdx.x) * BC;
  const XT *ag = static_cast<const XT *>(g.a);

  // ---- global -> register staging ---------------------------------------------------------
  // A tile: 128 rows x 8 chunks (8 values each); thread handles chunks q = tid + 256*i, i < 4
  constexpr int kAVecs = (sizeof(XT) == 4) ? 8 : 4;     // 16-byte loads per thread per step
  u32x4_t areg[kAVecs];
  int a_row[4], a_chunk[4];
  const XT *a_ptr[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int q = tid + kThreads * i;
    a_row[i] = q >> 3;
    a_chunk[i] = q & 7;
    int64_t m = row_lo + a_row[i];
    if (m >= row_hi) m = row_hi - 1;                    // clamp: rows past the end are never stored
    a_ptr[i] = ag + m * R + a_chunk[i] * 8;
  }
  auto load_a = [&](int64_t r0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (sizeof(XT) == 4) {
        areg[2 * i] = *reinterpret_cast<const u32x4_t *>(a_ptr[i] + r0);
        areg[2 * i + 1] = *reinterpret_cast<const u32x4_t *>(a_ptr[i] + r0 + 4);
      } else {
        areg[i] = *reinterpret_cast<const u32x4_t *>(a_ptr[i] + r0);
      }
    }
  };
  auto store_a = [&](unsigned char *dst) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      u32x4_t v;
      if constexpr (sizeof(XT) == 4) {
        const float *f0 = reinterpret_cast<const float *>(&areg[2 * i]);
        const float *f1 = reinterpret_cast<const float *>(&areg[2 * i + 1]);
        v[0] = pack2<CT>(f0[0], f0[1]);
        v[1] = pack2<CT>(f0[2], f0[3]);
        v[2] = pack2<CT>(f1[0], f1[1]);
        v[3] = pack2<CT>(f1[2], f1[3]);
      } else {
        v = areg[i];
      }
      *reinterpret_cast<u32x4_t *>(dst + swz(a_row[i], a_chunk[i])) = v;
    }
  };

  // W piece.  Registers hold raw codes (+ int4 scales); dequantisation happens at store time.
  //   forward  int4: row c = tid/2, 32 codes (16 B) at r = (tid%2)*32           -> 4 chunks
  //   forward  int8: rows c = tid/4 (+64), 16 codes (16 B) at r = (tid%4)*16    -> 2 x 2 chunks
  //   backward int4: rows r = (tid/16)*4 .. +3, 8 codes (4 B) at c = (tid%16)*8 -> 8 runs of 4
  //   backward int8: same rows, 8 codes (8 B)
  u32x4_t wreg[2];
  f16_t wscale[4];
  int64_t w_flat[4];       // flat index n*K + k of each register row's first code at step 0
  const f16_t *s16 = static_cast<const f16_t *>(scales);
  const float *s32 = static_cast<const float *>(scales);
  int wf_c = 0, wf_r = 0;  // forward: tile-local column / first r;  backward: first r row / first c
  if constexpr (!kBackward) {
    if constexpr (kInt4) {
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
  auto load_w = [&](int64_t r0) {
    if constexpr (!kBackward) {
      if constexpr (kInt4) {
        const int64_t f = w_flat[0] + r0;
        wreg[0] = *reinterpret_cast<const u32x4_t *>(wq + (f >> 1));
        wscale[0] = s16[f >> g.group_shift];
      } else {
#pragma unroll
        for (int i = 0; i < 2; ++i) wreg[i] = *reinterpret_cast<const u32x4_t *>(wq + w_flat[i] + r0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t f = w_flat[i] + r0 * g.K;
        if constexpr (kInt4) {
          reinterpret_cast<uint32_t *>(wreg)[i] = *reinterpret_cast<const uint32_t *>(wq + (f >> 1));
          wscale[i] = s16[f >> g.group_shift];
        } else {
          const u32x2_t v = *reinterpret_cast<const u32x2_t *>(wq + f);
          reinterpret_cast<uint32_t *>(wreg)[2 * i] = v[0];
          reinterpret_cast<uint32_t *>(wreg)[2 * i + 1] = v[1];
        }
      }
    }
  };
  // int8: fp32 value of 4 codes of dword p whose first code has flat index f
  auto deq8 = [&](uint32_t p, int64_t f, float (&out)[4]) {
    float q[4];
    int8x4_to_f32(p, q);
    if (g.scale_mode == SM_VEC4) {
      const floatx4_t s = *reinterpret_cast<const floatx4_t *>(s32 + (f % g.period));
#pragma unroll
      for (int j = 0; j < 4; ++j) out[j] = q[j] * s[j];
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) out[j] = q[j] * int8_scale_at(s32, g.scale_mode, g.period, f + j);
    }
  };
  auto store_w = [&](unsigned char *dst, int64_t r0) {
    if constexpr (!kBackward) {
      if constexpr (kInt4) {
        const float s = to_f32(wscale[0]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float e[8];
          dequant_int4x8(wreg[0][j], s, e);
          u32x4_t v;
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = pack2<CT>(e[2 * q], e[2 * q + 1]);
          *reinterpret_cast<u32x4_t *>(dst + swz(wf_c, (wf_r >> 3) + j)) = v;
        }
      } else {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            float lo[4], hi[4];
            deq8(wreg[i][2 * j], w_flat[i] + r0 + 8 * j, lo);
            deq8(wreg[i][2 * j + 1], w_flat[i] + r0 + 8 * j + 4, hi);
            u32x4_t v;
            v[0] = pack2<CT>(lo[0], lo[1]);
            v[1] = pack2<CT>(lo[2], lo[3]);
            v[2] = pack2<CT>(hi[0], hi[1]);
            v[3] = pack2<CT>(hi[2], hi[3]);
            *reinterpret_cast<u32x4_t *>(dst + swz(wf_c + 64 * i, (wf_r >> 3) + j)) = v;
          }
        }
      }
    } else {
      // e[i][j]: weight row (reduction index) wf_r + i, column wf_c + j
      float e[4][8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (kInt4) {
          dequant_int4x8(reinterpret_cast<const uint32_t *>(wreg)[i], to_f32(wscale[i]), e[i]);
        } else {
          const int64_t f = w_flat[i] + r0 * g.K;
          float lo[4], hi[4];
          deq8(reinterpret_cast<const uint32_t *>(wreg)[2 * i], f, lo);
          deq8(reinterpret_cast<const uint32_t *>(wreg)[2 * i + 1], f + 4, hi);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            e[i][j] = lo[j];
            e[i][4 + j] = hi[j];
          }
        }
      }
      // transposed write: LDS row = column c, run of 4 values along R at r = wf_r .. wf_r+3
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        u32x2_t v;
        v[0] = pack2<CT>(e[0][j], e[1][j]);
        v[1] = pack2<CT>(e[2][j], e[3][j]);
        const int row = wf_c + j;
        *reinterpret_cast<u32x2_t *>(dst + swz(row, wf_r >> 3) + ((wf_r & 4) << 1)) = v;
      }
    }
  };

  // ---- main loop ------------------------------------------------------------------------
  floatx16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int steps = static_cast<int>(R / BR);
  load_a(0);
  load_w(0);
  store_a(smem);
  store_w(smem + kTileBytes, 0);
  __syncthreads();

  const int frow = lane & 31;    // row of the operand tile this lane supplies
  const int fh = lane >> 5;      // which half of the 16-wide k step
  for (int s = 0; s < steps; ++s) {
    const unsigned char *abuf = smem + (s & 1) * 2 * kTileBytes;
    const unsigned char *bbuf = abuf + kTileBytes;
    const bool more = (s + 1 < steps);
    if (more) {
      load_a(static_cast<int64_t>(s + 1) * BR);
      load_w(static_cast<int64_t>(s + 1) * BR);
    }
#pragma unroll
    for (int ks = 0; ks < BR / 16; ++ks) {
      vec_t af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        af[i] = *reinterpret_cast<const vec_t *>(abuf + swz(wm * 64 + i * 32 + frow, ks * 2 + fh));
        bf[i] = *reinterpret_cast<const vec_t *>(bbuf + swz(wc * 64 + i * 32 + frow, ks * 2 + fh));
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = Mfma32<CT>::run(af[i], bf[j], acc[i][j]);
    }
    if (more) {
      unsigned char *nbuf = smem + ((s + 1) & 1) * 2 * kTileBytes;
      store_a(nbuf);
      store_w(nbuf + kTileBytes, static_cast<int64_t>(s + 1) * BR);
    }
    __syncthreads();
  }

  // ---- epilogue: acc[i][j][r] = D[row][col], row = 8*(r/4) + 4*(lane/32) + r%4, col = lane%32
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t col = col0 + wc * 64 + j * 32 + (lane & 31);
      if (col < C) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t row = row_lo + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          if (row < row_hi) {
            const int64_t o = row * C + col;
            const float v = acc[i][j][r];
            if (g.d_dtype == CAIFX_F32) static_cast<float *>(g.d)[o] = v;
            else if (g.d_dtype == CAIFX_BF16) static_cast<bf16_t *>(g.d)[o] = from_f32<bf16_t>(v);
            else static_cast<f16_t *>(g.d)[o] = from_f32<f16_t>(v);
          }
        }
      }
    }
  }
}

template <typename CT, typename XT, bool kInt4, bool kBackward>
int launch_tile(const TileArgs &t, bool grouped, int64_t max_row_tiles, hipStream_t s)
{
  const int64_t C = kBackward ? t.K : t.N;
  dim3 grid(static_cast<unsigned>((C + BC - 1) / BC), static_cast<unsigned>(max_row_tiles));
  if (grouped) hipLaunchKernelGGL((qgemm_kernel<CT, XT, kInt4, kBackward, true>), grid, dim3(kThreads), 0, s, t);
  else hipLaunchKernelGGL((qgemm_kernel<CT, XT, kInt4, kBackward, false>), grid, dim3(kThreads), 0, s, t);
  return launch_status();
}

template <typename CT, typename XT>
int pick_kind(const TileArgs &t, bool int4, bool backward, bool grouped, int64_t tiles, hipStream_t s)
{
  if (int4) return backward ? launch_tile<CT, XT, true, true>(t, grouped, tiles, s) : launch_tile<CT, XT, true, false>(t, grouped, tiles, s);
  return backward ? launch_tile<CT, XT, false, true>(t, grouped, tiles, s) : launch_tile<CT, XT, false, false>(t, grouped, tiles, s);
}

int run(const GemmArgs &a, bool backward, hipStream_t s)
{
  if (a.compute_dtype == CAIFX_F32) return CAIFX_ERR_UNSUPPORTED;
  if (a.x_dtype != a.compute_dtype && a.x_dtype != CAIFX_F32) return CAIFX_ERR_UNSUPPORTED;
  const bool grouped = a.offsets != nullptr;
  const bool int4 = a.w.kind == CAIFX_W_INT4_GROUP;
  const int64_t R = backward ? a.N : a.K;
  if (R % BR != 0 || a.K % 32 != 0 || a.K < 64 || a.N < 1) return CAIFX_ERR_UNSUPPORTED;
  if (a.M > (int64_t{1} << 30) || a.N > (int64_t{1} << 30) || a.K > (int64_t{1} << 30)) return CAIFX_ERR_UNSUPPORTED;
  if (!aligned_to(a.x, 16)) return CAIFX_ERR_UNSUPPORTED;

  TileArgs t{};
  t.M = a.M;
  t.N = a.N;
  t.K = a.K;
  t.a = a.x;
  t.d = a.y;
  t.d_dtype = a.y_dtype;
  t.wq = a.w.q;
  t.scales = a.w.scales;
  t.offsets = a.offsets;
  t.wq_ptrs = a.wq_ptrs;
  t.scales_ptrs = a.scales_ptrs;
  t.num_experts = a.num_experts;
  if (int4) {
    const int gs = a.w.group_size;
    if (gs < 32 || (gs & (gs - 1)) != 0) return CAIFX_ERR_UNSUPPORTED;
    t.group_shift = __builtin_ctz(static_cast<unsigned>(gs));
    if (!grouped && !aligned_to(a.w.q, 16)) return CAIFX_ERR_UNSUPPORTED;
  } else {
    if (!grouped && !aligned_to(a.w.q, 16)) return CAIFX_ERR_UNSUPPORTED;
    const bool has_scales = grouped ? a.scales_ptrs != nullptr : a.w.scales != nullptr;
    t.period = a.w.scale_period;
    if (!has_scales || t.period == 1) {
      t.scale_mode = SM_SCALAR;
    } else if (t.period % 4 == 0 && (grouped || aligned_to(a.w.scales, 16))) {
      t.scale_mode = SM_VEC4;     // flat index of every fetched quad is a multiple of 4 (K % 32 == 0)
    } else {
      t.scale_mode = SM_ANY;
    }
  }
  // grouped: every expert can add one partial row tile on top of the dense count
  const int64_t row_tiles = grouped ? (a.M + BM - 1) / BM + a.num_experts : (a.M + BM - 1) / BM;
  if (row_tiles > 65535) return CAIFX_ERR_UNSUPPORTED;
  if (a.compute_dtype == CAIFX_BF16) {
    if (a.x_dtype == CAIFX_F32) return pick_kind<bf16_t, float>(t, int4, backward, grouped, row_tiles, s);
    return pick_kind<bf16_t, bf16_t>(t, int4, backward, grouped, row_tiles, s);
  }
  if (a.x_dtype == CAIFX_F32) return pick_kind<f16_t, float>(t, int4, backward, grouped, row_tiles, s);
  return pick_kind<f16_t, f16_t>(t, int4, backward, grouped, row_tiles, s);
}

}  // namespace

int mfma_forward(const GemmArgs &a, hipStream_t s) { return run(a, false, s); }
int mfma_backward(const GemmArgs &a, hipStream_t s) { return run(a, true, s); }
size_t mfma_workspace_bytes(const GemmArgs &, bool) { return 0; }

}  // namespace caifx
