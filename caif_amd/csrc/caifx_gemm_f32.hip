// Dequant-GEMM for the fp32 compute type on the matrix cores: Y[M,N] = X[M,K] * W[N,K]^T and
// dX[M,K] = dY[M,N] * W[N,K] with W stored int8 or packed int4 and dequantised to fp32 exactly as the
// reference's dequantise kernels do (fp32 code * scale, no further rounding; ConvertToComputeDtype with
// ComputeT = float, src/caif_device_frozen_linear.cpp:289-378), activations widened to fp32, fp32
// accumulation (the reference's Accuracy_e matmul mode).
//
// v_mfma_f32_32x32x2_f32 runs at 1/16 of the bf16 rate, so this kernel is bound by the matrix pipes long
// before anything else and is kept simple: 256 threads, one BM x 128 tile of the result per workgroup, 32
// deep reduction steps, one LDS buffer per operand (the global loads of the next two steps are in flight in two
// register sets while the matrix cores work on the current one; two barriers per step cost little against the
// 1000-4000 MFMA cycles between them).  Plain and grouped (per-expert row segments) problems.  Both operands sit in LDS reduction-major ([r][row] with the row index contiguous),
// which is what the MFMA operands read: lane (i, h) of a 32x32x2 step takes element [2p + h][i].
// Up to 32 activation rows a workgroup takes a 32 x 32 tile with 128-deep steps and its four waves split each
// step's reduction (partial tiles are added through LDS in a fixed order at the end): four times as many
// workgroups for the same result and a quarter of the barriers.
#include <type_traits>

#include "caifx_internal.hpp"

namespace caifx {
namespace {

constexpr int kStep = 32;    // the reduction advances in multiples of this (host-side checks, scale-index steps)
constexpr int kSplitTileRows = 128;   // up to this many rows the 32 x 32 split tile is used (M = 64: 256 workgroups instead of 64)

struct F32Args {
  int64_t M, N, K;
  const void *a;         // activations [M, R]
  void *d;               // result [M, C]
  int d_dtype;
  const uint8_t *wq;
  const void *scales;
  int group_shift;       // int4: log2(group_size), group_size >= 16
  int64_t period;        // int8: 0 = no scales, 1 = one scale, otherwise the length of the scale vector (>= 32, % 4 == 0)
  uint32_t step;         // int8 scale vector: how far the scale index moves per 32 reduction elements, modulo period
  // grouped form: rows [offsets[e], offsets[e+1]) of a and d belong to expert e and its own weight
  const int32_t *offsets;
  const void *const *wq_ptrs;
  const void *const *scales_ptrs;
  int num_experts;
  // split tile only: `parts` workgroups share a tile's reduction, part_steps 128-deep steps each (blockIdx.z is the
  // part), and write fp32 partial tiles to d + part * M * C (d is then the caller's workspace)
  int parts;
  int part_steps;
  int round_dt;          // float storage with a 16-bit compute type: operands are rounded to it (CAIFX_F32: not)
};

__device__ __forceinline__ void store_result(void *p, int dt, int64_t i, float v)
{
  if (dt == CAIFX_BF16) static_cast<bf16_t *>(p)[i] = from_f32<bf16_t>(v);
  else if (dt == CAIFX_F16) static_cast<f16_t *>(p)[i] = from_f32<f16_t>(v);
  else static_cast<float *>(p)[i] = v;
}

// Tile shapes (BM x kBN result, kBK deep steps; kBN * kBK = 4096 so that every thread dequantises 16 codes per step):
//   128 x 128 x 32: waves 2 x 2 over the tile, 64 x 64 each
//    32 x 128 x 32: waves 1 x 4, 32 x 32 each
//    32 x  32 x 128: every wave works on the whole tile and takes a quarter of each step's reduction
// kVec: int8 with a scale vector (length a multiple of 4, 16-byte aligned: four scales per load)
// WT: void for quantised storage; float, f16_t or bf16_t for a weight stored undequantised (the float-storage cells of
// the layer grid, src/caif_device_frozen_linear.cpp:301-318 and the .To(target) branch after them): its elements are
// widened to fp32 and, like the activations, rounded to g.round_dt when that is a 16-bit type, so that the fp32
// products and sums are those of a GEMM in that type with fp32 accumulation.
template <typename XT, bool kInt4, bool kVec, bool kBackward, int BM, int kBN, int kBK, typename WT = void>
__global__ __launch_bounds__(256) void qgemm_f32_kernel(F32Args g)
{
  static_assert(kBN * kBK == 4096, "16 codes per thread and step");
  constexpr bool kFloatW = !std::is_void<WT>::value;
  constexpr int kWBytes = kFloatW ? static_cast<int>(sizeof(std::conditional_t<kFloatW, WT, char>)) : 1;
  constexpr bool kSplit = kBN == 32;       // the waves split the reduction instead of the tile
  constexpr int WM = BM == 128 ? 2 : 1;
  constexpr int WN = kSplit ? 1 : 4 / WM;
  constexpr int kWaveRows = BM / WM;
  constexpr int kWaveCols = kBN / WN;
  constexpr int TM = kWaveRows / 32;
  constexpr int TN = kWaveCols / 32;
  // row pitches in floats, chosen so that the transposing writes spread over the banks; the input gradient
  // writes its weight rows 16 bytes at a time and needs the pitch to keep that alignment
  constexpr int SA = BM == 32 ? BM + 1 : BM + 4;
  constexpr int SB = (kBN == 32 && !kBackward) ? kBN + 1 : kBN + 4;
  constexpr int EA = BM * kBK / 256;       // activation elements per thread per step (16 or 4)
  constexpr int TPR = kBK / EA;            // threads per activation row
  constexpr int kPairs = kSplit ? kBK / 8 : kBK / 2;     // 32x32x2 steps per wave and step
  static_assert(!kSplit || kBK * SA >= 4 * 16 * 64, "the partial tiles of the four waves fit the activation buffer");
  __shared__ __attribute__((aligned(16))) float As[kBK * SA];
  __shared__ __attribute__((aligned(16))) float Bs[kBK * SB];

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = t >> 6;
  const int wm = kSplit ? 0 : wave / WN;
  const int wn = kSplit ? 0 : wave % WN;
  const int64_t R = kBackward ? g.N : g.K;
  const int64_t C = kBackward ? g.K : g.N;
  int64_t row0 = static_cast<int64_t>(blockIdx.y) * BM;
  const int part = kSplit ? static_cast<int>(blockIdx.z) : 0;
  int64_t row_hi = g.M;                                          // rows this workgroup may touch end here
  const int64_t col0 = static_cast<int64_t>(blockIdx.x) * kBN;
  int steps = static_cast<int>(R / kBK);
  const uint8_t *wq = g.wq;
  const void *scales = g.scales;
  if (g.offsets) {
    // blockIdx.y counts row tiles over all experts (the grid is an upper bound: every expert can add one
    // partial tile); each thread walks the offsets, which a handful of cache lines hold
    int tile = blockIdx.y;
    int e = 0, lo = 0, hi = 0;
    for (; e < g.num_experts; ++e) {
      segment_rows(g.offsets, e, g.M, lo, hi);
      const int tiles = (hi - lo + BM - 1) / BM;
      if (tile < tiles) break;
      tile -= tiles;
    }
    if (e == g.num_experts) return;                              // the whole workgroup, before any barrier
    row0 = lo + static_cast<int64_t>(tile) * BM;
    row_hi = hi;
    wq = static_cast<const uint8_t *>(g.wq_ptrs[e]);
    scales = g.scales_ptrs ? g.scales_ptrs[e] : nullptr;
  }

  // ---- activations: thread (a_row, a_col) holds EA consecutive reduction elements of one row
  const int a_row = t / TPR;
  const int a_col = (t % TPR) * EA;
  int64_t am = row0 + a_row;
  if (am >= row_hi) am = row_hi - 1;                             // rows past the end are never stored
  const XT *ap = static_cast<const XT *>(g.a) + am * R + a_col;
  int64_t r_begin = 0;                                           // first reduction element of this workgroup's part
  if constexpr (kSplit) {
    if (g.parts > 1) {
      const int first = part * g.part_steps;
      r_begin = static_cast<int64_t>(first) * kBK;
      steps = steps - first < g.part_steps ? steps - first : g.part_steps;
      ap += r_begin;
    }
  }
  // two register sets: the loads of steps s+1 and s+2 are in flight while the matrix cores work on step s
  float areg[2][EA];
  auto load_a = [&](auto set_, int64_t r0) {
    constexpr int set = decltype(set_)::value;
    if constexpr (sizeof(XT) == 4) {
#pragma unroll
      for (int i = 0; i < EA / 4; ++i) {
        const floatx4_t v = *reinterpret_cast<const floatx4_t *>(ap + r0 + 4 * i);
#pragma unroll
        for (int e = 0; e < 4; ++e) areg[set][4 * i + e] = v[e];
      }
    } else if constexpr (EA == 16) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const u32x4_t v = *reinterpret_cast<const u32x4_t *>(ap + r0 + 8 * i);
        const XT *h = reinterpret_cast<const XT *>(&v);
#pragma unroll
        for (int e = 0; e < 8; ++e) areg[set][8 * i + e] = to_f32<XT>(h[e]);
      }
    } else {
      const u32x2_t v = *reinterpret_cast<const u32x2_t *>(ap + r0);
      const XT *h = reinterpret_cast<const XT *>(&v);
#pragma unroll
      for (int e = 0; e < 4; ++e) areg[set][e] = to_f32<XT>(h[e]);
    }
  };
  auto rounded = [&](float v) {
    if constexpr (kFloatW) {
      if (g.round_dt == CAIFX_BF16) return round_through<bf16_t>(v);
      if (g.round_dt == CAIFX_F16) return round_through<f16_t>(v);
    }
    return v;
  };
  auto store_a = [&](auto set_) {
    constexpr int set = decltype(set_)::value;
#pragma unroll
    for (int e = 0; e < EA; ++e) As[(a_col + e) * SA + a_row] = rounded(areg[set][e]);
  };

  // ---- weights: 16 consecutive codes (along k) per thread and step
  //   forward : weight row n = col0 + t/(kBK/16), k = r0 + (t%(kBK/16))*16 .. +16    -> Bs[k][n]   (transposing write)
  //   backward: weight row n = r0 + t/(kBN/16),   k = col0 + (t%(kBN/16))*16 .. +16  -> Bs[n][k]   (row write)
  constexpr int kPerRow = (kBackward ? kBN : kBK) / 16;          // threads per weight row of the piece
  const int b_major = t / kPerRow;
  const int b_minor = (t % kPerRow) * 16;
  int64_t flat0;                                                 // flat index n*K + k of the first code at step 0
  if constexpr (!kBackward) {
    int64_t n = col0 + b_major;
    if (n >= g.N) n = g.N - 1;                                   // columns past the end are never stored
    flat0 = n * g.K + b_minor;
  } else {
    int64_t k = col0 + b_minor;
    if (k + 16 > g.K) k = g.K - 16;                              // lands in LDS columns that are never stored
    flat0 = static_cast<int64_t>(b_major) * g.K + k;
  }
  flat0 += kBackward ? r_begin * g.K : r_begin;
  const int64_t flat_step = kBackward ? static_cast<int64_t>(kBK) * g.K : kBK;
  const float *s32 = static_cast<const float *>(scales);
  const f16_t *s16 = static_cast<const f16_t *>(scales);
  constexpr bool vec_scales = !kInt4 && kVec;
  const uint32_t period = static_cast<uint32_t>(g.period);
  uint32_t sidx = vec_scales ? static_cast<uint32_t>(flat0 % g.period) : 0u;
  const float s_one = (!kInt4 && g.period == 1) ? s32[0] : 1.0f;

  uint32_t wreg[2][kFloatW ? 4 * kWBytes : (kInt4 ? 2 : 4)];
  float sc[2][kInt4 ? 1 : 16];
  auto load_b = [&](auto set_, int s) {
    constexpr int set = decltype(set_)::value;
    const int64_t f = flat0 + static_cast<int64_t>(s) * flat_step;
    if constexpr (kFloatW) {
#pragma unroll
      for (int i = 0; i < kWBytes; ++i) {
        const u32x4_t v = *reinterpret_cast<const u32x4_t *>(wq + f * kWBytes + 16 * i);
#pragma unroll
        for (int e = 0; e < 4; ++e) wreg[set][4 * i + e] = v[e];
      }
    } else if constexpr (kInt4) {
      const u32x2_t v = *reinterpret_cast<const u32x2_t *>(wq + (f >> 1));
      wreg[set][0] = v[0];
      wreg[set][1] = v[1];
      sc[set][0] = to_f32(s16[f >> g.group_shift]);
    } else {
      const u32x4_t v = *reinterpret_cast<const u32x4_t *>(wq + f);
#pragma unroll
      for (int i = 0; i < 4; ++i) wreg[set][i] = v[i];
      if constexpr (vec_scales) {
        // the first code's flat index is a multiple of 16 and so is every step: quads never straddle the wrap
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          uint32_t idx = sidx + 4 * q;
          if (idx >= period) idx -= period;
          const floatx4_t v4 = *reinterpret_cast<const floatx4_t *>(s32 + idx);
#pragma unroll
          for (int e = 0; e < 4; ++e) sc[set][4 * q + e] = v4[e];
        }
#pragma unroll
        for (int q = 0; q < kBK / kStep; ++q) {
          sidx += g.step;
          if (sidx >= period) sidx -= period;
        }
      }
    }
  };
  auto store_b = [&](auto set_) {
    constexpr int set = decltype(set_)::value;
    float w[16];
    if constexpr (kFloatW) {
      typedef std::conditional_t<kFloatW, WT, float> W_t;
      const W_t *h = reinterpret_cast<const W_t *>(&wreg[set][0]);
#pragma unroll
      for (int e = 0; e < 16; ++e) w[e] = rounded(to_f32<W_t>(h[e]));
    } else if constexpr (kInt4) {
      float e0[8], e1[8];
      dequant_int4x8(wreg[set][0], sc[set][0], e0);
      dequant_int4x8(wreg[set][1], sc[set][0], e1);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        w[e] = e0[e];
        w[8 + e] = e1[e];
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float q[4];
        int8x4_to_f32(wreg[set][i], q);
#pragma unroll
        for (int e = 0; e < 4; ++e) w[4 * i + e] = vec_scales ? q[e] * sc[set][4 * i + e] : q[e] * s_one;
      }
    }
    if constexpr (!kBackward) {
#pragma unroll
      for (int e = 0; e < 16; ++e) Bs[(b_minor + e) * SB + b_major] = w[e];
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        floatx4_t v = {w[4 * i], w[4 * i + 1], w[4 * i + 2], w[4 * i + 3]};
        *reinterpret_cast<floatx4_t *>(&Bs[b_major * SB + b_minor + 4 * i]) = v;
      }
    }
  };

  floatx16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int li = lane & 31;
  const int lh = lane >> 5;
  typedef std::integral_constant<int, 0> I0;
  typedef std::integral_constant<int, 1> I1;
  // No load sits behind a branch (a step past the end re-reads the last one; its registers are never stored),
  // so the compiler can count the outstanding requests and a wait for one set leaves the other in flight.
  auto clamped = [&](int s) { return s < steps ? s : steps - 1; };
  auto one_step = [&](auto set_, int s) {
    store_a(set_);
    store_b(set_);
    __syncthreads();
    load_a(set_, static_cast<int64_t>(clamped(s + 2)) * kBK);
    load_b(set_, clamped(s + 2));
#pragma unroll
    for (int pp = 0; pp < kPairs; ++pp) {
      const int p = kSplit ? wave * kPairs + pp : pp;
      const int r = 2 * p + lh;
      float av[TM], bv[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) av[i] = As[r * SA + wm * kWaveRows + i * 32 + li];
#pragma unroll
      for (int j = 0; j < TN; ++j) bv[j] = Bs[r * SB + wn * kWaveCols + j * 32 + li];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], bv[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();              // the next step overwrites both buffers
  };
  load_a(I0{}, 0);
  load_b(I0{}, 0);
  load_a(I1{}, static_cast<int64_t>(clamped(1)) * kBK);
  load_b(I1{}, clamped(1));
  {
    int s = 0;
    for (; s + 2 <= steps; s += 2) {
      one_step(I0{}, s);
      one_step(I1{}, s + 1);
    }
    if (s < steps) one_step(I0{}, s);
  }

  // acc[i][j][r] = D[row][col], row = 8*(r/4) + 4*(lane/32) + r%4, col = lane%32
  if constexpr (kSplit) {
    // the loop's last barrier has passed: the activation buffer is free.  Partial tiles [wave][r][lane], then
    // every thread adds the four partials of four results in wave order.
#pragma unroll
    for (int r = 0; r < 16; ++r) As[(wave * 16 + r) * 64 + lane] = acc[0][0][r];
    __syncthreads();
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int o = t + 256 * q;
      const int r = o >> 6;
      const int ln = o & 63;
      float v = As[r * 64 + ln];
#pragma unroll
      for (int w = 1; w < 4; ++w) v += As[(w * 16 + r) * 64 + ln];
      const int64_t row = row0 + 8 * (r >> 2) + 4 * (ln >> 5) + (r & 3);
      const int64_t col = col0 + (ln & 31);
      if (row < row_hi && col < C) store_result(g.d, g.d_dtype, static_cast<int64_t>(part) * g.M * C + row * C + col, v);
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int64_t col = col0 + wn * kWaveCols + j * 32 + li;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t row = row0 + wm * kWaveRows + i * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
        if (row < row_hi && col < C) store_result(g.d, g.d_dtype, row * C + col, acc[i][j][r]);
      }
    }
}

template <typename XT, bool kInt4, bool kVec, bool kBackward, typename WT = void>
int launch_bm(const F32Args &f, hipStream_t s)
{
  const int64_t C = kBackward ? f.K : f.N;
  const int64_t R = kBackward ? f.N : f.K;
  const int64_t col_tiles = (C + 127) / 128;
  if (f.offsets) {
    // segment lengths live on the device; the host knows their mean: 128-row tiles when an expert has that
    // many rows on average, 32-row tiles otherwise; every expert can add one partial tile
    const bool tall_tiles = f.M >= static_cast<int64_t>(f.num_experts) * 128;
    const int64_t row_tiles = (f.M + (tall_tiles ? 127 : 31)) / (tall_tiles ? 128 : 32) + f.num_experts;
    if (row_tiles > 65535) return CAIFX_ERR_UNSUPPORTED;
    const dim3 grid(static_cast<unsigned>(col_tiles), static_cast<unsigned>(row_tiles));
    if (tall_tiles) hipLaunchKernelGGL((qgemm_f32_kernel<XT, kInt4, kVec, kBackward, 128, 128, 32, WT>), grid, dim3(256), 0, s, f);
    else hipLaunchKernelGGL((qgemm_f32_kernel<XT, kInt4, kVec, kBackward, 32, 128, 32, WT>), grid, dim3(256), 0, s, f);
    return launch_status();
  }
  // few rows: 32 x 32 tiles whose waves split the reduction (128-deep steps)
  if (f.M <= kSplitTileRows && R % 128 == 0) {
    hipLaunchKernelGGL((qgemm_f32_kernel<XT, kInt4, kVec, kBackward, 32, 32, 128, WT>),
                       dim3(static_cast<unsigned>((C + 31) / 32), static_cast<unsigned>((f.M + 31) / 32), static_cast<unsigned>(f.parts)),
                       dim3(256), 0, s, f);
    return launch_status();
  }
  // 128-row tiles once there are enough of them to give every compute unit one; below that 32-row tiles
  // put four times as many workgroups on the chip for the same weight traffic through L2
  const int64_t tall = (f.M + 127) / 128;
  if (tall * col_tiles >= 256 && tall <= 65535) {
    hipLaunchKernelGGL((qgemm_f32_kernel<XT, kInt4, kVec, kBackward, 128, 128, 32, WT>), dim3(static_cast<unsigned>(col_tiles), static_cast<unsigned>(tall)),
                       dim3(256), 0, s, f);
    return launch_status();
  }
  const int64_t low = (f.M + 31) / 32;
  if (low > 65535) return CAIFX_ERR_UNSUPPORTED;
  hipLaunchKernelGGL((qgemm_f32_kernel<XT, kInt4, kVec, kBackward, 32, 128, 32, WT>), dim3(static_cast<unsigned>(col_tiles), static_cast<unsigned>(low)),
                     dim3(256), 0, s, f);
  return launch_status();
}

template <typename XT>
int launch_kind(const F32Args &f, int kind, bool int4, bool backward, hipStream_t s)
{
  if (kind == CAIFX_W_F32) return backward ? launch_bm<XT, false, false, true, float>(f, s) : launch_bm<XT, false, false, false, float>(f, s);
  if (kind == CAIFX_W_F16) return backward ? launch_bm<XT, false, false, true, f16_t>(f, s) : launch_bm<XT, false, false, false, f16_t>(f, s);
  if (kind == CAIFX_W_BF16) return backward ? launch_bm<XT, false, false, true, bf16_t>(f, s) : launch_bm<XT, false, false, false, bf16_t>(f, s);
  if (int4) return backward ? launch_bm<XT, true, false, true>(f, s) : launch_bm<XT, true, false, false>(f, s);
  if (f.period > 1) return backward ? launch_bm<XT, false, true, true>(f, s) : launch_bm<XT, false, true, false>(f, s);
  return backward ? launch_bm<XT, false, false, true>(f, s) : launch_bm<XT, false, false, false>(f, s);
}

// Up to 32 rows there are C / 32 split tiles, 128 at C = 4096 (more rows: that many per 32 rows): a chain of R / 128 dependent steps on half of the
// chip.  With a workspace from the caller up to 4 workgroups share a tile's reduction (at least 8 steps each, about
// one workgroup per compute unit in total) and a second launch adds their partial tiles in a fixed order.
struct F32Plan {
  int parts;
  int part_steps;
  size_t bytes;
};
F32Plan plan_f32(int64_t M, int64_t C, int64_t R, bool grouped)
{
  F32Plan p{1, 0, 0};
  if (grouped || M > kSplitTileRows || R % 128 != 0) return p;
  const int64_t tiles = ((C + 31) / 32) * ((M + 31) / 32);
  if (tiles > 128) return p;
  const int64_t steps = R / 128;
  int64_t k = 256 / tiles;
  if (k > 4) k = 4;
  if (k > steps / 8) k = steps / 8;
  if (k < 2) return p;
  const int64_t per = (steps + k - 1) / k;
  k = (steps + per - 1) / per;
  if (k < 2) return p;
  p.parts = static_cast<int>(k);
  p.part_steps = static_cast<int>(per);
  p.bytes = static_cast<size_t>(k) * static_cast<size_t>(M) * static_cast<size_t>(C) * sizeof(float);
  return p;
}

int run_f32(const GemmArgs &a, bool backward, hipStream_t s)
{
  const bool float_w = a.w.kind == CAIFX_W_F32 || a.w.kind == CAIFX_W_F16 || a.w.kind == CAIFX_W_BF16;
  if ((a.compute_dtype != CAIFX_F32 && !float_w) || a.addend || a.epilogue) return CAIFX_ERR_UNSUPPORTED;
  const bool grouped = a.offsets != nullptr;
  if (grouped && (a.num_experts < 1 || !a.wq_ptrs)) return CAIFX_ERR_UNSUPPORTED;
  const int64_t R = backward ? a.N : a.K;
  if (R % kStep != 0 || a.K % 32 != 0 || a.K < 32 || a.M < 1 || a.N < 1) return CAIFX_ERR_UNSUPPORTED;
  if (a.M > (int64_t{1} << 30) || a.N > (int64_t{1} << 30) || a.K > (int64_t{1} << 30)) return CAIFX_ERR_UNSUPPORTED;
  if (a.N * a.K >= (int64_t{1} << 40)) return CAIFX_ERR_UNSUPPORTED;
  if (!aligned_to(a.x, 16) || (!grouped && !aligned_to(a.w.q, 16))) return CAIFX_ERR_UNSUPPORTED;
  const bool int4 = a.w.kind == CAIFX_W_INT4_GROUP;

  F32Args f{};
  f.M = a.M;
  f.N = a.N;
  f.K = a.K;
  f.a = a.x;
  f.d = a.y;
  f.d_dtype = a.y_dtype;
  f.wq = static_cast<const uint8_t *>(a.w.q);
  f.scales = a.w.scales;
  f.offsets = a.offsets;
  f.wq_ptrs = a.wq_ptrs;
  f.scales_ptrs = a.scales_ptrs;
  f.num_experts = a.num_experts;
  // grouped: the per-expert pointers live on the device; one allocation per expert keeps them 16-byte aligned
  const bool has_scales = grouped ? a.scales_ptrs != nullptr : a.w.scales != nullptr;
  if (int4) {
    const int gs = a.w.group_size;
    if (!has_scales || gs < 16 || (gs & (gs - 1)) != 0) return CAIFX_ERR_UNSUPPORTED;   // 16 codes of a thread share a scale
    f.group_shift = __builtin_ctz(static_cast<unsigned>(gs));
  } else if (a.w.kind == CAIFX_W_INT8) {
    if (!has_scales) {
      f.period = 0;
    } else if (a.w.scale_period == 1) {
      f.period = 1;
    } else {
      // one conditional subtraction per index: the vector must be at least one step (and one thread's run) long
      if (a.w.scale_period < 32 || a.w.scale_period % 4 != 0 || a.w.scale_period > (int64_t{1} << 30) || (!grouped && !aligned_to(a.w.scales, 16)))
        return CAIFX_ERR_UNSUPPORTED;
      f.period = a.w.scale_period;
      f.step = static_cast<uint32_t>((backward ? static_cast<int64_t>(kStep) * a.K : kStep) % a.w.scale_period);
    }
  } else if (!float_w) {
    return CAIFX_ERR_UNSUPPORTED;
  }
  f.round_dt = float_w ? a.compute_dtype : CAIFX_F32;
  f.parts = 1;
  const int64_t cols = backward ? a.K : a.N;
  const F32Plan plan = plan_f32(a.M, cols, R, grouped);
  const bool shared = plan.parts > 1 && a.workspace && a.workspace_bytes >= plan.bytes && aligned_to(a.workspace, 4);
  if (shared) {
    f.parts = plan.parts;
    f.part_steps = plan.part_steps;
    f.d = a.workspace;
    f.d_dtype = CAIFX_F32;
  }
  int st;
  if (a.x_dtype == CAIFX_F32) st = launch_kind<float>(f, a.w.kind, int4, backward, s);
  else if (a.x_dtype == CAIFX_BF16) st = launch_kind<bf16_t>(f, a.w.kind, int4, backward, s);
  else if (a.x_dtype == CAIFX_F16) st = launch_kind<f16_t>(f, a.w.kind, int4, backward, s);
  else return CAIFX_ERR_UNSUPPORTED;
  if (!shared || st != CAIFX_OK) return st;
  return splitk_reduce(static_cast<const float *>(a.workspace), plan.parts, a.M * cols, a.y, a.y_dtype, nullptr, s);
}

}  // namespace

size_t mfma_f32_workspace_bytes(const GemmArgs &a, bool backward)
{
  const bool float_w = a.w.kind == CAIFX_W_F32 || a.w.kind == CAIFX_W_F16 || a.w.kind == CAIFX_W_BF16;
  if (a.compute_dtype != CAIFX_F32 && !float_w) return 0;
  return plan_f32(a.M, backward ? a.K : a.N, backward ? a.N : a.K, a.offsets != nullptr).bytes;
}

int mfma_f32_forward(const GemmArgs &a, hipStream_t s) { return run_f32(a, false, s); }
int mfma_f32_backward(const GemmArgs &a, hipStream_t s) { return run_f32(a, true, s); }

}  // namespace caifx
