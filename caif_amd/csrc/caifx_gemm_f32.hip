// Dequant-GEMM for the fp32 compute type on the matrix cores: Y[M,N] = X[M,K] * W[N,K]^T and
// dX[M,K] = dY[M,N] * W[N,K] with W stored int8 or packed int4 and dequantised to fp32 exactly as the
// reference's dequantise kernels do (fp32 code * scale, no further rounding; ConvertToComputeDtype with
// ComputeT = float, src/caif_device_frozen_linear.cpp:289-378), activations widened to fp32, fp32
// accumulation (the reference's Accuracy_e matmul mode).
//
// v_mfma_f32_32x32x2_f32 runs at 1/16 of the bf16 rate, so this kernel is bound by the matrix pipes long
// before anything else and is kept simple: 256 threads, one BM x 128 tile of the result per workgroup, 32
// deep reduction steps, one LDS buffer per operand (the next step's global loads are in flight while the
// matrix cores work on the current one; two barriers per step cost little against the 1000-4000 MFMA
// cycles between them).  Both operands sit in LDS reduction-major ([r][row] with the row index contiguous),
// which is what the MFMA operands read: lane (i, h) of a 32x32x2 step takes element [2p + h][i].
#include "caifx_internal.hpp"

namespace caifx {
namespace {

constexpr int kBK = 32;      // reduction elements per step
constexpr int kBN = 128;     // result columns per workgroup

struct F32Args {
  int64_t M, N, K;
  const void *a;         // activations [M, R]
  void *d;               // result [M, C]
  int d_dtype;
  const uint8_t *wq;
  const void *scales;
  int group_shift;       // int4: log2(group_size), group_size >= 16
  int64_t period;        // int8: 0 = no scales, 1 = one scale, otherwise the length of the scale vector (>= 32)
  uint32_t step;         // int8 scale vector: how far the scale index moves per reduction step, modulo period
};

__device__ __forceinline__ void store_result(void *p, int dt, int64_t i, float v)
{
  if (dt == CAIFX_BF16) static_cast<bf16_t *>(p)[i] = from_f32<bf16_t>(v);
  else if (dt == CAIFX_F16) static_cast<f16_t *>(p)[i] = from_f32<f16_t>(v);
  else static_cast<float *>(p)[i] = v;
}

// BM = 128: waves 2 x 2 over the tile, 64 x 64 each; BM = 32: waves 1 x 4, 32 x 32 each (small M).
template <typename XT, bool kInt4, bool kBackward, int BM>
__global__ __launch_bounds__(256) void qgemm_f32_kernel(F32Args g)
{
  constexpr int WM = BM == 128 ? 2 : 1;
  constexpr int WN = 4 / WM;
  constexpr int kWaveRows = BM / WM;
  constexpr int kWaveCols = kBN / WN;
  constexpr int TM = kWaveRows / 32;
  constexpr int TN = kWaveCols / 32;
  constexpr int SA = BM + 4;               // row pitch in floats: the transposing writes spread over the banks
  constexpr int SB = kBN + 4;
  constexpr int EA = BM * kBK / 256;       // activation elements per thread per step (16 or 4)
  constexpr int TPR = kBK / EA;            // threads per activation row
  __shared__ __attribute__((aligned(16))) float As[kBK * SA];
  __shared__ __attribute__((aligned(16))) float Bs[kBK * SB];

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = t >> 6;
  const int wm = wave / WN;
  const int wn = wave % WN;
  const int64_t R = kBackward ? g.N : g.K;
  const int64_t C = kBackward ? g.K : g.N;
  const int64_t row0 = static_cast<int64_t>(blockIdx.y) * BM;
  const int64_t col0 = static_cast<int64_t>(blockIdx.x) * kBN;
  const int steps = static_cast<int>(R / kBK);

  // ---- activations: thread (a_row, a_col) holds EA consecutive reduction elements of one row
  const int a_row = t / TPR;
  const int a_col = (t % TPR) * EA;
  int64_t am = row0 + a_row;
  if (am >= g.M) am = g.M - 1;                                   // rows past the end are never stored
  const XT *ap = static_cast<const XT *>(g.a) + am * R + a_col;
  float areg[EA];
  auto load_a = [&](int64_t r0) {
    if constexpr (sizeof(XT) == 4) {
#pragma unroll
      for (int i = 0; i < EA / 4; ++i) {
        const floatx4_t v = *reinterpret_cast<const floatx4_t *>(ap + r0 + 4 * i);
#pragma unroll
        for (int e = 0; e < 4; ++e) areg[4 * i + e] = v[e];
      }
    } else if constexpr (EA == 16) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const u32x4_t v = *reinterpret_cast<const u32x4_t *>(ap + r0 + 8 * i);
        const XT *h = reinterpret_cast<const XT *>(&v);
#pragma unroll
        for (int e = 0; e < 8; ++e) areg[8 * i + e] = to_f32<XT>(h[e]);
      }
    } else {
      const u32x2_t v = *reinterpret_cast<const u32x2_t *>(ap + r0);
      const XT *h = reinterpret_cast<const XT *>(&v);
#pragma unroll
      for (int e = 0; e < 4; ++e) areg[e] = to_f32<XT>(h[e]);
    }
  };
  auto store_a = [&]() {
#pragma unroll
    for (int e = 0; e < EA; ++e) As[(a_col + e) * SA + a_row] = areg[e];
  };

  // ---- weights: 16 consecutive codes (along k) per thread and step
  //   forward : weight row n = col0 + t/2, k = r0 + (t%2)*16 .. +16      -> Bs[k][n]   (transposing write)
  //   backward: weight row n = r0 + t/8,   k = col0 + (t%8)*16 .. +16    -> Bs[n][k]   (row write)
  const int b_major = kBackward ? t >> 3 : t >> 1;
  const int b_minor = kBackward ? (t & 7) * 16 : (t & 1) * 16;
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
  const int64_t flat_step = kBackward ? static_cast<int64_t>(kBK) * g.K : kBK;
  const float *s32 = static_cast<const float *>(g.scales);
  const f16_t *s16 = static_cast<const f16_t *>(g.scales);
  const bool vec_scales = !kInt4 && g.period > 1;
  const uint32_t period = static_cast<uint32_t>(g.period);
  uint32_t sidx = vec_scales ? static_cast<uint32_t>(flat0 % g.period) : 0u;
  const float s_one = (!kInt4 && g.period == 1) ? s32[0] : 1.0f;

  uint32_t wreg[kInt4 ? 2 : 4];
  float sc[kInt4 ? 1 : 16];
  auto load_b = [&](int s) {
    const int64_t f = flat0 + static_cast<int64_t>(s) * flat_step;
    if constexpr (kInt4) {
      const u32x2_t v = *reinterpret_cast<const u32x2_t *>(g.wq + (f >> 1));
      wreg[0] = v[0];
      wreg[1] = v[1];
      sc[0] = to_f32(s16[f >> g.group_shift]);
    } else {
      const u32x4_t v = *reinterpret_cast<const u32x4_t *>(g.wq + f);
#pragma unroll
      for (int i = 0; i < 4; ++i) wreg[i] = v[i];
      if (vec_scales) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          uint32_t idx = sidx + e;
          if (idx >= period) idx -= period;
          sc[e] = s32[idx];
        }
        sidx += g.step;
        if (sidx >= period) sidx -= period;
      }
    }
  };
  auto store_b = [&]() {
    float w[16];
    if constexpr (kInt4) {
      float e0[8], e1[8];
      dequant_int4x8(wreg[0], sc[0], e0);
      dequant_int4x8(wreg[1], sc[0], e1);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        w[e] = e0[e];
        w[8 + e] = e1[e];
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float q[4];
        int8x4_to_f32(wreg[i], q);
#pragma unroll
        for (int e = 0; e < 4; ++e) w[4 * i + e] = vec_scales ? q[e] * sc[4 * i + e] : q[e] * s_one;
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
  load_a(0);
  load_b(0);
  for (int s = 0; s < steps; ++s) {
    store_a();
    store_b();
    __syncthreads();
    if (s + 1 < steps) {          // same for every thread
      load_a(static_cast<int64_t>(s + 1) * kBK);
      load_b(s + 1);
    }
#pragma unroll
    for (int p = 0; p < kBK / 2; ++p) {
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
  }

  // acc[i][j][r] = D[row][col], row = 8*(r/4) + 4*(lane/32) + r%4, col = lane%32
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int64_t col = col0 + wn * kWaveCols + j * 32 + li;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t row = row0 + wm * kWaveRows + i * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
        if (row < g.M && col < C) store_result(g.d, g.d_dtype, row * C + col, acc[i][j][r]);
      }
    }
}

template <typename XT, bool kInt4, bool kBackward>
int launch_bm(const F32Args &f, hipStream_t s)
{
  const int64_t C = kBackward ? f.K : f.N;
  const int64_t col_tiles = (C + kBN - 1) / kBN;
  // 128-row tiles once there are enough of them to give every compute unit one; below that 32-row tiles
  // put four times as many workgroups on the chip for the same weight traffic through L2
  const int64_t tall = (f.M + 127) / 128;
  if (tall * col_tiles >= 256 && tall <= 65535) {
    hipLaunchKernelGGL((qgemm_f32_kernel<XT, kInt4, kBackward, 128>), dim3(static_cast<unsigned>(col_tiles), static_cast<unsigned>(tall)),
                       dim3(256), 0, s, f);
    return launch_status();
  }
  const int64_t low = (f.M + 31) / 32;
  if (low > 65535) return CAIFX_ERR_UNSUPPORTED;
  hipLaunchKernelGGL((qgemm_f32_kernel<XT, kInt4, kBackward, 32>), dim3(static_cast<unsigned>(col_tiles), static_cast<unsigned>(low)),
                     dim3(256), 0, s, f);
  return launch_status();
}

template <typename XT>
int launch_kind(const F32Args &f, bool int4, bool backward, hipStream_t s)
{
  if (int4) return backward ? launch_bm<XT, true, true>(f, s) : launch_bm<XT, true, false>(f, s);
  return backward ? launch_bm<XT, false, true>(f, s) : launch_bm<XT, false, false>(f, s);
}

int run_f32(const GemmArgs &a, bool backward, hipStream_t s)
{
  if (a.compute_dtype != CAIFX_F32 || a.offsets || a.addend || a.epilogue) return CAIFX_ERR_UNSUPPORTED;
  const int64_t R = backward ? a.N : a.K;
  if (R % kBK != 0 || a.K % 32 != 0 || a.K < 32 || a.M < 1 || a.N < 1) return CAIFX_ERR_UNSUPPORTED;
  if (a.M > (int64_t{1} << 30) || a.N > (int64_t{1} << 30) || a.K > (int64_t{1} << 30)) return CAIFX_ERR_UNSUPPORTED;
  if (a.N * a.K >= (int64_t{1} << 40)) return CAIFX_ERR_UNSUPPORTED;
  if (!aligned_to(a.x, 16) || !aligned_to(a.w.q, 16)) return CAIFX_ERR_UNSUPPORTED;
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
  if (int4) {
    const int gs = a.w.group_size;
    if (!a.w.scales || gs < 16 || (gs & (gs - 1)) != 0) return CAIFX_ERR_UNSUPPORTED;   // 16 codes of a thread share a scale
    f.group_shift = __builtin_ctz(static_cast<unsigned>(gs));
  } else if (a.w.kind == CAIFX_W_INT8) {
    if (!a.w.scales) {
      f.period = 0;
    } else if (a.w.scale_period == 1) {
      f.period = 1;
    } else {
      // one conditional subtraction per index: the vector must be at least one step (and one thread's run) long
      if (a.w.scale_period < 32 || a.w.scale_period > (int64_t{1} << 30) || !aligned_to(a.w.scales, 4)) return CAIFX_ERR_UNSUPPORTED;
      f.period = a.w.scale_period;
      f.step = static_cast<uint32_t>((backward ? static_cast<int64_t>(kBK) * a.K : kBK) % a.w.scale_period);
    }
  } else {
    return CAIFX_ERR_UNSUPPORTED;
  }
  if (a.x_dtype == CAIFX_F32) return launch_kind<float>(f, int4, backward, s);
  if (a.x_dtype == CAIFX_BF16) return launch_kind<bf16_t>(f, int4, backward, s);
  if (a.x_dtype == CAIFX_F16) return launch_kind<f16_t>(f, int4, backward, s);
  return CAIFX_ERR_UNSUPPORTED;
}

}  // namespace

int mfma_f32_forward(const GemmArgs &a, hipStream_t s) { return run_f32(a, false, s); }
int mfma_f32_backward(const GemmArgs &a, hipStream_t s) { return run_f32(a, true, s); }

}  // namespace caifx
