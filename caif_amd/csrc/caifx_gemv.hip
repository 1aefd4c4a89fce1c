// Decode-regime dequant-GEMM (M <= 16 rows of activations): Y[M,N] = X[M,K] * W[N,K]^T.
//
// The weight matrix is read exactly once from HBM and nothing else of that size moves, so the
// kernel is judged on bytes per second.  Layout of the work:
//   * one workgroup = 16 consecutive weight rows (output features) x the whole K range;
//   * its NW waves split K in 64-byte row chunks, chunk ch belongs to wave ch % NW, so the
//     chunks the waves fetch at the same time are adjacent in memory;
//   * inside a wave, lane (r = lane%16, c = lane/16) fetches 16 bytes of row r: one 128-bit
//     load = 32 int4 codes or 16 int8 codes, up to 8 such loads in flight per lane before the
//     first one is consumed (the whole weight fits in flight across the chip);
//   * codes are unpacked and scaled in registers to the compute dtype (bit-identical to the
//     reference's dequantise-then-cast) and fed to v_mfma_f32_16x16x32 as the A operand
//     (16 rows x 32 k); the activations are the B operand (32 k x 16 columns, columns >= M
//     are don't-care).  The k order inside a chunk is permuted the same way for A and B;
//   * the NW partial 16x16 fp32 tiles meet in LDS and wave order fixes the summation order,
//     so results are deterministic and no atomics or workspace are needed.
#include "caifx_internal.hpp"

namespace caifx {
namespace {

template <typename CT> struct Mfma16;
template <> struct Mfma16<bf16_t> {
  typedef bf16x8_t vec_t;
  static __device__ __forceinline__ floatx4_t run(vec_t a, vec_t b, floatx4_t c)
  {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma16<f16_t> {
  typedef f16x8_t vec_t;
  static __device__ __forceinline__ floatx4_t run(vec_t a, vec_t b, floatx4_t c)
  {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

enum { WS_INT4 = 0, WS_INT8_SCALAR = 1, WS_INT8_VEC = 2 };

struct SkinnyArgs {
  const uint8_t *wq;
  const void *scales;
  const void *x;
  void *y;
  int M;
  int y_dtype;
  int64_t N, K;
  int group_shift;       // int4: log2(group_size)
  int period;            // int8 vec: scale index = flat % period
  int step_mod;          // int8 vec: (NW * chunk elements) % period
  int xpitch;            // elements between rows of the staged activations
};

template <typename CT, typename XT>
__device__ __forceinline__ typename Mfma16<CT>::vec_t load_x8(const XT *p)
{
  typename Mfma16<CT>::vec_t v;
  if constexpr (sizeof(XT) == 2 && dtype_code<XT>::value == dtype_code<CT>::value) {
    v = *reinterpret_cast<const typename Mfma16<CT>::vec_t *>(p);
  } else if constexpr (sizeof(XT) == 4) {
    const floatx4_t a = *reinterpret_cast<const floatx4_t *>(p);
    const floatx4_t b = *reinterpret_cast<const floatx4_t *>(p + 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[j] = from_f32<CT>(a[j]);
      v[4 + j] = from_f32<CT>(b[j]);
    }
  } else {   // fp16 <-> bf16 go through fp32, like Tensor::To()
    const u32x4_t raw = *reinterpret_cast<const u32x4_t *>(p);
    const XT *e = reinterpret_cast<const XT *>(&raw);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = from_f32<CT>(to_f32<XT>(e[j]));
  }
  return v;
}

template <typename CT, typename XT, int WS, int NW, bool XLDS>
__global__ __launch_bounds__(NW * 64) void skinny_forward_kernel(SkinnyArgs a)
{
  typedef typename Mfma16<CT>::vec_t vec_t;
  constexpr int EPB = (WS == WS_INT4) ? 2 : 1;   // elements per byte
  constexpr int EPL = 16 * EPB;                  // elements in one lane's 16-byte load
  constexpr int KC = 4 * EPL;                    // k extent of one chunk (64 bytes of a row)
  constexpr int SUB = EPL / 8;                   // MFMA steps per chunk
  constexpr int U = (WS == WS_INT8_VEC) ? 4 : 8; // chunk loads in flight per lane

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float *red = reinterpret_cast<float *>(smem);                 // [NW][16*16]
  CT *xs = reinterpret_cast<CT *>(smem + NW * 1024);            // [M][xpitch] when XLDS

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 15;
  const int c = lane >> 4;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * 16;
  const int64_t n = (n0 + r < a.N) ? n0 + r : a.N - 1;
  const int nchunks = static_cast<int>(a.K / KC);
  const int my_chunks = (nchunks - wave + NW - 1) / NW;
  const int64_t rowflat = n * a.K;
  const uint8_t *wrow = a.wq + rowflat / EPB + c * 16;
  const int mrow = (r < a.M) ? r : a.M - 1;

  u32x4_t wreg[U];
  float sreg[U];
  floatx4_t svec[U][4];
  int sidx = 0;
  float s_scalar = 1.0f;
  if constexpr (WS == WS_INT8_SCALAR) {
    if (a.scales) s_scalar = static_cast<const float *>(a.scales)[0];
  }
  if constexpr (WS == WS_INT8_VEC) {
    sidx = static_cast<int>((rowflat + static_cast<int64_t>(wave) * KC + c * EPL) % a.period);
  }

  auto issue = [&](int u, int ch) {
    wreg[u] = *reinterpret_cast<const u32x4_t *>(wrow + static_cast<int64_t>(ch) * 64);
    if constexpr (WS == WS_INT4) {
      const int64_t g = (rowflat + static_cast<int64_t>(ch) * KC + c * EPL) >> a.group_shift;
      sreg[u] = to_f32(static_cast<const f16_t *>(a.scales)[g]);
    }
    if constexpr (WS == WS_INT8_VEC) {
      const float *sp = static_cast<const float *>(a.scales);
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        int i = sidx + 4 * t;
        if (i >= a.period) i -= a.period;
        svec[u][t] = *reinterpret_cast<const floatx4_t *>(sp + i);
      }
      sidx += a.step_mod;
      if (sidx >= a.period) sidx -= a.period;
    }
  };

#pragma unroll
  for (int u = 0; u < U; ++u)
    if (u < my_chunks) issue(u, wave + u * NW);

  if constexpr (XLDS) {
    const XT *xg = static_cast<const XT *>(a.x);
    const int64_t total = static_cast<int64_t>(a.M) * a.K;
    for (int64_t idx = static_cast<int64_t>(threadIdx.x) * 8; idx < total; idx += NW * 64 * 8) {
      const int m = static_cast<int>(idx / a.K);
      const int k = static_cast<int>(idx - static_cast<int64_t>(m) * a.K);
      *reinterpret_cast<vec_t *>(xs + m * a.xpitch + k) = load_x8<CT, XT>(xg + idx);
    }
    __syncthreads();
  }

  floatx4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int i0 = 0; i0 < my_chunks; i0 += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u;
      if (i < my_chunks) {
        const int ch = wave + i * NW;
        const u32x4_t w = wreg[u];
        const float s = (WS == WS_INT4) ? sreg[u] : s_scalar;
        floatx4_t sv[4];
        if constexpr (WS == WS_INT8_VEC) {
#pragma unroll
          for (int t = 0; t < 4; ++t) sv[t] = svec[u][t];
        }
        if (i + U < my_chunks) issue(u, ch + U * NW);
        const int kb = ch * KC + c * EPL;
#pragma unroll
        for (int j = 0; j < SUB; ++j) {
          vec_t av;
          if constexpr (WS == WS_INT4) {
            float e[8];
            dequant_int4x8(w[j], s, e);
#pragma unroll
            for (int q = 0; q < 8; ++q) av[q] = from_f32<CT>(e[q]);
          } else {
            float lo[4], hi[4];
            int8x4_to_f32(w[2 * j], lo);
            int8x4_to_f32(w[2 * j + 1], hi);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float s0 = (WS == WS_INT8_VEC) ? sv[2 * j][q] : s;
              const float s1 = (WS == WS_INT8_VEC) ? sv[2 * j + 1][q] : s;
              av[q] = from_f32<CT>(lo[q] * s0);
              av[4 + q] = from_f32<CT>(hi[q] * s1);
            }
          }
          vec_t bv;
          if constexpr (XLDS) {
            bv = *reinterpret_cast<const vec_t *>(xs + mrow * a.xpitch + kb + 8 * j);
          } else {
            bv = load_x8<CT, XT>(static_cast<const XT *>(a.x) + static_cast<int64_t>(mrow) * a.K + kb + 8 * j);
          }
          acc = Mfma16<CT>::run(av, bv, acc);
        }
      }
    }
  }

  // acc[i] = partial Y for weight row 4*c + i of the tile, activation row r
#pragma unroll
  for (int i = 0; i < 4; ++i) red[wave * 256 + (4 * c + i) * 16 + r] = acc[i];
  __syncthreads();
  for (int t = threadIdx.x; t < 256; t += NW * 64) {
    const int m = t >> 4;
    const int nl = t & 15;
    float v = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; ++w) v += red[w * 256 + nl * 16 + m];
    if (m < a.M && n0 + nl < a.N) {
      const int64_t o = static_cast<int64_t>(m) * a.N + n0 + nl;
      if (a.y_dtype == CAIFX_F32) static_cast<float *>(a.y)[o] = v;
      else if (a.y_dtype == CAIFX_BF16) static_cast<bf16_t *>(a.y)[o] = from_f32<bf16_t>(v);
      else static_cast<f16_t *>(a.y)[o] = from_f32<f16_t>(v);
    }
  }
}

template <typename CT, typename XT, int WS, int NW, bool XLDS>
int launch_skinny(const SkinnyArgs &sa, hipStream_t s)
{
  const size_t lds = NW * 1024 + (XLDS ? static_cast<size_t>(sa.M) * sa.xpitch * sizeof(CT) : 0);
  const unsigned grid = static_cast<unsigned>((sa.N + 15) / 16);
  hipLaunchKernelGGL((skinny_forward_kernel<CT, XT, WS, NW, XLDS>), dim3(grid), dim3(NW * 64), lds, s, sa);
  return launch_status();
}

template <typename CT, typename XT, int WS>
int pick_waves(const SkinnyArgs &sa, bool xlds, int nw, hipStream_t s)
{
  if (xlds) {
    if (nw == 8) return launch_skinny<CT, XT, WS, 8, true>(sa, s);
    return launch_skinny<CT, XT, WS, 4, true>(sa, s);
  }
  if constexpr (dtype_code<XT>::value == dtype_code<CT>::value) {
    if (nw == 8) return launch_skinny<CT, XT, WS, 8, false>(sa, s);
    return launch_skinny<CT, XT, WS, 4, false>(sa, s);
  } else {
    return CAIFX_ERR_UNSUPPORTED;
  }
}

template <typename CT, typename XT>
int pick_weight(const SkinnyArgs &sa, int ws, bool xlds, int nw, hipStream_t s)
{
  switch (ws) {
    case WS_INT4: return pick_waves<CT, XT, WS_INT4>(sa, xlds, nw, s);
    case WS_INT8_SCALAR: return pick_waves<CT, XT, WS_INT8_SCALAR>(sa, xlds, nw, s);
    default: return pick_waves<CT, XT, WS_INT8_VEC>(sa, xlds, nw, s);
  }
}

template <typename CT>
int pick_x(const SkinnyArgs &sa, int x_dtype, int ws, bool xlds, int nw, hipStream_t s)
{
  switch (x_dtype) {
    case CAIFX_F32: return pick_weight<CT, float>(sa, ws, xlds, nw, s);
    case CAIFX_F16: return pick_weight<CT, f16_t>(sa, ws, xlds, nw, s);
    default: return pick_weight<CT, bf16_t>(sa, ws, xlds, nw, s);
  }
}

}  // namespace

int skinny_forward(const GemmArgs &g, hipStream_t s)
{
  if (g.offsets || g.M < 1 || g.M > 16 || g.compute_dtype == CAIFX_F32) return CAIFX_ERR_UNSUPPORTED;
  if (g.N < 1 || g.N > (int64_t{1} << 31) || g.K > (int64_t{1} << 30)) return CAIFX_ERR_UNSUPPORTED;
  const bool int4 = g.w.kind == CAIFX_W_INT4_GROUP;
  const int kc = int4 ? 128 : 64;
  if (g.K % kc != 0) return CAIFX_ERR_UNSUPPORTED;
  if (!aligned_to(g.w.q, 16) || !aligned_to(g.x, 16)) return CAIFX_ERR_UNSUPPORTED;

  SkinnyArgs sa{};
  sa.wq = static_cast<const uint8_t *>(g.w.q);
  sa.scales = g.w.scales;
  sa.x = g.x;
  sa.y = g.y;
  sa.M = static_cast<int>(g.M);
  sa.y_dtype = g.y_dtype;
  sa.N = g.N;
  sa.K = g.K;
  int ws;
  if (int4) {
    const int gs = g.w.group_size;
    if (gs < 32 || (gs & (gs - 1)) != 0 || !g.w.scales) return CAIFX_ERR_UNSUPPORTED;
    sa.group_shift = __builtin_ctz(static_cast<unsigned>(gs));
    ws = WS_INT4;
  } else if (!g.w.scales || g.w.scale_period == 1) {
    ws = WS_INT8_SCALAR;
  } else {
    if (g.w.scale_period % 4 != 0 || g.w.scale_period < 16 || g.w.scale_period > (int64_t{1} << 30) ||
        !aligned_to(g.w.scales, 16))
      return CAIFX_ERR_UNSUPPORTED;
    ws = WS_INT8_VEC;
    sa.period = static_cast<int>(g.w.scale_period);
  }
  const int64_t tiles = (g.N + 15) / 16;
  const int nchunks = static_cast<int>(g.K / kc);
  int nw = (tiles * 4 >= 2048 || nchunks < 8) ? 4 : 8;
  if (ws == WS_INT8_VEC) sa.step_mod = static_cast<int>((static_cast<int64_t>(nw) * kc) % sa.period);
  sa.xpitch = static_cast<int>(g.K) + 8;
  const bool xlds = static_cast<size_t>(sa.M) * sa.xpitch * 2 <= 48 * 1024;
  if (g.compute_dtype == CAIFX_BF16) return pick_x<bf16_t>(sa, g.x_dtype, ws, xlds, nw, s);
  return pick_x<f16_t>(sa, g.x_dtype, ws, xlds, nw, s);
}

}  // namespace caifx
