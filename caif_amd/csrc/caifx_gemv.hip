// Decode-regime dequant-GEMM (M <= 16 rows of activations): Y[M,N] = X[M,K] * W[N,K]^T.
//
// The weight matrix is read exactly once from HBM and nothing else of that size moves, so the
// kernel is judged on bytes per second.  Layout of the work:
//   * a wave owns a tile of 16 weight rows (output features) and a share of K; a workgroup is
//     RS row tiles x KS shares of K.  K is cut in 64-byte row chunks and chunk ch belongs to
//     share ch % KS, so the chunks fetched at the same time are adjacent in memory;
//   * lane (r = lane%16, c = lane/16) fetches 16 bytes of row r per chunk: one 128-bit load =
//     32 int4 codes or 16 int8 codes, up to 8 such loads in flight per lane before the first is
//     consumed, so the whole weight is in flight across the chip;
//   * codes become matrix-core operands in registers and feed v_mfma_f32_16x16x32 as the A
//     operand (16 rows x 32 k); the activations, staged once per workgroup in LDS, are the B
//     operand (32 k x 16 columns; columns >= M are don't-care).  The k order inside a chunk is
//     permuted the same way for A and B, which a sum over k does not see;
//   * the KS partial 16x16 fp32 tiles meet in LDS in a fixed order: deterministic, no atomics,
//     no workspace.
//
// Three ways of turning codes into operands:
//   INT4_POST  (group_size % 128 == 0): the VALU cannot unpack, scale and round 32 codes per
//              16 bytes at HBM speed (about 3 ops per code against a budget of 2), so codes go
//              to the matrix core unscaled: nibble n becomes the 16-bit float 128+(n^8) (bf16)
//              or 1024+(n^8) (fp16) with one bit-op per two codes, each 128-k chunk is
//              accumulated on its own, and  scale * (chunk_sum - offset * sum_k x)  is added to
//              the running total.  Mathematically sum_k code*scale*x with the products formed
//              exactly; it differs from the reference's dequantise-round-multiply only by the
//              bf16/fp16 rounding of code*scale that the reference applies to each weight.
//   INT4_EXACT (other power-of-two group sizes >= 32): code*scale in fp32, rounded to the
//              compute dtype, bit-identical to the reference's dequantise-then-cast.
//   INT8       : float(code) * scale[(n*K+k) % period] in fp32, rounded to the compute dtype,
//              bit-identical to the reference.  Rows whose flat index is congruent modulo the
//              period share their scale stream, so a tile takes rows n = v + V*i with
//              V = period / gcd(K, period): its 16 rows then read the same scale addresses.
#include "caifx_internal.hpp"

namespace caifx {
namespace {

template <typename CT> struct Mfma16;
template <> struct Mfma16<bf16_t> {
  typedef bf16x8_t vec_t;
  static constexpr uint32_t kMagic = 0x43084308u;   // bf16 128.0 in both halves, xor 8 folded in
  static constexpr float kOffset = 136.0f;          // 128 + 8
  static __device__ __forceinline__ floatx4_t run(vec_t a, vec_t b, floatx4_t c)
  {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma16<f16_t> {
  typedef f16x8_t vec_t;
  static constexpr uint32_t kMagic = 0x64086408u;   // fp16 1024.0 in both halves, xor 8 folded in
  static constexpr float kOffset = 1032.0f;         // 1024 + 8
  static __device__ __forceinline__ floatx4_t run(vec_t a, vec_t b, floatx4_t c)
  {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

enum { WS_INT4_POST = 0, WS_INT4_EXACT = 1, WS_INT8_SCALAR = 2, WS_INT8_VEC = 3 };

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
  int step_mod;          // int8 vec: (KS * chunk elements) % period
  int xpitch;            // elements between rows of the staged activations
  int row_stride;        // V: rows of a tile are n = v + V*i
  int tiles_per_res;     // T: tiles per residue class v
  int num_tiles;         // V*T
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

template <typename CT, typename XT, int WS, int RS, int KS, bool XLDS>
__global__ __launch_bounds__(RS * KS * 64) void skinny_forward_kernel(SkinnyArgs a)
{
  typedef typename Mfma16<CT>::vec_t vec_t;
  constexpr bool kInt4 = (WS == WS_INT4_POST || WS == WS_INT4_EXACT);
  constexpr int NT = RS * KS * 64;               // threads per workgroup
  constexpr int EPB = kInt4 ? 2 : 1;             // elements per byte
  constexpr int EPL = 16 * EPB;                  // elements in one lane's 16-byte load
  constexpr int KC = 4 * EPL;                    // k extent of one chunk (64 bytes of a row)
  constexpr int SUB = EPL / 8;                   // MFMA steps per chunk
  constexpr int U = (WS == WS_INT8_VEC) ? 4 : 8; // chunk loads in flight per lane
  static_assert(WS != WS_INT4_POST || XLDS, "post-scaled int4 needs the staged activations");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float *red = reinterpret_cast<float *>(smem);                         // [KS][RS][16*16]
  float *xsum = red + KS * RS * 256;                                    // [M][nchunks] (INT4_POST)
  const int nchunks = static_cast<int>(a.K / KC);
  CT *xs = reinterpret_cast<CT *>(xsum + (WS == WS_INT4_POST ? ((a.M * nchunks + 3) & ~3) : 0));   // [M][xpitch]

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int rs = wave % RS;
  const int ks = wave / RS;
  const int r = lane & 15;
  const int c = lane >> 4;
  int tile = blockIdx.x * RS + rs;
  const bool tile_ok = tile < a.num_tiles;
  if (!tile_ok) tile = a.num_tiles - 1;
  const int res = tile / a.tiles_per_res;                          // residue class v
  const int64_t i0 = static_cast<int64_t>(tile - res * a.tiles_per_res) * 16;
  auto row_of = [&](int local) -> int64_t {                        // weight row of tile-local row index
    const int64_t n = res + static_cast<int64_t>(a.row_stride) * (i0 + local);
    return n < a.N ? n : res;
  };
  const int64_t n = row_of(r);
  const int my_chunks = (nchunks - ks + KS - 1) / KS;
  const int64_t rowflat = n * a.K;
  const uint8_t *wrow = a.wq + rowflat / EPB + c * 16;
  const int mrow = (r < a.M) ? r : a.M - 1;

  u32x4_t wreg[U];
  float sreg[U];              // INT4_EXACT: scale of this lane's row
  f16_t spost[U][4];          // INT4_POST: scales of the four rows this lane accumulates
  floatx4_t svec[U][4];       // INT8_VEC
  int sidx = 0;
  float s_scalar = 1.0f;
  int64_t gbase[4] = {0, 0, 0, 0};
  if constexpr (WS == WS_INT8_SCALAR) {
    if (a.scales) s_scalar = static_cast<const float *>(a.scales)[0];
  }
  if constexpr (WS == WS_INT8_VEC) {
    sidx = static_cast<int>((rowflat + static_cast<int64_t>(ks) * KC + c * EPL) % a.period);
  }
  if constexpr (WS == WS_INT4_POST) {
#pragma unroll
    for (int i = 0; i < 4; ++i) gbase[i] = row_of(4 * c + i) * a.K;
  }

  auto issue = [&](int u, int ch) {
    wreg[u] = *reinterpret_cast<const u32x4_t *>(wrow + static_cast<int64_t>(ch) * 64);
    if constexpr (WS == WS_INT4_EXACT) {
      const int64_t g = (rowflat + static_cast<int64_t>(ch) * KC + c * EPL) >> a.group_shift;
      sreg[u] = to_f32(static_cast<const f16_t *>(a.scales)[g]);
    }
    if constexpr (WS == WS_INT4_POST) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        spost[u][i] = static_cast<const f16_t *>(a.scales)[(gbase[i] + static_cast<int64_t>(ch) * KC) >> a.group_shift];
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
    if (u < my_chunks) issue(u, ks + u * KS);

  if constexpr (XLDS) {
    // Stage X as compute-dtype values.  INT4_POST stores every aligned run of 8 in the order
    // 0,4,1,5,2,6,3,7 (the order its bit-ops produce codes in) and keeps sum_k x per 128-k chunk.
    const XT *xg = static_cast<const XT *>(a.x);
    const int64_t total = static_cast<int64_t>(a.M) * a.K;
    for (int64_t idx = static_cast<int64_t>(threadIdx.x) * 8; idx < total; idx += NT * 8) {
      const int m = static_cast<int>(idx / a.K);
      const int k = static_cast<int>(idx - static_cast<int64_t>(m) * a.K);
      vec_t v = load_x8<CT, XT>(xg + idx);
      if constexpr (WS == WS_INT4_POST) {
        float part = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) part += to_f32<CT>(v[j]);
        part += __shfl_xor(part, 1, 64);
        part += __shfl_xor(part, 2, 64);
        part += __shfl_xor(part, 4, 64);
        part += __shfl_xor(part, 8, 64);
        if ((lane & 15) == 0) xsum[m * nchunks + (k >> 7)] = part;
        vec_t p;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          p[2 * t] = v[t];
          p[2 * t + 1] = v[t + 4];
        }
        v = p;
      }
      *reinterpret_cast<vec_t *>(xs + m * a.xpitch + k) = v;
    }
    __syncthreads();
  }

  floatx4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int i0c = 0; i0c < my_chunks; i0c += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0c + u;
      if (i < my_chunks) {
        const int ch = ks + i * KS;
        const u32x4_t w = wreg[u];
        const float s = (WS == WS_INT4_EXACT) ? sreg[u] : s_scalar;
        floatx4_t sv[4];
        f16_t sp4[4];
        if constexpr (WS == WS_INT8_VEC) {
#pragma unroll
          for (int t = 0; t < 4; ++t) sv[t] = svec[u][t];
        }
        if constexpr (WS == WS_INT4_POST) {
#pragma unroll
          for (int t = 0; t < 4; ++t) sp4[t] = spost[u][t];
        }
        if (i + U < my_chunks) issue(u, ch + U * KS);
        const int kb = ch * KC + c * EPL;
        floatx4_t part = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < SUB; ++j) {
          vec_t av;
          if constexpr (WS == WS_INT4_POST) {
            u32x4_t t;
            const uint32_t p = w[j];
            t[0] = (p & 0x000F000Fu) ^ Mfma16<CT>::kMagic;           // codes 0,4
            t[1] = ((p >> 4) & 0x000F000Fu) ^ Mfma16<CT>::kMagic;    // codes 1,5
            t[2] = ((p >> 8) & 0x000F000Fu) ^ Mfma16<CT>::kMagic;    // codes 2,6
            t[3] = ((p >> 12) & 0x000F000Fu) ^ Mfma16<CT>::kMagic;   // codes 3,7
            av = *reinterpret_cast<const vec_t *>(&t);
          } else if constexpr (WS == WS_INT4_EXACT) {
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
          if constexpr (WS == WS_INT4_POST) part = Mfma16<CT>::run(av, bv, part);
          else acc = Mfma16<CT>::run(av, bv, acc);
        }
        if constexpr (WS == WS_INT4_POST) {
          const float corr = Mfma16<CT>::kOffset * xsum[mrow * nchunks + ch];
#pragma unroll
          for (int t = 0; t < 4; ++t) acc[t] = __builtin_fmaf(to_f32(sp4[t]), part[t] - corr, acc[t]);
        }
      }
    }
  }

  // acc[i] = partial Y for tile-local weight row 4*c + i, activation row r
#pragma unroll
  for (int i = 0; i < 4; ++i) red[(ks * RS + rs) * 256 + (4 * c + i) * 16 + r] = acc[i];
  __syncthreads();
  for (int t = threadIdx.x; t < RS * 256; t += NT) {
    const int trs = t >> 8;
    const int m = (t >> 4) & 15;
    const int nl = t & 15;
    float v = 0.0f;
#pragma unroll
    for (int w = 0; w < KS; ++w) v += red[(w * RS + trs) * 256 + nl * 16 + m];
    const int ttile = blockIdx.x * RS + trs;
    if (ttile < a.num_tiles && m < a.M) {
      const int tres = ttile / a.tiles_per_res;
      const int64_t nn = tres + static_cast<int64_t>(a.row_stride) *
                                    (static_cast<int64_t>(ttile - tres * a.tiles_per_res) * 16 + nl);
      if (nn < a.N) {
        const int64_t o = static_cast<int64_t>(m) * a.N + nn;
        if (a.y_dtype == CAIFX_F32) static_cast<float *>(a.y)[o] = v;
        else if (a.y_dtype == CAIFX_BF16) static_cast<bf16_t *>(a.y)[o] = from_f32<bf16_t>(v);
        else static_cast<f16_t *>(a.y)[o] = from_f32<f16_t>(v);
      }
    }
  }
}

size_t lds_bytes(const SkinnyArgs &sa, int ws, int rs, int ks, bool xlds, int kc)
{
  size_t b = static_cast<size_t>(rs) * ks * 1024;
  if (ws == WS_INT4_POST) b += static_cast<size_t>((sa.M * (sa.K / kc) + 3) & ~int64_t{3}) * 4;
  if (xlds) b += static_cast<size_t>(sa.M) * sa.xpitch * 2;
  return b;
}

template <typename CT, typename XT, int WS, int RS, int KS, bool XLDS>
int launch_skinny(const SkinnyArgs &sa, hipStream_t s)
{
  constexpr int kc = (WS == WS_INT4_POST || WS == WS_INT4_EXACT) ? 128 : 64;
  const size_t lds = lds_bytes(sa, WS, RS, KS, XLDS, kc);
  auto kern = skinny_forward_kernel<CT, XT, WS, RS, KS, XLDS>;
  if (lds > 64 * 1024) {
    static bool raised = false;   // once per instantiation is enough; the call is idempotent
    if (!raised) {
      if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              160 * 1024) != hipSuccess)
        return CAIFX_ERR_LAUNCH_FAILED;
      raised = true;
    }
  }
  const unsigned grid = static_cast<unsigned>((sa.num_tiles + RS - 1) / RS);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(RS * KS * 64), lds, s, sa);
  return launch_status();
}

// shape of the workgroup: 0 = one row tile, K split 4 ways; 1 = one row tile, K split 8 ways;
// 2 = four row tiles sharing the staged activations, K split 2 ways
template <typename CT, typename XT, int WS>
int pick_shape(const SkinnyArgs &sa, bool xlds, int shape, hipStream_t s)
{
  if (xlds) {
    if (shape == 2) return launch_skinny<CT, XT, WS, 4, 2, true>(sa, s);
    if (shape == 1) return launch_skinny<CT, XT, WS, 1, 8, true>(sa, s);
    return launch_skinny<CT, XT, WS, 1, 4, true>(sa, s);
  }
  if constexpr (WS != WS_INT4_POST && dtype_code<XT>::value == dtype_code<CT>::value) {
    if (shape == 1) return launch_skinny<CT, XT, WS, 1, 8, false>(sa, s);
    return launch_skinny<CT, XT, WS, 1, 4, false>(sa, s);
  } else {
    return CAIFX_ERR_UNSUPPORTED;
  }
}

template <typename CT, typename XT>
int pick_weight(const SkinnyArgs &sa, int ws, bool xlds, int shape, hipStream_t s)
{
  switch (ws) {
    case WS_INT4_POST: return pick_shape<CT, XT, WS_INT4_POST>(sa, xlds, shape, s);
    case WS_INT4_EXACT: return pick_shape<CT, XT, WS_INT4_EXACT>(sa, xlds, shape, s);
    case WS_INT8_SCALAR: return pick_shape<CT, XT, WS_INT8_SCALAR>(sa, xlds, shape, s);
    default: return pick_shape<CT, XT, WS_INT8_VEC>(sa, xlds, shape, s);
  }
}

template <typename CT>
int pick_x(const SkinnyArgs &sa, int x_dtype, int ws, bool xlds, int shape, hipStream_t s)
{
  switch (x_dtype) {
    case CAIFX_F32: return pick_weight<CT, float>(sa, ws, xlds, shape, s);
    case CAIFX_F16: return pick_weight<CT, f16_t>(sa, ws, xlds, shape, s);
    default: return pick_weight<CT, bf16_t>(sa, ws, xlds, shape, s);
  }
}

int64_t gcd64(int64_t a, int64_t b)
{
  while (b) {
    const int64_t t = a % b;
    a = b;
    b = t;
  }
  return a;
}

}  // namespace

int skinny_forward(const GemmArgs &g, hipStream_t s)
{
  if (g.offsets || g.M < 1 || g.M > 16 || g.compute_dtype == CAIFX_F32) return CAIFX_ERR_UNSUPPORTED;
  if (g.N < 1 || g.N > (int64_t{1} << 30) || g.K > (int64_t{1} << 30)) return CAIFX_ERR_UNSUPPORTED;
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
  sa.row_stride = 1;
  sa.xpitch = static_cast<int>(g.K) + 8;
  const int nchunks = static_cast<int>(g.K / kc);
  int ws;
  if (int4) {
    const int gs = g.w.group_size;
    if (gs < 32 || (gs & (gs - 1)) != 0 || !g.w.scales) return CAIFX_ERR_UNSUPPORTED;
    sa.group_shift = __builtin_ctz(static_cast<unsigned>(gs));
    ws = (gs % 128 == 0) ? WS_INT4_POST : WS_INT4_EXACT;
  } else if (!g.w.scales || g.w.scale_period == 1) {
    ws = WS_INT8_SCALAR;
  } else {
    const int64_t P = g.w.scale_period;
    if (P % 4 != 0 || P < 16 || P > (int64_t{1} << 30) || !aligned_to(g.w.scales, 16)) return CAIFX_ERR_UNSUPPORTED;
    ws = WS_INT8_VEC;
    sa.period = static_cast<int>(P);
    const int64_t V = P / gcd64(g.K % P == 0 ? P : g.K % P, P);   // rows n, n+V share their scale stream
    if (V * 64 <= g.N) sa.row_stride = static_cast<int>(V);       // else too few rows per class: plain tiles
  }

  // staged activations + partial tiles must fit LDS; prefer the layout that keeps occupancy
  const size_t xbytes = static_cast<size_t>(sa.M) * sa.xpitch * 2;
  const size_t xsum_bytes = (ws == WS_INT4_POST) ? static_cast<size_t>(sa.M) * nchunks * 4 + 16 : 0;
  int shape;
  bool xlds = true;
  if (xbytes + xsum_bytes + 8 * 1024 <= 48 * 1024) {
    const int64_t tiles = (g.N + 15) / 16;
    shape = (tiles * 4 >= 2048 || nchunks < 8) ? 0 : 1;
  } else if (xbytes + xsum_bytes + 8 * 1024 <= 150 * 1024) {
    shape = 2;
  } else {
    if (ws == WS_INT4_POST) ws = WS_INT4_EXACT;
    xlds = false;
    shape = 0;
  }
  const int ks = (shape == 0) ? 4 : (shape == 1 ? 8 : 2);
  if (ws == WS_INT8_VEC) sa.step_mod = static_cast<int>((static_cast<int64_t>(ks) * kc) % sa.period);
  const int64_t rows_per_res = (g.N + sa.row_stride - 1) / sa.row_stride;   // rows in residue class 0 (the largest)
  sa.tiles_per_res = static_cast<int>((rows_per_res + 15) / 16);
  sa.num_tiles = sa.tiles_per_res * sa.row_stride;
  if (g.compute_dtype == CAIFX_BF16) return pick_x<bf16_t>(sa, g.x_dtype, ws, xlds, shape, s);
  return pick_x<f16_t>(sa, g.x_dtype, ws, xlds, shape, s);
}

}  // namespace caifx
