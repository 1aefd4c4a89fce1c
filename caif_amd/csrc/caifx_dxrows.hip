// Input gradient for a handful of rows (M <= 16): dX[M,K] = dY[M,N] * W[N,K] with W stored as int8 codes, memory
// bound on the weight stream like the decode forward, but with the reduction running down the weight's rows.
//
// v_mfma_f32_16x16x4_f32 holds one value per lane in both operands, so a weight row needs no transposition: a
// lane (j = lane % 16, q = lane / 16) loads 8 consecutive codes of row n + q at k = k0 + 8j, and code b of that
// load is the B operand of matrix instruction b, whose 16 columns are then k0 + 8*col + b.  The A operand is
// dY[m = j][n + q].  Eight instructions consume one 8-byte load per lane; the sums stay in fp32, the codes are
// exact in fp32 and the weight's scale is applied to the finished column, so nothing is rounded to a 16-bit type
// on the way (the reference rounds code*scale to the compute dtype first; results differ by that rounding, a
// few 1e-3 of the largest output for bf16, 1e-7 for the fp32 compute type).
// That needs the scale of W[n][k] not to depend on n among the rows a workgroup visits: scale index
// (n*K + k) mod period with K a multiple of the period (the per-output-channel scales of a square weight), one
// scale, none, or any period with the rows split into residue classes (see DxArgs::V).
// Packed int4 codes in groups of 128 or more take the same route with the scale on the other operand: a slab of
// 128 columns lies inside one group, so the scale of (row, group) multiplies the row's gradient before it enters
// the A operand.
//
// A workgroup of 16 waves owns a slab of 128 columns (one cache line of every weight row it visits) and a range
// of rows; the waves split the rows 16 at a time, add their 16 partial tiles through LDS in a fixed order and
// write [M][128] sums.  Enough row ranges to fill the chip meet in the caller's workspace (fixed order again).
#include "caifx_internal.hpp"

namespace caifx {
namespace {

constexpr int kDxWaves = 16;
constexpr int kDxThreads = kDxWaves * 64;
constexpr int kDxSlab = 128;                 // columns of dX per workgroup
// 8-byte weight loads per stage of a wave's ring (4 rows each) and stages.  Measured at N = K = 4096 / N = 14336,
// 16 rows: 4 x 2: 15.6 / 33.4 us; 2 x 4: 16.1 / 32.6; 4 x 3: 19.8 / 36.5; 4 x 4: 24.4 / 35.6; 8 x 2: 23.4 / 35.5
// (a deeper ring only adds passes past the last row, which still cost their multiplications).
constexpr int kDxIter = 4;
constexpr int kDxStages = 2;
constexpr int kDxWaveRows = 4 * kDxIter;     // rows a wave takes per pass
constexpr int kDxPassRows = kDxWaves * kDxWaveRows;

struct DxArgs {
  const int8_t *wq;         // int8 codes, or packed int4 (two codes per byte, even k in the low nibble)
  const void *scales;       // int8: fp32 vector (see period); int4: fp16, one per row and group
  const void *dy;
  void *dx;
  int M;
  int y_dtype;
  int64_t N, K;
  int period;              // int8: 0: no scale, 1: scales[0], else scales[k % period]
  int group_shift;         // int4: log2 of the group size (>= 7: a slab lies inside one group)
  // int8 scale vectors whose index depends on the weight row: rows n with equal n mod V see the same scales along
  // k (V = period / gcd(K mod period, period)), so a workgroup only visits rows n = cls + V*i of one residue class
  // and its columns still have one scale each, scales[(cls*K + k) mod period].  V = 1 otherwise.
  int V;
  int ranges;              // row ranges per class: blockIdx.y = cls * ranges + range
  int64_t rows_per_wg;     // rows of a class per workgroup
  float *partial;          // [gridDim.y][M][K] when the rows are split among workgroups, else null
};

// XT: type of dY in memory; CT: compute type dY is rounded to first, as the layer's cast of its input does.
// kInt4: packed int4 codes; a lane's 8 codes are one dword, and the scale of (row, group) multiplies the row's
// gradient on its way into the A operand (the slab's 128 columns share the group).
template <typename XT, typename CT, bool kInt4>
__global__ __launch_bounds__(kDxThreads) void dxrows_kernel(DxArgs a)
{
  extern __shared__ __attribute__((aligned(16))) float tiles[];      // [16 waves][8 codes][4][64], then [16][128] sums
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int j = lane & 15;
  const int q = lane >> 4;
  const int64_t k0 = static_cast<int64_t>(blockIdx.x) * kDxSlab;
  const int cls = blockIdx.y / a.ranges;
  const int64_t rows_class = (a.N - cls + a.V - 1) / a.V;              // rows n = cls + V*i, i < rows_class
  const int64_t n_lo = static_cast<int64_t>(blockIdx.y - cls * a.ranges) * a.rows_per_wg;      // (i, not n, from here on)
  const int64_t n_hi = n_lo + a.rows_per_wg < rows_class ? n_lo + a.rows_per_wg : rows_class;
  const XT *dy = static_cast<const XT *>(a.dy) + static_cast<int64_t>(j < a.M ? j : a.M - 1) * a.N;
  const int8_t *wcol = a.wq + (kInt4 ? (k0 >> 1) + 4 * j : k0 + 8 * j);
  const int64_t row_bytes = kInt4 ? a.K >> 1 : a.K;
  const f16_t *s16 = static_cast<const f16_t *>(a.scales);
  const bool row_live = j < a.M;

  floatx4_t acc[8];
#pragma unroll
  for (int b = 0; b < 8; ++b) acc[b] = floatx4_t{0.0f, 0.0f, 0.0f, 0.0f};

  // A ring of kDxStages stages of kDxIter loads: later passes are on their way while this one is multiplied.
  // Every pass issues its loads whether or not rows are left (the address is clamped, the gradient zero), so the
  // number of loads in flight is known when the code is compiled and a stage is waited for without draining the
  // others.
  u32x2_t w[kDxStages][kDxIter];
  f16_t ws[kDxStages][kDxIter];          // int4: scale of the row in this slab's group
  XT av[kDxStages][kDxIter];             // dY as loaded
  uint32_t keep[kDxStages][kDxIter];     // all ones where the row and the gradient row exist, else 0
  auto issue = [&](int st, int64_t base) {
#pragma unroll
    for (int it = 0; it < kDxIter; ++it) {
      const int64_t n = base + 4 * it + q;
      const int64_t nn = cls + a.V * (n < n_hi ? n : n_hi - 1);          // rows past the range: a valid address, a zero gradient
      if constexpr (kInt4) {
        w[st][it][0] = *reinterpret_cast<const uint32_t *>(wcol + nn * row_bytes);
        ws[st][it] = s16[(nn * a.K + k0) >> a.group_shift];
      } else {
        w[st][it] = *reinterpret_cast<const u32x2_t *>(wcol + nn * row_bytes);
      }
      av[st][it] = dy[nn];
      // (a mask on the bits, not a conditional expression: the compiler turns that into a load under a branch
      // with a full wait behind it)
      keep[st][it] = static_cast<uint32_t>(-static_cast<int>((n < n_hi) & row_live));
    }
  };
  auto multiply = [&](int st) {
#pragma unroll
    for (int it = 0; it < kDxIter; ++it) {
      float g = round_through<CT>(to_f32<XT>(av[st][it]));
      if constexpr (kInt4) g *= to_f32(ws[st][it]);
      g = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, g) & keep[st][it]);
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const int code = kInt4 ? static_cast<int>(w[st][it][0] << (28 - 4 * b)) >> 28
                               : static_cast<int>(w[st][it][b >> 2] << (24 - 8 * (b & 3))) >> 24;
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(g, static_cast<float>(code), acc[b], 0, 0, 0);
      }
    }
  };
  int64_t base = n_lo + static_cast<int64_t>(wave) * kDxWaveRows;
  // (the fences keep the compiler from sinking a stage's loads down to their first use, which it otherwise does
  // to save registers, with a full wait in front of every multiplication)
#pragma unroll
  for (int st = 0; st < kDxStages - 1; ++st) issue(st, base + st * kDxPassRows);
  for (; base < n_hi; base += kDxStages * kDxPassRows) {       // the same trip count for every lane of a wave
#pragma unroll
    for (int st = 0; st < kDxStages; ++st) {
      issue((st + kDxStages - 1) % kDxStages, base + (st + kDxStages - 1) * kDxPassRows);
      __builtin_amdgcn_sched_barrier(0);
      multiply(st);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // acc[b][v] = this wave's share of dX[4*(lane/16) + v][k0 + 8*(lane%16) + b]
#pragma unroll
  for (int b = 0; b < 8; ++b)
#pragma unroll
    for (int v = 0; v < 4; ++v) tiles[((wave * 8 + b) * 4 + v) * 64 + lane] = acc[b][v];
  __syncthreads();
  constexpr int kPer = 2048 / kDxThreads;      // sums per thread
  float sum[kPer];
#pragma unroll
  for (int h = 0; h < kPer; ++h) {
    const int idx = threadIdx.x + h * kDxThreads;        // (b*4 + v) * 64 + lane
    float s = 0.0f;
#pragma unroll
    for (int wv = 0; wv < kDxWaves; ++wv) s += tiles[wv * 2048 + idx];
    sum[h] = s;
  }
  __syncthreads();
#pragma unroll
  for (int h = 0; h < kPer; ++h) {
    const int idx = threadIdx.x + h * kDxThreads;
    const int bv = idx >> 6;
    const int l = idx & 63;
    tiles[(4 * (l >> 4) + (bv & 3)) * kDxSlab + 8 * (l & 15) + (bv >> 2)] = sum[h];
  }
  __syncthreads();
#pragma unroll
  for (int h = 0; h < kPer; ++h) {
    const int o = threadIdx.x + h * kDxThreads;
    const int m = o >> 7;
    const int64_t k = k0 + (o & (kDxSlab - 1));
    if (m >= a.M) continue;
    float s = 1.0f;
    if constexpr (!kInt4) {
      const float *s32 = static_cast<const float *>(a.scales);
      if (a.period == 1) s = s32[0];
      else if (a.period > 1) s = s32[(static_cast<int64_t>(cls) * a.K + k) % a.period];
    }
    const float v = tiles[o] * s;
    const int64_t at = static_cast<int64_t>(m) * a.K + k;
    if (a.partial) a.partial[static_cast<int64_t>(blockIdx.y) * a.M * a.K + at] = v;
    else if (a.y_dtype == CAIFX_F32) static_cast<float *>(a.dx)[at] = v;
    else if (a.y_dtype == CAIFX_BF16) static_cast<bf16_t *>(a.dx)[at] = from_f32<bf16_t>(v);
    else static_cast<f16_t *>(a.dx)[at] = from_f32<f16_t>(v);
  }
}

int compute_units()
{
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
    return n;
  return 256;
}

template <typename CT, bool kInt4>
int launch_xt(const DxArgs &a, int x_dtype, dim3 grid, size_t lds, hipStream_t s)
{
  if (x_dtype == CAIFX_F32) hipLaunchKernelGGL((dxrows_kernel<float, CT, kInt4>), grid, dim3(kDxThreads), lds, s, a);
  else if (x_dtype == CAIFX_BF16) hipLaunchKernelGGL((dxrows_kernel<bf16_t, CT, kInt4>), grid, dim3(kDxThreads), lds, s, a);
  else hipLaunchKernelGGL((dxrows_kernel<f16_t, CT, kInt4>), grid, dim3(kDxThreads), lds, s, a);
  return launch_status();
}

template <typename CT>
int launch_ct(const DxArgs &a, bool int4, int x_dtype, dim3 grid, size_t lds, hipStream_t s)
{
  return int4 ? launch_xt<CT, true>(a, x_dtype, grid, lds, s) : launch_xt<CT, false>(a, x_dtype, grid, lds, s);
}

struct DxPlan {
  bool ok;
  int period;
  int group_shift;
  int V;                   // residue classes of the rows (int8 scale vectors), else 1
  int64_t rows_per_wg;
  int64_t ranges;          // workgroups along the rows of a class
};

DxPlan plan(const GemmArgs &g)
{
  DxPlan p{false, 0, 0, 1, 0, 0};
  if (g.offsets || g.M < 1 || g.M > 16 || (g.w.kind != CAIFX_W_INT8 && g.w.kind != CAIFX_W_INT4_GROUP)) return p;
  if (g.K % kDxSlab != 0 || g.N < 1 || g.N > (int64_t{1} << 30) || g.K > (int64_t{1} << 30)) return p;
  if (g.w.kind == CAIFX_W_INT4_GROUP) {
    // groups of 128 or more (a power of two): a slab of 128 columns has one scale per row.  (The size query
    // comes without a group size and is answered for such groups.)
    const int gs = g.w.group_size;
    if (gs != 0 && (gs < kDxSlab || (gs & (gs - 1)) != 0)) return p;
    p.group_shift = gs != 0 ? __builtin_ctz(static_cast<unsigned>(gs)) : 7;
  } else if (g.w.scales && g.w.scale_period > 1) {
    const int64_t P = g.w.scale_period;
    if (P > (int64_t{1} << 30)) return p;
    int64_t a = g.K % P == 0 ? P : g.K % P, b = P;       // V = P / gcd(K mod P, P)
    while (b) {
      const int64_t t = a % b;
      a = b;
      b = t;
    }
    const int64_t V = P / a;
    if (V > 64 || V * kDxPassRows > g.N) return p;       // too many classes, or too few rows in each
    p.V = static_cast<int>(V);
    p.period = static_cast<int>(P);
  } else if (g.w.scales) {
    p.period = 1;
  }
  const int64_t slabs = g.K / kDxSlab;
  static const int cus = compute_units();
  const int64_t rows_class = (g.N + p.V - 1) / p.V;                 // of the largest class
  int64_t ranges = (cus + slabs * p.V - 1) / (slabs * p.V);
  const int64_t most = (rows_class + kDxPassRows - 1) / kDxPassRows;      // every workgroup gets at least one full pass
  if (ranges > most) ranges = most;
  if (ranges < 1) ranges = 1;
  int64_t rows = (rows_class + ranges - 1) / ranges;
  rows = (rows + kDxWaveRows - 1) / kDxWaveRows * kDxWaveRows;
  p.rows_per_wg = rows;
  p.ranges = (rows_class + rows - 1) / rows;
  p.ok = slabs <= 0x7fffffff && p.ranges * p.V <= 65535;
  return p;
}

}  // namespace

static size_t plan_bytes(const GemmArgs &g)
{
  const DxPlan p = plan(g);
  if (!p.ok || p.ranges * p.V < 2) return 0;
  return static_cast<size_t>(p.ranges * p.V) * static_cast<size_t>(g.M) * static_cast<size_t>(g.K) * sizeof(float);
}

size_t dxrows_workspace_bytes(const GemmArgs &g)
{
  size_t bytes = plan_bytes(g);
  if (g.w.kind == CAIFX_W_INT8 && !g.w.scales) {
    // a size query knows no scales: also cover a vector of one scale per output feature (period N), the usual
    // int8 layout, whose residue classes each bring their own partial sums
    GemmArgs c = g;
    c.w.scales = &c;              // any non-null address; only its presence is looked at
    c.w.scale_period = g.N;
    const size_t per_feature = plan_bytes(c);
    if (per_feature > bytes) bytes = per_feature;
  }
  return bytes;
}

int dxrows_backward(const GemmArgs &g, hipStream_t s)
{
  const DxPlan p = plan(g);
  if (!p.ok) return CAIFX_ERR_UNSUPPORTED;
  const bool int4 = g.w.kind == CAIFX_W_INT4_GROUP;
  if (int4 && (!g.w.scales || g.w.group_size == 0)) return CAIFX_ERR_UNSUPPORTED;
  if (!aligned_to(g.w.q, 8) || (g.w.scales && !aligned_to(g.w.scales, int4 ? 2 : 4))) return CAIFX_ERR_UNSUPPORTED;
  const bool split = p.ranges * p.V > 1;
  if (split && (!g.workspace || !aligned_to(g.workspace, 4) || g.workspace_bytes < dxrows_workspace_bytes(g)))
    return CAIFX_ERR_UNSUPPORTED;
  DxArgs a{};
  a.wq = static_cast<const int8_t *>(g.w.q);
  a.scales = g.w.scales;
  a.dy = g.x;
  a.dx = g.y;
  a.M = static_cast<int>(g.M);
  a.y_dtype = g.y_dtype;
  a.N = g.N;
  a.K = g.K;
  a.period = p.period;
  a.group_shift = p.group_shift;
  a.rows_per_wg = p.rows_per_wg;
  a.V = p.V;
  a.ranges = static_cast<int>(p.ranges);
  a.partial = split ? static_cast<float *>(g.workspace) : nullptr;
  const dim3 grid(static_cast<unsigned>(g.K / kDxSlab), static_cast<unsigned>(p.ranges * p.V));
  const size_t lds = static_cast<size_t>(kDxWaves) * 8 * 4 * 64 * sizeof(float);
  const int st = g.compute_dtype == CAIFX_F32 ? launch_ct<float>(a, int4, g.x_dtype, grid, lds, s)
                 : g.compute_dtype == CAIFX_BF16 ? launch_ct<bf16_t>(a, int4, g.x_dtype, grid, lds, s)
                                                 : launch_ct<f16_t>(a, int4, g.x_dtype, grid, lds, s);
  if (st != CAIFX_OK || !split) return st;
  return splitk_reduce(a.partial, static_cast<int>(p.ranges * p.V), g.M * g.K, g.y, g.y_dtype, nullptr, s);
}

}  // namespace caifx
