// Input gradient for a handful of rows (M <= 16): dX[M,K] = dY[M,N] * W[N,K] with W stored as int8 codes, memory
// bound on the weight stream like the decode forward, but with the reduction running down the weight's rows.
//
// The 16-bit and integer matrix instructions hold several consecutive reduction elements of one column per lane,
// here several weight rows of one column, while a weight row is stored along k.  v_mfma_f32_16x16x16 (bf16 / fp16)
// holds four: lane (j = lane % 16, q = lane / 16) loads 8 consecutive codes of four rows at k = k0 + 8j (four
// 8-byte loads, row 4q + i of the stage's 16 for load i; which rows meet in one instruction is free as long as
// both operands agree), and code position b of the four loads is the B operand of matrix instruction b, whose 16
// columns are then k0 + 8*col + b: no transposition, the byte (or nibble) is picked when the code is converted.
// The A operand is dY[m = j][those four rows].  Eight instructions consume a stage of four loads per lane.
//   * 16-bit compute type: dY is in that type (or rounded to it first, as the layer's cast of its input does), int8
//     codes are exact in it and the weight's scale is applied to the finished column, so the weight is never rounded
//     to the compute type (the reference rounds code*scale first; results differ by that rounding, a few 1e-3 of the
//     largest output for bf16).  int4 codes meet their scale before the product, code * scale rounded once to the
//     compute type: the reference's operand.
//   * fp32 compute type: dY (times the int4 scale) is cut into three bf16 pieces that add up to it, the codes are
//     exact in bf16, and three instructions per code position form the fp32 products (1e-7 of the largest output).
// The scale of an int8 column must not depend on the weight row among the rows a workgroup visits: scale index
// (n*K + k) mod period with K a multiple of the period (the per-output-channel scales of a square weight), one
// scale, none, or any period with the rows split into residue classes (see DxArgs::V).
// Packed int4 codes come in groups of 128 or more: a slab of 128 columns lies inside one group, so a row has one
// scale per slab (fp32 compute: it multiplies the row's gradient on its way into the A operand).
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
// 8-byte weight loads per stage of a wave's ring (the four rows of one matrix instruction) and stages.  Three
// stages measured slower than two at every shape (16 rows of int8: 12.1 -> 13.8 us at N = K = 4096, 22.2 -> 22.8 at
// N = 4096 / K = 14336, 24.1 -> 25.0 at N = 14336 / K = 4096; int4 21.8 -> 23.3).
// matrix instructions' worth of rows (four each) a lane loads per stage; two measured slower or equal at every shape
// (16 rows of int8, N = K = 4096: 11.2 -> 14.8 us; int4, N = 4096 / K = 14336: 21.7 -> 25.0)
constexpr int kDxGroups = 1;
constexpr int kDxIter = 4 * kDxGroups;
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
  int staged_pitch;        // GRAD_STAGED: elements per gradient row of the piece of dY kept in LDS
};

// XT: type of dY in memory; CT: compute type dY is rounded to first, as the layer's cast of its input does.
// kInt4: packed int4 codes; a lane's 8 codes are one dword, and the scale of (row, group) multiplies the row's
// gradient on its way into the A operand (the slab's 128 columns share the group).
// kGrad: how a lane gets its four gradient values of a stage (rows 4q .. 4q+3 of the stage's 16).  A wave's gradient
// load touches 16 cache lines, one per gradient row, whatever its width, so four scalar loads per stage cost the
// L1 four times what the weight loads do.
//   GRAD_VECTOR  one load of four: the rows are neighbours in memory (no residue classes) and the vector is aligned
//   GRAD_STAGED  residue classes put the rows V columns apart: the workgroup first copies its class's piece of dY
//                into LDS (behind the first weight requests, which are in flight meanwhile) and reads four from there
//   GRAD_SCALAR  four loads (whatever the other two do not take)
enum { GRAD_SCALAR = 0, GRAD_VECTOR = 1, GRAD_STAGED = 2 };
template <typename XT, typename CT, bool kInt4, int kGrad>
__global__ __launch_bounds__(kDxThreads) void dxrows_kernel(DxArgs a)
{
  constexpr bool kVecA = kGrad == GRAD_VECTOR;
  // [16 waves][8 codes][4][64] partial tiles, then [16][128] sums; GRAD_STAGED: before those, the gradient piece
  extern __shared__ __attribute__((aligned(16))) float tiles[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int j = lane & 15;
  const int q = lane >> 4;
  // Packed int4: a slab's 128 columns are half a cache line of every weight row, and the other half belongs to the
  // neighbouring slab.  Workgroups go to the 8 XCDs (each with its own L2) in turn by their linear id, so neighbours
  // would fetch every line into two L2s; slabs 2p and 2p + 1 are therefore given to workgroups 8 apart (the same
  // XCD, dispatched together), in blocks of 16 slabs, when the grid's width keeps that pairing (a multiple of 8).
  int slab = blockIdx.x;
  if constexpr (kInt4) {
    if ((gridDim.x & 7) == 0 && slab < static_cast<int>(gridDim.x & ~15u)) {
      const int t = slab >> 4, h = (slab >> 3) & 1, x = slab & 7;
      slab = 16 * t + 2 * x + h;
    }
  }
  const int64_t k0 = static_cast<int64_t>(slab) * kDxSlab;
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
  struct alignas(kDxIter * sizeof(XT) > 16 ? 16 : kDxIter * sizeof(XT)) XT4 {      // a lane's gradient values of a stage
    XT v[kDxIter];
  };
  uint32_t keep[kDxStages][kDxIter];     // all ones where the row and the gradient row exist, else 0
  // GRAD_STAGED: staged[m][i - n_lo] for the rows i of this workgroup's range, zero past the range's end; the row
  // pitch is 16 bytes past a multiple of 256, so the 16 gradient rows of one pass of a read use different banks
  const int staged_pitch = a.staged_pitch;          // elements
  XT *staged = reinterpret_cast<XT *>(tiles);
  auto issue_a = [&](int st, int64_t base) {
    if constexpr (kVecA) {        // V == 1: rows base + 4q .. + 3 are four consecutive gradient columns
      const int64_t n4 = base + kDxIter * q;
      const XT4 g4 = *reinterpret_cast<const XT4 *>(dy + (n4 + kDxIter <= a.N ? n4 : a.N - kDxIter));       // past the end: masked below
#pragma unroll
      for (int it = 0; it < kDxIter; ++it) av[st][it] = g4.v[it];
    } else if constexpr (kGrad == GRAD_STAGED) {
      int64_t i4 = base - n_lo + kDxIter * q;
      if (i4 > staged_pitch - kDxIter) i4 = staged_pitch - kDxIter;       // passes past the range read the zeros at its end
      const XT4 g4 = *reinterpret_cast<const XT4 *>(staged + j * staged_pitch + i4);
#pragma unroll
      for (int it = 0; it < kDxIter; ++it) av[st][it] = g4.v[it];
    }
  };
  auto issue = [&](int st, int64_t base) {
#pragma unroll
    for (int it = 0; it < kDxIter; ++it) {
      const int64_t n = base + kDxIter * q + it;
      const int64_t nn = cls + a.V * (n < n_hi ? n : n_hi - 1);          // rows past the range: a valid address, a zero gradient
      if constexpr (kInt4) {
        w[st][it][0] = *reinterpret_cast<const uint32_t *>(wcol + nn * row_bytes);
        ws[st][it] = s16[(nn * a.K + k0) >> a.group_shift];
      } else {
        w[st][it] = *reinterpret_cast<const u32x2_t *>(wcol + nn * row_bytes);
      }
      if constexpr (kGrad == GRAD_SCALAR) av[st][it] = dy[nn];
      // (a mask on the bits, not a conditional expression: the compiler turns that into a load under a branch
      // with a full wait behind it)
      keep[st][it] = static_cast<uint32_t>(-static_cast<int>((n < n_hi) & row_live));
    }
  };
  // 16-bit compute types: one v_mfma_f32_16x16x16 per code position takes the stage's four rows at once.  Its lanes
  // hold four consecutive reduction elements; which weight rows those are is free as long as both operands agree,
  // so element e of lane (j, q) is row 4q + e of the stage: the loads above as they are.  The gradient is in the
  // compute type already and an int8 code is exact in it, so the sums are those of the fp32 form; an int4 code meets
  // its scale on this side, code * scale rounded once to the compute type: the reference's dequantised weight.
  auto multiply16 = [&](int st) {
   if constexpr (sizeof(CT) == 2) {
    typedef short short4_t __attribute__((ext_vector_type(4)));
    typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int grp = 0; grp < kDxGroups; ++grp) {
      float g[4];
#pragma unroll
      for (int e = 0; e < 4; ++e)
        g[e] = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, to_f32<XT>(av[st][4 * grp + e])) & keep[st][4 * grp + e]);
      u32x2_t av2;
      av2[0] = pack2<CT>(g[0], g[1]);
      av2[1] = pack2<CT>(g[2], g[3]);
      float c[4][8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int it = 4 * grp + e;
        if constexpr (kInt4) {
          dequant_int4x8(w[st][it][0], to_f32(ws[st][it]), c[e]);
        } else {
          float lo[4], hi[4];
          int8x4_to_f32(w[st][it][0], lo);
          int8x4_to_f32(w[st][it][1], hi);
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            c[e][b] = lo[b];
            c[e][4 + b] = hi[b];
          }
        }
      }
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        u32x2_t bv;
        bv[0] = pack2<CT>(c[0][b], c[1][b]);
        bv[1] = pack2<CT>(c[2][b], c[3][b]);
        if constexpr (dtype_code<CT>::value == CAIFX_BF16)
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, av2), __builtin_bit_cast(short4_t, bv), acc[b], 0, 0, 0);
        else
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4_t, av2), __builtin_bit_cast(half4_t, bv), acc[b], 0, 0, 0);
      }
    }
   }
  };
  // fp32 compute type: the gradient (times the int4 scale) is cut into three bf16 pieces, g = h + m + l to the last
  // bit of its mantissa or better (each piece is the rounded remainder of the one before, and the remainders are
  // exact), the codes are exact in bf16, so three v_mfma_f32_16x16x16 per code position form the same fp32 products
  // as 32 v_mfma_f32_16x16x4_f32 would, in a third of the matrix time.
  auto multiply_split = [&](int st) {
    typedef short short4_t __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int grp = 0; grp < kDxGroups; ++grp) {
      float h[4], m[4], l[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int it = 4 * grp + e;
        float g = to_f32<XT>(av[st][it]);
        if constexpr (kInt4) g *= to_f32(ws[st][it]);
        g = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, g) & keep[st][it]);
        h[e] = round_through<bf16_t>(g);
        const float r1 = g - h[e];
        m[e] = round_through<bf16_t>(r1);
        l[e] = r1 - m[e];               // rounded to bf16 by the pack below
      }
      u32x2_t ah, am, al;
      ah[0] = pack2<bf16_t>(h[0], h[1]);
      ah[1] = pack2<bf16_t>(h[2], h[3]);
      am[0] = pack2<bf16_t>(m[0], m[1]);
      am[1] = pack2<bf16_t>(m[2], m[3]);
      al[0] = pack2<bf16_t>(l[0], l[1]);
      al[1] = pack2<bf16_t>(l[2], l[3]);
      float c[4][8];
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int b = 0; b < 8; ++b)
          c[e][b] = static_cast<float>(kInt4 ? static_cast<int>(w[st][4 * grp + e][0] << (28 - 4 * b)) >> 28
                                             : static_cast<int>(w[st][4 * grp + e][b >> 2] << (24 - 8 * (b & 3))) >> 24);
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        u32x2_t bv;
        bv[0] = pack2<bf16_t>(c[0][b], c[1][b]);
        bv[1] = pack2<bf16_t>(c[2][b], c[3][b]);
        const short4_t bb = __builtin_bit_cast(short4_t, bv);
        // smallest piece first
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, al), bb, acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, am), bb, acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, ah), bb, acc[b], 0, 0, 0);
      }
    }
  };
  auto multiply = [&](int st) {
    if constexpr (sizeof(CT) == 2) {
      multiply16(st);
      return;
    } else {
      multiply_split(st);
    }
  };
  int64_t base = n_lo + static_cast<int64_t>(wave) * kDxWaveRows;
  // (the fences keep the compiler from sinking a stage's loads down to their first use, which it otherwise does
  // to save registers, with a full wait in front of every multiplication)
#pragma unroll
  for (int st = 0; st < kDxStages - 1; ++st) issue(st, base + st * kDxPassRows);
  if constexpr (kGrad == GRAD_STAGED) {
    // the piece of dY this workgroup's rows meet: 16 gradient rows (zero from M on) x the range's rows of the class
    // (eight loads at a time per thread, all issued before the first is stored: one at a time the copy would take
    // a memory round trip per element)
    const XT *src = static_cast<const XT *>(a.dy) + cls + a.V * n_lo;
    const int64_t last = (n_hi - n_lo - 1) * a.V;            // offset of the range's last row
    for (int i0 = 0; i0 < staged_pitch; i0 += kDxThreads) {
      const int i = i0 + static_cast<int>(threadIdx.x);
      const int64_t off = static_cast<int64_t>(i) * a.V;
      const XT *col = src + (off < last ? off : last);
#pragma unroll
      for (int m0 = 0; m0 < 16; m0 += 8) {
        XT v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = col[static_cast<int64_t>(m0 + u < a.M ? m0 + u : a.M - 1) * a.N];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (i < staged_pitch) staged[(m0 + u) * staged_pitch + i] = (m0 + u < a.M && n_lo + i < n_hi) ? v[u] : from_f32<XT>(0.0f);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int st = 0; st < kDxStages - 1; ++st) issue_a(st, base + st * kDxPassRows);
  for (; base < n_hi; base += kDxStages * kDxPassRows) {       // the same trip count for every lane of a wave
#pragma unroll
    for (int st = 0; st < kDxStages; ++st) {
      issue((st + kDxStages - 1) % kDxStages, base + (st + kDxStages - 1) * kDxPassRows);
      issue_a((st + kDxStages - 1) % kDxStages, base + (st + kDxStages - 1) * kDxPassRows);
      __builtin_amdgcn_sched_barrier(0);
      multiply(st);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  if constexpr (kGrad == GRAD_STAGED) __syncthreads();      // the partial tiles go where other waves may still read gradients
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

template <typename XT, typename CT, bool kInt4>
int launch_vec(const DxArgs &a, dim3 grid, size_t lds, hipStream_t s)
{
  // one vector load per stage for the gradient when its four values are neighbours and the vector is aligned;
  // with residue classes the workgroup's piece of dY goes through LDS when it fits where the partial tiles go later
  const size_t vbytes = kDxIter * sizeof(XT) > 16 ? 16 : kDxIter * sizeof(XT);
  const bool vec = a.V == 1 && a.N % kDxIter == 0 && a.N >= kDxIter && aligned_to(a.dy, vbytes);
  if (vec) {
    hipLaunchKernelGGL((dxrows_kernel<XT, CT, kInt4, GRAD_VECTOR>), grid, dim3(kDxThreads), lds, s, a);
    return launch_status();
  }
  if (a.V > 1 && a.M > 1) {
    // pitch: the range's rows, rounded up to 16 bytes past a multiple of 256
    const int64_t per256 = 256 / static_cast<int64_t>(sizeof(XT));
    const int64_t pitch = (a.rows_per_wg + per256 - 1) / per256 * per256 + 16 / static_cast<int64_t>(sizeof(XT));
    const size_t piece = 16 * static_cast<size_t>(pitch) * sizeof(XT);
    if (piece <= 160 * 1024) {
      DxArgs b = a;
      b.staged_pitch = static_cast<int>(pitch);
      hipLaunchKernelGGL((dxrows_kernel<XT, CT, kInt4, GRAD_STAGED>), grid, dim3(kDxThreads), piece > lds ? piece : lds, s, b);
      return launch_status();
    }
  }
  hipLaunchKernelGGL((dxrows_kernel<XT, CT, kInt4, GRAD_SCALAR>), grid, dim3(kDxThreads), lds, s, a);
  return launch_status();
}

template <typename CT, bool kInt4>
int launch_xt(const DxArgs &a, int x_dtype, dim3 grid, size_t lds, hipStream_t s)
{
  if (x_dtype == CAIFX_F32) return launch_vec<float, CT, kInt4>(a, grid, lds, s);
  if (x_dtype == CAIFX_BF16) return launch_vec<bf16_t, CT, kInt4>(a, grid, lds, s);
  return launch_vec<f16_t, CT, kInt4>(a, grid, lds, s);
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
  // Row ranges per class: one workgroup fills a compute unit (its partial tiles take 128 KB of LDS), so the launch
  // runs in rounds of `cus` workgroups, each round as long as a range plus what a workgroup spends before and after
  // its rows (about 470 rows' worth of streaming).  The fewest rounds of the shortest ranges win: 16 rows, N = 4096,
  // K = 14336, int8 in two classes (224 workgroups per range): one range 22.7 us, two 27.3, three 33.6; int4 (112):
  // one 32.8, two 21.9, three 31.0.
  const int64_t most = (rows_class + kDxPassRows - 1) / kDxPassRows;      // every workgroup gets at least one full pass
  const int64_t items = slabs * p.V;
  int64_t ranges = 1;
  int64_t best = -1;
  for (int64_t r = 1; r <= most && r <= 64; ++r) {
    const int64_t rounds = (items * r + cus - 1) / cus;
    const int64_t cost = rounds * (rows_class / r + 470);
    if (best < 0 || cost < best) {
      best = cost;
      ranges = r;
    }
  }
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
