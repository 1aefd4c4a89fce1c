// Decode path for a handful of activation rows (2 <= M <= 16): Y[M,N] = X[M,K] * W[N,K]^T with W
// stored int8 or packed int4, memory bound on the weight stream.
//
// The matrix cores do the dot products with the activation rows as the 16 rows of the A operand
// of v_mfma_f32_16x16x32 (rows past M are zero) and 16 weight rows as the columns of B, so the
// cost per weight byte does not depend on M.  A workgroup is 16 waves; wave w owns the k range
// [w*GPW*128, (w+1)*GPW*128) for every weight row the workgroup visits and keeps the matching
// slice of X in registers, already laid out as A operands, for the whole kernel.  Per block of 16
// weight rows a lane (j = lane%16, q = lane/16) loads 16 bytes of row j:
//   int4: 32 codes at k = group*128 + q*32; dword t of the load feeds MFMA t, its nibbles unpack
//         pairwise (order 0,4,1,5,2,6,3,7, X is stored in the same order) to the compute dtype as
//         OFFSET + (code + 8) with one AND/XOR each; the fp32 sum over a 128-k group is corrected by
//         OFFSET' * sum(x) and multiplied by the group's scale ("post-scaling": the weight is never
//         rounded to the compute dtype, so results differ from the dequantise-then-cast reference
//         by that rounding, a few 1e-3 of the largest output);
//   int8: 16 codes at k = group*128 + half*64 + q*16, fed to v_mfma_i32_16x16x64_i8 exactly as loaded
//         (no unpacking arithmetic).  The scales are folded into the activations instead: a scale
//         vector of period P is addressed by the flat index n*K + k modulo P; rows n with equal
//         n mod V, V = P / gcd(K mod P, P), see the same scales along k, so a workgroup only visits
//         rows of one residue class, stages that class's K scales in LDS once and forms
//         x'[m][k] = x[m][k] * scale[k] in fp32.  x' is split into three signed 8-bit digit planes
//         relative to a power-of-two unit per activation row and wave (x' ~ unit * (d0 + d1/256 +
//         d2/65536), |d0| <= 32, error <= unit * 2^-17); the three exact int32 sums are combined in fp32 per block.
//         The weight is therefore never rounded to the compute dtype: results differ from the
//         dequantise-then-cast reference by that rounding (a few 1e-3 of the largest output), like int4.
// After the last group every wave holds a partial 16x16 tile; the 16 partials are added through LDS
// in a fixed order (results do not depend on scheduling) and written as Y[token][row].
#include "caifx_internal.hpp"

namespace caifx {
namespace {

template <typename CT> struct Mfma16;
template <> struct Mfma16<bf16_t> {
  typedef bf16x8_t vec_t;
  static constexpr uint32_t kMagic = 0x43084308u;      // bf16 128 + (code ^ 8) in both halves
  static constexpr float kOffset = 136.0f;             // 128 + 8
  static __device__ __forceinline__ floatx4_t run(vec_t a, vec_t b, floatx4_t c)
  {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma16<f16_t> {
  typedef f16x8_t vec_t;
  static constexpr uint32_t kMagic = 0x64086408u;      // fp16 1024 + (code ^ 8)
  static constexpr float kOffset = 1032.0f;
  static __device__ __forceinline__ floatx4_t run(vec_t a, vec_t b, floatx4_t c)
  {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

constexpr int kMbWaves = 16;
constexpr int kMbThreads = kMbWaves * 64;
constexpr int kPartialFloats = kMbWaves * 4 * 64;     // one buffer of per-wave partial tiles

struct MbArgs {
  const uint8_t *wq;
  const void *scales;
  const void *x;
  void *y;
  int M;
  int y_dtype;
  int64_t N, K;
  int groups;            // K / 128
  int group_shift;       // int4: log2(group_size)
  int period;            // int8: length of the scale vector, 0 = one scale (or none)
  int V;                 // residue classes the rows are split into (1 unless period > 0)
  int blocks_per_class;  // gridDim.x = blocks_per_class * V
  int scale_step;        // int8 scale vector: 1024 mod period (staging stride of the workgroup)
  // K beyond one workgroup's reach: blockIdx.y takes the k range [y * slice_groups * 128, ...) and writes its
  // share of the sums as fp32 to partial + y * M * N; a second launch adds the shares in a fixed order
  int slice_groups;      // 128-k groups per slice (= groups when there is one slice)
  float *partial;        // null with one slice
};

// 8 consecutive activations as compute-dtype values
template <typename CT, typename XT>
__device__ __forceinline__ typename Mfma16<CT>::vec_t load_x8(const XT *p)
{
  typedef typename Mfma16<CT>::vec_t vec_t;
  if constexpr (dtype_code<XT>::value == dtype_code<CT>::value) {
    return *reinterpret_cast<const vec_t *>(p);
  } else if constexpr (sizeof(XT) == 4) {
    const floatx4_t a = *reinterpret_cast<const floatx4_t *>(p);
    const floatx4_t b = *reinterpret_cast<const floatx4_t *>(p + 4);
    vec_t v;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[i] = from_f32<CT>(a[i]);
      v[4 + i] = from_f32<CT>(b[i]);
    }
    return v;
  } else {
    const u32x4_t raw = *reinterpret_cast<const u32x4_t *>(p);
    const XT *h = reinterpret_cast<const XT *>(&raw);
    vec_t v;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = from_f32<CT>(to_f32<XT>(h[i]));
    return v;
  }
}

__device__ __forceinline__ void store_out(void *y, int y_dtype, int64_t o, float v)
{
  if (y_dtype == CAIFX_F32) static_cast<float *>(y)[o] = v;
  else if (y_dtype == CAIFX_BF16) static_cast<bf16_t *>(y)[o] = from_f32<bf16_t>(v);
  else static_cast<f16_t *>(y)[o] = from_f32<f16_t>(v);
}

// (a & mask) | base in one instruction (the compiler splits it in two when both constants are literals)
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t base)
{
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(base));
  return r;
}

typedef int i32x4_t __attribute__((ext_vector_type(4)));

// the low bytes of four words as one word (a in byte 0)
__device__ __forceinline__ uint32_t pack_low_bytes(int a, int b, int c, int d)
{
  const uint32_t ab = __builtin_amdgcn_perm(static_cast<uint32_t>(b), static_cast<uint32_t>(a), 0x0c0c0400u);
  const uint32_t cd = __builtin_amdgcn_perm(static_cast<uint32_t>(d), static_cast<uint32_t>(c), 0x0c0c0400u);
  return __builtin_amdgcn_perm(cd, ab, 0x05040100u);
}

// row blocks between two additions of the waves' partial tiles
constexpr int mb_reduce_blocks(bool int4, int mt) { return int4 && mt == 1 ? 4 : 2; }

constexpr int kSegBlocks = 16;                         // row blocks between two flushes of the output staging buffer
constexpr int kSegRows = kSegBlocks * 16;

// GPW: 128-k groups per wave (K <= 16 * GPW * 128); 1 and 2 fit the 128 registers of a 1024-thread workgroup
//
// Memory requests are arranged so that the compiler can count them: the weight loads are never
// behind a branch (lanes past the last row re-read the last row, row blocks past the end read the
// first bytes of the weight) and no global store happens between them (results are staged in LDS
// and written once per kSegRows rows).  A wait for one block of the ring then leaves the younger
// block in flight instead of draining the queue.
// kF32 (int8 only): fp32 compute type.  The activations are not rounded to a 16-bit type: the digit planes are cut
// from x * scale in fp32, read from memory in both passes over them instead of being kept in registers (CT then
// only names a vector type nothing is stored in).
// MT: tiles of 16 activation rows that share one pass over the weight (M <= 16 * MT); every weight fragment is
// unpacked once and multiplied with each tile's operands.
// wq / scales: the weight; xrows / yrows: the first of the M activation and result rows; slice: which part of
// the reduction (see MbArgs).  Every thread of the workgroup makes the same calls (the body has barriers).
// D: row blocks a wave keeps requested (1 or 2; the launch code picks by measurement)
template <typename CT, typename XT, bool kInt4, int GPW, bool kF32, int MT = 1, int D = 2>
__device__ __forceinline__ void mblock_body(const MbArgs &a, const uint8_t *wq, const void *scales, const void *xrows,
                                            void *yrows, int M, int slice)
{
  static_assert(!(kF32 && kInt4), "the fp32 compute type is for int8 storage");
  typedef typename Mfma16<CT>::vec_t vec_t;
  constexpr int LPG = kInt4 ? 1 : 2;           // 16-byte loads per lane per 128-k group
  constexpr int LPR = GPW * LPG;               // ... per block of 16 weight rows
  constexpr int RBB = mb_reduce_blocks(kInt4, MT);      // row blocks between two reductions (a multiple of D, divides kSegBlocks)
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float *partial = reinterpret_cast<float *>(smem);      // [RBB][MT][16 waves][4][64]
  float *ybuf = partial + RBB * MT * kPartialFloats;     // [16 * MT activation rows][kSegRows]
  float *svec = ybuf + 16 * MT * kSegRows;               // int8: the scale vector of this slice [slice k]; int4 with
                                                         // MT > 1: the group-sum corrections [MT][GPW][16 waves][16]

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int j = lane & 15;        // weight row within the block (B column) / activation row (A row)
  const int q = lane >> 4;        // quarter of the 32-wide k step
  const int cls = blockIdx.x / a.blocks_per_class;
  const int bc = blockIdx.x - cls * a.blocks_per_class;
  const int64_t rows_class = (a.N - cls + a.V - 1) / a.V;          // rows n = cls + V*i, i < rows_class
  // every workgroup of a class takes the same number of consecutive rows (the last block of 16 may
  // be partly masked): equal bytes per compute unit matter more than full MFMA tiles
  const int64_t per_block = (rows_class + a.blocks_per_class - 1) / a.blocks_per_class;
  const int64_t i_lo = bc * per_block;
  const int64_t i_hi = i_lo + per_block < rows_class ? i_lo + per_block : rows_class;
  const int nrb = i_hi > i_lo ? static_cast<int>((i_hi - i_lo + 15) / 16) : 0;
  if (nrb == 0) return;           // the whole workgroup; nothing has been started yet
  const int g0 = wave * GPW;
  const int kbase = slice * a.slice_groups * 128;          // first k of this workgroup's slice
  const int groups = a.groups - slice * a.slice_groups < a.slice_groups ? a.groups - slice * a.slice_groups
                                                                               : a.slice_groups;
  const f16_t *s16 = static_cast<const f16_t *>(scales);
  const float *s32 = static_cast<const float *>(scales);

  u32x4_t w[D][LPR];
  f16_t sc[D][GPW];
  auto issue = [&](int d, int rb) {
    int64_t i = i_lo + static_cast<int64_t>(rb) * 16 + j;
    if (i >= i_hi) i = i_hi - 1;                                   // masked lanes: their columns of the tile are never stored
    const int64_t f0 = (rb < nrb ? (cls + a.V * i) * a.K : 0) + kbase;       // (wave uniform) past the end: the first weight row
#pragma unroll
    for (int g = 0; g < GPW; ++g) {
      const int gg = g0 + g < groups ? g0 + g : groups - 1;   // waves without a k range compute on zero activations
      const int64_t f = f0 + gg * 128;
      if constexpr (kInt4) {
        w[d][g] = *reinterpret_cast<const u32x4_t *>(wq + (f >> 1) + q * 16);
        sc[d][g] = s16[f >> a.group_shift];
      } else {
        w[d][2 * g] = *reinterpret_cast<const u32x4_t *>(wq + f + q * 16);
        w[d][2 * g + 1] = *reinterpret_cast<const u32x4_t *>(wq + f + 64 + q * 16);
      }
    }
  };
  // Order of the requests: this wave's slice of X and (int8) the scale vector first, they come from
  // L2 and are needed first; then the first weight blocks.  Loads return in order, so the prologue
  // runs while the weights are still on their way from HBM.
  vec_t xa[MT][GPW][4];
  const XT *xg[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
    xg[mt] = static_cast<const XT *>(xrows) + static_cast<int64_t>(16 * mt + j < M ? 16 * mt + j : M - 1) * a.K + kbase;
  if constexpr (!kF32) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int g = 0; g < GPW; ++g) {
        const int gg = g0 + g < groups ? g0 + g : groups - 1;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int k = kInt4 ? gg * 128 + q * 32 + 8 * t : gg * 128 + (t >> 1) * 64 + q * 16 + 8 * (t & 1);
          xa[mt][g][t] = load_x8<CT, XT>(xg[mt] + k);
        }
      }
  }
  // int8 scale vector of this residue class: svec[k] = scales[(cls*K + k) mod period], K <= 4096
  float s_one = 1.0f;
  float sv[4] = {1.0f, 1.0f, 1.0f, 1.0f};     // without a scale vector the staged scales are 1
  if constexpr (!kInt4) {
    if (a.period > 0) {
      int idx = static_cast<int>((static_cast<int64_t>(cls) * a.K + kbase + threadIdx.x) % a.period);
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        sv[t] = s32[idx];
        idx += a.scale_step;
        if (idx >= a.period) idx -= a.period;
      }
    } else if (scales) {
      s_one = s32[0];
    }
  }
#pragma unroll
  for (int d = 0; d < D; ++d) issue(d, d);

  if constexpr (!kF32) {
    vec_t zero;
#pragma unroll
    for (int i = 0; i < 8; ++i) zero[i] = from_f32<CT>(0.0f);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int g = 0; g < GPW; ++g) {
        const bool live = g0 + g < groups && 16 * mt + j < M;
#pragma unroll
        for (int t = 0; t < 4; ++t) xa[mt][g][t] = live ? xa[mt][g][t] : zero;
      }
  }
  if constexpr (!kInt4) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int k = threadIdx.x + t * kMbThreads;
      if (k < groups * 128) svec[k] = sv[t];
    }
  }

  // int4: the nibbles unpack in the order 0,4,1,5,2,6,3,7, so X is stored that way; and
  // cor = OFFSET * (sum of x over each group) for the four activation rows this lane holds results of
  // (one tile keeps them in registers; with more tiles they wait in LDS, a wave reads back only what it wrote)
  float cor[MT == 1 ? GPW : 1][4];
  float *corbuf = svec + wave * 16;
  if constexpr (kInt4) {
    vec_t ones;
#pragma unroll
    for (int i = 0; i < 8; ++i) ones[i] = from_f32<CT>(1.0f);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int g = 0; g < GPW; ++g) {
        // the group sums come out of the matrix core in the layout of the results: X times a matrix of ones
        floatx4_t xsum = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const vec_t v = xa[mt][g][t];
          xsum = Mfma16<CT>::run(v, ones, xsum);
          vec_t p;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            p[2 * i] = v[i];
            p[2 * i + 1] = v[i + 4];
          }
          xa[mt][g][t] = p;
        }
        if constexpr (MT == 1) {
#pragma unroll
          for (int r = 0; r < 4; ++r) cor[g][r] = Mfma16<CT>::kOffset * xsum[r];
        } else if (j == 0) {
#pragma unroll
          for (int r = 0; r < 4; ++r) corbuf[(mt * GPW + g) * (kMbWaves * 16) + 4 * q + r] = Mfma16<CT>::kOffset * xsum[r];
        }
      }
    if constexpr (MT > 1) __syncthreads();
  }
  // int8: digit planes of x' = x * scale as A operands of the integer matrix core, dg[step][plane];
  // step t covers k = (g0 + t/2)*128 + (t%2)*64 + q*16 .. +16 of activation row j
  constexpr int kSteps = 2 * GPW;
  constexpr int kPlanes = 3;              // signed 8-bit digits: x' to 2^-21 of the largest |x'| of the row in this wave's k range
  i32x4_t dg[kInt4 ? 1 : MT][kInt4 ? 1 : kSteps][kPlanes];
  float ur[MT][4];            // unit of the activation rows 4q..4q+3 of each tile, which this lane holds results of
  bool poison[MT][4];         // those rows have a non-finite scaled activation in this wave's k range
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      ur[mt][r] = 1.0f;
      poison[mt][r] = false;
    }
  if constexpr (!kInt4) {
    __syncthreads();       // svec is complete
    // four consecutive x' values: quad c (0..3) of step t of tile mt
    auto xprime4 = [&](int mt, int t, int c, float (&v)[4]) {
      const int g = t >> 1;
      const int gg = g0 + g < groups ? g0 + g : groups - 1;
      if constexpr (kF32) {
        const bool live = g0 + g < groups && 16 * mt + j < M;
        const XT *px = xg[mt] + gg * 128 + (t & 1) * 64 + q * 16 + 4 * c;
        if constexpr (sizeof(XT) == 4) {
          const floatx4_t xv = *reinterpret_cast<const floatx4_t *>(px);
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = live ? xv[i] : 0.0f;
        } else {
          const u32x2_t raw = *reinterpret_cast<const u32x2_t *>(px);
          const XT *h = reinterpret_cast<const XT *>(&raw);
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = live ? to_f32<XT>(h[i]) : 0.0f;
        }
      } else {
        const vec_t xv = xa[mt][g][2 * (t & 1) + (c >> 1)];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = to_f32<CT>(xv[4 * (c & 1) + i]);
      }
      const floatx4_t sc4 = *reinterpret_cast<const floatx4_t *>(svec + gg * 128 + (t & 1) * 64 + q * 16 + 4 * c);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] *= sc4[i];
    };
    // One byte permute per pair of values and one per plane gather the bytes of four values.
    auto gather = [&](uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3, uint32_t sel) __attribute__((always_inline)) {
      const uint32_t lo = __builtin_amdgcn_perm(a1, a0, sel);
      const uint32_t hi = __builtin_amdgcn_perm(a3, a2, sel);
      return static_cast<int>(__builtin_amdgcn_perm(hi, lo, 0x05040100u));
    };
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      // first pass: x' = x * scale, kept in registers for the second pass; the largest |x'| and whether all are finite
      float xp[kSteps][16];
      float mx = 0.0f;
      bool finite = true;
#pragma unroll
      for (int t = 0; t < kSteps; ++t)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          float v[4];
          xprime4(mt, t, c, v);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            xp[t][4 * c + i] = v[i];
            mx = fmaxf(mx, fabsf(v[i]));                       // ignores a NaN
            finite = finite && fabsf(v[i]) <= 3.4028235e38f;    // false for NaN and infinities
          }
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16));
      mx = fmaxf(mx, __shfl_xor(mx, 32));      // over the four k quarters: row j's largest |x'| in this wave's k range
      // A NaN or an infinity among row j's scaled activations has no digits.  The reference's GEMM returns NaN or an
      // infinity in every output of that activation row; here this wave's share of them, and so their sum, is NaN.
      const int bad = (__ballot(!finite) >> j & 0x0001000100010001ull) != 0 ? 1 : 0;
      mx = bad ? 1.0f : mx;
#pragma unroll
      for (int r = 0; r < 4; ++r) poison[mt][r] = __shfl(bad, 4 * q + r) != 0;
      int e = 0;
      (void)frexpf(mx, &e);                     // mx = f * 2^e, f in [0.5, 1)
      const float unit = mx > 0.0f ? ldexpf(1.0f, e - 5) : 1.0f;    // |x'| / unit < 32
      const float inv16 = 65536.0f / unit;      // exact: a power of two
      // second pass: n = round(x' / unit * 2^16) sits in the low mantissa bits of b = x' * inv16 + 1.5 * 2^23
      // (|n| <= 2^21), and n = 2^16 d0 + 2^8 d1 + d2 with d1, d2 in [-128, 127]: d2 is byte 0 of b, d1 byte 1 of
      // b + 0x80, d0 byte 2 of b + 0x8080 less the 0x40 that the constant leaves there (adding 0xC00000 removes it).
#pragma unroll
      for (int t = 0; t < kSteps; ++t) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          uint32_t b0[4], b1[4], b2[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            b0[i] = __builtin_bit_cast(uint32_t, __builtin_fmaf(xp[t][4 * c + i], inv16, 12582912.0f));
            b1[i] = b0[i] + 0x80u;
            b2[i] = b0[i] + 0xC08080u;
          }
          dg[mt][t][0][c] = gather(b2[0], b2[1], b2[2], b2[3], 0x0c0c0602u);
          dg[mt][t][1][c] = gather(b1[0], b1[1], b1[2], b1[3], 0x0c0c0501u);
          dg[mt][t][2][c] = gather(b0[0], b0[1], b0[2], b0[3], 0x0c0c0400u);
        }
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) ur[mt][r] = __shfl(unit, 4 * q + r) * s_one;
    }
  }

  // The waves run freely through RBB blocks of 16 rows (no barrier in between, so one wave's
  // arithmetic overlaps another's wait for HBM), then the 16 partial tiles of each block are added
  // through LDS in a fixed order into the staging buffer.
  for (int seg0 = 0; seg0 < nrb; seg0 += kSegBlocks) {
    const int seg_end = seg0 + kSegBlocks < nrb ? seg0 + kSegBlocks : nrb;
    for (int base = seg0; base < seg_end; base += RBB) {
      floatx4_t tot[RBB][MT];
#pragma unroll
      for (int u = 0; u < RBB; ++u) {
        const int d = u % D;
        const int rb = base + u;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) tot[u][mt] = floatx4_t{0.0f, 0.0f, 0.0f, 0.0f};
        if (rb < nrb) {          // same for every thread of the workgroup
          if constexpr (kInt4) {
#pragma unroll
            for (int g = 0; g < GPW; ++g) {
              floatx4_t acc[MT];
#pragma unroll
              for (int mt = 0; mt < MT; ++mt) acc[mt] = floatx4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                // one xor turns the eight two's-complement nibbles into code + 8; every pair of
                // nibbles then takes a shift and one and-or to become OFFSET-biased values
                const uint32_t p = w[d][g][t] ^ 0x88888888u;
                constexpr uint32_t kBase = Mfma16<CT>::kMagic & 0xFFF0FFF0u;
                u32x4_t c4;
                c4[0] = and_or(p, 0x000F000Fu, kBase);
                c4[1] = and_or(p >> 4, 0x000F000Fu, kBase);
                c4[2] = and_or(p >> 8, 0x000F000Fu, kBase);
                c4[3] = and_or(p >> 12, 0x000F000Fu, kBase);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                  acc[mt] = Mfma16<CT>::run(xa[mt][g][t], *reinterpret_cast<const vec_t *>(&c4), acc[mt]);
              }
              const float sr = to_f32(sc[d][g]);
#pragma unroll
              for (int mt = 0; mt < MT; ++mt) {
                if constexpr (MT == 1) {
#pragma unroll
                  for (int r = 0; r < 4; ++r) tot[u][mt][r] = __builtin_fmaf(sr, acc[mt][r] - cor[g][r], tot[u][mt][r]);
                } else {
                  const floatx4_t cr = *reinterpret_cast<const floatx4_t *>(corbuf + (mt * GPW + g) * (kMbWaves * 16) + 4 * q);
#pragma unroll
                  for (int r = 0; r < 4; ++r) tot[u][mt][r] = __builtin_fmaf(sr, acc[mt][r] - cr[r], tot[u][mt][r]);
                }
              }
            }
          } else {
            i32x4_t s0[MT], s1[MT], s2[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) s0[mt] = s1[mt] = s2[mt] = i32x4_t{0, 0, 0, 0};
#pragma unroll
            for (int t = 0; t < kSteps; ++t) {
              const i32x4_t bw = __builtin_bit_cast(i32x4_t, w[d][t]);
#pragma unroll
              for (int mt = 0; mt < MT; ++mt) {
                s0[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(dg[mt][t][0], bw, s0[mt], 0, 0, 0);
                s1[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(dg[mt][t][1], bw, s1[mt], 0, 0, 0);
                s2[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(dg[mt][t][2], bw, s2[mt], 0, 0, 0);
              }
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                float v = static_cast<float>(s0[mt][r]);
                v = __builtin_fmaf(static_cast<float>(s1[mt][r]), 1.0f / 256.0f, v);
                v = __builtin_fmaf(static_cast<float>(s2[mt][r]), 1.0f / 65536.0f, v);
                tot[u][mt][r] = poison[mt][r] ? __builtin_nanf("") : v * ur[mt][r];
              }
          }
        }
        issue(d, rb + D);      // into the registers just consumed; the other block of the ring stays in flight
      }

      // tot[u][mt][r] = this wave's share of Y[activation row 16 mt + 4q + r][weight row j of block base+u]
#pragma unroll
      for (int u = 0; u < RBB; ++u)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int r = 0; r < 4; ++r) partial[(((u * MT + mt) * kMbWaves + wave) * 4 + r) * 64 + lane] = tot[u][mt][r];
      __syncthreads();
      for (int idx = threadIdx.x; idx < RBB * MT * 256; idx += kMbThreads) {
        const int um = idx >> 8;             // u * MT + mt
        const int r = (idx >> 6) & 3;
        const int l = idx & 63;
        float v = 0.0f;
#pragma unroll
        for (int wv = 0; wv < kMbWaves; ++wv) v += partial[((um * kMbWaves + wv) * 4 + r) * 64 + l];
        const int m = 16 * (um % MT) + 4 * (l >> 4) + r;
        ybuf[m * kSegRows + (base - seg0 + um / MT) * 16 + (l & 15)] = v;
      }
      __syncthreads();            // the next round overwrites the partial tiles; the flush reads ybuf
    }
    // flush: Y[m][cls + V*i] for the rows of this segment
    const int64_t i_seg = i_lo + static_cast<int64_t>(seg0) * 16;
    const int seg_rows = static_cast<int>(i_hi - i_seg < kSegRows ? i_hi - i_seg : kSegRows);
    float *part = a.partial ? a.partial + static_cast<int64_t>(slice) * M * a.N : nullptr;
    for (int idx = threadIdx.x; idx < M * seg_rows; idx += kMbThreads) {
      const int m = idx / seg_rows;
      const int r = idx - m * seg_rows;
      const int64_t o = static_cast<int64_t>(m) * a.N + cls + a.V * (i_seg + r);
      if (part) part[o] = ybuf[m * kSegRows + r];
      else store_out(yrows, a.y_dtype, o, ybuf[m * kSegRows + r]);
    }
  }
}

template <typename CT, typename XT, bool kInt4, int GPW, bool kF32 = false, int MT = 1, int D = 2>
__global__ __launch_bounds__(kMbThreads) void mblock_kernel(MbArgs a)
{
  mblock_body<CT, XT, kInt4, GPW, kF32, MT, D>(a, a.wq, a.scales, a.x, a.y, a.M, blockIdx.y);
}

// Token-sorted expert segments with few rows each (MoE decode): blockIdx.y is the expert, whose weight is streamed
// once per 16 rows of its segment; an expert without rows costs nothing.  The host only knows the total row
// count, so routing may hand one expert most of the rows: the 16-row passes of a segment are dealt out over
// blockIdx.z, and a long segment is worked on by gridDim.z times as many workgroups instead of gridDim.z times
// as long (its weight then comes from L2 after the first pass).
struct MbGroup {
  const int32_t *offsets;
  const void *const *wq_ptrs;
  const void *const *scales_ptrs;
  int64_t total_rows;
};
template <typename CT, typename XT, bool kInt4, int GPW>
__global__ __launch_bounds__(kMbThreads) void mblock_grouped_kernel(MbArgs a, MbGroup g)
{
  const int e = blockIdx.y;
  int lo, hi;
  segment_rows(g.offsets, e, g.total_rows, lo, hi);
  if (hi <= lo) return;
  const uint8_t *wq = static_cast<const uint8_t *>(g.wq_ptrs[e]);
  const void *scales = g.scales_ptrs ? g.scales_ptrs[e] : nullptr;
  const size_t ybytes = a.y_dtype == CAIFX_F32 ? 4 : 2;
  const int first = lo + 16 * static_cast<int>(blockIdx.z);
  for (int r = first; r < hi; r += 16 * static_cast<int>(gridDim.z)) {
    if (r > first) __syncthreads();      // the pass before has read its staging buffers
    mblock_body<CT, XT, kInt4, GPW, false>(a, wq, scales, static_cast<const XT *>(a.x) + static_cast<int64_t>(r) * a.K,
                                           static_cast<char *>(a.y) + static_cast<int64_t>(r) * a.N * ybytes,
                                           hi - r < 16 ? hi - r : 16, 0);
  }
}

int64_t gcd64(int64_t x, int64_t y)
{
  while (y) {
    const int64_t t = x % y;
    x = y;
    y = t;
  }
  return x;
}

// groups per wave that a kernel with MT tiles is built for: the operands of 32 rows (bf16 values or int8 digit
// planes) fit the 128 registers at one group per wave; with two, the int4 kernel spills 28-35 registers in its main loop
constexpr int mb_max_gpw(bool /*int4*/, int mt) { return mt == 1 ? 2 : 1; }

template <typename CT, typename XT, bool kInt4, bool kF32 = false>
int launch_gpw(const MbArgs &m, size_t lds, hipStream_t s)
{
  const dim3 grid(static_cast<unsigned>(m.blocks_per_class * m.V),
                  static_cast<unsigned>((m.groups + m.slice_groups - 1) / m.slice_groups));
  const int gpw = (m.slice_groups + kMbWaves - 1) / kMbWaves;
  if (m.M <= 16) {
    // One row block requested at a time instead of two, by measurement (K = 4096, N = 2048 ... 28672, times in us):
    // int4 with 4 rows 7.2 -> 6.6, 7.9 -> 7.1, 9.6 -> 9.1, 11.0 -> 10.6, 12.7 -> 12.4, 20.4 -> 19.7; with 16 rows
    // 9.0 -> 8.4, 9.4 -> 8.9, 11.3 -> 11.2, 12.8 -> 13.1, 14.7 -> 14.9, 23.0 -> 22.4, so two stay only for more than 8
    // rows with 33..64 weight rows per workgroup; int8 gains up to 32 weight rows per workgroup (10.8 -> 10.6,
    // 11.5 -> 11.35 at N = 4096) and loses 1.5 us beyond.
    const int64_t rows_class = (m.N + m.V - 1) / m.V;
    const int64_t rows_wg = (rows_class + m.blocks_per_class - 1) / m.blocks_per_class;
    const bool one_block = kInt4 ? (m.M <= 8 || rows_wg <= 32 || rows_wg > 64) : rows_wg <= 32;
    if (gpw > 2) return CAIFX_ERR_UNSUPPORTED;
    if (one_block) {
      if (gpw <= 1) hipLaunchKernelGGL((mblock_kernel<CT, XT, kInt4, 1, kF32, 1, 1>), grid, dim3(kMbThreads), lds, s, m);
      else hipLaunchKernelGGL((mblock_kernel<CT, XT, kInt4, 2, kF32, 1, 1>), grid, dim3(kMbThreads), lds, s, m);
    } else if (gpw <= 1) hipLaunchKernelGGL((mblock_kernel<CT, XT, kInt4, 1, kF32>), grid, dim3(kMbThreads), lds, s, m);
    else hipLaunchKernelGGL((mblock_kernel<CT, XT, kInt4, 2, kF32>), grid, dim3(kMbThreads), lds, s, m);
  } else {
    if (gpw <= 1) hipLaunchKernelGGL((mblock_kernel<CT, XT, kInt4, 1, kF32, 2>), grid, dim3(kMbThreads), lds, s, m);
    else if constexpr (mb_max_gpw(kInt4, 2) >= 2) {
      if (gpw <= 2) hipLaunchKernelGGL((mblock_kernel<CT, XT, kInt4, 2, kF32, 2>), grid, dim3(kMbThreads), lds, s, m);
      else return CAIFX_ERR_UNSUPPORTED;
    } else return CAIFX_ERR_UNSUPPORTED;
  }
  return launch_status();
}

template <typename CT, typename XT, bool kInt4>
int launch_grouped_gpw(const MbArgs &m, const MbGroup &g, int experts, size_t lds, hipStream_t s)
{
  // up to eight passes of a segment side by side: with every row in one expert a segment has g.total_rows / 16 passes
  const int64_t passes = (g.total_rows + 15) / 16;
  const dim3 grid(static_cast<unsigned>(m.blocks_per_class * m.V), static_cast<unsigned>(experts),
                  static_cast<unsigned>(passes < 8 ? (passes < 1 ? 1 : passes) : 8));
  const int gpw = (m.groups + kMbWaves - 1) / kMbWaves;
  if (gpw <= 1) hipLaunchKernelGGL((mblock_grouped_kernel<CT, XT, kInt4, 1>), grid, dim3(kMbThreads), lds, s, m, g);
  else if (gpw <= 2) hipLaunchKernelGGL((mblock_grouped_kernel<CT, XT, kInt4, 2>), grid, dim3(kMbThreads), lds, s, m, g);
  else return CAIFX_ERR_UNSUPPORTED;
  return launch_status();
}

template <typename CT>
int launch_grouped_xt(const MbArgs &m, const MbGroup &g, int experts, int x_dtype, bool int4, size_t lds, hipStream_t s)
{
  if (x_dtype == CAIFX_F32)
    return int4 ? launch_grouped_gpw<CT, float, true>(m, g, experts, lds, s) : launch_grouped_gpw<CT, float, false>(m, g, experts, lds, s);
  if (x_dtype == CAIFX_F16)
    return int4 ? launch_grouped_gpw<CT, f16_t, true>(m, g, experts, lds, s) : launch_grouped_gpw<CT, f16_t, false>(m, g, experts, lds, s);
  return int4 ? launch_grouped_gpw<CT, bf16_t, true>(m, g, experts, lds, s) : launch_grouped_gpw<CT, bf16_t, false>(m, g, experts, lds, s);
}

template <typename XT>
int launch_f32(const MbArgs &m, size_t lds, hipStream_t s)
{
  return launch_gpw<bf16_t, XT, false, true>(m, lds, s);
}

template <typename CT>
int launch_xt(const MbArgs &m, int x_dtype, bool int4, size_t lds, hipStream_t s)
{
  if (x_dtype == CAIFX_F32) return int4 ? launch_gpw<CT, float, true>(m, lds, s) : launch_gpw<CT, float, false>(m, lds, s);
  if (x_dtype == CAIFX_F16) return int4 ? launch_gpw<CT, f16_t, true>(m, lds, s) : launch_gpw<CT, f16_t, false>(m, lds, s);
  return int4 ? launch_gpw<CT, bf16_t, true>(m, lds, s) : launch_gpw<CT, bf16_t, false>(m, lds, s);
}

int compute_units()
{
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      cus = n;
    else
      cus = 256;
  }
  return cus;
}

}  // namespace

constexpr int kMbMaxRows = 32;                          // two tiles of 16 activation rows
constexpr int64_t kMbMaxSlices = 64;

// longest reduction one workgroup covers: 16 waves times the groups a wave can hold operands for
static int64_t mb_reach(int64_t M) { return kMbWaves * 128 * mb_max_gpw(false, M > 16 ? 2 : 1); }

// Reduction length per workgroup the launch is planned with.  The int8 prologue (scaled activations cut into digit
// planes) costs a workgroup time in proportion to its k range, while its share of the weight shrinks with N: at
// K = 4096, 16 rows, half the reach plus the pass that adds the two slices measured 17.6 -> 12.5 us (fp32 compute,
// N = 4096), 26.1 -> 21.9 us (fp32, N = 14336), 13.5 -> 11.7 us (bf16, N = 4096), 18.7 -> 18.9 us (bf16, N = 14336).
// int4 has no such prologue and loses (9.3 -> 9.0 us at N = 4096 but 14.4 -> 15.2 us at N = 14336).
static int64_t mb_slice_k(const GemmArgs &g)
{
  const int64_t reach = mb_reach(g.M);
  if (g.M > 16 || g.w.kind == CAIFX_W_INT4_GROUP) return reach;
  const int64_t n_max = g.compute_dtype == CAIFX_F32 ? 32768 : 8192;
  return g.N <= n_max ? reach / 2 : reach;
}

static size_t mb_lds_bytes(bool int4, int mt, int slice_groups)
{
  size_t floats = static_cast<size_t>(mb_reduce_blocks(int4, mt)) * mt * kPartialFloats + static_cast<size_t>(16) * mt * kSegRows;
  if (!int4) floats += static_cast<size_t>(slice_groups) * 128;      // staged scales (ones without a scale vector)
  else if (mt > 1) floats += static_cast<size_t>(mt) * mb_max_gpw(true, mt) * kMbWaves * 16;      // group-sum corrections
  return floats * sizeof(float);
}

size_t mblock_workspace_bytes(const GemmArgs &g)
{
  if (g.offsets || g.M < 1 || g.M > kMbMaxRows || g.K % 128 != 0) return 0;
  const bool int4 = g.w.kind == CAIFX_W_INT4_GROUP;
  if (g.compute_dtype == CAIFX_F32 && int4) return 0;
  int64_t reach = mb_slice_k(g);
  int64_t slices = (g.K + reach - 1) / reach;
  if (slices > kMbMaxSlices) {
    reach = mb_reach(g.M);
    slices = (g.K + reach - 1) / reach;
  }
  if (slices < 2 || slices > kMbMaxSlices) return 0;
  return static_cast<size_t>(slices) * static_cast<size_t>(g.M) * static_cast<size_t>(g.N) * sizeof(float);
}

int mblock_forward(const GemmArgs &g, hipStream_t s)
{
  if (g.offsets || g.M < 1 || g.M > kMbMaxRows) return CAIFX_ERR_UNSUPPORTED;
  if (g.N < 16 || g.N > (int64_t{1} << 30) || g.K % 128 != 0) return CAIFX_ERR_UNSUPPORTED;
  if (!aligned_to(g.w.q, 16) || !aligned_to(g.x, 16)) return CAIFX_ERR_UNSUPPORTED;
  const bool int4 = g.w.kind == CAIFX_W_INT4_GROUP;
  if (g.compute_dtype == CAIFX_F32 && int4) return CAIFX_ERR_UNSUPPORTED;
  // a reduction longer than one workgroup's reach is cut into slices whose sums meet in the caller's workspace
  // (a shorter slice than the workgroup's reach is a choice: without room for its sums the full reach is used)
  const int mt = g.M > 16 ? 2 : 1;
  int64_t reach = mb_slice_k(g);
  int64_t slices = (g.K + reach - 1) / reach;
  const bool room = g.workspace && aligned_to(g.workspace, 4) &&
                    g.workspace_bytes / sizeof(float) / static_cast<size_t>(g.M) / static_cast<size_t>(g.N) >= static_cast<size_t>(slices);
  if (slices > kMbMaxSlices || (slices > 1 && !room)) {
    reach = mb_reach(g.M);
    slices = (g.K + reach - 1) / reach;
    if (slices > kMbMaxSlices) return CAIFX_ERR_UNSUPPORTED;
    if (slices > 1 && (!g.workspace || !aligned_to(g.workspace, 4) ||
                       g.workspace_bytes < static_cast<size_t>(slices) * static_cast<size_t>(g.M) * static_cast<size_t>(g.N) * sizeof(float)))
      return CAIFX_ERR_UNSUPPORTED;
  }

  MbArgs m{};
  m.wq = static_cast<const uint8_t *>(g.w.q);
  m.scales = g.w.scales;
  m.x = g.x;
  m.y = g.y;
  m.M = static_cast<int>(g.M);
  m.y_dtype = g.y_dtype;
  m.N = g.N;
  m.K = g.K;
  m.groups = static_cast<int>(g.K / 128);
  m.slice_groups = static_cast<int>((m.groups + slices - 1) / slices);      // slices of equal length, the last may be shorter
  slices = (m.groups + m.slice_groups - 1) / m.slice_groups;
  m.partial = slices > 1 ? static_cast<float *>(g.workspace) : nullptr;
  m.V = 1;
  if (int4) {
    const int gs = g.w.group_size;
    if (!g.w.scales || gs < 128 || (gs & (gs - 1)) != 0) return CAIFX_ERR_UNSUPPORTED;
    m.group_shift = __builtin_ctz(static_cast<unsigned>(gs));
  } else if (g.w.scales && g.w.scale_period > 1) {
    const int64_t P = g.w.scale_period;
    if (P > (int64_t{1} << 30) || !aligned_to(g.w.scales, 4)) return CAIFX_ERR_UNSUPPORTED;
    const int64_t V = P / gcd64(g.K % P == 0 ? P : g.K % P, P);
    if (V * 64 > g.N) return CAIFX_ERR_UNSUPPORTED;      // too few rows per residue class
    m.period = static_cast<int>(P);
    m.scale_step = static_cast<int>(kMbThreads % P);
    m.V = static_cast<int>(V);
  }
  const size_t lds = mb_lds_bytes(int4, mt, m.slice_groups);
  // one workgroup per compute unit over all slices: the prologue (the slice of X as operands, for int8 its digit
  // planes) is paid per workgroup, so each should own as many rows as the chip allows
  int target = static_cast<int>((compute_units() + slices - 1) / slices);
  const int64_t nrb_class = ((g.N + m.V - 1) / m.V + 15) / 16;
  int64_t bpc = target / m.V;
  if (bpc < 1) bpc = 1;
  if (bpc > nrb_class) bpc = nrb_class;        // at least 16 rows per workgroup
  m.blocks_per_class = static_cast<int>(bpc);
  int st;
  if (g.compute_dtype == CAIFX_F32)
    st = g.x_dtype == CAIFX_F32 ? launch_f32<float>(m, lds, s)
                                : (g.x_dtype == CAIFX_F16 ? launch_f32<f16_t>(m, lds, s) : launch_f32<bf16_t>(m, lds, s));
  else
    st = g.compute_dtype == CAIFX_BF16 ? launch_xt<bf16_t>(m, g.x_dtype, int4, lds, s)
                                       : launch_xt<f16_t>(m, g.x_dtype, int4, lds, s);
  if (st != CAIFX_OK || slices == 1) return st;
  return splitk_reduce(m.partial, static_cast<int>(slices), g.M * g.N, g.y, g.y_dtype, nullptr, s);
}

int mblock_grouped_forward(const GemmArgs &g, hipStream_t s)
{
  if (!g.offsets || !g.wq_ptrs || g.num_experts < 1 || g.num_experts > 65535 || g.compute_dtype == CAIFX_F32 || g.addend ||
      g.epilogue != 0)
    return CAIFX_ERR_UNSUPPORTED;
  // worth it while a segment takes one or two passes of 16 rows; the tiled kernel streams an expert's weight
  // once per 128 rows
  if (g.M > 16 * static_cast<int64_t>(g.num_experts)) return CAIFX_ERR_UNSUPPORTED;
  if (g.N < 16 || g.N > (int64_t{1} << 30) || g.K % 128 != 0 || g.K > mb_reach(16) || !aligned_to(g.x, 16)) return CAIFX_ERR_UNSUPPORTED;
  const bool int4 = g.w.kind == CAIFX_W_INT4_GROUP;
  MbArgs m{};
  m.x = g.x;
  m.y = g.y;
  m.M = 16;
  m.y_dtype = g.y_dtype;
  m.N = g.N;
  m.K = g.K;
  m.groups = static_cast<int>(g.K / 128);
  m.slice_groups = m.groups;
  m.V = 1;
  if (int4) {
    const int gs = g.w.group_size;
    if (!g.scales_ptrs || gs < 128 || (gs & (gs - 1)) != 0) return CAIFX_ERR_UNSUPPORTED;
    m.group_shift = __builtin_ctz(static_cast<unsigned>(gs));
  } else if (g.scales_ptrs && g.w.scale_period > 1) {
    const int64_t P = g.w.scale_period;
    if (P > (int64_t{1} << 30)) return CAIFX_ERR_UNSUPPORTED;
    const int64_t V = P / gcd64(g.K % P == 0 ? P : g.K % P, P);
    if (V * 64 > g.N) return CAIFX_ERR_UNSUPPORTED;
    m.period = static_cast<int>(P);
    m.scale_step = static_cast<int>(kMbThreads % P);
    m.V = static_cast<int>(V);
  }
  const size_t lds = mb_lds_bytes(int4, 1, m.groups);
  const int64_t nrb_class = ((g.N + m.V - 1) / m.V + 15) / 16;
  int64_t bpc = 2 * static_cast<int64_t>(compute_units()) / (static_cast<int64_t>(g.num_experts) * m.V);
  if (bpc < 1) bpc = 1;
  if (bpc > nrb_class) bpc = nrb_class;
  m.blocks_per_class = static_cast<int>(bpc);
  MbGroup grp{g.offsets, g.wq_ptrs, g.scales_ptrs, g.M};
  return g.compute_dtype == CAIFX_BF16 ? launch_grouped_xt<bf16_t>(m, grp, g.num_experts, g.x_dtype, int4, lds, s)
                                       : launch_grouped_xt<f16_t>(m, grp, g.num_experts, g.x_dtype, int4, lds, s);
}

}  // namespace caifx
