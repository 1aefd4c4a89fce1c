// Decode-regime dequant-GEMV for M <= 4 activation rows, streaming every weight row linearly.
//
// Why a second decode kernel: on MI355X a plain linear read of the 29 MB int4 weight of the
// K=4096 x N=14336 case takes about 6 us, and any pattern that touches 64-byte pieces of 16
// different rows per instruction is 20-50 % slower than that.  Here one load instruction of a
// wave covers 1 KiB of ONE weight row (lane l reads bytes [16 l, 16 l + 16)), a wave walks a
// few whole rows through a small ring of rows in flight.
//
// The matrix core still does the multiply-adds.  v_mfma_f32_16x16x32 wants, per lane
// (i = lane%16, c = lane/16), 8 consecutive-k values of "row i" of A and of "column i" of B.
// Here A's 16 rows are 16 different k-segments of the same weight row and B's 16 columns are the
// same 16 k-segments of the activation row: lane l holds the codes of k-slot l in A and the
// activations of k-slot l in B, and D[i][i] = sum over the 4 lanes (c) of segment i.  Only the
// diagonal of D is meaningful; the other 240 products are wasted matrix-core work, which is
// free here (the kernel is bound by HBM and by the VALU work of unpacking, not by MFMA rate).
// Each extra activation row costs one more MFMA per step with its own B.
//
//   int4 (group_size % 128 == 0): a k-slot is 32 codes, segment i of a 2048-k chunk is exactly
//     one 128-k scale group, so D[i][i] is a per-group sum of (code+136 or code+1032) * x and
//     the lane holding it applies  scale * (D[i][i] - offset * sum_k x)  -- the post-scaled form
//     (see caifx_gemv.hip for the numerics note).
//   int8 (two to four activation rows, and one row when the shape does not fit the kernel below):
//     a k-slot is 16 codes; float(code)*scale is rounded to the compute dtype exactly as the
//     reference does.  With per-channel scales the index (n*K+k) % period depends on the
//     row only through (n*K) % period, so a wave takes rows of one residue class
//     n = v + V*i (V = period / gcd(K, period)) and keeps that class's scales in registers.
//   int8, one activation row, K a multiple of 1024: the scales are folded into the activations and
//     the codes go into the integer matrix core as loaded (rowlin_int8_digits_kernel below).
#include "caifx_internal.hpp"

#include <atomic>

namespace caifx {
namespace {

template <typename CT> struct Mfma16;
template <> struct Mfma16<bf16_t> {
  typedef bf16x8_t vec_t;
  static constexpr uint32_t kMagic = 0x43084308u;
  static constexpr float kOffset = 136.0f;
  static __device__ __forceinline__ floatx4_t run(vec_t a, vec_t b, floatx4_t c)
  {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma16<f16_t> {
  typedef f16x8_t vec_t;
  static constexpr uint32_t kMagic = 0x64086408u;
  static constexpr float kOffset = 1032.0f;
  static __device__ __forceinline__ floatx4_t run(vec_t a, vec_t b, floatx4_t c)
  {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

struct RowArgs {
  const uint8_t *wq;
  const void *scales;
  const void *x;
  void *y;
  int M;
  int y_dtype;
  int64_t N, K;
  int group_shift;      // int4
  int period;           // int8 vec
  int row_stride;       // int8 vec: V
  int rows_per_wave;
  int waves_per_class;  // int8: waves that share one residue class
  int total_waves;
  int cpr;              // chunks (one load instruction of a wave) per weight row
  int xpitch;           // staged activations: elements per row (cpr * k-per-chunk)
  int digits;           // int8, one activation row: take the integer-matrix-core kernel
  int round_x;          // that kernel only: activations pass through this dtype first (caifx_dtype), -1 = they are of it already
  int slices;           // its form for K > 4096: parts a weight row is cut into (2 or 4), 0 otherwise
};

template <typename CT, typename XT>
__device__ __forceinline__ typename Mfma16<CT>::vec_t load_x8g(const XT *p)
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
  } else {
    const u32x4_t raw = *reinterpret_cast<const u32x4_t *>(p);
    const XT *e = reinterpret_cast<const XT *>(&raw);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = from_f32<CT>(to_f32<XT>(e[j]));
  }
  return v;
}

// v + (v moved across lanes by DPP control kCtrl); lanes outside kRowMask add 0
template <int kCtrl, int kRowMask = 0xF>
__device__ __forceinline__ float dpp_add(float v)
{
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, kRowMask, 0xF, false);
  return v + __builtin_bit_cast(float, moved);
}

// sum over each aligned group of 16 lanes, result in all 16 (4 VALU ops, no LDS)
__device__ __forceinline__ float row16_sum(float v)
{
  v = dpp_add<0xB1>(v);    // quad_perm [1,0,3,2]
  v = dpp_add<0x4E>(v);    // quad_perm [2,3,0,1]
  v = dpp_add<0x141>(v);   // row_half_mirror
  v = dpp_add<0x140>(v);   // row_mirror
  return v;
}

// sum over the wave; valid in lanes 48..63 (read it from lane 63)
__device__ __forceinline__ float wave_sum_hi(float v)
{
  v = row16_sum(v);
  v = dpp_add<0x142, 0xA>(v);   // row_bcast:15 into rows 1 and 3
  v = dpp_add<0x143, 0xC>(v);   // row_bcast:31 into rows 2 and 3
  return v;
}

// (a & mask) | base in one instruction (the compiler splits it in two when both constants are literals)
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t base)
{
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(base));
  return r;
}

// the low bytes of four words as one word (a in byte 0)
__device__ __forceinline__ uint32_t pack_low_bytes(int a, int b, int c, int d)
{
  const uint32_t ab = __builtin_amdgcn_perm(static_cast<uint32_t>(b), static_cast<uint32_t>(a), 0x0c0c0400u);
  const uint32_t cd = __builtin_amdgcn_perm(static_cast<uint32_t>(d), static_cast<uint32_t>(c), 0x0c0c0400u);
  return __builtin_amdgcn_perm(cd, ab, 0x05040100u);
}

// `acc` with lane `dst_lane` (wave uniform) replaced by the wave sum that wave_sum_hi left in lane 63
__device__ __forceinline__ float lane_insert(float acc, float sum_hi, int dst_lane)
{
  const int s = __builtin_amdgcn_readlane(__builtin_bit_cast(int, sum_hi), 63);
  return static_cast<int>(threadIdx.x & 63) == dst_lane ? __builtin_bit_cast(float, s) : acc;
}

__device__ __forceinline__ void store_y(void *y, int y_dtype, int64_t o, float v)
{
  if (y_dtype == CAIFX_F32) static_cast<float *>(y)[o] = v;
  else if (y_dtype == CAIFX_BF16) static_cast<bf16_t *>(y)[o] = from_f32<bf16_t>(v);
  else static_cast<f16_t *>(y)[o] = from_f32<f16_t>(v);
}

// D[i][i] of the 16x16 tile lives on lane i + 16*(i/4) in element i%4; other lanes return 0.
__device__ __forceinline__ float diag_of(floatx4_t d, int lane)
{
  const int r = lane & 15;
  const int t = r & 3;
  float v = d[0];
  v = (t == 1) ? d[1] : v;
  v = (t == 2) ? d[2] : v;
  v = (t == 3) ? d[3] : v;
  return ((lane >> 4) == (r >> 2)) ? v : 0.0f;
}

// Stage X[MT rows][K] as compute-dtype values into LDS, zero padded to `xpitch` per row, in the
// order the MFMA B operand is read: row m is a sequence of 1 KiB blocks (chunk, step j), and in
// each block lane l owns 16 bytes at l*16, so the ds_read_b128 of a wave is conflict free.
// kInt4: a k-slot is 32 values (4 steps), the slot of lane l is 4*(l%16) + l/16, every aligned
// run of 8 is stored in the order 0,4,1,5,2,6,3,7 and the per-128-k sums of the rounded values
// go to xsum[m][xpitch/128].  Otherwise (int8): a k-slot is 16 values (2 steps), slot = lane.
template <typename CT, typename XT, int MT, bool kInt4>
__device__ __forceinline__ void stage_x(const RowArgs &a, CT *xs, float *xsum)
{
  typedef typename Mfma16<CT>::vec_t vec_t;
  constexpr int kSteps = kInt4 ? 4 : 2;
  const XT *xg = static_cast<const XT *>(a.x);
  const int lane = threadIdx.x & 63;
  const int per_row = a.xpitch / 8;                      // 8-element pieces per staged row
  for (int p = threadIdx.x; p < MT * per_row; p += blockDim.x) {
    const int m = p / per_row;
    const int piece = p - m * per_row;
    const int k = piece * 8;
    const int msrc = m < a.M ? m : a.M - 1;
    vec_t v;
    if (k < a.K) {
      v = load_x8g<CT, XT>(xg + static_cast<int64_t>(msrc) * a.K + k);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = from_f32<CT>(0.0f);
    }
    const int j = piece % kSteps;
    const int slot_all = piece / kSteps;                 // chunk*64 + slot
    const int chunk = slot_all >> 6;
    const int slot = slot_all & 63;
    int l = slot;
    if constexpr (kInt4) {
      l = (slot & 3) * 16 + (slot >> 2);
      float part = 0.0f;
#pragma unroll
      for (int t = 0; t < 8; ++t) part += to_f32<CT>(v[t]);
      part = row16_sum(part);
      if ((lane & 15) == 0) xsum[m * (a.xpitch >> 7) + (k >> 7)] = part;
      vec_t q;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        q[2 * t] = v[t];
        q[2 * t + 1] = v[t + 4];
      }
      v = q;
    }
    *reinterpret_cast<vec_t *>(xs + m * a.xpitch + ((chunk * kSteps + j) * 64 + l) * 8) = v;
  }
}

// ------------------------------------------------------------------ int4, post-scaled
template <typename CT, typename XT, int MT>
__global__ __launch_bounds__(256) void rowlin_int4_kernel(RowArgs a)
{
  typedef typename Mfma16<CT>::vec_t vec_t;
  constexpr int U = 8;                                   // 16-byte loads in flight per lane
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int groups_pad = a.xpitch >> 7;
  float *xsum = reinterpret_cast<float *>(smem);                        // [MT][groups_pad]
  CT *xs = reinterpret_cast<CT *>(xsum + ((MT * groups_pad + 3) & ~3)); // [MT][xpitch]

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int gw = blockIdx.x * 4 + wave;
  const int64_t row0 = static_cast<int64_t>(gw) * a.rows_per_wave;
  int nrows = 0;
  if (row0 < a.N) nrows = static_cast<int>(a.N - row0 < a.rows_per_wave ? a.N - row0 : a.rows_per_wave);
  const int cpr = a.cpr;
  const int ntasks = nrows * cpr;
  const int slots = static_cast<int>(a.K >> 5);          // 32-code slots per row
  const int64_t rowbytes = a.K >> 1;
  const bool is_diag = (lane >> 4) == ((lane & 15) >> 2);
  const int di = lane & 15;
  const int pslot = (lane & 15) * 4 + (lane >> 4);       // k-slot of this lane inside a chunk

  u32x4_t wreg[U];
  f16_t sreg[U];
  // task t = (row t / cpr, chunk t % cpr); keep the issue cursor incrementally
  int irow = 0, ichunk = 0;
  auto issue = [&](int u) {
    const int slot = ichunk * 64 + pslot;
    u32x4_t w = {0u, 0u, 0u, 0u};
    if (slot < slots)
      w = *reinterpret_cast<const u32x4_t *>(a.wq + (row0 + irow) * rowbytes + static_cast<int64_t>(slot) * 16);
    wreg[u] = w;
    f16_t s = static_cast<f16_t>(0.0f);
    const int gslot = ichunk * 64 + di * 4;              // first slot of the group this lane's diagonal covers
    if (is_diag && gslot < slots)
      s = static_cast<const f16_t *>(a.scales)[((row0 + irow) * a.K + (static_cast<int64_t>(gslot) << 5)) >> a.group_shift];
    sreg[u] = s;
    if (++ichunk == cpr) {
      ichunk = 0;
      ++irow;
    }
  };

#pragma unroll
  for (int u = 0; u < U; ++u)
    if (u < ntasks) issue(u);

  stage_x<CT, XT, MT, true>(a, xs, xsum);
  __syncthreads();

  float tot[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) tot[m] = 0.0f;
  int crow = 0, cchunk = 0;
  for (int t0 = 0; t0 < ntasks; t0 += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int t = t0 + u;
      if (t < ntasks) {
        const u32x4_t w = wreg[u];
        const float s = to_f32(sreg[u]);
        if (t + U < ntasks) issue(u);
        floatx4_t part[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) part[m] = floatx4_t{0.0f, 0.0f, 0.0f, 0.0f};
        const CT *xb = xs + (cchunk * 4 * 64 + lane) * 8;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          u32x4_t c4;
          const uint32_t p = w[j];
          c4[0] = (p & 0x000F000Fu) ^ Mfma16<CT>::kMagic;           // codes 0,4
          c4[1] = ((p >> 4) & 0x000F000Fu) ^ Mfma16<CT>::kMagic;    // codes 1,5
          c4[2] = ((p >> 8) & 0x000F000Fu) ^ Mfma16<CT>::kMagic;    // codes 2,6
          c4[3] = ((p >> 12) & 0x000F000Fu) ^ Mfma16<CT>::kMagic;   // codes 3,7
          const vec_t av = *reinterpret_cast<const vec_t *>(&c4);
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            const vec_t bv = *reinterpret_cast<const vec_t *>(xb + m * a.xpitch + j * 64 * 8);
            part[m] = Mfma16<CT>::run(av, bv, part[m]);
          }
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const float corr = Mfma16<CT>::kOffset * xsum[m * groups_pad + cchunk * 16 + di];
          tot[m] = __builtin_fmaf(s, diag_of(part[m], lane) - corr, tot[m]);
        }
        if (++cchunk == cpr) {
          cchunk = 0;
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            const float v = wave_sum_hi(tot[m]);
            if (lane == 63 && m < a.M) store_y(a.y, a.y_dtype, static_cast<int64_t>(m) * a.N + row0 + crow, v);
            tot[m] = 0.0f;
          }
          ++crow;
        }
      }
    }
  }
}

// ------------------------------------------------------------------ fixed-shape fast paths
// Same arithmetic as the kernels above for rows made of whole chunks (K = CPR * 2048 for int4,
// CPR * 1024 for int8).  Every inner trip count is a compile-time constant.  What the prologue needs
// (activations, int8 scales) is requested BEFORE the first weight rows, because loads return in
// order; a wave then walks `rows_per_wave` rows through a ring of D rows: it computes a row out of
// the registers it arrived in and requests the row D further on into the same registers, so D-1
// rows are on their way from HBM while one is unpacked.  No load sits behind a branch (rows past the
// end read a cache-resident dummy) and nothing is stored inside the loop (lane r keeps the result of
// row r until one coalesced store at the end): only then does the compiler know how many requests
// are outstanding at each wait and leaves the younger ones in flight.

// Activation pieces (8 values) a thread stages: piece p = threadIdx.x + i*kThreads of MT*PIECES_PER_ROW.
template <typename CT, int MT, int kPiecesPerRow, int kThreads = 256>
struct XPieces {
  static constexpr int kTotal = MT * kPiecesPerRow;
  static constexpr int kPerThread = (kTotal + kThreads - 1) / kThreads;
  typename Mfma16<CT>::vec_t v[kPerThread];
};

template <typename CT, int MT, int kPiecesPerRow, int kThreads = 256>
__device__ __forceinline__ void x_request(const RowArgs &a, XPieces<CT, MT, kPiecesPerRow, kThreads> &xp)
{
  typedef typename Mfma16<CT>::vec_t vec_t;
  const CT *xg = static_cast<const CT *>(a.x);
#pragma unroll
  for (int i = 0; i < XPieces<CT, MT, kPiecesPerRow, kThreads>::kPerThread; ++i) {
    const int p = threadIdx.x + i * kThreads;
    const int m = p / kPiecesPerRow;
    const int piece = p - m * kPiecesPerRow;
    const int msrc = m < a.M ? m : a.M - 1;
    if (XPieces<CT, MT, kPiecesPerRow, kThreads>::kTotal % kThreads == 0 || p < MT * kPiecesPerRow)
      xp.v[i] = *reinterpret_cast<const vec_t *>(xg + static_cast<int64_t>(msrc) * a.K + piece * 8);
  }
}

template <typename CT, int MT, int kPiecesPerRow, bool kInt4, int kThreads = 256>
__device__ __forceinline__ void x_commit(const XPieces<CT, MT, kPiecesPerRow, kThreads> &xp, CT *xs, float *xsum)
{
  typedef typename Mfma16<CT>::vec_t vec_t;
  constexpr int kSteps = kInt4 ? 4 : 2;
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < XPieces<CT, MT, kPiecesPerRow, kThreads>::kPerThread; ++i) {
    const int p = threadIdx.x + i * kThreads;
    if (XPieces<CT, MT, kPiecesPerRow, kThreads>::kTotal % kThreads == 0 || p < MT * kPiecesPerRow) {
      const int m = p / kPiecesPerRow;
      const int piece = p - m * kPiecesPerRow;
      vec_t v = xp.v[i];
      const int j = piece % kSteps;
      const int slot_all = piece / kSteps;
      const int chunk = slot_all >> 6;
      const int slot = slot_all & 63;
      int l = slot;
      if constexpr (kInt4) {
        l = (slot & 3) * 16 + (slot >> 2);
        float part = 0.0f;
#pragma unroll
        for (int t = 0; t < 8; ++t) part += to_f32<CT>(v[t]);
        part = row16_sum(part);
        if ((lane & 15) == 0) xsum[m * (kPiecesPerRow / 16) + (piece >> 4)] = part;
        vec_t q;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          q[2 * t] = v[t];
          q[2 * t + 1] = v[t + 4];
        }
        v = q;
      }
      *reinterpret_cast<vec_t *>(xs + m * (kPiecesPerRow * 8) + ((chunk * kSteps + j) * 64 + l) * 8) = v;
    }
  }
}

constexpr int kInt4FastWaves = 4;   // waves per workgroup of the kernel below (8 and 16 measured no better)

template <typename CT, int MT, int CPR>
__global__ __launch_bounds__(kInt4FastWaves * 64) void rowlin_int4_fast_kernel(RowArgs a)
{
  constexpr int kThreads = kInt4FastWaves * 64;
  typedef typename Mfma16<CT>::vec_t vec_t;
  constexpr int D = (CPR >= 2) ? 2 : 4;   // rows in the ring (2 for K = 4096 measured best against 1, 3, 4 and 8)
  constexpr int kPieces = CPR * 256;         // 8-value pieces per activation row
  constexpr int kGroupsPad = CPR * 16;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float *xsum = reinterpret_cast<float *>(smem);                        // [MT][CPR*16]
  CT *xs = reinterpret_cast<CT *>(xsum + ((MT * kGroupsPad + 3) & ~3)); // [MT][CPR*2048]

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * kInt4FastWaves + wave) * a.rows_per_wave;
  int nrows = 0;
  if (row0 < a.N) nrows = static_cast<int>(a.N - row0 < a.rows_per_wave ? a.N - row0 : a.rows_per_wave);
  const bool is_diag = (lane >> 4) == ((lane & 15) >> 2);
  const int di = lane & 15;
  const int pslot = di * 4 + (lane >> 4);
  constexpr int64_t kRowBytes = static_cast<int64_t>(CPR) * 1024;
  constexpr int groups_per_row = CPR * 16;       // group size 128

  XPieces<CT, MT, kPieces, kThreads> xp;
  x_request<CT, MT, kPieces, kThreads>(a, xp);

  const uint8_t *wp = a.wq + row0 * kRowBytes + pslot * 16;
  const f16_t *sp = static_cast<const f16_t *>(a.scales) + row0 * groups_per_row;
  u32x4_t w[D][CPR];
  f16_t sc[D][CPR];
  // Every load below is issued unconditionally (a row index past the wave's range reads the start of
  // the activation row instead, which is cache resident and large enough): with no branch around a
  // load the compiler knows how many requests are in flight at every wait and lets the newer ones
  // stay outstanding, which is what keeps the ring of rows in flight.
  const uint8_t *wdummy = static_cast<const uint8_t *>(a.x) + pslot * 16;
  const f16_t *sdummy = static_cast<const f16_t *>(a.x) + di;
  auto issue = [&](int d, int r) {
    const bool ok = r < nrows;
    const uint8_t *wsrc = ok ? wp + r * kRowBytes : wdummy;
    const f16_t *ssrc = ok ? sp + r * groups_per_row + di : sdummy;
#pragma unroll
    for (int c = 0; c < CPR; ++c) {
      w[d][c] = *reinterpret_cast<const u32x4_t *>(wsrc + c * 1024);
      sc[d][c] = ssrc[c * 16];
    }
  };
#pragma unroll
  for (int d = 0; d < D; ++d) issue(d, d);

  x_commit<CT, MT, kPieces, true, kThreads>(xp, xs, xsum);
  __syncthreads();

  float corr[MT][CPR];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int c = 0; c < CPR; ++c) corr[m][c] = Mfma16<CT>::kOffset * xsum[m * kGroupsPad + c * 16 + di];
  const int tsel = di & 3;
  // lane r keeps the result of the wave's row r: one coalesced store per wave after the loop, and no
  // store (which would count against the same in-flight counter as the loads) inside it
  float res[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) res[m] = 0.0f;

  for (int r0 = 0; r0 < nrows; r0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int r = r0 + d;
      if (r < nrows) {
        float tot[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) tot[m] = 0.0f;
#pragma unroll
        for (int c = 0; c < CPR; ++c) {
          floatx4_t part[MT];
#pragma unroll
          for (int m = 0; m < MT; ++m) part[m] = floatx4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            u32x4_t c4;
            // one xor turns all eight two's-complement nibbles into code + 8; each pair of nibbles then
            // needs a shift and one and-or to become two compute-dtype values 128 (or 1024) + code + 8
            const uint32_t p = w[d][c][j] ^ 0x88888888u;
            constexpr uint32_t kBase = Mfma16<CT>::kMagic & 0xFFF0FFF0u;
            c4[0] = and_or(p, 0x000F000Fu, kBase);
            c4[1] = and_or(p >> 4, 0x000F000Fu, kBase);
            c4[2] = and_or(p >> 8, 0x000F000Fu, kBase);
            c4[3] = and_or(p >> 12, 0x000F000Fu, kBase);
            const vec_t av = *reinterpret_cast<const vec_t *>(&c4);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
              const vec_t bv = *reinterpret_cast<const vec_t *>(xs + m * (CPR * 2048) + ((c * 4 + j) * 64 + lane) * 8);
              part[m] = Mfma16<CT>::run(av, bv, part[m]);
            }
          }
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            float dsel = part[m][0];
            dsel = (tsel == 1) ? part[m][1] : dsel;
            dsel = (tsel == 2) ? part[m][2] : dsel;
            dsel = (tsel == 3) ? part[m][3] : dsel;
            tot[m] = __builtin_fmaf(to_f32(sc[d][c]), dsel - corr[m][c], tot[m]);
          }
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const float v = wave_sum_hi(is_diag ? tot[m] : 0.0f);
          res[m] = lane_insert(res[m], v, r);
        }
      }
      issue(d, r + D);      // into the registers just consumed: the other D-1 rows stay in flight meanwhile
    }
  }
  if (lane < nrows) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
      if (MT != 4 || m < a.M) static_cast<float *>(a.y)[static_cast<int64_t>(m) * a.N + row0 + lane] = res[m];
  }
}

template <typename CT, int MT, bool kVec, int CPR>
__global__ __launch_bounds__(256) void rowlin_int8_fast_kernel(RowArgs a)
{
  typedef typename Mfma16<CT>::vec_t vec_t;
  constexpr int D = (CPR >= 4) ? 2 : 4;   // rows in the ring
  constexpr int kPieces = CPR * 128;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  CT *xs = reinterpret_cast<CT *>(smem);     // [MT][CPR*1024]

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int gw = blockIdx.x * 4 + wave;
  const int cls = gw / a.waves_per_class;
  const int64_t i0 = static_cast<int64_t>(gw - cls * a.waves_per_class) * a.rows_per_wave;
  const int64_t V = a.row_stride;
  int nrows = 0;
  if (gw < a.total_waves) {
    const int64_t first = cls + V * i0;
    if (first < a.N) {
      const int64_t avail = (a.N - first + V - 1) / V;
      nrows = static_cast<int>(avail < a.rows_per_wave ? avail : a.rows_per_wave);
    }
  }
  constexpr int64_t kRowBytes = static_cast<int64_t>(CPR) * 1024;

  XPieces<CT, MT, kPieces> xp;
  x_request<CT, MT, kPieces>(a, xp);

  floatx4_t sc[CPR][4];
  float s_scalar = 1.0f;
  if constexpr (kVec) {
    const float *sp = static_cast<const float *>(a.scales);
#pragma unroll
    for (int c = 0; c < CPR; ++c) {
      const int idx = static_cast<int>((static_cast<uint32_t>(cls) * (CPR * 1024) + (c * 64 + lane) * 16) % static_cast<uint32_t>(a.period));
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        int i = idx + 4 * q;
        if (i >= a.period) i -= a.period;
        sc[c][q] = *reinterpret_cast<const floatx4_t *>(sp + i);
      }
    }
  } else {
    if (a.scales) s_scalar = static_cast<const float *>(a.scales)[0];
  }

  // unconditional loads (a row past the wave's range reads the start of the activation row): see the
  // int4 kernel above
  const uint8_t *wp = a.wq + (cls + V * i0) * kRowBytes + lane * 16;
  const uint8_t *wdummy = static_cast<const uint8_t *>(a.x) + lane * 16;
  const int64_t rstep = V * kRowBytes;
  u32x4_t w[D][CPR];
  auto issue = [&](int d, int r) {
    const uint8_t *wsrc = r < nrows ? wp + r * rstep : wdummy;
#pragma unroll
    for (int c = 0; c < CPR; ++c) w[d][c] = *reinterpret_cast<const u32x4_t *>(wsrc + c * 1024);
  };
#pragma unroll
  for (int d = 0; d < D; ++d) issue(d, d);

  x_commit<CT, MT, kPieces, false>(xp, xs, nullptr);
  __syncthreads();

  float res[MT];             // lane r: results of the wave's row r
#pragma unroll
  for (int m = 0; m < MT; ++m) res[m] = 0.0f;
  for (int r0 = 0; r0 < nrows; r0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int r = r0 + d;
      if (r < nrows) {
        floatx4_t acc[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[m] = floatx4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int c = 0; c < CPR; ++c) {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            float lo[4], hi[4];
            int8x4_to_f32(w[d][c][2 * j], lo);
            int8x4_to_f32(w[d][c][2 * j + 1], hi);
            vec_t av;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float s0 = kVec ? sc[c][2 * j][q] : s_scalar;
              const float s1 = kVec ? sc[c][2 * j + 1][q] : s_scalar;
              av[q] = from_f32<CT>(lo[q] * s0);
              av[4 + q] = from_f32<CT>(hi[q] * s1);
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) {
              const vec_t bv = *reinterpret_cast<const vec_t *>(xs + m * (CPR * 1024) + ((c * 2 + j) * 64 + lane) * 8);
              acc[m] = Mfma16<CT>::run(av, bv, acc[m]);
            }
          }
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const float v = wave_sum_hi(diag_of(acc[m], lane));
          res[m] = lane_insert(res[m], v, r);
        }
      }
      issue(d, r + D);
    }
  }
  if (lane < nrows) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
      if (MT != 4 || m < a.M) static_cast<float *>(a.y)[static_cast<int64_t>(m) * a.N + cls + V * (i0 + lane)] = res[m];
  }
}

// ------------------------------------------------------------------ int8, one activation row, integer matrix core
// Y[n] = sum_k q[n,k] * scale[(n*K+k) mod P] * x[k].  All rows of one residue class see the same
// scales along k, so the scales are folded into the activations once per workgroup:
// x'[k] = scale[(cls*K+k) mod P] * x[k] (fp32), and x' is split into three signed 7-bit "digits"
// relative to a power-of-two scale per diagonal element (the 256 k values of lanes i, i+16, i+32,
// i+48): x' ~ 2^(e-6) * (d0 + d1/128 + d2/16384), |error| <= 2^(e-21).  The int8 codes then go into
// v_mfma_i32_16x16x64_i8 exactly as they were loaded (one 16-byte load = one A operand, no
// unpacking arithmetic at all) against the digit planes as B operands; the three int32 sums are exact
// and are combined in fp32 once per weight row.  As in the kernels above only the diagonal of the
// 16x16 result is used.  The result is sum_k q*scale*x with every product exact to ~2^-21 of the
// largest |x'| of its 256-k set; it differs from the reference's dequantise-round-GEMM by the rounding
// of q*scale to the compute dtype that the reference applies and this kernel does not.
typedef int i32x4_t __attribute__((ext_vector_type(4)));

// Waves per workgroup of the kernel below.  The prologue (activations times scales, digit planes) is
// paid once per workgroup and reads 24 KB for K = 4096, so a workgroup should own many rows: 16 waves
// measured 12.2 us against 12.9 (8) and 13.1 (4) on the K=4096, N=14336 case.
constexpr int kDigitWaves = 16;

template <typename XT, bool kVec, int CPR>
__global__ __launch_bounds__(kDigitWaves * 64) void rowlin_int8_digits_kernel(RowArgs a)
{
  constexpr int D = (CPR >= 4) ? 2 : 4;   // rows in the ring (2 for K = 4096 measured best against 1 and 4)
  __shared__ float mx[4][16];                                  // per chunk: max |x'| of every diagonal element
  __shared__ __attribute__((aligned(16))) i32x4_t dig[4][3][64];   // [chunk][digit][lane]

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int gw = blockIdx.x * kDigitWaves + wave;
  const int cls = (blockIdx.x * kDigitWaves) / a.waves_per_class;        // waves_per_class is a multiple of kDigitWaves: one class per workgroup
  const int64_t i0 = static_cast<int64_t>(gw - cls * a.waves_per_class) * a.rows_per_wave;
  const int64_t V = a.row_stride;
  int nrows = 0;
  {
    const int64_t first = cls + V * i0;
    if (first < a.N) {
      const int64_t avail = (a.N - first + V - 1) / V;
      nrows = static_cast<int>(avail < a.rows_per_wave ? avail : a.rows_per_wave);
    }
  }
  constexpr int64_t kRowBytes = static_cast<int64_t>(CPR) * 1024;

  // this lane's activations of chunk `wave` (chunks beyond CPR do not exist; their waves only join the
  // barriers) and their scales are requested BEFORE the first weight rows: loads return in order, so
  // everything the prologue needs must be ahead of the long HBM latency of the weights in the queue
  float xv[16];
  floatx4_t scv[4];
  const bool has_chunk = wave < CPR;
  if (has_chunk) {
    const XT *xg = static_cast<const XT *>(a.x) + (wave * 64 + lane) * 16;
#pragma unroll
    for (int t = 0; t < 16; ++t) xv[t] = to_f32<XT>(xg[t]);
    // the layer casts its input to the compute dtype before the GEMM (src/caif_device_frozen_linear.cpp:459)
    if (a.round_x == CAIFX_BF16) {
#pragma unroll
      for (int t = 0; t < 16; ++t) xv[t] = round_through<bf16_t>(xv[t]);
    } else if (a.round_x == CAIFX_F16) {
#pragma unroll
      for (int t = 0; t < 16; ++t) xv[t] = round_through<f16_t>(xv[t]);
    }
    if constexpr (kVec) {
      const float *sp = static_cast<const float *>(a.scales);
      // 32-bit arithmetic: cls < N / 256 and K <= 4096, so cls * K + k stays far below 2^31
      const int idx = static_cast<int>((static_cast<uint32_t>(cls) * (CPR * 1024) + (wave * 64 + lane) * 16) % static_cast<uint32_t>(a.period));
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        int i = idx + 4 * q;
        if (i >= a.period) i -= a.period;
        scv[q] = *reinterpret_cast<const floatx4_t *>(sp + i);
      }
    }
  }
  float s_scalar = 1.0f;
  if constexpr (!kVec) {
    if (a.scales) s_scalar = static_cast<const float *>(a.scales)[0];
  }

  const uint8_t *wp = a.wq + (cls + V * i0) * kRowBytes + lane * 16;
  const int64_t rstep = V * kRowBytes;
  i32x4_t w[D][CPR];
  // unconditional loads (a row past the wave's range reads the start of the activation row): see the
  // int4 kernel above
  const uint8_t *wdummy = static_cast<const uint8_t *>(a.x) + lane * 16;
  auto issue = [&](int d, int r) {
    const uint8_t *wsrc = r < nrows ? wp + r * rstep : wdummy;
#pragma unroll
    for (int c = 0; c < CPR; ++c) w[d][c] = *reinterpret_cast<const i32x4_t *>(wsrc + c * 1024);
  };
#pragma unroll
  for (int d = 0; d < D; ++d) issue(d, d);

  if (has_chunk) {
    if constexpr (kVec) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int t = 0; t < 4; ++t) xv[4 * q + t] *= scv[q][t];
    }
    float m = 0.0f;
    bool finite = true;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      m = fmaxf(m, fabsf(xv[t]));                       // ignores a NaN
      finite = finite && fabsf(xv[t]) <= 3.4028235e38f;  // false for NaN and infinities
    }
    m = finite ? m : __builtin_inff();
    m = fmaxf(m, __shfl_xor(m, 16));
    m = fmaxf(m, __shfl_xor(m, 32));
    if (lane < 16) mx[wave][lane] = m;
  }
  __syncthreads();

  // power-of-two unit of diagonal element i: the largest |x'| of its CPR*64 values maps into [32, 64]
  float unit;
  bool poisoned;       // wave uniform, and the same in every wave of the workgroup
  {
    float m = 0.0f;
#pragma unroll
    for (int c = 0; c < CPR; ++c) m = fmaxf(m, mx[c][lane & 15]);
    // A NaN or an infinity among the scaled activations has no digits.  The reference's GEMM returns NaN or an
    // infinity in every output then (each output multiplies every activation); here every output becomes NaN.
    poisoned = __any(!(m <= 3.4028235e38f));
    int e = 0;
    (void)frexpf(poisoned ? 1.0f : m, &e);    // m = f * 2^e, f in [0.5, 1)
    unit = (m > 0.0f && !poisoned) ? ldexpf(1.0f, e - 6) : 1.0f;
  }
  if (has_chunk) {
    // n = round(x' / unit * 2^14) as the low mantissa bits of x' * (2^14 / unit) + 1.5 * 2^23 (|n| <= 2^20);
    // n = 2^14 d0 + 2^7 d1 + d2 with d1, d2 in [-64, 63]: three signed bit-field extracts, the carries
    // supplied by adding half a digit below each field
    const float inv14 = 16384.0f / unit;      // exact: a power of two
    i32x4_t d0, d1, d2;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int e0[4], e1[4], e2[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int b = __builtin_bit_cast(int, __builtin_fmaf(xv[4 * q + t], inv14, 12582912.0f));
        e2[t] = __builtin_amdgcn_sbfe(b, 0, 7);
        e1[t] = __builtin_amdgcn_sbfe(b + 64, 7, 7);
        e0[t] = __builtin_amdgcn_sbfe(b + 64 + 8192, 14, 8);
      }
      d0[q] = static_cast<int>(pack_low_bytes(e0[0], e0[1], e0[2], e0[3]));
      d1[q] = static_cast<int>(pack_low_bytes(e1[0], e1[1], e1[2], e1[3]));
      d2[q] = static_cast<int>(pack_low_bytes(e2[0], e2[1], e2[2], e2[3]));
    }
    dig[wave][0][lane] = d0;
    dig[wave][1][lane] = d1;
    dig[wave][2][lane] = d2;
  }
  __syncthreads();
  i32x4_t xb[CPR][3];
#pragma unroll
  for (int c = 0; c < CPR; ++c)
#pragma unroll
    for (int d = 0; d < 3; ++d) xb[c][d] = dig[c][d][lane];
  const float u0 = unit * s_scalar, u1 = u0 * (1.0f / 128.0f), u2 = u0 * (1.0f / 16384.0f);
  const int tsel = lane & 3;
  const bool is_diag = (lane >> 4) == ((lane & 15) >> 2);

  float res = 0.0f;          // lane r: result of the wave's row r
  for (int r0 = 0; r0 < nrows; r0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int r = r0 + d;
      if (r < nrows) {
        i32x4_t s0 = {0, 0, 0, 0}, s1 = {0, 0, 0, 0}, s2 = {0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < CPR; ++c) {
          s0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[d][c], xb[c][0], s0, 0, 0, 0);
          s1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[d][c], xb[c][1], s1, 0, 0, 0);
          s2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[d][c], xb[c][2], s2, 0, 0, 0);
        }
        // D[i][i] sits in element i%4 of lane i + 16*(i/4)
        int p0 = s0[0], p1 = s1[0], p2 = s2[0];
        p0 = tsel == 1 ? s0[1] : p0;  p1 = tsel == 1 ? s1[1] : p1;  p2 = tsel == 1 ? s2[1] : p2;
        p0 = tsel == 2 ? s0[2] : p0;  p1 = tsel == 2 ? s1[2] : p1;  p2 = tsel == 2 ? s2[2] : p2;
        p0 = tsel == 3 ? s0[3] : p0;  p1 = tsel == 3 ? s1[3] : p1;  p2 = tsel == 3 ? s2[3] : p2;
        float v = static_cast<float>(p0) * u0;
        v = __builtin_fmaf(static_cast<float>(p1), u1, v);
        v = __builtin_fmaf(static_cast<float>(p2), u2, v);
        v = wave_sum_hi(is_diag ? v : 0.0f);
        res = lane_insert(res, v, r);
      }
      issue(d, r + D);
    }
  }
  if (lane < nrows) static_cast<float *>(a.y)[cls + V * (i0 + lane)] = poisoned ? __builtin_nanf("") : res;
}


// The same for reductions of 4097..16384 (a down projection at decode time).  The row no longer fits one wave's
// registers, so the 16 waves of a workgroup split it: wave w takes slice w % nsl of every row of row group w / nsl,
// a slice being `cps` <= 4 chunks of 1 KiB (the last slice may have fewer), and keeps that slice's digit planes in
// registers for the whole kernel.  The power-of-two unit is taken per slice.  The nsl partial sums of a row meet in
// LDS after the loop and are added in slice order.  a.cpr = chunks per row (K / 1024 <= 16), a.slices = nsl (2 or
// 4), a.waves_per_class = row groups per residue class (a multiple of 16 / nsl).
template <typename XT, bool kVec>
__global__ __launch_bounds__(kDigitWaves * 64) void rowlin_int8_digits_long_kernel(RowArgs a)
{
  constexpr int CPS = 4;                  // chunks per slice at most
  constexpr int D = 2;                    // row slices in the ring
  __shared__ float mx[16][16];                                      // per chunk: max |x'| of every diagonal element
  __shared__ __attribute__((aligned(16))) i32x4_t dig[16][3][64];   // [chunk][digit][lane]
  __shared__ float red[kDigitWaves][64];                             // per wave: partial sums of its rows

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nsl = a.slices;
  const int cps = (a.cpr + nsl - 1) / nsl;
  const int slice = wave % nsl;
  const int groups_per_block = kDigitWaves / nsl;
  const int grp = blockIdx.x * groups_per_block + wave / nsl;       // row group index over all classes
  const int cls = (blockIdx.x * groups_per_block) / a.waves_per_class;
  const int64_t i0 = static_cast<int64_t>(grp - cls * a.waves_per_class) * a.rows_per_wave;
  const int64_t V = a.row_stride;
  int nrows = 0;
  {
    const int64_t first = cls + V * i0;
    if (first < a.N) {
      const int64_t avail = (a.N - first + V - 1) / V;
      nrows = static_cast<int>(avail < a.rows_per_wave ? avail : a.rows_per_wave);
    }
  }
  const int64_t row_bytes = a.K;
  const int first_chunk = slice * cps;
  int my_chunks = a.cpr - first_chunk;                               // chunks of this wave's slice
  my_chunks = my_chunks < 0 ? 0 : (my_chunks > cps ? cps : my_chunks);

  // the activations and scales of chunk `wave` are requested before the first weight rows (see the kernel above)
  float xv[16];
  floatx4_t scv[4];
  const bool has_chunk = wave < a.cpr;
  if (has_chunk) {
    const XT *xg = static_cast<const XT *>(a.x) + (wave * 64 + lane) * 16;
#pragma unroll
    for (int t = 0; t < 16; ++t) xv[t] = to_f32<XT>(xg[t]);
    if (a.round_x == CAIFX_BF16) {
#pragma unroll
      for (int t = 0; t < 16; ++t) xv[t] = round_through<bf16_t>(xv[t]);
    } else if (a.round_x == CAIFX_F16) {
#pragma unroll
      for (int t = 0; t < 16; ++t) xv[t] = round_through<f16_t>(xv[t]);
    }
    if constexpr (kVec) {
      const float *sp = static_cast<const float *>(a.scales);
      const int idx = static_cast<int>((static_cast<int64_t>(cls) * a.K + (wave * 64 + lane) * 16) % a.period);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        int i = idx + 4 * q;
        if (i >= a.period) i -= a.period;
        scv[q] = *reinterpret_cast<const floatx4_t *>(sp + i);
      }
    }
  }
  float s_scalar = 1.0f;
  if constexpr (!kVec) {
    if (a.scales) s_scalar = static_cast<const float *>(a.scales)[0];
  }

  const uint8_t *wp = a.wq + (cls + V * i0) * row_bytes + first_chunk * 1024 + lane * 16;
  const int64_t rstep = V * row_bytes;
  i32x4_t w[D][CPS];
  // unconditional loads: a row past the wave's range, or a chunk past the slice, reads the activation row
  const uint8_t *wdummy = static_cast<const uint8_t *>(a.x) + lane * 16;
  auto issue = [&](int d, int r) {
    const uint8_t *wsrc = r < nrows ? wp + r * rstep : wdummy;
#pragma unroll
    for (int c = 0; c < CPS; ++c) w[d][c] = *reinterpret_cast<const i32x4_t *>(c < my_chunks ? wsrc + c * 1024 : wdummy);
  };
#pragma unroll
  for (int d = 0; d < D; ++d) issue(d, d);

  if (has_chunk) {
    if constexpr (kVec) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int t = 0; t < 4; ++t) xv[4 * q + t] *= scv[q][t];
    }
    float m = 0.0f;
    bool finite = true;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      m = fmaxf(m, fabsf(xv[t]));
      finite = finite && fabsf(xv[t]) <= 3.4028235e38f;
    }
    m = finite ? m : __builtin_inff();
    m = fmaxf(m, __shfl_xor(m, 16));
    m = fmaxf(m, __shfl_xor(m, 32));
    if (lane < 16) mx[wave][lane] = m;
  }
  __syncthreads();

  // unit of diagonal element i within slice sl: the largest |x'| of the slice's chunks maps into [32, 64]
  auto slice_max = [&](int sl) {
    float m = 0.0f;
    for (int c = sl * cps; c < (sl + 1) * cps && c < a.cpr; ++c) m = fmaxf(m, mx[c][lane & 15]);
    return m;
  };
  auto unit_of = [&](float m) {
    int e = 0;
    (void)frexpf(m, &e);
    return (m > 0.0f && m <= 3.4028235e38f) ? ldexpf(1.0f, e - 6) : 1.0f;
  };
  bool poisoned;       // the same in every wave of the workgroup
  {
    float m = 0.0f;
    for (int c = 0; c < a.cpr; ++c) m = fmaxf(m, mx[c][lane & 15]);
    poisoned = __any(!(m <= 3.4028235e38f));
  }
  if (has_chunk) {
    const float unit_c = poisoned ? 1.0f : unit_of(slice_max(wave / cps));
    const float inv14 = 16384.0f / unit_c;
    i32x4_t d0, d1, d2;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int e0[4], e1[4], e2[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int b = __builtin_bit_cast(int, __builtin_fmaf(xv[4 * q + t], inv14, 12582912.0f));
        e2[t] = __builtin_amdgcn_sbfe(b, 0, 7);
        e1[t] = __builtin_amdgcn_sbfe(b + 64, 7, 7);
        e0[t] = __builtin_amdgcn_sbfe(b + 64 + 8192, 14, 8);
      }
      d0[q] = static_cast<int>(pack_low_bytes(e0[0], e0[1], e0[2], e0[3]));
      d1[q] = static_cast<int>(pack_low_bytes(e1[0], e1[1], e1[2], e1[3]));
      d2[q] = static_cast<int>(pack_low_bytes(e2[0], e2[1], e2[2], e2[3]));
    }
    dig[wave][0][lane] = d0;
    dig[wave][1][lane] = d1;
    dig[wave][2][lane] = d2;
  }
  __syncthreads();
  const float unit = poisoned ? 1.0f : unit_of(slice_max(slice));
  i32x4_t xb[CPS][3];
#pragma unroll
  for (int c = 0; c < CPS; ++c)
#pragma unroll
    for (int d = 0; d < 3; ++d) xb[c][d] = c < my_chunks ? dig[first_chunk + c][d][lane] : i32x4_t{0, 0, 0, 0};
  const float u0 = unit * s_scalar, u1 = u0 * (1.0f / 128.0f), u2 = u0 * (1.0f / 16384.0f);
  const int tsel = lane & 3;
  const bool is_diag = (lane >> 4) == ((lane & 15) >> 2);

  float res = 0.0f;          // lane r: this slice's share of the result of the wave's row r
  for (int r0 = 0; r0 < nrows; r0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int r = r0 + d;
      if (r < nrows) {
        i32x4_t s0 = {0, 0, 0, 0}, s1 = {0, 0, 0, 0}, s2 = {0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < CPS; ++c) {
          s0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[d][c], xb[c][0], s0, 0, 0, 0);
          s1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[d][c], xb[c][1], s1, 0, 0, 0);
          s2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[d][c], xb[c][2], s2, 0, 0, 0);
        }
        int p0 = s0[0], p1 = s1[0], p2 = s2[0];
        p0 = tsel == 1 ? s0[1] : p0;  p1 = tsel == 1 ? s1[1] : p1;  p2 = tsel == 1 ? s2[1] : p2;
        p0 = tsel == 2 ? s0[2] : p0;  p1 = tsel == 2 ? s1[2] : p1;  p2 = tsel == 2 ? s2[2] : p2;
        p0 = tsel == 3 ? s0[3] : p0;  p1 = tsel == 3 ? s1[3] : p1;  p2 = tsel == 3 ? s2[3] : p2;
        float v = static_cast<float>(p0) * u0;
        v = __builtin_fmaf(static_cast<float>(p1), u1, v);
        v = __builtin_fmaf(static_cast<float>(p2), u2, v);
        v = wave_sum_hi(is_diag ? v : 0.0f);
        res = lane_insert(res, v, r);
      }
      issue(d, r + D);
    }
  }
  red[wave][lane] = res;
  __syncthreads();
  if (slice == 0 && lane < nrows) {
    float v = res;
    for (int sl = 1; sl < nsl; ++sl) v += red[wave + sl][lane];
    static_cast<float *>(a.y)[cls + V * (i0 + lane)] = poisoned ? __builtin_nanf("") : v;
  }
}


// ------------------------------------------------------------------ int8, exact
// kVec: per-channel scales (period > 1) cached in registers per residue class.
template <typename CT, typename XT, int MT, bool kVec, int CPR>
__global__ __launch_bounds__(256) void rowlin_int8_kernel(RowArgs a)
{
  typedef typename Mfma16<CT>::vec_t vec_t;
  constexpr int RB = (CPR == 1) ? 8 : (CPR == 2 ? 4 : 2);   // rows in flight (RB*CPR 16-byte loads per lane)
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  CT *xs = reinterpret_cast<CT *>(smem);                    // [MT][xpitch]

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int gw = blockIdx.x * 4 + wave;
  const int cls = gw / a.waves_per_class;                   // residue class v (0 when row_stride == 1)
  const int64_t i0 = static_cast<int64_t>(gw - cls * a.waves_per_class) * a.rows_per_wave;
  const int64_t V = a.row_stride;
  // rows of this wave: n = cls + V * (i0 + t), t < nrows
  int nrows = 0;
  if (gw < a.total_waves) {
    const int64_t first = cls + V * i0;
    if (first < a.N) {
      const int64_t avail = (a.N - first + V - 1) / V;
      nrows = static_cast<int>(avail < a.rows_per_wave ? avail : a.rows_per_wave);
    }
  }
  const int slots = static_cast<int>(a.K >> 4);             // 16-code slots per row

  // scales of this residue class for this lane's slots
  floatx4_t sc[CPR][4];
  float s_scalar = 1.0f;
  if constexpr (kVec) {
    const float *sp = static_cast<const float *>(a.scales);
#pragma unroll
    for (int c = 0; c < CPR; ++c) {
      const int slot = c * 64 + lane;
      const int64_t k0 = static_cast<int64_t>(slot < slots ? slot : 0) << 4;
      int idx = static_cast<int>((static_cast<int64_t>(cls) * a.K + k0) % a.period);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        int i = idx + 4 * q;
        if (i >= a.period) i -= a.period;
        sc[c][q] = *reinterpret_cast<const floatx4_t *>(sp + i);
      }
    }
  } else {
    if (a.scales) s_scalar = static_cast<const float *>(a.scales)[0];
  }

  u32x4_t wreg[RB][CPR];
  auto issue = [&](int rb, int t) {
    const uint8_t *rowp = a.wq + (cls + V * (i0 + t)) * a.K;
#pragma unroll
    for (int c = 0; c < CPR; ++c) {
      const int slot = c * 64 + lane;
      u32x4_t w = {0u, 0u, 0u, 0u};
      if (slot < slots) w = *reinterpret_cast<const u32x4_t *>(rowp + static_cast<int64_t>(slot) * 16);
      wreg[rb][c] = w;
    }
  };
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
    if (rb < nrows) issue(rb, rb);

  stage_x<CT, XT, MT, false>(a, xs, nullptr);
  __syncthreads();

  for (int t0 = 0; t0 < nrows; t0 += RB) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int t = t0 + rb;
      if (t < nrows) {
        u32x4_t w[CPR];
#pragma unroll
        for (int c = 0; c < CPR; ++c) w[c] = wreg[rb][c];
        if (t + RB < nrows) issue(rb, t + RB);
        floatx4_t acc[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[m] = floatx4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int c = 0; c < CPR; ++c) {
          const CT *xb = xs + (c * 2 * 64 + lane) * 8;
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            float lo[4], hi[4];
            int8x4_to_f32(w[c][2 * j], lo);
            int8x4_to_f32(w[c][2 * j + 1], hi);
            vec_t av;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float s0 = kVec ? sc[c][2 * j][q] : s_scalar;
              const float s1 = kVec ? sc[c][2 * j + 1][q] : s_scalar;
              av[q] = from_f32<CT>(lo[q] * s0);
              av[4 + q] = from_f32<CT>(hi[q] * s1);
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) {
              const vec_t bv = *reinterpret_cast<const vec_t *>(xb + m * a.xpitch + j * 64 * 8);
              acc[m] = Mfma16<CT>::run(av, bv, acc[m]);
            }
          }
        }
        const int64_t nrow = cls + V * (i0 + t);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const float v = wave_sum_hi(diag_of(acc[m], lane));
          if (lane == 63 && m < a.M) store_y(a.y, a.y_dtype, static_cast<int64_t>(m) * a.N + nrow, v);
        }
      }
    }
  }
}

template <typename CT, int MT, int CPR>
int launch_int4_fast(const RowArgs &ra, hipStream_t s)
{
  const size_t lds = static_cast<size_t>((MT * CPR * 16 + 3) & ~3) * 4 + static_cast<size_t>(MT) * CPR * 2048 * 2;
  hipLaunchKernelGGL((rowlin_int4_fast_kernel<CT, MT, CPR>),
                     dim3(static_cast<unsigned>((ra.total_waves + kInt4FastWaves - 1) / kInt4FastWaves)), dim3(kInt4FastWaves * 64),
                     lds, s, ra);
  return launch_status();
}

template <typename CT, int MT, bool kVec, int CPR>
int launch_int8_fast(const RowArgs &ra, hipStream_t s)
{
  const size_t lds = static_cast<size_t>(MT) * CPR * 1024 * 2;
  hipLaunchKernelGGL((rowlin_int8_fast_kernel<CT, MT, kVec, CPR>), dim3(static_cast<unsigned>((ra.total_waves + 3) / 4)),
                     dim3(256), lds, s, ra);
  return launch_status();
}

template <typename CT, typename XT, int MT>
int launch_int4(const RowArgs &ra, hipStream_t s)
{
  if constexpr (dtype_code<XT>::value == dtype_code<CT>::value) {
    const bool full = (ra.K % 2048 == 0) && ra.group_shift == 7 && ra.y_dtype == CAIFX_F32;
    if (full && ra.cpr == 1) return launch_int4_fast<CT, MT, 1>(ra, s);
    if (full && ra.cpr == 2) return launch_int4_fast<CT, MT, 2>(ra, s);
    if (full && ra.cpr == 4) return launch_int4_fast<CT, MT, 4>(ra, s);
    if constexpr (MT == 1) {      // long reductions with one activation row (a down projection at decode time)
      if (full && ra.cpr == 7) return launch_int4_fast<CT, MT, 7>(ra, s);
      if (full && ra.cpr == 8) return launch_int4_fast<CT, MT, 8>(ra, s);
    }
  }
  const size_t lds = static_cast<size_t>((MT * (ra.xpitch >> 7) + 3) & ~3) * 4 + static_cast<size_t>(MT) * ra.xpitch * 2;
  const unsigned grid = static_cast<unsigned>((ra.total_waves + 3) / 4);
  hipLaunchKernelGGL((rowlin_int4_kernel<CT, XT, MT>), dim3(grid), dim3(256), lds, s, ra);
  return launch_status();
}

template <typename XT, bool kVec, int CPR>
int launch_int8_digits(const RowArgs &ra, hipStream_t s)
{
  hipLaunchKernelGGL((rowlin_int8_digits_kernel<XT, kVec, CPR>), dim3(static_cast<unsigned>(ra.total_waves / kDigitWaves)), dim3(kDigitWaves * 64), 0, s, ra);
  return launch_status();
}

template <typename CT, typename XT, int MT, bool kVec>
int launch_int8(const RowArgs &ra, hipStream_t s)
{
  if constexpr (MT == 1) {
    if (ra.digits && ra.slices > 0) {
      hipLaunchKernelGGL((rowlin_int8_digits_long_kernel<XT, kVec>),
                         dim3(static_cast<unsigned>(ra.total_waves / (kDigitWaves / ra.slices))), dim3(kDigitWaves * 64), 0, s, ra);
      return launch_status();
    }
    if (ra.digits) {
      if (ra.cpr == 1) return launch_int8_digits<XT, kVec, 1>(ra, s);
      if (ra.cpr == 2) return launch_int8_digits<XT, kVec, 2>(ra, s);
      return launch_int8_digits<XT, kVec, 4>(ra, s);
    }
  }
  if constexpr (dtype_code<XT>::value == dtype_code<CT>::value) {
    const bool full = (ra.K % 1024 == 0) && ra.y_dtype == CAIFX_F32;
    if (full && ra.cpr == 1) return launch_int8_fast<CT, MT, kVec, 1>(ra, s);
    if (full && ra.cpr == 2) return launch_int8_fast<CT, MT, kVec, 2>(ra, s);
    if (full && ra.cpr == 4) return launch_int8_fast<CT, MT, kVec, 4>(ra, s);
  }
  const size_t lds = static_cast<size_t>(MT) * ra.xpitch * 2;
  const unsigned grid = static_cast<unsigned>((ra.total_waves + 3) / 4);
  switch (ra.cpr) {
    case 1: hipLaunchKernelGGL((rowlin_int8_kernel<CT, XT, MT, kVec, 1>), dim3(grid), dim3(256), lds, s, ra); break;
    case 2: hipLaunchKernelGGL((rowlin_int8_kernel<CT, XT, MT, kVec, 2>), dim3(grid), dim3(256), lds, s, ra); break;
    case 3: hipLaunchKernelGGL((rowlin_int8_kernel<CT, XT, MT, kVec, 3>), dim3(grid), dim3(256), lds, s, ra); break;
    case 4: hipLaunchKernelGGL((rowlin_int8_kernel<CT, XT, MT, kVec, 4>), dim3(grid), dim3(256), lds, s, ra); break;
    default: return CAIFX_ERR_UNSUPPORTED;
  }
  return launch_status();
}

template <typename CT, typename XT, int MT>
int pick_kind(const RowArgs &ra, int kind, hipStream_t s)
{
  if (kind == 0) return launch_int4<CT, XT, MT>(ra, s);
  if (kind == 1) return launch_int8<CT, XT, MT, false>(ra, s);
  return launch_int8<CT, XT, MT, true>(ra, s);
}

template <typename CT, typename XT>
int pick_m(const RowArgs &ra, int kind, hipStream_t s)
{
  if (ra.M == 1) return pick_kind<CT, XT, 1>(ra, kind, s);
  if (ra.M == 2) return pick_kind<CT, XT, 2>(ra, kind, s);
  return pick_kind<CT, XT, 4>(ra, kind, s);
}

template <typename CT>
int pick_xt(const RowArgs &ra, int x_dtype, int kind, hipStream_t s)
{
  switch (x_dtype) {
    case CAIFX_F32: return pick_m<CT, float>(ra, kind, s);
    case CAIFX_F16: return pick_m<CT, f16_t>(ra, kind, s);
    default: return pick_m<CT, bf16_t>(ra, kind, s);
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

int64_t compute_unit_count()
{
  static std::atomic<int> cached{0};
  int n = cached.load(std::memory_order_relaxed);
  if (n == 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached.store(n, std::memory_order_relaxed);
  }
  return n;
}

int pick_rows_per_wave(int64_t rows, int min_rows, int64_t target = 2048)
{
  // aim for two waves per SIMD (2048 waves): each walks its rows through a ring of loads, so
  // unpacking overlaps the HBM latency of the rows behind it
  int64_t rpw = (rows + target - 1) / target;
  if (rpw < min_rows) rpw = min_rows;
  if (rpw > 64) rpw = 64;
  return static_cast<int>(rpw);
}

}  // namespace

int rowlin_forward(const GemmArgs &g, hipStream_t s)
{
  if (g.offsets || g.M < 1 || g.M > 4 || g.compute_dtype == CAIFX_F32) return CAIFX_ERR_UNSUPPORTED;
  if (g.N < 1 || g.N > (int64_t{1} << 30) || g.K > (int64_t{1} << 20)) return CAIFX_ERR_UNSUPPORTED;
  if (!aligned_to(g.w.q, 16) || !aligned_to(g.x, 16)) return CAIFX_ERR_UNSUPPORTED;
  const bool int4 = g.w.kind == CAIFX_W_INT4_GROUP;

  RowArgs ra{};
  ra.wq = static_cast<const uint8_t *>(g.w.q);
  ra.scales = g.w.scales;
  ra.x = g.x;
  ra.y = g.y;
  ra.M = static_cast<int>(g.M);
  ra.y_dtype = g.y_dtype;
  ra.N = g.N;
  ra.K = g.K;
  ra.row_stride = 1;
  const int mt = g.M == 3 ? 4 : static_cast<int>(g.M);
  int kind;
  if (int4) {
    const int gs = g.w.group_size;
    if (!g.w.scales || gs < 128 || (gs & (gs - 1)) != 0 || g.K % 128 != 0) return CAIFX_ERR_UNSUPPORTED;
    ra.group_shift = __builtin_ctz(static_cast<unsigned>(gs));
    kind = 0;
    ra.cpr = static_cast<int>((g.K + 2047) / 2048);
    ra.xpitch = ra.cpr * 2048;
    ra.rows_per_wave = pick_rows_per_wave(g.N, (8 + ra.cpr - 1) / ra.cpr);
    ra.total_waves = static_cast<int>((g.N + ra.rows_per_wave - 1) / ra.rows_per_wave);
    ra.waves_per_class = ra.total_waves;
    if (static_cast<size_t>(mt) * ra.xpitch * 2 + 4096 > 64 * 1024) return CAIFX_ERR_UNSUPPORTED;
  } else {
    // one activation row and 4096 < K <= 16384: the integer-matrix-core kernel with the row split among waves
    const bool long_digits = g.M == 1 && g.K > 4096 && g.K <= 16384 && g.K % 1024 == 0 && g.y_dtype == CAIFX_F32;
    if (g.K % 16 != 0 || (g.K > 4096 && !long_digits)) return CAIFX_ERR_UNSUPPORTED;
    ra.cpr = static_cast<int>((g.K + 1023) / 1024);
    ra.xpitch = ra.cpr * 1024;
    if (!g.w.scales || g.w.scale_period == 1) {
      kind = 1;
    } else {
      const int64_t P = g.w.scale_period;
      if (P % 4 != 0 || P < 16 || P > (int64_t{1} << 30) || !aligned_to(g.w.scales, 16)) return CAIFX_ERR_UNSUPPORTED;
      kind = 2;
      ra.period = static_cast<int>(P);
      const int64_t V = P / gcd64(g.K % P == 0 ? P : g.K % P, P);
      if (V * 256 > g.N) return CAIFX_ERR_UNSUPPORTED;   // too few rows per residue class to amortise the scales
      ra.row_stride = static_cast<int>(V);
    }
    const int64_t rows_class = (g.N + ra.row_stride - 1) / ra.row_stride;
    const int rb = ra.cpr == 1 ? 8 : (ra.cpr == 2 ? 4 : 2);
    const bool digits = long_digits || (g.M == 1 && g.K % 1024 == 0 && (ra.cpr == 1 || ra.cpr == 2 || ra.cpr == 4) && g.y_dtype == CAIFX_F32);
    if (long_digits) {
      // wave w of a workgroup takes slice w % slices of the rows of row group w / slices; waves_per_class and
      // total_waves count row groups here
      ra.slices = ra.cpr > 8 ? 4 : 2;
      ra.digits = 1;
      ra.round_x = g.x_dtype != g.compute_dtype ? g.compute_dtype : -1;
      const int groups_per_block = kDigitWaves / ra.slices;
      const int64_t cus = compute_unit_count();
      ra.rows_per_wave = 1;
      while (ra.rows_per_wave < 64 &&
             ra.row_stride * (((rows_class + ra.rows_per_wave - 1) / ra.rows_per_wave + groups_per_block - 1) / groups_per_block) > cus)
        ++ra.rows_per_wave;
      ra.waves_per_class = static_cast<int>((rows_class + ra.rows_per_wave - 1) / ra.rows_per_wave);
      ra.waves_per_class = (ra.waves_per_class + groups_per_block - 1) / groups_per_block * groups_per_block;
      ra.total_waves = ra.waves_per_class * ra.row_stride;
      if (g.compute_dtype == CAIFX_BF16) return pick_xt<bf16_t>(ra, g.x_dtype, kind, s);
      return pick_xt<f16_t>(ra, g.x_dtype, kind, s);
    }
    // the integer-matrix-core kernel is light on registers and arithmetic: four waves per SIMD measured best
    ra.rows_per_wave = digits ? pick_rows_per_wave(g.N, 1, 4096) : pick_rows_per_wave(g.N, kind == 2 ? 2 * rb : rb);
    if (digits) {
      // one workgroup per compute unit at a time (16 waves): keep the grid within one round when the rows allow
      const int64_t cus = compute_unit_count();
      while (ra.rows_per_wave < 64 &&
             ra.row_stride * (((rows_class + ra.rows_per_wave - 1) / ra.rows_per_wave + kDigitWaves - 1) / kDigitWaves) > cus)
        ++ra.rows_per_wave;
    }
    ra.waves_per_class = static_cast<int>((rows_class + ra.rows_per_wave - 1) / ra.rows_per_wave);
    if (digits) {
      ra.digits = 1;
      ra.round_x = g.x_dtype != g.compute_dtype ? g.compute_dtype : -1;
      ra.waves_per_class = (ra.waves_per_class + kDigitWaves - 1) / kDigitWaves * kDigitWaves;      // a workgroup stays inside one class
    }
    ra.total_waves = ra.waves_per_class * ra.row_stride;
    if (static_cast<size_t>(mt) * ra.xpitch * 2 > 64 * 1024) return CAIFX_ERR_UNSUPPORTED;
  }
  if (g.compute_dtype == CAIFX_BF16) return pick_xt<bf16_t>(ra, g.x_dtype, kind, s);
  return pick_xt<f16_t>(ra, g.x_dtype, kind, s);
}

}  // namespace caifx
