// Large-M forward dequant-GEMM for int8 weights, Y = X * W^T, plain and over token-sorted expert segments, with
// the weight kept out of the shared operand tiles: the int8 form of caifx_gemm_regw.hip.
//
// A workgroup of eight waves owns a 128 x 256 tile of Y and walks K in steps of 64; wave w owns the 32 columns
// [32w, 32w+32) of the tile for all of its rows.  Lane (c = lane % 32, h = lane / 32) dequantises the 32 codes
// W[n0 + c][k0 + 32h .. + 31] of a step in registers (float(code) * scale in fp32, one rounding to the compute
// type: the reference's dequantise-then-cast weight, bit for bit) into the four B operands of the step's four
// v_mfma_f32_32x32x16; the activations follow the same permutation of the step's 64 reduction indices.
//   * codes: one request moves 8 weight rows x 128 bytes (the codes of two steps) into one of ten 1 KiB slots of
//     the wave's private LDS ring; two requests per wave and step, ten requests ahead.  Request u (rows 8 (u % 4) ..,
//     block u / 4) is issued in step (u - 10) / 2, has landed when the barrier of step (u - 10) / 2 + 2 is passed
//     and is first read in step 2 (u / 4) - 1; its slot was last read in step 2 ((u - 10) / 4) <= (u - 10) / 2.
//   * scales: the reference addresses an int8 scale vector of P entries by the flat index (n K + k) mod P, so along
//     a weight row the scales change with k, and from row to row the run starts K mod P further on: the starts of
//     all rows differ by multiples of G = gcd(K mod P, P).  The vector sits in LDS for the whole tile, cut into
//     rows of G entries (one row when P divides K) with a pitch of 4 mod 64 floats, so the 16 lanes of one pass of
//     a 128-bit LDS read (16 consecutive weight rows) either read the same address or, with different table
//     rows, banks 16 bytes apart per table row instead of the same bank.  A lane reads the 32 scales of its 32
//     codes as eight such reads from one address.  One scale (or none) is a table of 64 equal entries.
//   * activations, barrier placement, hand-counted waits and the store are those of the int4 kernel.
// A tile with fewer than 128 valid rows (the last row tile of a segment or of M) runs the matrix cores over its
// 32-row blocks that hold rows only; the dequantisation is the same, so such a tile is bound by it.
// Grouped form: tiles are numbered expert by expert, row tile by row tile, column tile last, and XCD x (workgroup
// id mod 8) takes the x-th contiguous eighth of the list, so one expert's weight is fetched into one L2.
#include "caifx_gemm_regw.hpp"

#include <atomic>
#include <type_traits>

namespace caifx {
namespace {

using regw::kBK;
using regw::kBN;
using regw::kStages;
using regw::swz;
constexpr int BM = 128;
constexpr int WR = BM / 32;
constexpr int kWSlots = 10;
constexpr int kWAheadReq = 10;
constexpr int kStageBytes = BM * kBK * 2;
constexpr int kDma = BM / 64;          // activation requests per wave and step (8 rows each)
constexpr int kWBase = kStages * kStageBytes;            // LDS: activation ring, code rings, scale table
constexpr int kTBase = kWBase + 8 * kWSlots * 1024;
constexpr int kTableBytes = 16 * 1024;

struct Regw8Args {
  int64_t M, N, K;
  const void *a;             // X [M, K] in the compute type
  void *d;                   // Y [M, N]
  int d_dtype;
  const void *addend;        // optional [M, N] of d_dtype: d = T(float(T(acc)) + float(addend))
  const void *gate;          // optional, with d2 (16-bit results): d2 = T(T(silu(gate)) * d), the gated expert's hidden
  void *d2;
  const uint8_t *wq;         // plain form
  const float *scales;
  int has_vector;            // 0: the table is 64 copies of scales[0] (1 without scales)
  int period;                // entries of the table
  int row_len;               // the table is cut into rows of this many entries ...
  int row_pitch;             // ... this many floats apart
  const int32_t *offsets;    // grouped form
  const void *const *wq_ptrs;
  const void *const *scales_ptrs;
  int num_experts;
  unsigned long long *stamps;       // grouped form, measurement only
  long long stamps_capacity;
};

// a 64-bit value every lane holds alike, moved to scalar registers (the direct-to-LDS requests take their base there)
__device__ __forceinline__ uint64_t uniform64(uint64_t v)
{
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
  return (static_cast<uint64_t>(hi) << 32) | lo;
}

template <typename CT, bool kGrouped>
__global__ __launch_bounds__(512, 2) void qgemm_regw8_kernel(Regw8Args g)
{
  typedef typename Mfma32<CT>::vec_t vec_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int frow = lane & 31;
  const int fh = lane >> 5;

  // ---- which tile
  int64_t row0, row_end, col0;
  const uint8_t *wq = g.wq;
  const float *scales = g.scales;
  int64_t stamp_pos = -1;
  const int64_t col_tiles = (g.N + kBN - 1) / kBN;
  if constexpr (kGrouped) {
    GroupedTile gt;
    if (!grouped_tile<BM>(g.offsets, g.num_experts, g.M, col_tiles, g.wq_ptrs, g.scales_ptrs, lane, gt)) return;
    const int e = gt.e;
    const int64_t pos = gt.pos;
    col0 = gt.col_tile * kBN;
    row0 = gt.row0;
    row_end = gt.row_end;
    wq = static_cast<const uint8_t *>(gt.wq);
    scales = static_cast<const float *>(gt.scales);
    if (g.stamps && threadIdx.x == 0 && pos < g.stamps_capacity) {
      const int64_t rows = row_end - row0 < BM ? row_end - row0 : BM;
      g.stamps[4 * pos] = static_cast<unsigned long long>(e);
      g.stamps[4 * pos + 1] = static_cast<unsigned long long>(rows) | (1ull << 32);      // one workgroup per compute unit
      g.stamps[4 * pos + 2] = wall_clock64();
      stamp_pos = pos;
    }
  } else {
    // as in the int4 kernel: 512-row bands column by column, one contiguous eighth of the list per XCD
    constexpr int kBandTiles = 512 / BM;
    const int64_t row_tiles = (g.M + BM - 1) / BM;
    const unsigned bid = blockIdx.x;
    const int64_t per_xcd = gridDim.x >> 3;
    const int64_t pos = static_cast<int64_t>(bid & 7) * per_xcd + (bid >> 3);
    if (pos >= row_tiles * col_tiles) return;
    const int64_t band = pos / (kBandTiles * col_tiles);
    const int64_t within = pos - band * kBandTiles * col_tiles;
    const int64_t left = row_tiles - band * kBandTiles;
    const int64_t band_rows = left < kBandTiles ? left : kBandTiles;
    col0 = (within / band_rows) * kBN;
    row0 = (band * kBandTiles + within % band_rows) * BM;
    row_end = g.M;
  }
  const int valid_rows = static_cast<int>(row_end - row0 < BM ? row_end - row0 : BM);
  const int nblk = __builtin_amdgcn_readfirstlane((valid_rows + 31) >> 5);        // 32-row blocks that hold rows

  // ---- request set-up (see the int4 kernel)
  uint32_t a_voff[kDma];
#pragma unroll
  for (int i = 0; i < kDma; ++i) {
    const int row = 8 * (wave + 8 * i) + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row ^ (row >> 3)) & 7);
    int64_t m = row0 + row;
    if (m >= row_end) m = row_end - 1;                // rows past the end are loaded from the last row and never stored
    a_voff[i] = static_cast<uint32_t>((m - row0) * g.K * 2 + chunk * 16);
  }
  const uint64_t a_base = uniform64(reinterpret_cast<uint64_t>(g.a) + static_cast<uint64_t>(row0 * g.K * 2));
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem));
  // code request with u % 4 == i moves weight rows 8i .. 8i+7 of this wave's 32: lane L asks for piece
  // (L % 8) ^ r ^ (i & 1) of row r = L / 8, so piece p of that row sits at position p ^ r ^ (i & 1) of its LDS row
  uint32_t w_voff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = lane >> 3;
    int64_t n = col0 + wave * 32 + 8 * i + r;
    if (n >= g.N) n = g.N - 1;                        // columns past the end: loaded, never stored
    w_voff[i] = static_cast<uint32_t>(n * g.K) + 16 * ((lane & 7) ^ r ^ (i & 1));       // N * K < 2^32 (host)
  }
  const uint64_t w_base = uniform64(reinterpret_cast<uint64_t>(wq));

  const int steps = static_cast<int>(g.K / kBK);
  const int last = steps - 1;
  const int last_block = static_cast<int>(g.K / 128) - 1;

  int issue_slot = 0;      // u % kWSlots of the next code request
  auto issue_a = [&](auto set_, int t) __attribute__((always_inline)) {
    constexpr int set = decltype(set_)::value;
    const uint32_t k0 = static_cast<uint32_t>(t < last ? t : last) * kBK;       // past the end: the last step again
    const uint64_t a_src = a_base + 2 * k0;
#pragma unroll
    for (int i = 0; i < kDma; ++i) {
      const uint32_t dst = lds0 + set * kStageBytes + (wave + 8 * i) * 1024;
      const uint32_t voff = a_voff[i];
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(voff), "s"(a_src) : "memory");
    }
  };
  auto issue_w = [&](auto i_, int block) __attribute__((always_inline)) {
    constexpr int i = decltype(i_)::value;
    const uint32_t b = static_cast<uint32_t>(block < last_block ? block : last_block);   // past the end: the last block again
    const uint64_t w_src = w_base + 128 * b;
    const uint32_t dst = lds0 + kWBase + (wave * kWSlots + issue_slot) * 1024;
    const uint32_t wv = w_voff[i];
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(wv), "s"(w_src) : "memory");
    issue_slot = issue_slot + 1 == kWSlots ? 0 : issue_slot + 1;
  };

  typedef std::integral_constant<int, 0> I0;
  typedef std::integral_constant<int, 1> I1;
  typedef std::integral_constant<int, 2> I2;
  typedef std::integral_constant<int, 3> I3;

  // before anything else: code requests 0..9 (blocks 0 and 1, half of block 2), activation stages 0..2
  issue_w(I0{}, 0);
  issue_w(I1{}, 0);
  issue_w(I2{}, 0);
  issue_w(I3{}, 0);
  issue_w(I0{}, 1);
  issue_w(I1{}, 1);
  issue_w(I2{}, 1);
  issue_w(I3{}, 1);
  issue_w(I0{}, 2);
  issue_w(I1{}, 2);
  issue_a(I0{}, 0);
  issue_a(I1{}, 1);
  issue_a(I2{}, 2);

  // ---- the scale table
  float *table = reinterpret_cast<float *>(smem + kTBase);
  if (g.has_vector) {
    for (int idx = 4 * static_cast<int>(threadIdx.x); idx < g.period; idx += 4 * 512) {
      const int ta = idx / g.row_len;
      const int tb = idx - ta * g.row_len;
      *reinterpret_cast<floatx4_t *>(table + ta * g.row_pitch + tb) = *reinterpret_cast<const floatx4_t *>(scales + idx);
    }
  } else if (threadIdx.x < 64) {
    table[threadIdx.x] = scales ? scales[0] : 1.0f;
  }
  // this lane's position in the table: flat index si of the first of its 32 codes of the coming step, as row sa
  // and offset sb of the layout; every step moves it on by 64
  int si, sa, sb;
  {
    int64_t n = col0 + wave * 32 + frow;
    if (n >= g.N) n = g.N - 1;
    si = static_cast<int>(static_cast<uint64_t>(n * g.K) % static_cast<uint64_t>(g.period)) + 32 * fh;
    if (si >= g.period) si -= g.period;
    sa = si / g.row_len;
    sb = si - sa * g.row_len;
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");

  // Step t's codes and scales of this lane; q = t % 2 says which half of the block's 128 codes
  const int my_req = frow >> 3;                                       // which of a block's four requests holds this lane's row
  const int my_row = (frow & 7) * 128;
  const int my_x = (frow & 7) ^ (my_req & 1);
  struct WRaw {
    u32x4_t c[2];
    floatx4_t s[8];
    int so;              // byte offset of the lane's 32 scales in the table
  };
  auto fetch_w = [&](auto q_, int t, WRaw &w) __attribute__((always_inline)) {
    constexpr int q = decltype(q_)::value;
    const int block = t >> 1;
    int slot = (4 * block) % kWSlots + my_req;
    if (slot >= kWSlots) slot -= kWSlots;
    const unsigned char *row = smem + kWBase + wave * (kWSlots * 1024) + slot * 1024 + my_row;
    w.c[0] = *reinterpret_cast<const u32x4_t *>(row + (((4 * q + 2 * fh) ^ my_x) << 4));
    w.c[1] = *reinterpret_cast<const u32x4_t *>(row + (((4 * q + 2 * fh + 1) ^ my_x) << 4));
    w.so = (sa * g.row_pitch + sb) * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) w.s[e] = *reinterpret_cast<const floatx4_t *>(smem + kTBase + w.so + 16 * e);
    sb += 64;
    if (sb >= g.row_len) {
      sb -= g.row_len;
      sa += 1;
    }
    si += 64;
    if (si >= g.period) {
      si -= g.period;
      sa = 0;
      sb = si;
    }
  };
  auto fetch_w_rest = [&](WRaw &w) __attribute__((always_inline)) {
#pragma unroll
    for (int e = 4; e < 8; ++e) w.s[e] = *reinterpret_cast<const floatx4_t *>(smem + kTBase + w.so + 16 * e);
  };
  // codes 8j .. 8j+7 of the lane's 32 times their scales, rounded to CT: B operand j of the step
  auto dequant_one = [&](const WRaw &w, int j, vec_t &out) __attribute__((always_inline)) {
    u32x4_t v;
#pragma unroll
    for (int hw = 0; hw < 2; ++hw) {
      float f[4];
      int8x4_to_f32(w.c[j >> 1][2 * (j & 1) + hw], f);
      const floatx4_t sc = w.s[2 * j + hw];
      v[2 * hw] = pack2<CT>(f[0] * sc[0], f[1] * sc[1]);
      v[2 * hw + 1] = pack2<CT>(f[2] * sc[2], f[3] * sc[3]);
    }
    out = __builtin_bit_cast(vec_t, v);
  };

  floatx16_t acc[WR];
#pragma unroll
  for (int i = 0; i < WR; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;

  // the reduction over K with the matrix cores running over NB 32-row blocks
  auto run = [&](auto nb_) __attribute__((always_inline)) {
    constexpr int NB = decltype(nb_)::value;
    auto read_a = [&](auto set_, int j, vec_t (&out)[WR]) __attribute__((always_inline)) {
      constexpr int set = decltype(set_)::value;
      const unsigned char *abuf = smem + set * kStageBytes;
#pragma unroll
      for (int i = 0; i < NB; ++i) out[i] = *reinterpret_cast<const vec_t *>(abuf + swz(i * 32 + frow, 4 * fh + j));
    };
    auto mfma_row = [&](const vec_t (&a)[WR], const vec_t &b) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < NB; ++i) acc[i] = Mfma32<CT>::run(a[i], b, acc[i]);
    };
    if constexpr (NB == 0) {
      // a wave whose 32 columns lie beyond N: it only moves its share of the activation tiles and keeps the barriers
      auto idle_step = [&](auto ph_, int s) __attribute__((always_inline)) {
        constexpr int ph = decltype(ph_)::value;
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kDma) : "memory");
        issue_a(std::integral_constant<int, (ph + 3) % 4>{}, s + 3);
      };
      int s = 0;
      for (; s + 4 <= steps; s += 4) {
        idle_step(I0{}, s);
        idle_step(I1{}, s + 1);
        idle_step(I2{}, s + 2);
        idle_step(I3{}, s + 3);
      }
      if (s < steps) {
        idle_step(I0{}, s);
        idle_step(I1{}, s + 1);
      }
      return;
    }
    vec_t bfr[4];      // B operands of the current step
    vec_t afa[WR];     // A operands of its first MFMA row
    {
      WRaw w0;
      fetch_w(I0{}, 0, w0);
      fetch_w_rest(w0);
#pragma unroll
      for (int j = 0; j < 4; ++j) dequant_one(w0, j, bfr[j]);
    }
    read_a(I0{}, 0, afa);
    // Step s works on stage ph = s % 4; on entry its B operands are in registers and its first A operands on
    // their way.  Each of the step's four MFMA rows is written next to the LDS requests of the row after it and
    // a part of the dequantisation of step s + 1, and the compiler's scheduler is kept from moving work between rows.
    auto step = [&](auto ph_, int s) __attribute__((always_inline)) {
      constexpr int ph = decltype(ph_)::value;
      typedef std::integral_constant<int, (ph + 1) % 4> Next;
      typedef std::integral_constant<int, (ph + 1) % 2> NextHalf;
      vec_t afb[WR], bnext[4];
      WRaw wn;
      // row 0
      read_a(ph_, 1, afb);
      fetch_w(NextHalf{}, s + 1, wn);
      mfma_row(afa, bfr[0]);
      __builtin_amdgcn_sched_barrier(0);
      // row 1
      read_a(ph_, 2, afa);
      fetch_w_rest(wn);
      dequant_one(wn, 0, bnext[0]);
      mfma_row(afb, bfr[1]);
      __builtin_amdgcn_sched_barrier(0);
      // This wave's requests of every step but the last one have landed (requests complete in issue order);
      // behind the barrier stage s + 1 is there for everybody and stage s - 1 is free.
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kDma + 2) : "memory");
      issue_a(std::integral_constant<int, (ph + 3) % 4>{}, s + 3);
      {
        const int block = (s + kWAheadReq / 2) >> 1;
        if constexpr (ph % 2 == 0) {
          issue_w(I2{}, block);
          issue_w(I3{}, block);
        } else {
          issue_w(I0{}, block);
          issue_w(I1{}, block);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      // row 2
      read_a(ph_, 3, afb);
      dequant_one(wn, 1, bnext[1]);
      mfma_row(afa, bfr[2]);
      __builtin_amdgcn_sched_barrier(0);
      // row 3
      read_a(Next{}, 0, afa);
      dequant_one(wn, 2, bnext[2]);
      dequant_one(wn, 3, bnext[3]);
      mfma_row(afb, bfr[3]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < 4; ++j) bfr[j] = bnext[j];
    };
    int s = 0;
    for (; s + 4 <= steps; s += 4) {
      step(I0{}, s);
      step(I1{}, s + 1);
      step(I2{}, s + 2);
      step(I3{}, s + 3);
    }
    if (s < steps) {          // K is a multiple of 128: the steps come in pairs
      step(I0{}, s);
      step(I1{}, s + 1);
    }
  };
  const int idle = __builtin_amdgcn_readfirstlane(col0 + wave * 32 >= g.N ? 1 : 0);      // scalar: the branches hold barriers
  if (idle) run(std::integral_constant<int, 0>{});
  else if (nblk == 4) run(std::integral_constant<int, 4>{});
  else if (nblk == 3) run(std::integral_constant<int, 3>{});
  else if (nblk == 2) run(std::integral_constant<int, 2>{});
  else run(std::integral_constant<int, 1>{});
  // requests past the last step may still be writing LDS, and other waves may still be reading
  asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");

  if (g.d_dtype == CAIFX_BF16)
    regw::store_tile<bf16_t, WR>(smem, acc, wave, lane, row0, row_end, col0, g.N, static_cast<bf16_t *>(g.d), static_cast<const bf16_t *>(g.addend),
                                 static_cast<const bf16_t *>(g.gate), static_cast<bf16_t *>(g.d2));
  else if (g.d_dtype == CAIFX_F16)
    regw::store_tile<f16_t, WR>(smem, acc, wave, lane, row0, row_end, col0, g.N, static_cast<f16_t *>(g.d), static_cast<const f16_t *>(g.addend),
                                static_cast<const f16_t *>(g.gate), static_cast<f16_t *>(g.d2));
  else
    regw::store_tile<float, WR>(smem, acc, wave, lane, row0, row_end, col0, g.N, static_cast<float *>(g.d), static_cast<const float *>(g.addend));
  if constexpr (kGrouped) {
    if (stamp_pos >= 0) g.stamps[4 * stamp_pos + 3] = wall_clock64();
  }
}

template <typename CT, bool kGrouped> int launch(const Regw8Args &t, int64_t row_tiles, hipStream_t s)
{
  const size_t ring = static_cast<size_t>(kTBase) + kTableBytes;
  const size_t staging = regw::store_bytes(BM);
  const size_t lds = ring > staging ? ring : staging;
  auto kern = qgemm_regw8_kernel<CT, kGrouped>;
  static std::atomic<bool> raised{false};
  if (!raised.load(std::memory_order_relaxed)) {
    // the attribute is per kernel and sticky; two threads racing here both set it, which is harmless
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(lds)) != hipSuccess)
      return CAIFX_ERR_LAUNCH_FAILED;
    raised.store(true, std::memory_order_relaxed);
  }
  const int64_t tiles = row_tiles * ((t.N + kBN - 1) / kBN);
  const int64_t padded = (tiles + 7) / 8 * 8;
  if (padded > 0x7fffffff) return CAIFX_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(padded)), dim3(512), lds, s, t);
  return launch_status();
}

}  // namespace

int mfma_regw8_forward(const GemmArgs &a, hipStream_t s)
{
  const bool grouped = a.offsets != nullptr;
  if (a.w.kind != CAIFX_W_INT8) return CAIFX_ERR_UNSUPPORTED;
  if (a.epilogue != 0) {
    // the forward gating in the store: grouped launches with 16-bit results in 16-byte pieces
    if (a.epilogue != 1 || !grouped || a.addend || a.y_dtype == CAIFX_F32 || a.N % 8 != 0 || !a.e1 || !a.y2 ||
        !aligned_to(a.e1, 16) || !aligned_to(a.y2, 16))
      return CAIFX_ERR_UNSUPPORTED;
  }
  if (a.compute_dtype == CAIFX_F32 || a.x_dtype != a.compute_dtype) return CAIFX_ERR_UNSUPPORTED;
  if (a.K % 128 != 0 || a.K < 256 || a.K > (int64_t{1} << 22)) return CAIFX_ERR_UNSUPPORTED;
  if (a.N < 1 || a.N * a.K >= (int64_t{1} << 32) || a.M < 1 || a.M > (int64_t{1} << 30)) return CAIFX_ERR_UNSUPPORTED;
  if (!aligned_to(a.x, 16) || !aligned_to(a.y, 16) || (a.addend && !aligned_to(a.addend, 16))) return CAIFX_ERR_UNSUPPORTED;
  if (grouped) {
    if (!a.wq_ptrs || a.num_experts < 1) return CAIFX_ERR_UNSUPPORTED;
  } else if (!aligned_to(a.w.q, 16)) {
    return CAIFX_ERR_UNSUPPORTED;
  }
  // enough 128 x 256 tiles to give most compute units one; below that the tiled kernel's shared reduction wins
  const int64_t col_tiles = (a.N + kBN - 1) / kBN;
  if (((a.M + BM - 1) / BM) * col_tiles < 128) return CAIFX_ERR_UNSUPPORTED;

  Regw8Args t{};
  t.M = a.M;
  t.N = a.N;
  t.K = a.K;
  t.a = a.x;
  t.d = a.y;
  t.d_dtype = a.y_dtype;
  t.addend = a.addend;
  if (a.epilogue == 1) {
    t.gate = a.e1;
    t.d2 = a.y2;
  }
  t.wq = static_cast<const uint8_t *>(a.w.q);
  t.scales = static_cast<const float *>(a.w.scales);
  t.offsets = a.offsets;
  t.wq_ptrs = a.wq_ptrs;
  t.scales_ptrs = a.scales_ptrs;
  t.num_experts = a.num_experts;
  const bool has_scales = grouped ? a.scales_ptrs != nullptr : a.w.scales != nullptr;
  const int64_t P = a.w.scale_period;
  if (!has_scales || P <= 1) {
    t.has_vector = 0;
    t.period = 64;
    t.row_len = 64;
    t.row_pitch = 64;
  } else {
    // rows of gcd(K mod P, P) entries: the runs of different weight rows start whole table rows apart
    if (P % 32 != 0 || P > 4096 || (!grouped && !aligned_to(a.w.scales, 16))) return CAIFX_ERR_UNSUPPORTED;
    int64_t len = P;
    for (int64_t r = a.K % P; r != 0;) {
      const int64_t t2 = len % r;
      len = r;
      r = t2;
    }
    if (len < 64) return CAIFX_ERR_UNSUPPORTED;
    const int64_t rows = (P + len - 1) / len;
    const int64_t pitch = rows == 1 ? len : len + ((4 - len % 64) + 64) % 64;
    if (rows * pitch * 4 > kTableBytes) return CAIFX_ERR_UNSUPPORTED;
    t.has_vector = 1;
    t.period = static_cast<int>(P);
    t.row_len = static_cast<int>(len);
    t.row_pitch = static_cast<int>(pitch);
  }
  if (grouped) {
    mfma_grouped_stamp_target(&t.stamps, &t.stamps_capacity);
    // segment lengths live on the device: the grid is an upper bound, every expert can add one partial tile
    const int64_t row_tiles = (a.M + BM - 1) / BM + a.num_experts;
    return a.compute_dtype == CAIFX_BF16 ? launch<bf16_t, true>(t, row_tiles, s) : launch<f16_t, true>(t, row_tiles, s);
  }
  const int64_t row_tiles = (a.M + BM - 1) / BM;
  return a.compute_dtype == CAIFX_BF16 ? launch<bf16_t, false>(t, row_tiles, s) : launch<f16_t, false>(t, row_tiles, s);
}

}  // namespace caifx
