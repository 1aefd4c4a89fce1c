// Large-M forward dequant-GEMM for packed int4 weights (groups of 128), Y = X * W^T, with the weight kept out of
// the shared operand tiles.
//
// A workgroup of eight waves owns a 128 x 256 tile of Y and walks K in steps of 64.  Wave w owns the 32 columns
// [32w, 32w+32) of the tile for all of its rows:
//   * the weight: lane (c = lane % 32, h = lane / 32) dequantises the 32 codes W[n0 + c][k0 + 32h .. + 31] of a
//     step in registers (code * scale in fp32, one rounding to the compute type: the reference's
//     dequantise-then-cast weight, bit for bit) into the four B operands of the step's four v_mfma_f32_32x32x16.
//     MFMA j of a step therefore reduces over k0 + 32h + 8j .. + 7 for lane half h: a permutation of the step's
//     64 reduction indices, which a sum does not care about as long as the A operand follows it.  No wave ever
//     needs another wave's weights: nothing dequantised is written anywhere and W needs no barrier;
//   * the packed codes reach the wave in whole cache lines: one request moves 8 weight rows x 128 bytes (256
//     codes of each row, the reduction range of four steps) into one of ten 1 KiB slots of the wave's private
//     LDS ring, one request per wave and step, seven steps ahead.  Asking for the 32 bytes a step needs when it
//     needs them makes every line travel from L2 four times and measured 2.5 times the cost of the activations,
//     which are twice the bytes;
//   * the activations: the 128 x 64 tile of X of a step is brought into a four-stage LDS ring by
//     global_load_lds_dwordx4 as well (each wave moves 8 rows of 128 bytes per request; no registers, no VALU).
//     A lane asks for the global 16-byte chunk that belongs into its LDS slot under the XOR swizzle, so the
//     128-bit operand reads are conflict free; the code slots are swizzled likewise.
// Requests run two steps ahead of the barrier that publishes them.  That barrier sits in the middle of a step:
// behind the first half of step s's MFMAs every wave waits for its own requests of stage s + 1 and meets the
// others, which also proves that everybody has left stage s - 1, so the requests of stage s + 3 go there.  The
// second half of the step's MFMAs then runs beside the first operand reads and the dequantisation of stage
// s + 1, so the matrix pipe is not drained at a step's edge.
// Every global request of the loop is written as inline asm and none returns into a register: requests complete
// in issue order, so "all but the newest n" is an exact s_waitcnt, which the compiler cannot know while a direct
// load is pending (it would drain the queue before every LDS read), and a register result would have to stay
// untouched between its request and the hand-placed wait, which the compiler does not promise.
// The store goes through LDS as a whole tile so that one wave instruction writes one contiguous row piece of the
// tile (1 KiB of fp32) instead of eight 128-byte pieces.
#include "caifx_gemm_regw.hpp"

#include <atomic>
#include <type_traits>

namespace caifx {
namespace {

using regw::kBK;
using regw::kBN;
using regw::kStages;
using regw::swz;
constexpr int kWAhead = 7;     // code request u (8 weight rows x 256 codes: rows 8 (u % 4) .., block u / 4) is issued in step u - 7
constexpr int kWSlots = 10;    // ... into slot u % 10 of the wave's ring
constexpr int kGroup = 128;    // int4 group size this kernel is written for: one scale dword per weight row and block

struct RegwArgs {
  int64_t M, N, K;
  const void *a;             // X [M, K] in the compute type
  void *d;                   // Y [M, N]
  int d_dtype;
  const void *addend;        // optional [M, N] of d_dtype: d = T(float(T(acc)) + float(addend))
  const uint8_t *wq;
  const f16_t *scales;
};

// eight int4 codes of one dword (nibble t = element t) times one scale, rounded to CT: fma(code + 8, s, -8 s) is
// the exact product float(code) * s (m8 = -8 s and s16 = s / 16 are exact), so the only rounding is the cast.
// The odd elements stay in the high nibbles of their bytes (16 (code + 8)) and meet s / 16 instead of a shift.
template <typename CT> __device__ __forceinline__ u32x4_t dequant_int4x8_packed(uint32_t p, float s, float s16, float m8)
{
  p ^= 0x88888888u;
  const uint32_t lo = p & 0x0F0F0F0Fu;
  const uint32_t hi = p & 0xF0F0F0F0u;
  u32x4_t v;
  v[0] = pack2<CT>(__builtin_fmaf(ubyte0_f32(lo), s, m8), __builtin_fmaf(ubyte0_f32(hi), s16, m8));
  v[1] = pack2<CT>(__builtin_fmaf(ubyte1_f32(lo), s, m8), __builtin_fmaf(ubyte1_f32(hi), s16, m8));
  v[2] = pack2<CT>(__builtin_fmaf(ubyte2_f32(lo), s, m8), __builtin_fmaf(ubyte2_f32(hi), s16, m8));
  v[3] = pack2<CT>(__builtin_fmaf(ubyte3_f32(lo), s, m8), __builtin_fmaf(ubyte3_f32(hi), s16, m8));
  return v;
}

template <typename CT, int WR>
__global__ __launch_bounds__(512, 2) void qgemm_regw_kernel(RegwArgs g)
{
  constexpr int BM = 32 * WR;
  constexpr int kStageBytes = BM * kBK * 2;
  constexpr int kDma = BM / 64;          // activation requests per wave and step (8 rows each)
  constexpr int kWBase = kStages * kStageBytes;            // LDS: activation ring, code rings, scale rings
  constexpr int kSBase = kWBase + 8 * kWSlots * 1024;
  typedef typename Mfma32<CT>::vec_t vec_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int frow = lane & 31;
  const int fh = lane >> 5;

  // ---- which tile: XCD x (workgroup id mod 8) walks the x-th contiguous eighth of a list that runs through
  // 512-row bands column by column, so the tiles an XCD works on at a time share rows of X and columns of W in its L2
  constexpr int kBandTiles = 512 / BM;
  const int64_t col_tiles = (g.N + kBN - 1) / kBN;
  const int64_t row_tiles = (g.M + BM - 1) / BM;
  int64_t row0, col0;
  {
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
  }

  // ---- request set-up ------------------------------------------------------------------------------------
  // activation request i of this wave fills LDS rows 8q .. 8q+7 of a stage, q = wave + 8 i; LDS slot (row, pos)
  // holds chunk pos ^ f(row) of the row, so that is the chunk this lane asks for
  uint32_t a_voff[BM / 64];
#pragma unroll
  for (int i = 0; i < BM / 64; ++i) {
    const int row = 8 * (wave + 8 * i) + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row ^ (row >> 3)) & 7);
    int64_t m = row0 + row;
    if (m >= g.M) m = g.M - 1;                        // rows past the end are loaded from the last row and never stored
    a_voff[i] = static_cast<uint32_t>((m - row0) * g.K * 2 + chunk * 16);
  }
  const uint64_t a_base = reinterpret_cast<uint64_t>(g.a) + static_cast<uint64_t>(row0 * g.K * 2);
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem));   // LDS byte address (low half of the flat address)
  // code request with u % 4 == i moves weight rows 8i .. 8i+7 of this wave's 32: lane L asks for piece
  // (L % 8) ^ r ^ (i & 1) of row r = L / 8, so that piece p of that row sits at position p ^ r ^ (i & 1) of its
  // 128-byte LDS row and the operand reads of 16 neighbouring lanes (two requests' rows) spread over all banks
  uint32_t w_voff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = lane >> 3;
    int64_t n = col0 + wave * 32 + 8 * i + r;
    if (n >= g.N) n = g.N - 1;                        // columns past the end: loaded, never stored
    w_voff[i] = static_cast<uint32_t>((n * g.K) >> 1) + 16 * ((lane & 7) ^ r ^ (i & 1));       // N * K < 2^32 (host)
  }
  // scale request: the dword with the two scales of this lane's weight row in a block of 256 codes
  uint32_t s_voff;
  {
    int64_t n = col0 + wave * 32 + frow;
    if (n >= g.N) n = g.N - 1;
    s_voff = static_cast<uint32_t>((n * g.K / kGroup) * 2);
  }
  const uint64_t w_base = reinterpret_cast<uint64_t>(g.wq);
  const uint64_t s_base = reinterpret_cast<uint64_t>(g.scales);

  const int steps = static_cast<int>(g.K / kBK);
  const int last = steps - 1;
  const int last_block = static_cast<int>(g.K / 256) - 1;

  // requests of one step, in this order: the activation tile of step t, code request u, and with u % 4 == 0 the
  // scales of block u / 4 (three scale slots per wave)
  int issue_slot = 0;      // u % kWSlots of the next code request
  auto issue_a = [&](auto set_, int t) __attribute__((always_inline)) {
    constexpr int set = decltype(set_)::value;
    const uint32_t k0 = static_cast<uint32_t>(t < last ? t : last) * kBK;       // past the end: the last step again
    // (asm operands inside a generic lambda must be the lambda's own variables)
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
    {
      const uint64_t w_src = w_base + 128 * b;
      const uint32_t dst = lds0 + kWBase + (wave * kWSlots + issue_slot) * 1024;
      const uint32_t wv = w_voff[i];
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(wv), "s"(w_src) : "memory");
    }
    issue_slot = issue_slot + 1 == kWSlots ? 0 : issue_slot + 1;
    if constexpr (i == 0) {
      const uint64_t s_src = s_base + 4 * b;
      const uint32_t dst = lds0 + kSBase + (wave * 3 + block % 3) * 256;
      const uint32_t sv = s_voff;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(dst), "v"(sv), "s"(s_src) : "memory");
    }
  };

  // Step t's codes and scale of this lane come from the wave's own rings (only this wave's requests wrote them, so
  // its own wait is enough); q = t % 4 says which 64 of the block's 256 codes.  fetch_w asks LDS for them,
  // dequant_one turns dword j into B operand j of the step.
  const int my_req = frow >> 3;                                       // which of a block's four requests holds this lane's row
  const int my_row = (frow & 7) * 128;
  const int my_x = (frow & 7) ^ (my_req & 1);
  struct WRaw {
    u32x4_t codes;
    uint32_t sdw;
  };
  auto fetch_w = [&](auto q_, int t, WRaw &w) __attribute__((always_inline)) {
    constexpr int q = decltype(q_)::value;
    const int block = t >> 2;
    int slot = (4 * block) % kWSlots + my_req;
    if (slot >= kWSlots) slot -= kWSlots;
    const unsigned char *wring = smem + kWBase + wave * (kWSlots * 1024);
    w.codes = *reinterpret_cast<const u32x4_t *>(wring + slot * 1024 + my_row + (((2 * q + fh) ^ my_x) << 4));
    w.sdw = *reinterpret_cast<const uint32_t *>(smem + kSBase + (wave * 3 + block % 3) * 256 + frow * 4);
  };
  struct WScale {
    float s, s16, m8;
  };
  auto scale_of = [&](auto q_, const WRaw &w) __attribute__((always_inline)) {
    constexpr int q = decltype(q_)::value;
    const uint32_t bits = (q & 2) ? (w.sdw >> 16) : (w.sdw & 0xffffu);
    WScale r;
    r.s = to_f32(__builtin_bit_cast(f16_t, static_cast<uint16_t>(bits)));
    r.s16 = r.s * 0.0625f;
    r.m8 = -8.0f * r.s;
    return r;
  };
  auto dequant_one = [&](const WRaw &w, const WScale &sc, int j, vec_t &out) __attribute__((always_inline)) {
    out = __builtin_bit_cast(vec_t, dequant_int4x8_packed<CT>(w.codes[j], sc.s, sc.s16, sc.m8));
  };

  floatx16_t acc[WR];
#pragma unroll
  for (int i = 0; i < WR; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;

  auto read_a = [&](auto set_, int j, vec_t (&out)[WR]) __attribute__((always_inline)) {
    constexpr int set = decltype(set_)::value;
    const unsigned char *abuf = smem + set * kStageBytes;
#pragma unroll
    for (int i = 0; i < WR; ++i) out[i] = *reinterpret_cast<const vec_t *>(abuf + swz(i * 32 + frow, 4 * fh + j));
  };
  auto mfma_row = [&](const vec_t (&a)[WR], const vec_t &b) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < WR; ++i) acc[i] = Mfma32<CT>::run(a[i], b, acc[i]);
  };

  typedef std::integral_constant<int, 0> I0;
  typedef std::integral_constant<int, 1> I1;
  typedef std::integral_constant<int, 2> I2;
  typedef std::integral_constant<int, 3> I3;

  // before the loop: code requests 0..6 (block 0 and three quarters of block 1, with their scales), activation
  // stages 0..2
  issue_w(I0{}, 0);
  issue_w(I1{}, 0);
  issue_w(I2{}, 0);
  issue_w(I3{}, 0);
  issue_w(I0{}, 1);
  issue_w(I1{}, 1);
  issue_w(I2{}, 1);
  issue_a(I0{}, 0);
  issue_a(I1{}, 1);
  issue_a(I2{}, 2);
  asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
  vec_t bfr[4];      // B operands of the current step
  vec_t afa[WR];     // A operands of its first MFMA row
  {
    WRaw w0;
    fetch_w(I0{}, 0, w0);
    const WScale sc = scale_of(I0{}, w0);
#pragma unroll
    for (int j = 0; j < 4; ++j) dequant_one(w0, sc, j, bfr[j]);
  }
  read_a(I0{}, 0, afa);
  // Step s works on stage ph = s % 4; on entry its B operands are in registers and its first A operands on their
  // way.  Each of the step's four MFMA rows is written next to the LDS requests of the row after it and a
  // quarter of the dequantisation of step s + 1, and the compiler's scheduler is kept from moving work between
  // rows (left alone it sinks every LDS read to just before its first use, and the wave then waits for LDS in
  // front of every MFMA).
  auto step = [&](auto ph_, int s) __attribute__((always_inline)) {
    constexpr int ph = decltype(ph_)::value;
    typedef std::integral_constant<int, (ph + 1) % 4> Next;
    vec_t afb[WR], bnext[4];
    WRaw wn;
    // row 0
    read_a(ph_, 1, afb);
    fetch_w(Next{}, s + 1, wn);
    mfma_row(afa, bfr[0]);
    __builtin_amdgcn_sched_barrier(0);
    // row 1
    read_a(ph_, 2, afa);
    const WScale sc = scale_of(Next{}, wn);
    dequant_one(wn, sc, 0, bnext[0]);
    mfma_row(afb, bfr[1]);
    __builtin_amdgcn_sched_barrier(0);
    // This wave's requests of every step but the last one have landed (requests complete in issue order); behind
    // the barrier stage s + 1 is there for everybody and stage s - 1 is free.  Step s - 1 issued a scale request
    // when its code request was the first of a block, (s - 1 + 7) % 4 == 0
    {
      constexpr int kPrev = kDma + 1 + (ph == 2 ? 1 : 0);
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kPrev) : "memory");
    }
    issue_a(std::integral_constant<int, (ph + 3) % 4>{}, s + 3);
    issue_w(std::integral_constant<int, (ph + kWAhead) % 4>{}, (s + kWAhead) >> 2);
    __builtin_amdgcn_sched_barrier(0);
    // row 2
    read_a(ph_, 3, afb);
    dequant_one(wn, sc, 1, bnext[1]);
    mfma_row(afa, bfr[2]);
    __builtin_amdgcn_sched_barrier(0);
    // row 3
    read_a(Next{}, 0, afa);
    dequant_one(wn, sc, 2, bnext[2]);
    dequant_one(wn, sc, 3, bnext[3]);
    mfma_row(afb, bfr[3]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 4; ++j) bfr[j] = bnext[j];
  };
  {
    int s = 0;
    for (; s + 4 <= steps; s += 4) {          // K is a multiple of 256: the steps come in fours
      step(I0{}, s);
      step(I1{}, s + 1);
      step(I2{}, s + 2);
      step(I3{}, s + 3);
    }
  }
  // requests past the last step may still be writing LDS, and other waves may still be reading
  asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");

  // ---- store (regw::store_tile: the whole tile through LDS, whole rows per wave instruction)
  if (g.d_dtype == CAIFX_BF16)
    regw::store_tile<bf16_t, WR>(smem, acc, wave, lane, row0, g.M, col0, g.N, static_cast<bf16_t *>(g.d), static_cast<const bf16_t *>(g.addend));
  else if (g.d_dtype == CAIFX_F16)
    regw::store_tile<f16_t, WR>(smem, acc, wave, lane, row0, g.M, col0, g.N, static_cast<f16_t *>(g.d), static_cast<const f16_t *>(g.addend));
  else
    regw::store_tile<float, WR>(smem, acc, wave, lane, row0, g.M, col0, g.N, static_cast<float *>(g.d), static_cast<const float *>(g.addend));
}

template <typename CT, int WR> int launch(const RegwArgs &t, hipStream_t s)
{
  constexpr int BM = 32 * WR;
  const size_t ring = static_cast<size_t>(kStages) * BM * kBK * 2 + 8 * kWSlots * 1024 + 8 * 3 * 256;
  const size_t staging = regw::store_bytes(BM);
  const size_t lds = ring > staging ? ring : staging;
  auto kern = qgemm_regw_kernel<CT, WR>;
  static std::atomic<bool> raised{false};
  if (!raised.load(std::memory_order_relaxed)) {
    // the attribute is per kernel and sticky; two threads racing here both set it, which is harmless
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(lds)) != hipSuccess)
      return CAIFX_ERR_LAUNCH_FAILED;
    raised.store(true, std::memory_order_relaxed);
  }
  const int64_t tiles = ((t.M + BM - 1) / BM) * ((t.N + kBN - 1) / kBN);
  const int64_t padded = (tiles + 7) / 8 * 8;
  if (padded > 0x7fffffff) return CAIFX_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(padded)), dim3(512), lds, s, t);
  return launch_status();
}

}  // namespace

int mfma_regw_forward(const GemmArgs &a, hipStream_t s)
{
  if (a.w.kind != CAIFX_W_INT4_GROUP || a.offsets != nullptr || a.epilogue != 0) return CAIFX_ERR_UNSUPPORTED;
  if (a.compute_dtype == CAIFX_F32 || a.x_dtype != a.compute_dtype) return CAIFX_ERR_UNSUPPORTED;
  if (a.w.group_size != kGroup) return CAIFX_ERR_UNSUPPORTED;
  if (a.K % 256 != 0 || a.K < 512 || a.K > (int64_t{1} << 22)) return CAIFX_ERR_UNSUPPORTED;
  if (a.N * a.K >= (int64_t{1} << 32) || a.M > (int64_t{1} << 30)) return CAIFX_ERR_UNSUPPORTED;
  if (!aligned_to(a.x, 16) || !aligned_to(a.w.q, 16) || !aligned_to(a.w.scales, 4) || !aligned_to(a.y, 16) ||
      (a.addend && !aligned_to(a.addend, 16)))
    return CAIFX_ERR_UNSUPPORTED;
  // enough 128 x 256 tiles to give most compute units one; below that the tiled kernel's shared reduction wins
  const int64_t tiles128 = ((a.M + 127) / 128) * ((a.N + kBN - 1) / kBN);
  if (tiles128 < 128) return CAIFX_ERR_UNSUPPORTED;
  RegwArgs t{};
  t.M = a.M;
  t.N = a.N;
  t.K = a.K;
  t.a = a.x;
  t.d = a.y;
  t.d_dtype = a.y_dtype;
  t.addend = a.addend;
  t.wq = static_cast<const uint8_t *>(a.w.q);
  t.scales = static_cast<const f16_t *>(a.w.scales);
  if (a.compute_dtype == CAIFX_BF16) return launch<bf16_t, 4>(t, s);
  return launch<f16_t, 4>(t, s);
}

int mfma_forward(const GemmArgs &a, hipStream_t s)
{
  int st = mfma_regw_forward(a, s);
  if (st == CAIFX_ERR_UNSUPPORTED) st = mfma_regw8_forward(a, s);
  return st == CAIFX_ERR_UNSUPPORTED ? mfma_tiled_forward(a, s) : st;
}

}  // namespace caifx
