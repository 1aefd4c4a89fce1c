// Shared device helpers for the gfx950 frozen quantized-linear kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "caifx.h"

namespace caifx {

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;

constexpr int kWave = 64;

inline hipStream_t as_stream(caifx_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline int launch_status()
{
  return hipGetLastError() == hipSuccess ? CAIFX_OK : CAIFX_ERR_LAUNCH_FAILED;
}

inline bool aligned_to(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

template <typename T> struct dtype_code;
template <> struct dtype_code<float> { static constexpr int value = CAIFX_F32; };
template <> struct dtype_code<f16_t> { static constexpr int value = CAIFX_F16; };
template <> struct dtype_code<bf16_t> { static constexpr int value = CAIFX_BF16; };

inline size_t dtype_size(int dt) { return dt == CAIFX_F32 ? 4 : 2; }
inline bool valid_dtype(int dt) { return dt == CAIFX_F32 || dt == CAIFX_F16 || dt == CAIFX_BF16; }

// fp32 -> T with round-to-nearest-even (v_cvt_pk_bf16_f32 / v_cvt_f16_f32), T -> fp32 exact.
template <typename T> __device__ __forceinline__ T from_f32(float v) { return static_cast<T>(v); }
template <typename T> __device__ __forceinline__ float to_f32(T v) { return static_cast<float>(v); }
// the value an fp32 number has after a cast to T and back
template <typename T> __device__ __forceinline__ float round_through(float v) { return to_f32<T>(from_f32<T>(v)); }
template <> __device__ __forceinline__ float round_through<float>(float v) { return v; }

// SiLU and its derivative (src/caif_cuda_kernels_activations.cu:513-514,558-561), shared by the element-wise
// kernels and the GEMM epilogues.  The one place where the compiler could choose between a fused and an
// unfused multiply-add is written out, so every user returns the same bits.
__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float silu_bwd_f32(float x, float g)
{
  const float s = 1.0f / (1.0f + expf(-x));
  return g * s * __builtin_fmaf(x, 1.0f - s, 1.0f);
}
// One element of the gated expert's backward between its down and up/gate projections
// (src/caif_device_moe_frozen_expert.cpp:252-290): h = grad of hidden, gate/up = the forward's projections,
// all already rounded to T; grad_up = T(h * T(silu(gate))), grad_gate = T(silu'(gate) * T(h * up)).
template <typename T> __device__ __forceinline__ void swiglu_bwd_one(T gate, T up, T h, T &grad_gate, T &grad_up)
{
  const float g = to_f32<T>(gate), u = to_f32<T>(up), hh = to_f32<T>(h);
  grad_up = from_f32<T>(hh * round_through<T>(silu_f32(g)));
  grad_gate = from_f32<T>(silu_bwd_f32(g, round_through<T>(hh * u)));
}
// hidden = T(T(silu(gate)) * up) (:119-153)
template <typename T> __device__ __forceinline__ T swiglu_fwd_one(T gate, T up)
{
  return from_f32<T>(round_through<T>(silu_f32(to_f32<T>(gate))) * to_f32<T>(up));
}

// Byte k of a dword as fp32 (v_cvt_f32_ubyteK: one VALU op, no shift/mask).
__device__ __forceinline__ float ubyte0_f32(uint32_t v) { float r; asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(r) : "v"(v)); return r; }
__device__ __forceinline__ float ubyte1_f32(uint32_t v) { float r; asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(r) : "v"(v)); return r; }
__device__ __forceinline__ float ubyte2_f32(uint32_t v) { float r; asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(r) : "v"(v)); return r; }
__device__ __forceinline__ float ubyte3_f32(uint32_t v) { float r; asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(r) : "v"(v)); return r; }

// Sign-extended nibble `i` (0 = low) of a byte-sized field, as the reference's dequantiser
// decodes it: code 0x8 is -8.
__device__ __forceinline__ int nibble_s4(uint32_t byte, int i)
{
  return (static_cast<int>(byte << (28 - 4 * i))) >> 28;
}

// Eight int4 codes of one dword, flat order (nibble j = element j), times one scale.
// (code * scale) is formed as fma(code + 8, scale, -8*scale): -8*scale is exact and the fused
// multiply-add rounds the exact product once, so each value equals the reference's
// float(code) * scale (the sign of a zero aside).  s must be finite.
__device__ __forceinline__ void dequant_int4x8(uint32_t p, float s, float (&e)[8])
{
  const float m8 = -8.0f * s;
  p ^= 0x88888888u;                       // two's complement nibble -> offset binary (code + 8)
  const uint32_t lo = p & 0x0F0F0F0Fu;    // elements 0,2,4,6 in bytes 0..3
  const uint32_t hi = (p >> 4) & 0x0F0F0F0Fu;  // elements 1,3,5,7
  e[0] = __builtin_fmaf(ubyte0_f32(lo), s, m8);
  e[1] = __builtin_fmaf(ubyte0_f32(hi), s, m8);
  e[2] = __builtin_fmaf(ubyte1_f32(lo), s, m8);
  e[3] = __builtin_fmaf(ubyte1_f32(hi), s, m8);
  e[4] = __builtin_fmaf(ubyte2_f32(lo), s, m8);
  e[5] = __builtin_fmaf(ubyte2_f32(hi), s, m8);
  e[6] = __builtin_fmaf(ubyte3_f32(lo), s, m8);
  e[7] = __builtin_fmaf(ubyte3_f32(hi), s, m8);
}

// Four int8 codes of one dword as fp32.
__device__ __forceinline__ void int8x4_to_f32(uint32_t p, float (&e)[4])
{
  e[0] = static_cast<float>(static_cast<int8_t>(p));
  e[1] = static_cast<float>(static_cast<int8_t>(p >> 8));
  e[2] = static_cast<float>(static_cast<int8_t>(p >> 16));
  e[3] = static_cast<float>(static_cast<int>(p) >> 24);
}

// Rows [lo, hi) of expert e, forced into 0 <= lo <= hi <= M: offsets that are not non-decreasing or that
// run past the buffer (a caller's mistake) then lose rows instead of sending loads and stores out of bounds.
__device__ __forceinline__ void segment_rows(const int32_t *offsets, int e, int64_t M, int &lo, int &hi)
{
  const int m = static_cast<int>(M);          // M <= 2^30 is checked on the host
  lo = offsets[e];
  hi = offsets[e + 1];
  lo = lo < 0 ? 0 : (lo > m ? m : lo);
  hi = hi < lo ? lo : (hi > m ? m : hi);
}

// Which tile of a grouped launch a workgroup owns.  Row tiles of BM rows are counted over all experts, expert by
// expert, and crossed with col_tiles column tiles, column tile last; XCD x (workgroup id mod 8, each XCD has its own
// L2) takes the x-th contiguous eighth of that list, so one expert's weight and one row tile's activations are
// fetched into one L2.  Every wave works the numbering out on its own: lane l takes expert base + l and a scan
// over the lanes gives the running tile count.  A tile starts with this search, and each dependent global load in
// it is a memory round trip during which the compute unit's share of the tile does nothing: with up to 64 experts
// every lane asks for its expert's offsets and pointers in one go, before the tile is known, and the owner's
// values are then read from its lane; with more, the offsets are walked twice and the pointers fetched last.
// False: the workgroup has no tile (the grid is an upper bound).  pos: the tile's index in the list.
struct GroupedTile {
  int e;                   // expert
  int64_t row0, row_end;   // first row of the tile, end of the expert's segment
  int64_t col_tile;
  int64_t pos;
  const void *wq;
  const void *scales;      // null when scales_ptrs is
};
template <int BM>
__device__ __forceinline__ bool grouped_tile(const int32_t *offsets, int num_experts, int64_t M, int64_t col_tiles,
                                             const void *const *wq_ptrs, const void *const *scales_ptrs, int lane,
                                             GroupedTile &out)
{
  if (num_experts <= 64) {
    int my_lo = 0, my_hi = 0;
    uint64_t my_w = 0, my_s = 0;
    if (lane < num_experts) {
      segment_rows(offsets, lane, M, my_lo, my_hi);
      my_w = reinterpret_cast<uint64_t>(wq_ptrs[lane]);
      if (scales_ptrs) my_s = reinterpret_cast<uint64_t>(scales_ptrs[lane]);
    }
    const int tiles = (my_hi - my_lo + BM - 1) / BM;
    int incl = tiles;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o, 64);
      if (lane >= o) incl += up;
    }
    const int64_t total = static_cast<int64_t>(__shfl(incl, 63, 64)) * col_tiles;
    const int64_t per_xcd = (total + 7) >> 3;
    const int64_t slot = blockIdx.x >> 3;
    const int64_t pos = static_cast<int64_t>(blockIdx.x & 7) * per_xcd + slot;
    if (slot >= per_xcd || pos >= total) return false;
    const int t = static_cast<int>(pos / col_tiles);
    const unsigned long long owners = __ballot(incl > t);
    if (owners == 0) return false;
    const int src = __builtin_ctzll(owners);
    out.e = src;
    out.pos = pos;
    out.col_tile = pos - static_cast<int64_t>(t) * col_tiles;
    out.row0 = __shfl(my_lo, src, 64) + static_cast<int64_t>(t - __shfl(incl - tiles, src, 64)) * BM;
    out.row_end = __shfl(my_hi, src, 64);
    const uint32_t wl = __shfl(static_cast<uint32_t>(my_w), src, 64), wh = __shfl(static_cast<uint32_t>(my_w >> 32), src, 64);
    const uint32_t sl = __shfl(static_cast<uint32_t>(my_s), src, 64), sh = __shfl(static_cast<uint32_t>(my_s >> 32), src, 64);
    out.wq = reinterpret_cast<const void *>((static_cast<uint64_t>(wh) << 32) | wl);
    out.scales = reinterpret_cast<const void *>((static_cast<uint64_t>(sh) << 32) | sl);
    return true;
  }
  int total_rt = 0;
  for (int base = 0; base < num_experts; base += 64) {
    const int my = base + lane;
    int tiles = 0;
    if (my < num_experts) {
      int slo, shi;
      segment_rows(offsets, my, M, slo, shi);
      tiles = (shi - slo + BM - 1) / BM;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) tiles += __shfl_xor(tiles, o, 64);
    total_rt += tiles;
  }
  const int64_t total = static_cast<int64_t>(total_rt) * col_tiles;
  const int64_t per_xcd = (total + 7) >> 3;
  const int64_t slot = blockIdx.x >> 3;
  const int64_t pos = static_cast<int64_t>(blockIdx.x & 7) * per_xcd + slot;
  if (slot >= per_xcd || pos >= total) return false;
  int t = static_cast<int>(pos / col_tiles);
  out.pos = pos;
  out.col_tile = pos - static_cast<int64_t>(t) * col_tiles;
  for (int base = 0; base < num_experts; base += 64) {
    const int my = base + lane;
    int my_lo = 0, my_hi = 0;
    if (my < num_experts) segment_rows(offsets, my, M, my_lo, my_hi);
    const int tiles = (my_hi - my_lo + BM - 1) / BM;
    int incl = tiles;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o, 64);
      if (lane >= o) incl += up;
    }
    const unsigned long long owners = __ballot(incl > t);
    if (owners != 0) {
      const int src = __builtin_ctzll(owners);
      out.e = base + src;
      out.row0 = __shfl(my_lo, src, 64) + static_cast<int64_t>(t - __shfl(incl - tiles, src, 64)) * BM;
      out.row_end = __shfl(my_hi, src, 64);
      out.wq = wq_ptrs[out.e];
      out.scales = scales_ptrs ? scales_ptrs[out.e] : nullptr;
      return true;
    }
    t -= __shfl(incl, 63, 64);
  }
  return false;
}

// v_mfma_f32_32x32x16 in the 16-bit compute type CT: A is 32 rows x 16 (lane l supplies row l % 32, reduction
// elements 8 * (l / 32) .. + 7), B likewise by column; of the 32 x 32 result lane l holds column l % 32 and, in
// register r, row 8 * (r / 4) + 4 * (l / 32) + r % 4.
template <typename CT> struct Mfma32;
template <> struct Mfma32<bf16_t> {
  typedef bf16x8_t vec_t;
  static __device__ __forceinline__ floatx16_t run(vec_t a, vec_t b, floatx16_t c)
  {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma32<f16_t> {
  typedef f16x8_t vec_t;
  static __device__ __forceinline__ floatx16_t run(vec_t a, vec_t b, floatx16_t c)
  {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// two fp32 values rounded to CT (nearest even), the first in the low half
template <typename CT> __device__ __forceinline__ uint32_t pack2(float lo, float hi)
{
  typedef __attribute__((__vector_size__(2 * sizeof(CT)))) CT pair_t;
  pair_t p;
  p[0] = from_f32<CT>(lo);
  p[1] = from_f32<CT>(hi);
  return __builtin_bit_cast(uint32_t, p);
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

}  // namespace caifx
