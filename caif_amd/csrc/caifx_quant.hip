// Quantise / dequantise / cast kernels for gfx950.
//
// Numerics contract (what makes codes and scales bit-identical to the reference's
// src/caif_cuda_kernels_quant.cu): IEEE binary32 division for max/127, max/7 and 1/scale,
// a single rounding for x * inv_scale, clamp before round, round-half-to-even (v_rndne_f32),
// fp32 -> fp16 scale by round-half-to-even (v_cvt_f16_f32), int4 codes from the UNROUNDED
// fp32 scale.  Max reductions are order independent, so parallelising them changes nothing.
// No multiply feeds an add in these kernels; contraction is switched off anyway.
#include "caifx_common.hpp"

#pragma clang fp contract(off)

namespace caifx {
namespace {

constexpr int kBlock = 256;
constexpr float kInt8Max = 127.0f;
constexpr float kInt4Max = 7.0f;

inline int grid_for(int64_t work_items, int block = kBlock)
{
  return static_cast<int>((work_items + block - 1) / block);
}

__device__ __forceinline__ float clamp_sym(float v, float limit)
{
  if (v > limit) v = limit;
  else if (v < -limit) v = -limit;
  return v;
}

// ------------------------------------------------------------------ casts
template <typename In, typename Out>
__global__ void cast_kernel(const In *__restrict__ in, Out *__restrict__ out, int64_t n)
{
  int64_t i = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
  if (i + 4 <= n) {
    In v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = in[i + j];
#pragma unroll
    for (int j = 0; j < 4; ++j) out[i + j] = static_cast<Out>(static_cast<float>(v[j]));
  } else {
    for (; i < n; ++i) out[i] = static_cast<Out>(static_cast<float>(in[i]));
  }
}

__global__ void cast_f32_to_int8_kernel(const float *__restrict__ in, int8_t *__restrict__ out, int64_t n)
{
  int64_t i = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
  int64_t end = i + 4 < n ? i + 4 : n;
  for (; i < end; ++i) out[i] = static_cast<int8_t>(rintf(clamp_sym(in[i], kInt8Max)));
}

template <typename In, typename Out>
int launch_cast(const In *in, Out *out, int64_t n, hipStream_t s)
{
  if (n <= 0) return CAIFX_OK;
  if (!in || !out) return CAIFX_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL((cast_kernel<In, Out>), dim3(grid_for((n + 3) / 4)), dim3(kBlock), 0, s, in, out, n);
  return launch_status();
}

// ------------------------------------------------------------------ absmax reductions
__global__ void fill_u32_kernel(uint32_t *p, int64_t n, uint32_t v)
{
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// max |x| over the whole tensor -> atomicMax on the bit pattern (non-negative floats order
// like unsigned integers).  `v > m` drops NaNs exactly like the reference's comparison.
// `vec`: the input is 16-byte aligned, so the body goes in 16-byte loads (four of them in flight per lane) and
// the last n % 4 elements are left to the first lanes.
__global__ void absmax_tensor_kernel(const float *__restrict__ in, uint32_t *__restrict__ acc, int64_t n, int vec)
{
  __shared__ float part[kBlock / kWave];
  float m = 0.0f;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t first = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  auto take = [&](float v) {
    v = fabsf(v);
    if (v > m) m = v;
  };
  if (vec) {
    const floatx4_t *in4 = reinterpret_cast<const floatx4_t *>(in);
    const int64_t n4 = n >> 2;
    int64_t i = first;
    for (; i + 3 * stride < n4; i += 4 * stride) {
      const floatx4_t a = in4[i], b = in4[i + stride], c = in4[i + 2 * stride], d = in4[i + 3 * stride];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        take(a[j]);
        take(b[j]);
        take(c[j]);
        take(d[j]);
      }
    }
    for (; i < n4; i += stride) {
      const floatx4_t a = in4[i];
#pragma unroll
      for (int j = 0; j < 4; ++j) take(a[j]);
    }
    if (first < (n & 3)) take(in[(n4 << 2) + first]);
  } else {
    for (int64_t i = first; i < n; i += stride) take(in[i]);
  }
  m = wave_max(m);
  if ((threadIdx.x & (kWave - 1)) == 0) part[threadIdx.x / kWave] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kBlock / kWave; ++w) m = fmaxf(m, part[w]);
    if (m > 0.0f) atomicMax(acc, __float_as_uint(m));
  }
}

// max over rows of |x[r, c]| for a [rows, cols] row-major tensor; one thread per column and
// a chunk of rows, coalesced across the columns of a block.
constexpr int kRowChunk = 64;
__global__ void absmax_columns_kernel(const float *__restrict__ in, uint32_t *__restrict__ acc, int rows, int cols)
{
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= cols) return;
  float m = 0.0f;
  // chunks of rows are strided over gridDim.y, which the launch caps at the grid limit
  for (int64_t r0 = static_cast<int64_t>(blockIdx.y) * kRowChunk; r0 < rows; r0 += static_cast<int64_t>(gridDim.y) * kRowChunk) {
    const int64_t r1 = r0 + kRowChunk < rows ? r0 + kRowChunk : rows;
    for (int64_t r = r0; r < r1; ++r) {
      float v = fabsf(in[r * cols + c]);
      if (v > m) m = v;
    }
  }
  if (m > 0.0f) atomicMax(acc + c, __float_as_uint(m));
}

// The same with four adjacent columns per thread (cols % 4 == 0, 16-byte aligned input): 16-byte loads, four
// rows in flight per lane.
__global__ void absmax_columns_x4_kernel(const float *__restrict__ in, uint32_t *__restrict__ acc, int rows, int cols)
{
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (c >= cols) return;
  const int r0 = blockIdx.y * kRowChunk;
  const int r1 = r0 + kRowChunk < rows ? r0 + kRowChunk : rows;
  float m[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  const float *p = in + static_cast<int64_t>(r0) * cols + c;
  auto take = [&](const floatx4_t &v) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float a = fabsf(v[j]);
      if (a > m[j]) m[j] = a;
    }
  };
  int r = r0;
  for (; r + 4 <= r1; r += 4, p += 4 * static_cast<int64_t>(cols)) {
    const floatx4_t a = *reinterpret_cast<const floatx4_t *>(p);
    const floatx4_t b = *reinterpret_cast<const floatx4_t *>(p + cols);
    const floatx4_t d = *reinterpret_cast<const floatx4_t *>(p + 2 * static_cast<int64_t>(cols));
    const floatx4_t e = *reinterpret_cast<const floatx4_t *>(p + 3 * static_cast<int64_t>(cols));
    take(a);
    take(b);
    take(d);
    take(e);
  }
  for (; r < r1; ++r, p += cols) take(*reinterpret_cast<const floatx4_t *>(p));
#pragma unroll
  for (int j = 0; j < 4; ++j)
    if (m[j] > 0.0f) atomicMax(acc + c + j, __float_as_uint(m[j]));
}

// in place: max|x| -> scale = max / 127 (1.0 when max is zero)
__global__ void finalize_int8_scale_kernel(float *scales, int count)
{
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= count) return;
  const float m = scales[c];
  scales[c] = (m > 0.0f) ? m / kInt8Max : 1.0f;
}

// q = rint(clamp(x * (1/scale[f % period], +-127)); four consecutive elements per thread
__global__ void quantize_int8_kernel(const float *__restrict__ in, int8_t *__restrict__ out,
                                     const float *__restrict__ scales, int64_t n, int period)
{
  int64_t i = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
  if (i >= n) return;
  int col = static_cast<int>(i % period);
  const int cnt = (n - i) < 4 ? static_cast<int>(n - i) : 4;
  for (int j = 0; j < cnt; ++j) {
    const float s = scales[col];
    const float inv_s = (s > 0.0f) ? 1.0f / s : 0.0f;
    out[i + j] = static_cast<int8_t>(rintf(clamp_sym(in[i + j] * inv_s, kInt8Max)));
    if (++col == period) col = 0;
  }
}

__device__ __forceinline__ uint32_t quantize_int8_x4(const floatx4_t &v, const float (&inv)[4])
{
  uint32_t w = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j)
    w |= (static_cast<uint32_t>(static_cast<int>(rintf(clamp_sym(v[j] * inv[j], kInt8Max)))) & 0xFFu) << (8 * j);
  return w;
}

// One scale for the whole tensor, 16 consecutive elements per thread (16-byte aligned input and output,
// n % 16 == 0): same arithmetic per element as quantize_int8_kernel, the reciprocal taken once per thread.
// The blocks walk the tensor from its end: the maximum pass before this one read it front to back, so its tail
// is what the memory-side cache still holds.
__global__ void quantize_int8_tensor_x16_kernel(const float *__restrict__ in, int8_t *__restrict__ out,
                                                const float *__restrict__ scale, int64_t n16)
{
  const int64_t i = static_cast<int64_t>(gridDim.x - 1 - blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n16) return;
  const float s = scale[0];
  const float one = (s > 0.0f) ? 1.0f / s : 0.0f;
  const float inv[4] = {one, one, one, one};
  const floatx4_t *p = reinterpret_cast<const floatx4_t *>(in) + i * 4;
  const floatx4_t a = p[0], b = p[1], c = p[2], d = p[3];
  u32x4_t w;
  w[0] = quantize_int8_x4(a, inv);
  w[1] = quantize_int8_x4(b, inv);
  w[2] = quantize_int8_x4(c, inv);
  w[3] = quantize_int8_x4(d, inv);
  reinterpret_cast<u32x4_t *>(out)[i] = w;
}

// One scale per column of a [rows, cols] tensor: a thread takes four adjacent columns (cols % 4 == 0, aligned
// pointers) and kQuantRows consecutive rows, so the four reciprocals are taken once for all of them.  The row
// blocks are walked from the last to the first: the maxima pass before this one read the tensor front to back,
// so its tail is what the caches still hold.
constexpr int kQuantRows = 16;
__global__ void quantize_int8_columns_x4_kernel(const float *__restrict__ in, int8_t *__restrict__ out,
                                                const float *__restrict__ scales, int rows, int cols)
{
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (c >= cols) return;
  const int r0 = (gridDim.y - 1 - blockIdx.y) * kQuantRows;
  const int r1 = r0 + kQuantRows < rows ? r0 + kQuantRows : rows;
  const floatx4_t s = *reinterpret_cast<const floatx4_t *>(scales + c);
  float inv[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) inv[j] = (s[j] > 0.0f) ? 1.0f / s[j] : 0.0f;
  const float *p = in + static_cast<int64_t>(r0) * cols + c;
  int8_t *q = out + static_cast<int64_t>(r0) * cols + c;
  int r = r0;
  for (; r + 4 <= r1; r += 4, p += 4 * static_cast<int64_t>(cols), q += 4 * static_cast<int64_t>(cols)) {
    const floatx4_t a = *reinterpret_cast<const floatx4_t *>(p);
    const floatx4_t b = *reinterpret_cast<const floatx4_t *>(p + cols);
    const floatx4_t d = *reinterpret_cast<const floatx4_t *>(p + 2 * static_cast<int64_t>(cols));
    const floatx4_t e = *reinterpret_cast<const floatx4_t *>(p + 3 * static_cast<int64_t>(cols));
    *reinterpret_cast<uint32_t *>(q) = quantize_int8_x4(a, inv);
    *reinterpret_cast<uint32_t *>(q + cols) = quantize_int8_x4(b, inv);
    *reinterpret_cast<uint32_t *>(q + 2 * static_cast<int64_t>(cols)) = quantize_int8_x4(d, inv);
    *reinterpret_cast<uint32_t *>(q + 3 * static_cast<int64_t>(cols)) = quantize_int8_x4(e, inv);
  }
  for (; r < r1; ++r, p += cols, q += cols)
    *reinterpret_cast<uint32_t *>(q) = quantize_int8_x4(*reinterpret_cast<const floatx4_t *>(p), inv);
}

__global__ void dequantize_int8_kernel(const int8_t *__restrict__ in, float *__restrict__ out,
                                       const float *__restrict__ scales, int64_t n, int period)
{
  int64_t i = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
  if (i >= n) return;
  int col = static_cast<int>(i % period);
  const int cnt = (n - i) < 4 ? static_cast<int>(n - i) : 4;
  for (int j = 0; j < cnt; ++j) {
    out[i + j] = static_cast<float>(in[i + j]) * scales[col];
    if (++col == period) col = 0;
  }
}

// Four consecutive codes per thread (4-byte aligned codes, 16-byte aligned output): one dword in, one 16-byte
// store out, consecutive lanes on consecutive addresses.  The scale vector has period `period`, a multiple of 4
// that divides n, so the four scales of a thread are consecutive and do not wrap (period 1: one scale).  Same
// product per element as dequantize_int8_kernel.
__global__ void dequantize_int8_x4_kernel(const int8_t *__restrict__ in, float *__restrict__ out,
                                          const float *__restrict__ scales, int64_t n4, int period)
{
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n4) return;
  const uint32_t w = reinterpret_cast<const uint32_t *>(in)[i];
  floatx4_t s;
  if (period == 1) {
    const float one = scales[0];
    s = floatx4_t{one, one, one, one};
  } else {
    s = *reinterpret_cast<const floatx4_t *>(scales + (i * 4) % period);
  }
  float e[4];
  int8x4_to_f32(w, e);
  reinterpret_cast<floatx4_t *>(out)[i] = floatx4_t{e[0] * s[0], e[1] * s[1], e[2] * s[2], e[3] * s[3]};
}

int launch_dequantize_int8(const int8_t *in, float *out, const float *scales, int64_t n, int period, hipStream_t s)
{
  const bool vec = aligned_to(in, 4) && aligned_to(out, 16) &&
                   (period == 1 || (period % 4 == 0 && n % period == 0 && aligned_to(scales, 16)));
  const int64_t body = vec ? n / 4 * 4 : 0;
  if (body > 0)
    hipLaunchKernelGGL(dequantize_int8_x4_kernel, dim3(grid_for(body / 4)), dim3(kBlock), 0, s, in, out, scales, body / 4,
                       period);
  // a tail is left only with one scale (period 1) or when nothing went the vector way: n is a multiple of the
  // period, so a period that is a multiple of 4 leaves none
  if (body < n)
    hipLaunchKernelGGL(dequantize_int8_kernel, dim3(grid_for((n - body + 3) / 4)), dim3(kBlock), 0, s, in + body,
                       out + body, scales, n - body, period);
  return launch_status();
}

// ------------------------------------------------------------------ int4 per-group
// Fast path: each thread owns 8 consecutive elements (one dword of packed output); a team of
// group_size/8 adjacent lanes owns one group and shares its max through wave shuffles.
// Needs group_size % 8 == 0 and group_size/8 a power of two <= 64.  `vec`: the input is 16-byte aligned (two
// 16-byte loads per thread).
__global__ void quantize_int4_team_kernel(const float *__restrict__ in, uint8_t *__restrict__ packed,
                                          f16_t *__restrict__ scales, int64_t n, int group_size, int team, int vec)
{
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t base = gid * 8;
  float x[8];
  if (vec && base + 8 <= n) {
    const floatx4_t lo = *reinterpret_cast<const floatx4_t *>(in + base);
    const floatx4_t hi = *reinterpret_cast<const floatx4_t *>(in + base + 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      x[j] = lo[j];
      x[4 + j] = hi[j];
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = (base + j < n) ? in[base + j] : 0.0f;
  }
  float m = 0.0f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    float a = fabsf(x[j]);
    if (a > m) m = a;
  }
  for (int o = team >> 1; o > 0; o >>= 1) {
    float other = __shfl_xor(m, o, 64);
    if (other > m) m = other;
  }
  if (base >= n) return;
  const float scale = (m == 0.0f) ? 0.0f : m / kInt4Max;
  if ((gid & (team - 1)) == 0) scales[base / group_size] = static_cast<f16_t>(scale);
  const float inv = (scale == 0.0f) ? 0.0f : 1.0f / scale;
  uint32_t word = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    int q = static_cast<int>(rintf(clamp_sym(x[j] * inv, kInt4Max))) & 0xF;
    if (base + j >= n) q = 0;
    word |= static_cast<uint32_t>(q) << (4 * j);
  }
  const int64_t byte0 = base / 2;
  const int64_t nbytes = (n + 1) / 2;
  if (byte0 + 4 <= nbytes) {
    *reinterpret_cast<uint32_t *>(packed + byte0) = word;
  } else {
    for (int64_t b = byte0; b < nbytes; ++b) packed[b] = static_cast<uint8_t>(word >> (8 * (b - byte0)));
  }
}

// Any (even) group size: one thread per group, serial over the group.
__global__ void quantize_int4_serial_kernel(const float *__restrict__ in, uint8_t *__restrict__ packed,
                                            f16_t *__restrict__ scales, int64_t n, int group_size)
{
  const int64_t g = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t num_groups = (n + group_size - 1) / group_size;
  if (g >= num_groups) return;
  const int64_t start = g * group_size;
  const int64_t end = start + group_size < n ? start + group_size : n;
  float m = 0.0f;
  for (int64_t i = start; i < end; ++i) {
    float a = fabsf(in[i]);
    if (a > m) m = a;
  }
  const float scale = (m == 0.0f) ? 0.0f : m / kInt4Max;
  scales[g] = static_cast<f16_t>(scale);
  const float inv = (scale == 0.0f) ? 0.0f : 1.0f / scale;
  for (int64_t i = start; i < end; i += 2) {
    int q0 = static_cast<int>(rintf(clamp_sym(in[i] * inv, kInt4Max))) & 0xF;
    int q1 = 0;
    if (i + 1 < end) q1 = static_cast<int>(rintf(clamp_sym(in[i + 1] * inv, kInt4Max))) & 0xF;
    packed[i / 2] = static_cast<uint8_t>(q0 | (q1 << 4));
  }
}

// out[f] = float(code) * float(scale[f / group]); 8 elements (one packed dword) per thread
__global__ void dequantize_int4_x8_kernel(const uint8_t *__restrict__ packed, const f16_t *__restrict__ scales,
                                          float *__restrict__ out, int64_t n, int group_size, int vec)
{
  const int64_t base = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 8;
  if (base >= n) return;
  if (base + 8 <= n) {
    const uint32_t w = *reinterpret_cast<const uint32_t *>(packed + base / 2);
    const float s = static_cast<float>(scales[base / group_size]);
    float e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) e[j] = static_cast<float>(nibble_s4(w >> (4 * j), 0)) * s;
    if (vec) {
      *reinterpret_cast<floatx4_t *>(out + base) = floatx4_t{e[0], e[1], e[2], e[3]};
      *reinterpret_cast<floatx4_t *>(out + base + 4) = floatx4_t{e[4], e[5], e[6], e[7]};
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) out[base + j] = e[j];
    }
  } else {
    for (int64_t f = base; f < n; ++f) {
      const uint32_t b = packed[f / 2];
      out[f] = static_cast<float>(nibble_s4(b, static_cast<int>(f & 1))) * static_cast<float>(scales[f / group_size]);
    }
  }
}

__global__ void dequantize_int4_scalar_kernel(const uint8_t *__restrict__ packed, const f16_t *__restrict__ scales,
                                              float *__restrict__ out, int64_t n, int group_size)
{
  const int64_t f = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (f >= n) return;
  const uint32_t b = packed[f / 2];
  out[f] = static_cast<float>(nibble_s4(b, static_cast<int>(f & 1))) * static_cast<float>(scales[f / group_size]);
}

}  // namespace
}  // namespace caifx

using namespace caifx;

extern "C" {

int caifx_convert_fp32_to_fp16(const float *input, void *output, int64_t n, caifx_stream_t stream)
{
  return launch_cast<float, f16_t>(input, static_cast<f16_t *>(output), n, as_stream(stream));
}
int caifx_convert_fp16_to_fp32(const void *input, float *output, int64_t n, caifx_stream_t stream)
{
  return launch_cast<f16_t, float>(static_cast<const f16_t *>(input), output, n, as_stream(stream));
}
int caifx_convert_fp32_to_bf16(const float *input, void *output, int64_t n, caifx_stream_t stream)
{
  return launch_cast<float, bf16_t>(input, static_cast<bf16_t *>(output), n, as_stream(stream));
}
int caifx_convert_bf16_to_fp32(const void *input, float *output, int64_t n, caifx_stream_t stream)
{
  return launch_cast<bf16_t, float>(static_cast<const bf16_t *>(input), output, n, as_stream(stream));
}
int caifx_convert_fp32_to_int8(const float *input, void *output, int64_t n, caifx_stream_t stream)
{
  if (n <= 0) return CAIFX_OK;
  if (!input || !output) return CAIFX_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(cast_f32_to_int8_kernel, dim3(grid_for((n + 3) / 4)), dim3(kBlock), 0, as_stream(stream),
                     input, static_cast<int8_t *>(output), n);
  return launch_status();
}
int caifx_convert_int8_to_fp32(const void *input, float *output, int64_t n, caifx_stream_t stream)
{
  return launch_cast<int8_t, float>(static_cast<const int8_t *>(input), output, n, as_stream(stream));
}

int caifx_quantize_int8_per_tensor(const float *input, void *output, void *scale, int64_t n,
                                   caifx_stream_t stream)
{
  if (n <= 0) return CAIFX_OK;
  if (!input || !output || !scale) return CAIFX_ERR_INVALID_ARGUMENT;
  if (!aligned_to(input, 4) || !aligned_to(scale, 4)) return CAIFX_ERR_MISALIGNED;
  hipStream_t s = as_stream(stream);
  // a fill kernel, not hipMemsetAsync: safe to record into a captured graph
  hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(64), 0, s, static_cast<uint32_t *>(scale), int64_t{1}, 0u);
  int blocks = grid_for(n);
  if (blocks > 2048) blocks = 2048;
  hipLaunchKernelGGL(absmax_tensor_kernel, dim3(blocks), dim3(kBlock), 0, s, input, static_cast<uint32_t *>(scale), n,
                     aligned_to(input, 16) ? 1 : 0);
  hipLaunchKernelGGL(finalize_int8_scale_kernel, dim3(1), dim3(64), 0, s, static_cast<float *>(scale), 1);
  const int64_t body = (aligned_to(input, 16) && aligned_to(output, 16)) ? n / 16 * 16 : 0;
  if (body > 0)
    hipLaunchKernelGGL(quantize_int8_tensor_x16_kernel, dim3(grid_for(body / 16)), dim3(kBlock), 0, s, input,
                       static_cast<int8_t *>(output), static_cast<const float *>(scale), body / 16);
  if (body < n)
    hipLaunchKernelGGL(quantize_int8_kernel, dim3(grid_for((n - body + 3) / 4)), dim3(kBlock), 0, s, input + body,
                       static_cast<int8_t *>(output) + body, static_cast<const float *>(scale), n - body, 1);
  return launch_status();
}

int caifx_dequantize_int8_per_tensor(const void *input, float *output, const void *scale, int64_t n,
                                     caifx_stream_t stream)
{
  if (n <= 0) return CAIFX_OK;
  if (!input || !output || !scale) return CAIFX_ERR_INVALID_ARGUMENT;
  return launch_dequantize_int8(static_cast<const int8_t *>(input), output, static_cast<const float *>(scale), n, 1,
                                as_stream(stream));
}

int caifx_quantize_int8_per_channel(const float *input, void *output, void *scales, int rows, int cols,
                                    caifx_stream_t stream)
{
  if (rows <= 0 || cols <= 0) return CAIFX_OK;
  if (!input || !output || !scales) return CAIFX_ERR_INVALID_ARGUMENT;
  if (!aligned_to(input, 4) || !aligned_to(scales, 4)) return CAIFX_ERR_MISALIGNED;
  hipStream_t s = as_stream(stream);
  const int64_t n = static_cast<int64_t>(rows) * cols;
  hipLaunchKernelGGL(fill_u32_kernel, dim3(grid_for(cols)), dim3(kBlock), 0, s, static_cast<uint32_t *>(scales),
                     static_cast<int64_t>(cols), 0u);
  // four columns per thread when every row starts 16-byte aligned (and the codes of a row 4-byte aligned)
  const bool x4 = cols % 4 == 0 && aligned_to(input, 16) && aligned_to(output, 4) && aligned_to(scales, 16) &&
                  (rows + kQuantRows - 1) / kQuantRows <= 65535;
  if (x4)
    hipLaunchKernelGGL(absmax_columns_x4_kernel, dim3(grid_for(cols / 4, 64), (rows + kRowChunk - 1) / kRowChunk), dim3(64),
                       0, s, input, static_cast<uint32_t *>(scales), rows, cols);
  else
    hipLaunchKernelGGL(absmax_columns_kernel,
                       dim3(grid_for(cols), (rows + kRowChunk - 1) / kRowChunk > 65535 ? 65535 : (rows + kRowChunk - 1) / kRowChunk),
                       dim3(kBlock), 0, s, input, static_cast<uint32_t *>(scales), rows, cols);
  hipLaunchKernelGGL(finalize_int8_scale_kernel, dim3(grid_for(cols)), dim3(kBlock), 0, s,
                     static_cast<float *>(scales), cols);
  if (x4)
    hipLaunchKernelGGL(quantize_int8_columns_x4_kernel, dim3(grid_for(cols / 4, 64), (rows + kQuantRows - 1) / kQuantRows),
                       dim3(64), 0, s, input, static_cast<int8_t *>(output), static_cast<const float *>(scales), rows,
                       cols);
  else
    hipLaunchKernelGGL(quantize_int8_kernel, dim3(grid_for((n + 3) / 4)), dim3(kBlock), 0, s, input,
                       static_cast<int8_t *>(output), static_cast<const float *>(scales), n, cols);
  return launch_status();
}

int caifx_dequantize_int8_per_channel(const void *input, float *output, const void *scales, int rows,
                                      int cols, caifx_stream_t stream)
{
  if (rows <= 0 || cols <= 0) return CAIFX_OK;
  if (!input || !output || !scales) return CAIFX_ERR_INVALID_ARGUMENT;
  const int64_t n = static_cast<int64_t>(rows) * cols;
  return launch_dequantize_int8(static_cast<const int8_t *>(input), output, static_cast<const float *>(scales), n, cols,
                                as_stream(stream));
}

int caifx_quantize_to_int4(const float *input, void *packed_output, void *scales_output,
                           int64_t num_elements, int group_size, caifx_stream_t stream)
{
  if (num_elements <= 0) return CAIFX_OK;
  if (!input || !packed_output || !scales_output || group_size <= 0) return CAIFX_ERR_INVALID_ARGUMENT;
  if ((group_size & 1) && num_elements > group_size) return CAIFX_ERR_INVALID_ARGUMENT;
  if (!aligned_to(input, 4) || !aligned_to(scales_output, 2)) return CAIFX_ERR_MISALIGNED;
  hipStream_t s = as_stream(stream);
  const int team = group_size / 8;
  const bool team_ok = (group_size % 8 == 0) && team >= 1 && team <= 64 && (team & (team - 1)) == 0 &&
                       aligned_to(packed_output, 4);
  if (team_ok) {
    const int64_t threads = (num_elements + 7) / 8;
    hipLaunchKernelGGL(quantize_int4_team_kernel, dim3(grid_for(threads)), dim3(kBlock), 0, s, input,
                       static_cast<uint8_t *>(packed_output), static_cast<f16_t *>(scales_output), num_elements,
                       group_size, team, aligned_to(input, 16) ? 1 : 0);
  } else {
    const int64_t groups = (num_elements + group_size - 1) / group_size;
    hipLaunchKernelGGL(quantize_int4_serial_kernel, dim3(grid_for(groups)), dim3(kBlock), 0, s, input,
                       static_cast<uint8_t *>(packed_output), static_cast<f16_t *>(scales_output), num_elements,
                       group_size);
  }
  return launch_status();
}

int caifx_dequantize_int4(const void *packed_data, const void *scales, float *output,
                          int64_t num_elements, int group_size, caifx_stream_t stream)
{
  if (num_elements <= 0) return CAIFX_OK;
  if (!packed_data || !scales || !output || group_size <= 0) return CAIFX_ERR_INVALID_ARGUMENT;
  if (!aligned_to(output, 4) || !aligned_to(scales, 2)) return CAIFX_ERR_MISALIGNED;
  hipStream_t s = as_stream(stream);
  if (group_size % 8 == 0 && aligned_to(packed_data, 4)) {
    hipLaunchKernelGGL(dequantize_int4_x8_kernel, dim3(grid_for((num_elements + 7) / 8)), dim3(kBlock), 0, s,
                       static_cast<const uint8_t *>(packed_data), static_cast<const f16_t *>(scales), output,
                       num_elements, group_size, aligned_to(output, 16) ? 1 : 0);
  } else {
    hipLaunchKernelGGL(dequantize_int4_scalar_kernel, dim3(grid_for(num_elements)), dim3(kBlock), 0, s,
                       static_cast<const uint8_t *>(packed_data), static_cast<const f16_t *>(scales), output,
                       num_elements, group_size);
  }
  return launch_status();
}

}  // extern "C"
