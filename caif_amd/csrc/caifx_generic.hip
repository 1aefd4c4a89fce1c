// Shape-agnostic dequant-GEMM kernels: any M, N, K, group size, scale period, dtype mix and
// the fp32 compute type.  They are the correctness floor the tuned kernels fall back to for
// shapes outside their tiling assumptions; they decode every weight exactly like the tuned
// kernels (fp32 code*scale, one rounding to the compute dtype) and accumulate in fp32.
#include "caifx_internal.hpp"

namespace caifx {
namespace {

__device__ __forceinline__ float round_rt(float v, int dt)
{
  if (dt == CAIFX_BF16) return round_through<bf16_t>(v);
  if (dt == CAIFX_F16) return round_through<f16_t>(v);
  return v;
}

__device__ __forceinline__ float load_rt(const void *p, int dt, int64_t i)
{
  if (dt == CAIFX_BF16) return to_f32(static_cast<const bf16_t *>(p)[i]);
  if (dt == CAIFX_F16) return to_f32(static_cast<const f16_t *>(p)[i]);
  return static_cast<const float *>(p)[i];
}

__device__ __forceinline__ void store_rt(void *p, int dt, int64_t i, float v)
{
  if (dt == CAIFX_BF16) static_cast<bf16_t *>(p)[i] = from_f32<bf16_t>(v);
  else if (dt == CAIFX_F16) static_cast<f16_t *>(p)[i] = from_f32<f16_t>(v);
  else static_cast<float *>(p)[i] = v;
}

// W[flat] in the compute dtype, widened to fp32
__device__ __forceinline__ float weight_rt(const QWeight &w, const void *wq, const void *scales, int64_t f,
                                           int compute_dtype)
{
  float v;
  if (w.kind == CAIFX_W_F32) {
    v = static_cast<const float *>(wq)[f];
  } else if (w.kind == CAIFX_W_F16) {
    v = to_f32(static_cast<const f16_t *>(wq)[f]);
  } else if (w.kind == CAIFX_W_BF16) {
    v = to_f32(static_cast<const bf16_t *>(wq)[f]);
  } else if (w.kind == CAIFX_W_INT4_GROUP) {
    const uint32_t b = static_cast<const uint8_t *>(wq)[f >> 1];
    v = static_cast<float>(nibble_s4(b, static_cast<int>(f & 1))) *
        to_f32(static_cast<const f16_t *>(scales)[f / w.group_size]);
  } else {
    v = static_cast<float>(static_cast<const int8_t *>(wq)[f]);
    if (scales) v *= static_cast<const float *>(scales)[f % w.scale_period];
  }
  return round_rt(v, compute_dtype);
}

constexpr int kMB = 8;   // rows of X / dY a block keeps accumulators for

// Y[m, n] = sum_k X[m,k] W[n,k].  One wave per output column n and block of kMB rows;
// lanes stride over k (coalesced), then a wave reduction.
__global__ void generic_forward_kernel(GemmArgs a)
{
  const int lane = threadIdx.x & 63;
  const int64_t n = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  int64_t row_lo = 0, row_hi = a.M;
  const void *wq = a.w.q;
  const void *scales = a.w.scales;
  if (a.offsets) {   // grouped: blockIdx.z = expert
    const int e = blockIdx.z;
    row_lo = a.offsets[e];
    row_hi = a.offsets[e + 1];
    // offsets that are not non-decreasing or run past the buffer lose rows instead of leaving it
    row_lo = row_lo < 0 ? 0 : (row_lo > a.M ? a.M : row_lo);
    row_hi = row_hi < row_lo ? row_lo : (row_hi > a.M ? a.M : row_hi);
    wq = a.wq_ptrs[e];
    scales = a.scales_ptrs ? a.scales_ptrs[e] : nullptr;
  }
  if (n >= a.N) return;
  // blocks of kMB rows are strided over gridDim.y, which the launch caps at the grid limit
  for (int64_t m0 = row_lo + static_cast<int64_t>(blockIdx.y) * kMB; m0 < row_hi; m0 += static_cast<int64_t>(gridDim.y) * kMB) {
    const int mcnt = static_cast<int>(row_hi - m0 < kMB ? row_hi - m0 : kMB);
    float acc[kMB];
#pragma unroll
    for (int i = 0; i < kMB; ++i) acc[i] = 0.0f;
    for (int64_t k = lane; k < a.K; k += 64) {
      const float wv = weight_rt(a.w, wq, scales, n * a.K + k, a.compute_dtype);
#pragma unroll
      for (int i = 0; i < kMB; ++i)
        if (i < mcnt) acc[i] = __builtin_fmaf(round_rt(load_rt(a.x, a.x_dtype, (m0 + i) * a.K + k), a.compute_dtype), wv, acc[i]);
    }
#pragma unroll
    for (int i = 0; i < kMB; ++i) {
      float v = acc[i];
      for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
      if (lane == 0 && i < mcnt) store_rt(a.y, a.y_dtype, (m0 + i) * a.N + n, v);
    }
  }
}

// dX[m, k] = sum_n dY[m,n] W[n,k].  One thread per k (coalesced over a weight row) and block
// of kMB rows; serial over n.
__global__ void generic_backward_kernel(GemmArgs a)
{
  const int64_t k = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  int64_t row_lo = 0, row_hi = a.M;
  const void *wq = a.w.q;
  const void *scales = a.w.scales;
  if (a.offsets) {
    const int e = blockIdx.z;
    row_lo = a.offsets[e];
    row_hi = a.offsets[e + 1];
    // offsets that are not non-decreasing or run past the buffer lose rows instead of leaving it
    row_lo = row_lo < 0 ? 0 : (row_lo > a.M ? a.M : row_lo);
    row_hi = row_hi < row_lo ? row_lo : (row_hi > a.M ? a.M : row_hi);
    wq = a.wq_ptrs[e];
    scales = a.scales_ptrs ? a.scales_ptrs[e] : nullptr;
  }
  if (k >= a.K) return;
  for (int64_t m0 = row_lo + static_cast<int64_t>(blockIdx.y) * kMB; m0 < row_hi; m0 += static_cast<int64_t>(gridDim.y) * kMB) {
    const int mcnt = static_cast<int>(row_hi - m0 < kMB ? row_hi - m0 : kMB);
    float acc[kMB];
#pragma unroll
    for (int i = 0; i < kMB; ++i) acc[i] = 0.0f;
    for (int64_t n = 0; n < a.N; ++n) {
      const float wv = weight_rt(a.w, wq, scales, n * a.K + k, a.compute_dtype);
#pragma unroll
      for (int i = 0; i < kMB; ++i)
        if (i < mcnt) acc[i] = __builtin_fmaf(round_rt(load_rt(a.x, a.x_dtype, (m0 + i) * a.N + n), a.compute_dtype), wv, acc[i]);
    }
#pragma unroll
    for (int i = 0; i < kMB; ++i)
      if (i < mcnt) store_rt(a.y, a.y_dtype, (m0 + i) * a.K + k, acc[i]);
  }
}

}  // namespace

// a.M is the row count for the plain call, or an upper bound of any one expert's segment
// length for the grouped call (offsets != nullptr, num_experts > 0).
// Grid limits: y and z hold at most 65535 blocks.  Row blocks beyond that are reached by the kernels' stride over
// gridDim.y; more experts than that have no launch here.
unsigned generic_row_blocks(int64_t M)
{
  const int64_t blocks = (M + kMB - 1) / kMB;
  return static_cast<unsigned>(blocks < 1 ? 1 : (blocks > 65535 ? 65535 : blocks));
}

int generic_forward(const GemmArgs &a, hipStream_t s)
{
  const int waves = 4;
  if (a.offsets && a.num_experts > 65535) return CAIFX_ERR_UNSUPPORTED;
  dim3 grid(static_cast<unsigned>((a.N + waves - 1) / waves), generic_row_blocks(a.M), a.offsets ? a.num_experts : 1);
  hipLaunchKernelGGL(generic_forward_kernel, grid, dim3(waves * 64), 0, s, a);
  return launch_status();
}

int generic_backward(const GemmArgs &a, hipStream_t s)
{
  if (a.offsets && a.num_experts > 65535) return CAIFX_ERR_UNSUPPORTED;
  dim3 grid(static_cast<unsigned>((a.K + 255) / 256), generic_row_blocks(a.M), a.offsets ? a.num_experts : 1);
  hipLaunchKernelGGL(generic_backward_kernel, grid, dim3(256), 0, s, a);
  return launch_status();
}

}  // namespace caifx
