// Measurement only: what the bf16 matrix pipes of the whole chip sustain on given operand values when they do
// nothing else.  The matrix pipes' clock follows the power the operands' bit patterns draw: all-zero operands
// run a third faster than normally distributed ones.  A dequant-GEMM's TFLOP/s on real activations is therefore
// priced against this figure on the same values, beside the published peak.
#include "caifx_internal.hpp"

namespace caifx {
namespace {

// every wave keeps four A and four B operands (16 bytes per lane each) and issues `iters` rounds of sixteen
// v_mfma_f32_32x32x16_bf16 over four independent accumulators; nothing is loaded or stored inside the loop
__global__ __launch_bounds__(512, 2) void mfma_alone_kernel(const u32x4_t *__restrict__ a_ops, const u32x4_t *__restrict__ b_ops,
                                                             int64_t iters, float *__restrict__ sink)
{
  floatx16_t acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
  bf16x8_t a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = __builtin_bit_cast(bf16x8_t, a_ops[threadIdx.x * 4 + i]);
    b[i] = __builtin_bit_cast(bf16x8_t, b_ops[threadIdx.x * 4 + i]);
  }
  for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = Mfma32<bf16_t>::run(a[i], b[r], acc[i]);
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  if (sink && blockIdx.x == 0) sink[threadIdx.x] = s;
}

}  // namespace
}  // namespace caifx

extern "C" int caifx_probe_mfma_bf16(const void *a_ops, const void *b_ops, int64_t iters, void *sink, int64_t *flops,
                                     caifx_stream_t stream)
{
  using namespace caifx;
  if (!a_ops || !b_ops || iters <= 0) return CAIFX_ERR_INVALID_ARGUMENT;
  if (!aligned_to(a_ops, 16) || !aligned_to(b_ops, 16) || !aligned_to(sink, 4)) return CAIFX_ERR_MISALIGNED;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return CAIFX_ERR_LAUNCH_FAILED;
  // one workgroup of eight waves per compute unit: two waves per SIMD, as in the GEMM kernels
  hipLaunchKernelGGL(mfma_alone_kernel, dim3(static_cast<unsigned>(cus)), dim3(512), 0, as_stream(stream),
                     static_cast<const u32x4_t *>(a_ops), static_cast<const u32x4_t *>(b_ops), iters,
                     static_cast<float *>(sink));
  if (flops) *flops = static_cast<int64_t>(cus) * 8 * iters * 16 * (2LL * 32 * 32 * 16);
  return launch_status();
}
