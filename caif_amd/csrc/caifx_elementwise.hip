// Element-wise ops that sit between the frozen-expert GEMMs (SiLU, its backward, multiply,
// add).  Each computes in fp32 and rounds once to the tensor dtype, like the reference's
// kernels; eight elements per thread on the aligned body, one per thread on the tail.
#include "caifx_common.hpp"

#pragma clang fp contract(off)

namespace caifx {
namespace {

constexpr int kBlock = 256;
constexpr int kVec = 8;

struct SiluOp {
  __device__ float operator()(float x, float) const { return silu_f32(x); }
};
struct SiluBwdOp {   // a = forward input x, b = upstream gradient
  __device__ float operator()(float x, float g) const { return silu_bwd_f32(x, g); }
};
struct MulOp {
  __device__ float operator()(float a, float b) const { return a * b; }
};
struct AddOp {
  __device__ float operator()(float a, float b) const { return a + b; }
};
template <typename T> struct SiluMulOp {   // a = gate, b = up; silu(gate) is rounded to T first
  __device__ float operator()(float g, float u) const { return round_through<T>(silu_f32(g)) * u; }
};

template <typename T, typename Op, bool kBinary>
__global__ void ew_kernel(const T *__restrict__ a, const T *__restrict__ b, T *__restrict__ out, int64_t n,
                          int64_t n_body, Op op)
{
  const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t i = t * kVec;
  if (i < n_body) {
    T va[kVec], vb[kVec], vo[kVec];
#pragma unroll
    for (int j = 0; j < kVec; ++j) va[j] = a[i + j];
    if (kBinary) {
#pragma unroll
      for (int j = 0; j < kVec; ++j) vb[j] = b[i + j];
    }
#pragma unroll
    for (int j = 0; j < kVec; ++j)
      vo[j] = from_f32<T>(op(to_f32<T>(va[j]), kBinary ? to_f32<T>(vb[j]) : 0.0f));
#pragma unroll
    for (int j = 0; j < kVec; ++j) out[i + j] = vo[j];
  } else {
    const int64_t k = n_body + (t - n_body / kVec);
    if (k < n) out[k] = from_f32<T>(op(to_f32<T>(a[k]), kBinary ? to_f32<T>(b[k]) : 0.0f));
  }
}

template <typename T, typename Op, bool kBinary>
int launch_ew(const void *a, const void *b, void *out, int64_t n, hipStream_t s, Op op)
{
  const int64_t n_body = (n / kVec) * kVec;
  const int64_t threads = n_body / kVec + (n - n_body);
  hipLaunchKernelGGL((ew_kernel<T, Op, kBinary>), dim3(static_cast<unsigned>((threads + kBlock - 1) / kBlock)), dim3(kBlock), 0, s,
                     static_cast<const T *>(a), static_cast<const T *>(b), static_cast<T *>(out), n, n_body, op);
  return launch_status();
}

// Backward of hidden = silu(gate) * up as the reference chains four kernels, with every intermediate
// rounded to T exactly where those kernels round:
//   act = T(silu(gate));  grad_up = T(grad_hidden * act);
//   t = T(grad_hidden * up);  grad_gate = T(silu'(gate) applied to t)
// Three tensors in, two out, one pass.
template <typename T>
__global__ void swiglu_bwd_kernel(const T *__restrict__ gate, const T *__restrict__ up, const T *__restrict__ gh,
                                  T *__restrict__ grad_gate, T *__restrict__ grad_up, int64_t n, int64_t n_body)
{
  const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  auto one = [&](T g16, T u16, T h16, T &gg, T &gu) { swiglu_bwd_one<T>(g16, u16, h16, gg, gu); };
  const int64_t i = t * kVec;
  if (i < n_body) {
    T vg[kVec], vu[kVec], vh[kVec], og[kVec], ou[kVec];
#pragma unroll
    for (int j = 0; j < kVec; ++j) vg[j] = gate[i + j];
#pragma unroll
    for (int j = 0; j < kVec; ++j) vu[j] = up[i + j];
#pragma unroll
    for (int j = 0; j < kVec; ++j) vh[j] = gh[i + j];
#pragma unroll
    for (int j = 0; j < kVec; ++j) one(vg[j], vu[j], vh[j], og[j], ou[j]);
#pragma unroll
    for (int j = 0; j < kVec; ++j) grad_gate[i + j] = og[j];
#pragma unroll
    for (int j = 0; j < kVec; ++j) grad_up[i + j] = ou[j];
  } else {
    const int64_t k = n_body + (t - n_body / kVec);
    if (k < n) one(gate[k], up[k], gh[k], grad_gate[k], grad_up[k]);
  }
}

template <typename T>
int launch_swiglu_bwd(const void *gate, const void *up, const void *gh, void *grad_gate, void *grad_up, int64_t n, hipStream_t s)
{
  const int64_t n_body = (n / kVec) * kVec;
  const int64_t threads = n_body / kVec + (n - n_body);
  hipLaunchKernelGGL((swiglu_bwd_kernel<T>), dim3(static_cast<unsigned>((threads + kBlock - 1) / kBlock)), dim3(kBlock), 0, s,
                     static_cast<const T *>(gate), static_cast<const T *>(up), static_cast<const T *>(gh),
                     static_cast<T *>(grad_gate), static_cast<T *>(grad_up), n, n_body);
  return launch_status();
}

template <typename Op, bool kBinary>
int dispatch_ew(const void *a, const void *b, void *out, int64_t n, int dtype, caifx_stream_t stream, Op op)
{
  if (n <= 0) return CAIFX_OK;
  if (!a || !out || (kBinary && !b)) return CAIFX_ERR_INVALID_ARGUMENT;
  hipStream_t s = as_stream(stream);
  switch (dtype) {
    case CAIFX_F32: return launch_ew<float, Op, kBinary>(a, b, out, n, s, op);
    case CAIFX_F16: return launch_ew<f16_t, Op, kBinary>(a, b, out, n, s, op);
    case CAIFX_BF16: return launch_ew<bf16_t, Op, kBinary>(a, b, out, n, s, op);
    default: return CAIFX_ERR_INVALID_ARGUMENT;
  }
}

}  // namespace
}  // namespace caifx

using namespace caifx;

extern "C" {

int caifx_silu(const void *input, void *output, int64_t n, int dtype, caifx_stream_t stream)
{
  return dispatch_ew<SiluOp, false>(input, nullptr, output, n, dtype, stream, SiluOp{});
}
int caifx_silu_backward(const void *input, const void *grad_output, void *grad_input, int64_t n, int dtype,
                        caifx_stream_t stream)
{
  return dispatch_ew<SiluBwdOp, true>(input, grad_output, grad_input, n, dtype, stream, SiluBwdOp{});
}
int caifx_multiply(const void *a, const void *b, void *output, int64_t n, int dtype, caifx_stream_t stream)
{
  return dispatch_ew<MulOp, true>(a, b, output, n, dtype, stream, MulOp{});
}
int caifx_add(const void *a, const void *b, void *output, int64_t n, int dtype, caifx_stream_t stream)
{
  return dispatch_ew<AddOp, true>(a, b, output, n, dtype, stream, AddOp{});
}
int caifx_silu_multiply(const void *gate, const void *up, void *hidden, int64_t n, int dtype,
                        caifx_stream_t stream)
{
  if (n <= 0) return CAIFX_OK;
  if (!gate || !up || !hidden) return CAIFX_ERR_INVALID_ARGUMENT;
  hipStream_t s = as_stream(stream);
  switch (dtype) {
    case CAIFX_F32: return launch_ew<float, SiluMulOp<float>, true>(gate, up, hidden, n, s, SiluMulOp<float>{});
    case CAIFX_F16: return launch_ew<f16_t, SiluMulOp<f16_t>, true>(gate, up, hidden, n, s, SiluMulOp<f16_t>{});
    case CAIFX_BF16: return launch_ew<bf16_t, SiluMulOp<bf16_t>, true>(gate, up, hidden, n, s, SiluMulOp<bf16_t>{});
    default: return CAIFX_ERR_INVALID_ARGUMENT;
  }
}

int caifx_swiglu_backward(const void *gate, const void *up, const void *grad_hidden, void *grad_gate, void *grad_up,
                          int64_t n, int dtype, caifx_stream_t stream)
{
  if (n <= 0) return CAIFX_OK;
  if (!gate || !up || !grad_hidden || !grad_gate || !grad_up) return CAIFX_ERR_INVALID_ARGUMENT;
  hipStream_t s = as_stream(stream);
  switch (dtype) {
    case CAIFX_F32: return launch_swiglu_bwd<float>(gate, up, grad_hidden, grad_gate, grad_up, n, s);
    case CAIFX_F16: return launch_swiglu_bwd<f16_t>(gate, up, grad_hidden, grad_gate, grad_up, n, s);
    case CAIFX_BF16: return launch_swiglu_bwd<bf16_t>(gate, up, grad_hidden, grad_gate, grad_up, n, s);
    default: return CAIFX_ERR_INVALID_ARGUMENT;
  }
}

}  // extern "C"
