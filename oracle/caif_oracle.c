/*
 * caif_oracle.c -- CPU restatement of the reference's frozen quantized-linear
 * arithmetic.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
 * compared against; nothing in the shipped library links, loads or calls it.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
 * use it.
 *
 * Every function restates, in scalar C with IEEE-754 binary32 semantics
 * (compile with -ffp-contract=off, no fast-math), what one reference routine
 * computes; the reference file:line it follows is cited at each function.
 * Citations are relative to the reference checkout (cppaif/caif).
 *
 * Parity status of each function (what pins it besides this restatement) is
 * listed in tests/test_oracle_*.py; there is no "parity unpinned" function for
 * value parity at the stated tolerances.  The one thing that cannot be derived
 * from the reference's sources is the summation order inside its vendor GEMM
 * (cuBLAS / OpenBLAS); the GEMMs here accumulate in binary64 and round once,
 * which is within 1 ulp(fp32)*sqrt(K) of any fp32 ordering.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* threads the parallel loops below run on (what a timed CPU baseline has to state) */
ORC_API int orc_max_threads(void)
{
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* dtype codes shared with include/caifx.h */
enum { ORC_F32 = 0, ORC_F16 = 1, ORC_BF16 = 2 };
/* weight kinds shared with include/caifx.h */
enum { ORC_W_INT8 = 0, ORC_W_INT4_GROUP = 1, ORC_W_F32 = 2, ORC_W_F16 = 3, ORC_W_BF16 = 4 };

/* include/caif/caif_cuda_kernels_constants.cuh:185-197 */
static const float k_int8_max = 127.0f;
static const float k_int4_max = 7.0f;

/* ------------------------------------------------------------------------ */
/* scalar float <-> 16-bit conversions                                       */
/* ------------------------------------------------------------------------ */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* fp32 -> bf16, round-to-nearest-even, NaN kept NaN.
 * Device: __float2bfloat16 (src/caif_cuda_kernels_quant.cu:84-96); the same
 * rounding is spelled out on the host in
 * include/caif/caif_host_dtype_convert.h:55-66. */
ORC_API uint16_t orc_f32_to_bf16(float f)
{
  uint32_t bits = f2u(f);
  if (((bits & 0x7f800000u) == 0x7f800000u) && (bits & 0x007fffffu))
    return (uint16_t)((bits >> 16) | 0x40u);
  uint32_t bias = 0x7fffu + ((bits >> 16) & 1u);
  return (uint16_t)((bits + bias) >> 16);
}

/* include/caif/caif_host_dtype_convert.h:143-149 */
ORC_API float orc_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* fp32 -> fp16, IEEE round-to-nearest-even (device __float2half,
 * src/caif_cuda_kernels_quant.cu:42-54 and :299).  This deliberately does NOT
 * follow include/caif/caif_host_dtype_convert.h:107-118, whose normalised
 * branch rounds exact ties upward; the device intrinsic rounds ties to even. */
ORC_API uint16_t orc_f32_to_f16(float f)
{
  uint32_t bits = f2u(f);
  uint32_t sign = (bits >> 16) & 0x8000u;
  uint32_t absb = bits & 0x7fffffffu;
  if (absb >= 0x7f800000u) {                     /* inf / NaN */
    if (absb > 0x7f800000u) {
      uint32_t m = (absb & 0x007fffffu) >> 13;
      return (uint16_t)(sign | 0x7c00u | m | (m == 0 ? 0x200u : 0u));
    }
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absb >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 -> inf */
  if (absb < 0x33000001u) return (uint16_t)sign;              /* <= 2^-25 -> 0 */
  int32_t e = (int32_t)(absb >> 23) - 127;       /* unbiased exponent */
  uint32_t mant = (absb & 0x007fffffu) | 0x00800000u;         /* 24-bit */
  int shift;                                      /* bits to drop */
  uint32_t base;
  if (e < -14) { shift = 13 + (-14 - e); base = 0; }          /* subnormal half */
  else { shift = 13; base = (uint32_t)(e + 15) << 10; mant &= 0x007fffffu; }
  uint32_t kept = mant >> shift;
  uint32_t rem = mant & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (kept & 1u))) kept += 1u;  /* carries into exponent correctly */
  return (uint16_t)(sign | (base + kept));
}

ORC_API float orc_f16_to_f32(uint16_t h)
{
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu;
  uint32_t m = h & 0x3ffu;
  if (e == 0) {
    if (m == 0) return u2f(sign);
    float v = (float)m * 5.9604644775390625e-08f;            /* m * 2^-24, exact */
    return sign ? -v : v;
  }
  if (e == 31) return u2f(sign | 0x7f800000u | (m << 13));
  return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

/* Round an fp32 value to `dtype` and widen it again (the value a tensor of
 * that dtype would hold).  CAIF_DeviceTensor::To() between float dtypes is a
 * plain cast kernel (src/caif_device_tensor.cpp:604-706 ->
 * src/caif_cuda_kernels_quant.cu:42-138). */
ORC_API float orc_round_scalar(float v, int dtype)
{
  if (dtype == ORC_BF16) return orc_bf16_to_f32(orc_f32_to_bf16(v));
  if (dtype == ORC_F16) return orc_f16_to_f32(orc_f32_to_f16(v));
  return v;
}

ORC_API void orc_round_to_dtype(float *buf, int64_t n, int dtype)
{
  if (dtype == ORC_F32) return;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) buf[i] = orc_round_scalar(buf[i], dtype);
}

/* src/caif_cuda_kernels_quant.cu:42-138 -- element casts */
ORC_API void orc_convert_fp32_to_fp16(const float *in, uint16_t *out, int64_t n)
{ for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_f16(in[i]); }
ORC_API void orc_convert_fp16_to_fp32(const uint16_t *in, float *out, int64_t n)
{ for (int64_t i = 0; i < n; ++i) out[i] = orc_f16_to_f32(in[i]); }
ORC_API void orc_convert_fp32_to_bf16(const float *in, uint16_t *out, int64_t n)
{ for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_bf16(in[i]); }
ORC_API void orc_convert_bf16_to_fp32(const uint16_t *in, float *out, int64_t n)
{ for (int64_t i = 0; i < n; ++i) out[i] = orc_bf16_to_f32(in[i]); }

/* clamp to +-limit (comparison order as in the reference: NaN passes through) */
static inline float clampf(float v, float limit)
{
  if (v > limit) v = limit;
  else if (v < -limit) v = -limit;
  return v;
}

/* src/caif_cuda_kernels_quant.cu:144-162 -- unscaled fp32 -> int8 cast */
ORC_API void orc_convert_fp32_to_int8(const float *in, int8_t *out, int64_t n)
{ for (int64_t i = 0; i < n; ++i) out[i] = (int8_t)rintf(clampf(in[i], k_int8_max)); }
/* src/caif_cuda_kernels_quant.cu:177-186 */
ORC_API void orc_convert_int8_to_fp32(const int8_t *in, float *out, int64_t n)
{ for (int64_t i = 0; i < n; ++i) out[i] = (float)in[i]; }

/* ------------------------------------------------------------------------ */
/* int8 symmetric quantisation                                               */
/* ------------------------------------------------------------------------ */

/* src/caif_cuda_kernels_quant.cu:384-444,458-483.
 * scale = max|x| / 127 (1.0 when the input is all zero); q = rint(clamp(x *
 * (1/scale))).  The max is order independent, so the atomicMax reduction of
 * the reference and this serial loop agree bit for bit. */
ORC_API void orc_quantize_int8_per_tensor(const float *in, int8_t *out, float *scale, int64_t n)
{
  if (n <= 0) return;
  float max_abs = 0.0f;
  for (int64_t i = 0; i < n; ++i) {
    float v = fabsf(in[i]);
    if (v > max_abs) max_abs = v;
  }
  float s = (max_abs > 0.0f) ? max_abs / k_int8_max : 1.0f;
  scale[0] = s;
  float inv_s = (s > 0.0f) ? 1.0f / s : 0.0f;
  for (int64_t i = 0; i < n; ++i)
    out[i] = (int8_t)rintf(clampf(in[i] * inv_s, k_int8_max));
}

/* src/caif_cuda_kernels_quant.cu:446-456 */
ORC_API void orc_dequantize_int8_per_tensor(const int8_t *in, float *out, const float *scale, int64_t n)
{
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) out[i] = (float)in[i] * scale[0];
}

/* src/caif_cuda_kernels_quant.cu:502-559,576-600.
 * scales[c] = max_r |x[r*cols+c]| / 127 (1.0 if zero); the scale of flat
 * element f is scales[f % cols]. */
ORC_API void orc_quantize_int8_per_channel(const float *in, int8_t *out, float *scales, int rows, int cols)
{
  if (rows <= 0 || cols <= 0) return;
  for (int c = 0; c < cols; ++c) {
    float max_abs = 0.0f;
    for (int r = 0; r < rows; ++r) {
      float v = fabsf(in[(int64_t)r * cols + c]);
      if (v > max_abs) max_abs = v;
    }
    scales[c] = (max_abs > 0.0f) ? max_abs / k_int8_max : 1.0f;
  }
  int64_t total = (int64_t)rows * cols;
  for (int64_t idx = 0; idx < total; ++idx) {
    float s = scales[idx % cols];
    float inv_s = (s > 0.0f) ? 1.0f / s : 0.0f;
    out[idx] = (int8_t)rintf(clampf(in[idx] * inv_s, k_int8_max));
  }
}

/* src/caif_cuda_kernels_quant.cu:561-574 */
ORC_API void orc_dequantize_int8_per_channel(const int8_t *in, float *out, const float *scales, int rows, int cols)
{
  int64_t total = (int64_t)rows * cols;
#pragma omp parallel for schedule(static)
  for (int64_t idx = 0; idx < total; ++idx) out[idx] = (float)in[idx] * scales[idx % cols];
}

/* ------------------------------------------------------------------------ */
/* int4 symmetric per-group quantisation, two nibbles per byte               */
/* ------------------------------------------------------------------------ */

/* src/caif_cuda_kernels_quant.cu:258-342.
 * Groups run over the flat index.  scale = max|x|/7 in fp32 (0 for an all-zero
 * group); the STORED scale is that value rounded to fp16, but the codes are
 * computed with 1/scale of the UNROUNDED fp32 scale.  Even flat index -> low
 * nibble, odd -> high nibble, two's complement; a group that ends on an odd
 * count leaves its last high nibble zero. */
ORC_API void orc_quantize_to_int4(const float *in, uint8_t *packed, uint16_t *scales_f16,
                                  int64_t n, int group_size)
{
  if (n <= 0) return;
  int64_t num_groups = (n + group_size - 1) / group_size;
  for (int64_t g = 0; g < num_groups; ++g) {
    int64_t start = g * group_size;
    int64_t end = start + group_size;
    if (end > n) end = n;
    float max_abs = 0.0f;
    for (int64_t i = start; i < end; ++i) {
      float a = fabsf(in[i]);
      if (a > max_abs) max_abs = a;
    }
    float scale = (max_abs == 0.0f) ? 0.0f : max_abs / k_int4_max;
    scales_f16[g] = orc_f32_to_f16(scale);
    float inv_scale = (scale == 0.0f) ? 0.0f : 1.0f / scale;
    for (int64_t i = start; i < end; i += 2) {
      int q0 = (int)rintf(clampf(in[i] * inv_scale, k_int4_max)) & 0x0F;
      int q1 = 0;
      if (i + 1 < end) q1 = (int)rintf(clampf(in[i + 1] * inv_scale, k_int4_max)) & 0x0F;
      packed[i / 2] = (uint8_t)(q0 | (q1 << 4));
    }
  }
}

static inline int nibble_at(const uint8_t *packed, int64_t idx)
{
  uint8_t b = packed[idx / 2];
  int v = (idx & 1) ? ((b >> 4) & 0x0F) : (b & 0x0F);
  if (v & 0x08) v |= (int)0xFFFFFFF0;            /* sign extend 4 -> 32 bits */
  return v;
}

/* src/caif_cuda_kernels_quant.cu:205-237 */
ORC_API void orc_dequantize_int4(const uint8_t *packed, const uint16_t *scales_f16, float *out,
                                 int64_t n, int group_size)
{
#pragma omp parallel for schedule(static)
  for (int64_t idx = 0; idx < n; ++idx)
    out[idx] = (float)nibble_at(packed, idx) * orc_f16_to_f32(scales_f16[idx / group_size]);
}

/* ------------------------------------------------------------------------ */
/* frozen linear: weight materialisation + GEMMs                             */
/* ------------------------------------------------------------------------ */

/* CAIF_DeviceFrozenLinear::ConvertToComputeDtype
 * (src/caif_device_frozen_linear.cpp:289-378): dequantise the stored weight
 * to fp32 with the launcher the storage kind selects, then cast to the
 * compute dtype.  The flat buffer is afterwards read as W[n,k] = buf[n*K+k]
 * (:345).  For int8 the layer calls the per-channel dequantiser with
 * rows=InputDim, cols=OutputDim (:356-361), i.e. scale index = f % N; that is
 * the `scale_period` here (1 for per-tensor).  scales == NULL reproduces the
 * int8-without-scales branch (:373-375), a plain widening cast.
 * Float storage (ORC_W_F32 / F16 / BF16): the buffer as it is when storage and
 * compute types agree (:301-318), otherwise its elements cast to the compute
 * type (the tensor's .To(target): widen to fp32, round to nearest even).
 * w_out holds the compute-dtype values widened to fp32. */
ORC_API void orc_frozen_weight_compute(const void *wq, int w_kind, const void *scales,
                                       int64_t N, int64_t K, int64_t scale_period, int group_size,
                                       int compute_dtype, float *w_out)
{
  int64_t total = N * K;
  if (w_kind == ORC_W_F32) {
    memcpy(w_out, wq, (size_t)total * sizeof(float));
  } else if (w_kind == ORC_W_F16 || w_kind == ORC_W_BF16) {
    const uint16_t *h = (const uint16_t *)wq;
#pragma omp parallel for schedule(static)
    for (int64_t f = 0; f < total; ++f)
      w_out[f] = w_kind == ORC_W_F16 ? orc_f16_to_f32(h[f]) : orc_bf16_to_f32(h[f]);
  } else if (w_kind == ORC_W_INT4_GROUP) {
    orc_dequantize_int4((const uint8_t *)wq, (const uint16_t *)scales, w_out, total, group_size);
  } else {
    const int8_t *q = (const int8_t *)wq;
    const float *s = (const float *)scales;
#pragma omp parallel for schedule(static)
    for (int64_t f = 0; f < total; ++f)
      w_out[f] = s ? (float)q[f] * s[f % scale_period] : (float)q[f];
  }
  orc_round_to_dtype(w_out, total, compute_dtype);
}

/* Forward GEMM of CAIF_DeviceFrozenLinear::ForwardImpl
 * (src/caif_device_frozen_linear.cpp:445-509): Y[M,N] = X[M,K] * W[N,K]^T,
 * operands already in the compute dtype (widened to fp32 here), fp32 output.
 * Host_e equivalent: cblas_sgemm(RowMajor, NoTrans, Trans, M,N,K, ...)
 * (src/caif_ops_host.cpp:112-139 -> src/caif_host_gemm.cpp:52-65).
 * Accumulates in binary64 and rounds once to fp32. */
ORC_API void orc_gemm_nt(int64_t M, int64_t N, int64_t K, const float *X, const float *W, float *Y)
{
#pragma omp parallel for schedule(static) collapse(2)
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      const float *x = X + m * K;
      const float *w = W + n * K;
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k) acc += (double)x[k] * (double)w[k];
      Y[m * N + n] = (float)acc;
    }
}

/* Backward GEMM of CAIF_DeviceFrozenLinear::BackwardImpl
 * (src/caif_device_frozen_linear.cpp:583-645): dX[M,K] = dY[M,N] * W[N,K],
 * fp32 output.  Host_e: cblas_sgemm(RowMajor, NoTrans, NoTrans, M,K,N, ...)
 * (src/caif_ops_host.cpp:54-81). */
ORC_API void orc_gemm_nn(int64_t M, int64_t N, int64_t K, const float *dY, const float *W, float *dX)
{
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    double *acc = (double *)calloc((size_t)K, sizeof(double));
    for (int64_t n = 0; n < N; ++n) {
      double g = (double)dY[m * N + n];
      const float *w = W + n * K;
      for (int64_t k = 0; k < K; ++k) acc[k] += g * (double)w[k];
    }
    for (int64_t k = 0; k < K; ++k) dX[m * K + k] = (float)acc[k];
    free(acc);
  }
}

/* ------------------------------------------------------------------------ */
/* element-wise ops between the expert GEMMs                                 */
/* ------------------------------------------------------------------------ */

/* SiLU forward, computed in fp32 and rounded once to the tensor dtype
 * (src/caif_cuda_kernels_activations.cu:513-514).  in/out hold dtype values
 * widened to fp32. */
ORC_API void orc_silu(const float *in, float *out, int64_t n, int dtype)
{
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float x = in[i];
    out[i] = orc_round_scalar(x / (1.0f + expf(-x)), dtype);
  }
}

/* SiLU backward (src/caif_cuda_kernels_activations.cu:558-561):
 * s = 1/(1+exp(-x)); r = g*s*(1+x*(1-s)), left-to-right fp32, one rounding to
 * the tensor dtype.  The reference's build leaves nvcc's multiply-add contraction
 * on (CMakeLists.txt:350-351 sets no --fmad), so 1+x*(1-s) is one fused
 * multiply-add there; fmaf states that here, whatever -ffp-contract says. */
ORC_API void orc_silu_backward(const float *x_in, const float *grad_out, float *grad_in, int64_t n, int dtype)
{
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float gv = grad_out[i];
    float x = x_in[i];
    float s = 1.0f / (1.0f + expf(-x));
    grad_in[i] = orc_round_scalar(gv * s * fmaf(x, 1.0f - s, 1.0f), dtype);
  }
}

/* Multiply / Add: T(float(a) op float(b)) per element
 * (src/caif_cuda_kernels_elementwise.cu:247-269 mul, :42-64 add). */
ORC_API void orc_multiply(const float *a, const float *b, float *out, int64_t n, int dtype)
{
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) out[i] = orc_round_scalar(a[i] * b[i], dtype);
}
ORC_API void orc_add(const float *a, const float *b, float *out, int64_t n, int dtype)
{
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) out[i] = orc_round_scalar(a[i] + b[i], dtype);
}

/* ------------------------------------------------------------------------ */
/* MoE token -> expert segment map                                           */
/* ------------------------------------------------------------------------ */

/* CAIF_Ops::MoEBuildDispatchMapDevice (src/caif_ops_device.cpp:4896-4942).
 * counts per expert (ids outside [0,E) ignored), optional capacity clamp,
 * prefix sum into offsets[E+1]; map[t*top_k+k] = arrival position of (t,k)
 * inside its expert in token-major, k-minor order, or -1 when dropped.
 * Returns total_assigned = offsets[E]. */
ORC_API uint32_t orc_moe_build_dispatch_map(const int32_t *indices, uint32_t num_tokens,
                                            uint32_t num_experts, uint32_t top_k,
                                            uint32_t capacity_per_expert,
                                            int32_t *dispatch_map, int32_t *offsets)
{
  uint32_t *counts = (uint32_t *)calloc(num_experts ? num_experts : 1, sizeof(uint32_t));
  uint32_t *pos = (uint32_t *)calloc(num_experts ? num_experts : 1, sizeof(uint32_t));
  for (uint32_t t = 0; t < num_tokens; ++t)
    for (uint32_t k = 0; k < top_k; ++k) {
      int32_t e = indices[t * top_k + k];
      if (e >= 0 && e < (int32_t)num_experts) ++counts[e];
    }
  offsets[0] = 0;
  for (uint32_t e = 0; e < num_experts; ++e) {
    if (capacity_per_expert > 0 && counts[e] > capacity_per_expert) counts[e] = capacity_per_expert;
    offsets[e + 1] = offsets[e] + (int32_t)counts[e];
  }
  for (uint32_t t = 0; t < num_tokens; ++t)
    for (uint32_t k = 0; k < top_k; ++k) {
      int32_t e = indices[t * top_k + k];
      dispatch_map[t * top_k + k] = -1;
      if (e >= 0 && e < (int32_t)num_experts && pos[e] < counts[e]) {
        dispatch_map[t * top_k + k] = (int32_t)pos[e];
        ++pos[e];
      }
    }
  uint32_t total = (uint32_t)offsets[num_experts];
  free(counts);
  free(pos);
  return total;
}
