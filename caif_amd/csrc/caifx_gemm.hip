// Host side of the tiled dequant-GEMM for integer codes (int8, packed int4): argument checks, tile and
// scale-mode choice, the shared reduction for launches with few tiles.  The kernel is in caifx_gemm_tile.hpp.
#include "caifx_gemm_regw.hpp"
#include "caifx_gemm_tile.hpp"


namespace caifx {
namespace {

using namespace gemm_tile;

template <typename CT, typename XT>
int pick_kind(const TileArgs &t, bool int4, bool backward, bool grouped, hipStream_t s)
{
  if (int4) return backward ? launch_tile<CT, XT, W_CODES4, true>(t, grouped, s) : launch_tile<CT, XT, W_CODES4, false>(t, grouped, s);
  return backward ? launch_tile<CT, XT, W_CODES8, true>(t, grouped, s) : launch_tile<CT, XT, W_CODES8, false>(t, grouped, s);
}

// y[i] = T(sum over the parts of partial[part][i]) in part order, then the optional addend with the roundings
// of the cast and the Add
template <typename T>
__global__ void splitk_reduce_kernel(const float *__restrict__ partial, int parts, int64_t n, T *__restrict__ y,
                                     const T *__restrict__ addend)
{
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float v = partial[i];
  for (int p = 1; p < parts; ++p) v += partial[p * n + i];
  if (addend) v = round_through<T>(v) + to_f32<T>(addend[i]);
  y[i] = from_f32<T>(v);
}

// The same for four neighbouring elements per thread (n a multiple of 4, 16-byte aligned partial sums): the parts
// are requested four at a time before the first is added, in the same order of additions.
template <typename T>
__global__ void splitk_reduce_x4_kernel(const float *__restrict__ partial, int parts, int64_t n, T *__restrict__ y,
                                        const T *__restrict__ addend)
{
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
  if (i >= n) return;
  const floatx4_t *src = reinterpret_cast<const floatx4_t *>(partial + i);
  const int64_t stride = n >> 2;
  floatx4_t v = src[0];
  int p = 1;
  for (; p + 4 <= parts; p += 4) {
    const floatx4_t a = src[p * stride], b = src[(p + 1) * stride], c = src[(p + 2) * stride], d = src[(p + 3) * stride];
    v += a;
    v += b;
    v += c;
    v += d;
  }
  for (; p < parts; ++p) v += src[p * stride];
  struct alignas(4 * sizeof(T)) T4 {
    T e[4];
  };
  T4 out;
  if (addend) {
    const T4 add = *reinterpret_cast<const T4 *>(addend + i);
#pragma unroll
    for (int e = 0; e < 4; ++e) out.e[e] = from_f32<T>(round_through<T>(v[e]) + to_f32<T>(add.e[e]));
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) out.e[e] = from_f32<T>(v[e]);
  }
  *reinterpret_cast<T4 *>(y + i) = out;
}

// With no more tiles than compute units the launch lasts one tile's whole reduction (43-70 us at K = 4096) however
// few rows there are.  Then up to 8 workgroups share a tile's reduction, each at least 8 steps of it, and write
// fp32 partial tiles to the caller's workspace; a second launch adds them in a fixed order.
struct SplitPlan {
  int ksplit;
  int split_steps;
  size_t bytes;
};
SplitPlan plan_split(int64_t M, int64_t C, int64_t R, bool grouped)
{
  SplitPlan p{1, 0, 0};
  if (grouped || R % BR != 0) return p;
  const int64_t tiles = ((M + 127) / 128) * ((C + BC - 1) / BC);
  const int64_t steps = R / BR;
  if (tiles > 128 || steps < 16) return p;
  // one workgroup per compute unit: two resident 128-row workgroups run about as fast as one after the other, so
  // parts beyond 256 workgroups only add partial tiles (224 tiles in 2 parts measured 90 us against 75 us unsplit)
  int64_t target = 256, most = 8, least = 8;
  int64_t k = target / tiles;
  if (k > most) k = most;
  if (k > steps / least) k = steps / least;
  if (k < 2) return p;
  const int64_t per = (steps + k - 1) / k;
  k = (steps + per - 1) / per;                   // every part has at least one step
  if (k < 2) return p;
  p.ksplit = static_cast<int>(k);
  p.split_steps = static_cast<int>(per);
  p.bytes = static_cast<size_t>(k) * static_cast<size_t>(M) * static_cast<size_t>(C) * sizeof(float);
  return p;
}

std::atomic<unsigned long long *> g_stamps{nullptr};
std::atomic<long long> g_stamps_capacity{0};

int run(const GemmArgs &a, bool backward, hipStream_t s)
{
  if (a.compute_dtype == CAIFX_F32) return CAIFX_ERR_UNSUPPORTED;
  if (a.x_dtype != a.compute_dtype && a.x_dtype != CAIFX_F32) return CAIFX_ERR_UNSUPPORTED;
  const bool grouped = a.offsets != nullptr;
  const bool int4 = a.w.kind == CAIFX_W_INT4_GROUP;
  // float storage in the 16-bit compute type: the same tiles with the dequantisation compiled out
  const bool dense = (a.w.kind == CAIFX_W_BF16 && a.compute_dtype == CAIFX_BF16) ||
                     (a.w.kind == CAIFX_W_F16 && a.compute_dtype == CAIFX_F16);
  if (!dense && !int4 && a.w.kind != CAIFX_W_INT8) return CAIFX_ERR_UNSUPPORTED;
  const int64_t R = backward ? a.N : a.K;
  if (R % BR != 0 || a.K % 32 != 0 || a.K < 64 || a.N < 1) return CAIFX_ERR_UNSUPPORTED;
  if (a.M > (int64_t{1} << 30) || a.N > (int64_t{1} << 30) || a.K > (int64_t{1} << 30)) return CAIFX_ERR_UNSUPPORTED;
  if (!aligned_to(a.x, 16)) return CAIFX_ERR_UNSUPPORTED;

  TileArgs t{};
  t.M = a.M;
  t.N = a.N;
  t.K = a.K;
  t.a = a.x;
  t.d = a.y;
  t.d_dtype = a.y_dtype;
  t.addend = a.addend;
  {
    const int64_t cols = backward ? a.K : a.N;
    t.vec_store = cols % 8 == 0 && aligned_to(a.y, 16) && (!a.addend || aligned_to(a.addend, 16));
  }
  if (a.epilogue != EPI_NONE) {
    // only the staged 16-byte store carries these; the caller falls back to separate launches otherwise
    if (!grouped || !t.vec_store || a.y_dtype == CAIFX_F32 || a.addend || !aligned_to(a.e1, 16) || !aligned_to(a.y2, 16) ||
        (a.epilogue == EPI_SWIGLU_BWD && !aligned_to(a.e2, 16)))
      return CAIFX_ERR_UNSUPPORTED;
    t.epilogue = a.epilogue;
    t.e1 = a.e1;
    t.e2 = a.e2;
    t.d2 = a.y2;
  }
  t.wq = a.w.q;
  t.scales = a.w.scales;
  t.offsets = a.offsets;
  t.wq_ptrs = a.wq_ptrs;
  t.scales_ptrs = a.scales_ptrs;
  t.num_experts = a.num_experts;
  if (dense) {
    if (!grouped && !aligned_to(a.w.q, 16)) return CAIFX_ERR_UNSUPPORTED;
    t.scales = nullptr;
    t.scales_ptrs = nullptr;
  } else if (int4) {
    const int gs = a.w.group_size;
    if (gs < 32 || (gs & (gs - 1)) != 0) return CAIFX_ERR_UNSUPPORTED;
    t.group_shift = __builtin_ctz(static_cast<unsigned>(gs));
    if (!grouped && !aligned_to(a.w.q, 16)) return CAIFX_ERR_UNSUPPORTED;
  } else {
    if (!grouped && !aligned_to(a.w.q, 16)) return CAIFX_ERR_UNSUPPORTED;
    const bool has_scales = grouped ? a.scales_ptrs != nullptr : a.w.scales != nullptr;
    t.period = a.w.scale_period;
    if (!has_scales || t.period == 1) {
      t.scale_mode = SM_SCALAR;
    } else if (t.period % 4 == 0 && t.period < (int64_t{1} << 31) && (grouped || aligned_to(a.w.scales, 16))) {
      t.scale_mode = SM_VEC4;     // flat index of every fetched quad is a multiple of 4 (K % 32 == 0)
      // one step moves the flat index by 64 (forward: along k) or by 64 rows of K codes (backward)
      t.scale_step = static_cast<uint32_t>((backward ? (static_cast<int64_t>(BR) * t.K) % t.period : BR % t.period));
    } else {
      t.scale_mode = SM_ANY;
    }
  }
  t.ksplit = 1;
  if (grouped) {
    t.stamps = g_stamps.load(std::memory_order_relaxed);
    t.stamps_capacity = t.stamps ? g_stamps_capacity.load(std::memory_order_relaxed) : 0;
  }
  const int64_t cols = backward ? a.K : a.N;
  const SplitPlan plan = plan_split(a.M, cols, R, grouped);
  const bool split = plan.ksplit > 1 && a.epilogue == EPI_NONE && a.workspace && a.workspace_bytes >= plan.bytes &&
                     aligned_to(a.workspace, 16);
  if (split) {
    t.ksplit = plan.ksplit;
    t.split_steps = plan.split_steps;
    t.d = a.workspace;
    t.d_dtype = CAIFX_F32;
    t.addend = nullptr;
    t.vec_store = cols % 8 == 0;
  }
  int st;
  if (dense) {
    st = dense_launch(t, a.compute_dtype, a.x_dtype, backward, grouped, s);
  } else if (a.compute_dtype == CAIFX_BF16) {
    st = a.x_dtype == CAIFX_F32 ? pick_kind<bf16_t, float>(t, int4, backward, grouped, s) : pick_kind<bf16_t, bf16_t>(t, int4, backward, grouped, s);
  } else {
    st = a.x_dtype == CAIFX_F32 ? pick_kind<f16_t, float>(t, int4, backward, grouped, s) : pick_kind<f16_t, f16_t>(t, int4, backward, grouped, s);
  }
  if (!split || st != CAIFX_OK) return st;
  return splitk_reduce(static_cast<const float *>(a.workspace), plan.ksplit, a.M * cols, a.y, a.y_dtype, a.addend, s);
}

}  // namespace

int splitk_reduce(const float *partial, int parts, int64_t n, void *y, int y_dtype, const void *addend, hipStream_t s)
{
  const size_t quad = 4 * (y_dtype == CAIFX_F32 ? 4 : 2);
  if (n % 4 == 0 && aligned_to(partial, 16) && aligned_to(y, quad) && (!addend || aligned_to(addend, quad))) {
    const dim3 grid4(static_cast<unsigned>((n / 4 + 255) / 256));
    if (y_dtype == CAIFX_F32)
      hipLaunchKernelGGL(splitk_reduce_x4_kernel<float>, grid4, dim3(256), 0, s, partial, parts, n, static_cast<float *>(y),
                         static_cast<const float *>(addend));
    else if (y_dtype == CAIFX_BF16)
      hipLaunchKernelGGL(splitk_reduce_x4_kernel<bf16_t>, grid4, dim3(256), 0, s, partial, parts, n, static_cast<bf16_t *>(y),
                         static_cast<const bf16_t *>(addend));
    else
      hipLaunchKernelGGL(splitk_reduce_x4_kernel<f16_t>, grid4, dim3(256), 0, s, partial, parts, n, static_cast<f16_t *>(y),
                         static_cast<const f16_t *>(addend));
    return launch_status();
  }
  const dim3 grid(static_cast<unsigned>((n + 255) / 256));
  if (y_dtype == CAIFX_F32)
    hipLaunchKernelGGL(splitk_reduce_kernel<float>, grid, dim3(256), 0, s, partial, parts, n, static_cast<float *>(y),
                       static_cast<const float *>(addend));
  else if (y_dtype == CAIFX_BF16)
    hipLaunchKernelGGL(splitk_reduce_kernel<bf16_t>, grid, dim3(256), 0, s, partial, parts, n, static_cast<bf16_t *>(y),
                       static_cast<const bf16_t *>(addend));
  else
    hipLaunchKernelGGL(splitk_reduce_kernel<f16_t>, grid, dim3(256), 0, s, partial, parts, n, static_cast<f16_t *>(y),
                       static_cast<const f16_t *>(addend));
  return launch_status();
}

int mfma_tiled_forward(const GemmArgs &a, hipStream_t s) { return run(a, false, s); }
int mfma_backward(const GemmArgs &a, hipStream_t s) { return run(a, true, s); }
void mfma_grouped_stamp_target(unsigned long long **buf, long long *capacity)
{
  *buf = g_stamps.load(std::memory_order_relaxed);
  *capacity = *buf ? g_stamps_capacity.load(std::memory_order_relaxed) : 0;
}

void mfma_grouped_tile_stamps(void *buf, int64_t tiles)
{
  g_stamps_capacity.store(buf ? tiles : 0, std::memory_order_relaxed);
  g_stamps.store(static_cast<unsigned long long *>(buf), std::memory_order_relaxed);
}
size_t mfma_workspace_bytes(const GemmArgs &a, bool backward)
{
  if (a.compute_dtype == CAIFX_F32) return 0;
  return plan_split(a.M, backward ? a.K : a.N, backward ? a.N : a.K, a.offsets != nullptr).bytes;
}

}  // namespace caifx
