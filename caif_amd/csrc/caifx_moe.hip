// MoE token routing around the grouped dequant-GEMMs: dispatch map, gather into the token-sorted
// expert buffer, weighted combine, and the backward passes of the two.  All of it is HBM-bound
// integer / row-copy work: one wave moves one row segment with 16-byte accesses; nothing is
// reshaped into a GEMM.
//
// The dispatch map is built in three small launches without touching the host:
//   1. every wave counts, per expert, the assignments of its 64-entry slice of the flat
//      [num_tokens*top_k] index array                         -> counts[wave][expert]
//   2. one thread per expert turns its column of counts into exclusive prefix sums over the waves
//      (arrival order) and clamps the total by the capacity; a single wave then scans the totals
//      into the offsets
//   3. every wave ranks its 64 entries among equal experts (stable, by lane order) and writes
//      base[wave][expert] + rank, or -1 past the clamped count.
// The result is the reference's: positions in token-major, k-minor arrival order.
#include "caifx_internal.hpp"

#include <atomic>

namespace caifx {
namespace {

constexpr int kRouteThreads = 256;

// number of lanes below `lane` in `mask`
__device__ __forceinline__ int rank_below(unsigned long long mask, int lane)
{
  return __builtin_popcountll(mask & ((1ull << lane) - 1ull));
}

// The lanes of the wave whose expert id equals this lane's (e < 0: no expert, an empty mask): one ballot per bit of
// the id, each lane keeping the side of the ballot its own bit is on, instead of one round per distinct id.
__device__ __forceinline__ unsigned long long lanes_with_same_expert(int e, int num_experts)
{
  const bool valid = e >= 0;
  unsigned long long same = __ballot(valid);
  const int bits = 32 - __builtin_clz(static_cast<unsigned>(num_experts > 1 ? num_experts - 1 : 1));
  for (int b = 0; b < bits; ++b) {
    const bool one = valid && ((e >> b) & 1);
    const unsigned long long with = __ballot(one);
    same &= one ? with : ~with;
  }
  return valid ? same : 0ull;
}

__global__ __launch_bounds__(kRouteThreads) void map_count_kernel(const int32_t *idx, int64_t total, int num_experts,
                                                                   int32_t *counts)
{
  const int lane = threadIdx.x & 63;
  const int64_t slice = (static_cast<int64_t>(blockIdx.x) * kRouteThreads + threadIdx.x) >> 6;
  const int64_t i = slice * 64 + lane;
  int e = -1;
  if (i < total) {
    e = idx[i];
    if (e < 0 || e >= num_experts) e = -1;
  }
  int32_t *row = counts + slice * num_experts;
  if (slice * 64 < total) {
    for (int x = lane; x < num_experts; x += 64) row[x] = 0;
  }
  __builtin_amdgcn_wave_barrier();
  // the first lane of every expert value writes how many lanes hold it
  const unsigned long long same = lanes_with_same_expert(e, num_experts);
  if (e >= 0 && rank_below(same, lane) == 0) row[e] = __builtin_popcountll(same);
}

// counts[w][e] -> exclusive prefix over w (in place), one wave per expert walking the slices 64 at a
// time; the total, clamped by the capacity, goes to clamped[e]
__global__ __launch_bounds__(64) void map_scan_kernel(int32_t *counts, int64_t slices, int num_experts, int capacity,
                                                       int32_t *clamped)
{
  const int e = blockIdx.x;
  const int lane = threadIdx.x;
  int32_t carry = 0;
  for (int64_t base = 0; base < slices; base += 64) {
    const int64_t w = base + lane;
    const int32_t c = w < slices ? counts[w * num_experts + e] : 0;
    int32_t v = c;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int32_t up = __shfl_up(v, o, 64);
      if (lane >= o) v += up;
    }
    if (w < slices) counts[w * num_experts + e] = carry + v - c;
    carry += __shfl(v, 63, 64);
  }
  if (capacity > 0 && carry > capacity) carry = capacity;
  if (lane == 0) clamped[e] = carry;
}

__global__ __launch_bounds__(64) void map_offsets_kernel(const int32_t *clamped, int num_experts, int32_t *offsets)
{
  const int lane = threadIdx.x;
  int32_t carry = 0;
  if (lane == 0) offsets[0] = 0;
  for (int base = 0; base < num_experts; base += 64) {
    const int e = base + lane;
    int32_t v = e < num_experts ? clamped[e] : 0;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int32_t up = __shfl_up(v, o, 64);
      if (lane >= o) v += up;
    }
    if (e < num_experts) offsets[e + 1] = carry + v;
    carry += __shfl(v, 63, 64);
  }
}

__global__ __launch_bounds__(kRouteThreads) void map_rank_kernel(const int32_t *idx, int64_t total, int num_experts,
                                                                  const int32_t *base, const int32_t *clamped,
                                                                  int32_t *map)
{
  const int lane = threadIdx.x & 63;
  const int64_t slice = (static_cast<int64_t>(blockIdx.x) * kRouteThreads + threadIdx.x) >> 6;
  const int64_t i = slice * 64 + lane;
  int e = -1;
  if (i < total) {
    e = idx[i];
    if (e < 0 || e >= num_experts) e = -1;
  }
  int pos = -1;
  const unsigned long long same = lanes_with_same_expert(e, num_experts);
  if (e >= 0) {
    pos = base[slice * num_experts + e] + rank_below(same, lane);
    if (pos >= clamped[e]) pos = -1;               // dropped by the capacity limit
  }
  if (i < total) map[i] = pos;
}

// The three steps above in one workgroup of 16 waves, for short index arrays (decode batches: up to 3072
// assignments, three 64-entry slices per wave) whose counts[slice][expert] table fits LDS: four launches back to back
// cost 10-12 us in a graph however little they do, this one 5.5 us at 16 x 6 assignments over 64 experts and 7.0 us at
// 340 x 6 (at 1024 x 6 it measured 12.8 us: no gain left).  A wave asks for all its slices' ids before it looks at
// the first (one memory round trip, not one per slice) and keeps them for the ranking.  Row pitch of the table odd,
// so that a wave walking one expert's column touches 64 different banks.
constexpr int kMapOneThreads = 1024;
constexpr int kMapOneWaves = kMapOneThreads / 64;
constexpr int kMapOneSlices = 3;                                  // slices per wave
constexpr size_t kMapOneLdsMax = 144 * 1024;
__global__ __launch_bounds__(kMapOneThreads) void map_one_kernel(const int32_t *idx, int64_t total, int num_experts, int capacity,
                                                                  int32_t *map, int32_t *offsets)
{
  extern __shared__ int32_t map_lds[];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int slices = static_cast<int>((total + 63) >> 6);
  const int pitch = num_experts | 1;
  int32_t *counts = map_lds;                                      // [slices][pitch]
  int32_t *clamped = map_lds + static_cast<size_t>(slices) * pitch;       // [num_experts]
  int ev[kMapOneSlices];                                          // slice wave + 16 u: this lane's expert id, -1 for none
#pragma unroll
  for (int u = 0; u < kMapOneSlices; ++u) {
    const int64_t i = static_cast<int64_t>(wave + kMapOneWaves * u) * 64 + lane;
    ev[u] = -1;
    if (i < total) ev[u] = idx[i];
    if (ev[u] >= num_experts) ev[u] = -1;
  }
  for (int i = threadIdx.x; i < slices * pitch; i += kMapOneThreads) counts[i] = 0;
  __syncthreads();
#pragma unroll
  for (int u = 0; u < kMapOneSlices; ++u) {
    const int slice = wave + kMapOneWaves * u;
    if (slice >= slices) break;                                   // the same for every lane of the wave
    const unsigned long long same = lanes_with_same_expert(ev[u], num_experts);
    if (ev[u] >= 0 && rank_below(same, lane) == 0) counts[slice * pitch + ev[u]] = __builtin_popcountll(same);
  }
  __syncthreads();
  // one wave per expert: exclusive prefix over the slices (arrival order), the total clamped by the capacity
  for (int e = wave; e < num_experts; e += kMapOneWaves) {
    int32_t carry = 0;
    for (int base = 0; base < slices; base += 64) {
      const int w = base + lane;
      const int32_t c = w < slices ? counts[w * pitch + e] : 0;
      int32_t v = c;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int32_t up = __shfl_up(v, o, 64);
        if (lane >= o) v += up;
      }
      if (w < slices) counts[w * pitch + e] = carry + v - c;
      carry += __shfl(v, 63, 64);
    }
    if (capacity > 0 && carry > capacity) carry = capacity;
    if (lane == 0) clamped[e] = carry;
  }
  __syncthreads();
  if (wave == 0) {
    int32_t carry = 0;
    if (lane == 0) offsets[0] = 0;
    for (int base = 0; base < num_experts; base += 64) {
      const int e = base + lane;
      int32_t v = e < num_experts ? clamped[e] : 0;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int32_t up = __shfl_up(v, o, 64);
        if (lane >= o) v += up;
      }
      if (e < num_experts) offsets[e + 1] = carry + v;
      carry += __shfl(v, 63, 64);
    }
  }
#pragma unroll
  for (int u = 0; u < kMapOneSlices; ++u) {
    const int slice = wave + kMapOneWaves * u;
    if (slice >= slices) break;
    const int64_t i = static_cast<int64_t>(slice) * 64 + lane;
    const unsigned long long same = lanes_with_same_expert(ev[u], num_experts);
    int pos = -1;
    if (ev[u] >= 0) {
      pos = counts[slice * pitch + ev[u]] + rank_below(same, lane);
      if (pos >= clamped[ev[u]]) pos = -1;           // dropped by the capacity limit
    }
    if (i < total) map[i] = pos;
  }
}

// destination / source row of assignment a = t*top_k + k, or -1
__device__ __forceinline__ int64_t routed_row(const int32_t *idx, const int32_t *map, const int32_t *offsets, int64_t a,
                                              int num_experts)
{
  const int e = idx[a];
  const int p = map[a];
  if (e < 0 || e >= num_experts || p < 0) return -1;
  return static_cast<int64_t>(offsets[e]) + p;
}

template <typename T> struct Vec16 {
  static constexpr int kN = 16 / sizeof(T);
  typedef T type __attribute__((ext_vector_type(16 / sizeof(T))));
};

// one wave per assignment: copy a row, 16 bytes per lane and step
template <typename T>
__global__ __launch_bounds__(kRouteThreads) void dispatch_kernel(const T *in, const int32_t *idx, const int32_t *map,
                                                                  const int32_t *offsets, T *buf, int64_t assignments,
                                                                  int64_t dim, int top_k, int num_experts, bool vec)
{
  const int lane = threadIdx.x & 63;
  const int64_t a = (static_cast<int64_t>(blockIdx.x) * kRouteThreads + threadIdx.x) >> 6;
  if (a >= assignments) return;
  const int64_t row = routed_row(idx, map, offsets, a, num_experts);
  if (row < 0) return;
  const T *src = in + (a / top_k) * dim;
  T *dst = buf + row * dim;
  if (vec) {
    typedef typename Vec16<T>::type v_t;
    constexpr int n = Vec16<T>::kN;
    for (int64_t d = lane * n; d < dim; d += 64 * n) *reinterpret_cast<v_t *>(dst + d) = *reinterpret_cast<const v_t *>(src + d);
  } else {
    for (int64_t d = lane; d < dim; d += 64) dst[d] = src[d];
  }
}

// grad_expert_buffer[row(t,k)] = T(w[t,k] * grad_output[t]); one wave per assignment
template <typename T, bool kVec>
__global__ __launch_bounds__(kRouteThreads) void combine_bwd_kernel(const T *gout, const int32_t *idx, const T *w,
                                                                     const int32_t *map, const int32_t *offsets, T *gbuf,
                                                                     int64_t assignments, int64_t dim, int top_k,
                                                                     int num_experts)
{
  const int lane = threadIdx.x & 63;
  const int64_t a = (static_cast<int64_t>(blockIdx.x) * kRouteThreads + threadIdx.x) >> 6;
  if (a >= assignments) return;
  const int64_t row = routed_row(idx, map, offsets, a, num_experts);
  if (row < 0) return;
  const float wt = to_f32<T>(w[a]);
  const T *src = gout + (a / top_k) * dim;
  T *dst = gbuf + row * dim;
  if constexpr (kVec) {
    typedef typename Vec16<T>::type v_t;
    constexpr int n = Vec16<T>::kN;
    for (int64_t d = lane * n; d < dim; d += 64 * n) {
      const v_t g = *reinterpret_cast<const v_t *>(src + d);
      v_t o;
#pragma unroll
      for (int i = 0; i < n; ++i) o[i] = from_f32<T>(wt * to_f32<T>(g[i]));
      *reinterpret_cast<v_t *>(dst + d) = o;
    }
  } else {
    for (int64_t d = lane; d < dim; d += 64) dst[d] = from_f32<T>(wt * to_f32<T>(src[d]));
  }
}

// one wave per token: out[t] = T(sum_k w[t,k] * buf[row(t,k)])  (kWeighted) or T(sum_k buf[row(t,k)]);
// per element the additions run over k in order.  The rows and weights of a token are fetched once per
// batch of 8 assignments by lanes 0..7 and broadcast.
template <typename T, bool kWeighted, bool kVec>
__global__ __launch_bounds__(kRouteThreads) void gather_sum_kernel(const T *buf, const int32_t *idx, const T *w,
                                                                    const int32_t *map, const int32_t *offsets, T *out,
                                                                    int64_t num_tokens, int64_t dim, int top_k,
                                                                    int num_experts)
{
  constexpr int n = kVec ? Vec16<T>::kN : 1;
  typedef typename Vec16<T>::type v_t;
  const int lane = threadIdx.x & 63;
  const int64_t t = (static_cast<int64_t>(blockIdx.x) * kRouteThreads + threadIdx.x) >> 6;
  if (t >= num_tokens) return;
  for (int64_t d0 = 0; d0 < dim; d0 += 64 * n) {          // the whole wave walks the row together
    const int64_t d = d0 + static_cast<int64_t>(lane) * n;
    float sum[n];
#pragma unroll
    for (int i = 0; i < n; ++i) sum[i] = 0.0f;
    for (int k0 = 0; k0 < top_k; k0 += 8) {
      int64_t my_row = -1;
      float my_w = 0.0f;
      if (lane < 8 && k0 + lane < top_k) {
        const int64_t a = t * top_k + k0 + lane;
        my_row = routed_row(idx, map, offsets, a, num_experts);
        if constexpr (kWeighted) my_w = to_f32<T>(w[a]);
      }
      const int kn = top_k - k0 < 8 ? top_k - k0 : 8;
      for (int k = 0; k < kn; ++k) {
        const int64_t row = __shfl(my_row, k, 64);
        const float wt = __shfl(my_w, k, 64);
        if (row < 0 || d >= dim) continue;
        if constexpr (kVec) {
          const v_t v = *reinterpret_cast<const v_t *>(buf + row * dim + d);
#pragma unroll
          for (int i = 0; i < n; ++i) {
            if constexpr (kWeighted) sum[i] = __builtin_fmaf(wt, to_f32<T>(v[i]), sum[i]);
            else sum[i] += to_f32<T>(v[i]);
          }
        } else {
          const float v = to_f32<T>(buf[row * dim + d]);
          if constexpr (kWeighted) sum[0] = __builtin_fmaf(wt, v, sum[0]);
          else sum[0] += v;
        }
      }
    }
    if (d < dim) {
      if constexpr (kVec) {
        v_t o;
#pragma unroll
        for (int i = 0; i < n; ++i) o[i] = from_f32<T>(sum[i]);
        *reinterpret_cast<v_t *>(out + t * dim + d) = o;
      } else {
        out[t * dim + d] = from_f32<T>(sum[0]);
      }
    }
  }
}

// one wave per assignment: grad_weights[t,k] = T(sum_d grad_output[t,d] * buffer[row(t,k),d]), fp32;
// 0 for assignments that moved no data.  Lane l adds elements l, l+64, ... in order, then the 64 partial
// sums are added pairwise (xor 32, 16, ..., 1): a fixed order, so results repeat bit for bit.
template <typename T>
__global__ __launch_bounds__(kRouteThreads) void combine_bwd_weights_kernel(const T *gout, const T *buf, const int32_t *idx,
                                                                             const int32_t *map, const int32_t *offsets,
                                                                             T *gw, int64_t assignments, int64_t dim,
                                                                             int top_k, int num_experts)
{
  const int lane = threadIdx.x & 63;
  const int64_t a = (static_cast<int64_t>(blockIdx.x) * kRouteThreads + threadIdx.x) >> 6;
  if (a >= assignments) return;
  const int64_t row = routed_row(idx, map, offsets, a, num_experts);
  float sum = 0.0f;
  if (row >= 0) {
    const T *g = gout + (a / top_k) * dim;
    const T *b = buf + row * dim;
    for (int64_t d = lane; d < dim; d += 64) sum = __builtin_fmaf(to_f32<T>(g[d]), to_f32<T>(b[d]), sum);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
  }
  if (lane == 0) gw[a] = from_f32<T>(sum);
}

int check_route(const void *a, const void *b, const int32_t *idx, const int32_t *map, const int32_t *offsets,
                int64_t num_tokens, int64_t dim, int top_k, int num_experts, int dtype)
{
  if (num_tokens < 0 || dim < 0 || top_k < 0 || num_experts <= 0 || !valid_dtype(dtype)) return CAIFX_ERR_INVALID_ARGUMENT;
  if (num_tokens == 0 || dim == 0 || top_k == 0) return CAIFX_OK;
  if (!a || !b || !idx || !map || !offsets) return CAIFX_ERR_INVALID_ARGUMENT;
  if (!aligned_to(a, dtype_size(dtype)) || !aligned_to(b, dtype_size(dtype)) || !aligned_to(idx, 4) || !aligned_to(map, 4) ||
      !aligned_to(offsets, 4))
    return CAIFX_ERR_MISALIGNED;
  return -1;      // go on
}

unsigned wave_blocks(int64_t waves) { return static_cast<unsigned>((waves * 64 + kRouteThreads - 1) / kRouteThreads); }

}  // namespace
}  // namespace caifx

using namespace caifx;

extern "C" {

size_t caifx_moe_dispatch_map_workspace_bytes(int64_t num_tokens, int top_k, int num_experts)
{
  if (num_tokens <= 0 || top_k <= 0 || num_experts <= 0) return 0;
  const int64_t slices = (num_tokens * top_k + 63) / 64;
  return static_cast<size_t>(slices + 1) * static_cast<size_t>(num_experts) * sizeof(int32_t);
}

int caifx_moe_build_dispatch_map(const int32_t *expert_indices, int64_t num_tokens, int top_k, int num_experts,
                                 int capacity_per_expert, int32_t *dispatch_map, int32_t *expert_offsets,
                                 void *workspace, size_t workspace_bytes, caifx_stream_t stream)
{
  if (num_tokens < 0 || top_k < 0 || num_experts <= 0 || capacity_per_expert < 0 || !expert_offsets) return CAIFX_ERR_INVALID_ARGUMENT;
  const int64_t total = num_tokens * top_k;
  if (total > (int64_t{1} << 31) - 64) return CAIFX_ERR_UNSUPPORTED;
  hipStream_t s = as_stream(stream);
  if (total > 0 && (!expert_indices || !dispatch_map)) return CAIFX_ERR_INVALID_ARGUMENT;
  if (!aligned_to(expert_indices, 4) || !aligned_to(dispatch_map, 4) || !aligned_to(expert_offsets, 4) || !aligned_to(workspace, 4))
    return CAIFX_ERR_MISALIGNED;
  const size_t need = total > 0 ? caifx_moe_dispatch_map_workspace_bytes(num_tokens, top_k, num_experts)
                                : static_cast<size_t>(num_experts) * sizeof(int32_t);
  if (!workspace || workspace_bytes < need) return CAIFX_ERR_WORKSPACE_TOO_SMALL;
  {
    // short index arrays: everything in one workgroup's LDS (the workspace is checked all the same and not used)
    const size_t one = ((static_cast<size_t>((total + 63) / 64)) * static_cast<size_t>(num_experts | 1) + static_cast<size_t>(num_experts)) *
                       sizeof(int32_t);
    if (one <= kMapOneLdsMax && (total + 63) / 64 <= kMapOneWaves * kMapOneSlices) {
      static std::atomic<bool> raised{false};
      if (!raised.load(std::memory_order_relaxed)) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(map_one_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(kMapOneLdsMax)) != hipSuccess)
          return CAIFX_ERR_LAUNCH_FAILED;
        raised.store(true, std::memory_order_relaxed);
      }
      hipLaunchKernelGGL(map_one_kernel, dim3(1), dim3(kMapOneThreads), one, s, expert_indices, total, num_experts,
                         capacity_per_expert, dispatch_map, expert_offsets);
      return launch_status();
    }
  }
  const int64_t slices = (total + 63) / 64;
  int32_t *counts = static_cast<int32_t *>(workspace);            // [slices][num_experts]
  int32_t *clamped = counts + slices * num_experts;               // [num_experts]
  if (total > 0)
    hipLaunchKernelGGL(map_count_kernel, dim3(wave_blocks(slices)), dim3(kRouteThreads), 0, s, expert_indices, total,
                       num_experts, counts);
  hipLaunchKernelGGL(map_scan_kernel, dim3(num_experts), dim3(64), 0, s, counts, slices, num_experts, capacity_per_expert,
                     clamped);
  hipLaunchKernelGGL(map_offsets_kernel, dim3(1), dim3(64), 0, s, clamped, num_experts, expert_offsets);
  if (total > 0)
    hipLaunchKernelGGL(map_rank_kernel, dim3(wave_blocks(slices)), dim3(kRouteThreads), 0, s, expert_indices, total,
                       num_experts, counts, clamped, dispatch_map);
  return launch_status();
}

int caifx_moe_dispatch(const void *input, const int32_t *expert_indices, const int32_t *dispatch_map,
                       const int32_t *expert_offsets, void *expert_buffer, int64_t num_tokens, int64_t dim, int top_k,
                       int num_experts, int dtype, caifx_stream_t stream)
{
  const int st = check_route(input, expert_buffer, expert_indices, dispatch_map, expert_offsets, num_tokens, dim, top_k,
                             num_experts, dtype);
  if (st >= 0) return st;
  const int64_t assignments = num_tokens * top_k;
  const size_t es = dtype_size(dtype);
  const bool vec = (dim * es) % 16 == 0 && aligned_to(input, 16) && aligned_to(expert_buffer, 16);
  const dim3 grid(wave_blocks(assignments)), block(kRouteThreads);
  hipStream_t s = as_stream(stream);
  if (dtype == CAIFX_F32)
    hipLaunchKernelGGL(dispatch_kernel<float>, grid, block, 0, s, static_cast<const float *>(input), expert_indices,
                       dispatch_map, expert_offsets, static_cast<float *>(expert_buffer), assignments, dim, top_k,
                       num_experts, vec);
  else      // fp16 and bf16 rows are copied as 16-bit patterns
    hipLaunchKernelGGL(dispatch_kernel<uint16_t>, grid, block, 0, s, static_cast<const uint16_t *>(input), expert_indices,
                       dispatch_map, expert_offsets, static_cast<uint16_t *>(expert_buffer), assignments, dim, top_k,
                       num_experts, vec);
  return launch_status();
}

int caifx_moe_combine(const void *expert_buffer, const int32_t *expert_indices, const void *expert_weights,
                      const int32_t *dispatch_map, const int32_t *expert_offsets, void *output, int64_t num_tokens,
                      int64_t dim, int top_k, int num_experts, int dtype, caifx_stream_t stream)
{
  const int st = check_route(expert_buffer, output, expert_indices, dispatch_map, expert_offsets, num_tokens, dim, top_k,
                             num_experts, dtype);
  if (st >= 0) return st;
  if (!expert_weights) return CAIFX_ERR_INVALID_ARGUMENT;
  const dim3 grid(wave_blocks(num_tokens)), block(kRouteThreads);
  hipStream_t s = as_stream(stream);
  const bool vec = (dim * dtype_size(dtype)) % 16 == 0 && aligned_to(expert_buffer, 16) && aligned_to(output, 16);
#define CAIFX_GO(T)                                                                                                    \
  if (vec)                                                                                                             \
    hipLaunchKernelGGL((gather_sum_kernel<T, true, true>), grid, block, 0, s, static_cast<const T *>(expert_buffer),   \
                       expert_indices, static_cast<const T *>(expert_weights), dispatch_map, expert_offsets,          \
                       static_cast<T *>(output), num_tokens, dim, top_k, num_experts);                                \
  else                                                                                                                 \
    hipLaunchKernelGGL((gather_sum_kernel<T, true, false>), grid, block, 0, s, static_cast<const T *>(expert_buffer),  \
                       expert_indices, static_cast<const T *>(expert_weights), dispatch_map, expert_offsets,          \
                       static_cast<T *>(output), num_tokens, dim, top_k, num_experts)
  if (dtype == CAIFX_F32) {
    CAIFX_GO(float);
  } else if (dtype == CAIFX_F16) {
    CAIFX_GO(f16_t);
  } else {
    CAIFX_GO(bf16_t);
  }
#undef CAIFX_GO
  return launch_status();
}

int caifx_moe_combine_backward_grad_expert(const void *grad_output, const int32_t *expert_indices,
                                           const void *expert_weights, const int32_t *dispatch_map,
                                           const int32_t *expert_offsets, void *grad_expert_buffer, int64_t num_tokens,
                                           int64_t dim, int top_k, int num_experts, int dtype, caifx_stream_t stream)
{
  const int st = check_route(grad_output, grad_expert_buffer, expert_indices, dispatch_map, expert_offsets, num_tokens, dim,
                             top_k, num_experts, dtype);
  if (st >= 0) return st;
  if (!expert_weights) return CAIFX_ERR_INVALID_ARGUMENT;
  const int64_t assignments = num_tokens * top_k;
  const dim3 grid(wave_blocks(assignments)), block(kRouteThreads);
  hipStream_t s = as_stream(stream);
  const bool vec = (dim * dtype_size(dtype)) % 16 == 0 && aligned_to(grad_output, 16) && aligned_to(grad_expert_buffer, 16);
#define CAIFX_GO(T)                                                                                                    \
  if (vec)                                                                                                             \
    hipLaunchKernelGGL((combine_bwd_kernel<T, true>), grid, block, 0, s, static_cast<const T *>(grad_output),          \
                       expert_indices, static_cast<const T *>(expert_weights), dispatch_map, expert_offsets,          \
                       static_cast<T *>(grad_expert_buffer), assignments, dim, top_k, num_experts);                   \
  else                                                                                                                 \
    hipLaunchKernelGGL((combine_bwd_kernel<T, false>), grid, block, 0, s, static_cast<const T *>(grad_output),         \
                       expert_indices, static_cast<const T *>(expert_weights), dispatch_map, expert_offsets,          \
                       static_cast<T *>(grad_expert_buffer), assignments, dim, top_k, num_experts)
  if (dtype == CAIFX_F32) {
    CAIFX_GO(float);
  } else if (dtype == CAIFX_F16) {
    CAIFX_GO(f16_t);
  } else {
    CAIFX_GO(bf16_t);
  }
#undef CAIFX_GO
  return launch_status();
}

int caifx_moe_combine_backward_grad_weights(const void *grad_output, const void *expert_buffer,
                                            const int32_t *expert_indices, const int32_t *dispatch_map,
                                            const int32_t *expert_offsets, void *grad_weights, int64_t num_tokens,
                                            int64_t dim, int top_k, int num_experts, int dtype, caifx_stream_t stream)
{
  const int st = check_route(grad_output, expert_buffer, expert_indices, dispatch_map, expert_offsets, num_tokens, dim, top_k,
                             num_experts, dtype);
  if (st >= 0) return st;
  if (!grad_weights) return CAIFX_ERR_INVALID_ARGUMENT;
  const int64_t assignments = num_tokens * top_k;
  const dim3 grid(wave_blocks(assignments)), block(kRouteThreads);
  hipStream_t s = as_stream(stream);
#define CAIFX_GO(T)                                                                                                    \
  hipLaunchKernelGGL(combine_bwd_weights_kernel<T>, grid, block, 0, s, static_cast<const T *>(grad_output),            \
                     static_cast<const T *>(expert_buffer), expert_indices, dispatch_map, expert_offsets,             \
                     static_cast<T *>(grad_weights), assignments, dim, top_k, num_experts)
  if (dtype == CAIFX_F32) {
    CAIFX_GO(float);
  } else if (dtype == CAIFX_F16) {
    CAIFX_GO(f16_t);
  } else {
    CAIFX_GO(bf16_t);
  }
#undef CAIFX_GO
  return launch_status();
}

int caifx_moe_dispatch_backward(const void *grad_expert_buffer, const int32_t *expert_indices, const int32_t *dispatch_map,
                                const int32_t *expert_offsets, void *grad_input, int64_t num_tokens, int64_t dim, int top_k,
                                int num_experts, int dtype, caifx_stream_t stream)
{
  const int st = check_route(grad_expert_buffer, grad_input, expert_indices, dispatch_map, expert_offsets, num_tokens, dim,
                             top_k, num_experts, dtype);
  if (st >= 0) return st;
  const dim3 grid(wave_blocks(num_tokens)), block(kRouteThreads);
  hipStream_t s = as_stream(stream);
  const bool vec = (dim * dtype_size(dtype)) % 16 == 0 && aligned_to(grad_expert_buffer, 16) && aligned_to(grad_input, 16);
#define CAIFX_GO(T)                                                                                                    \
  if (vec)                                                                                                             \
    hipLaunchKernelGGL((gather_sum_kernel<T, false, true>), grid, block, 0, s,                                         \
                       static_cast<const T *>(grad_expert_buffer), expert_indices, static_cast<const T *>(nullptr),   \
                       dispatch_map, expert_offsets, static_cast<T *>(grad_input), num_tokens, dim, top_k, num_experts); \
  else                                                                                                                 \
    hipLaunchKernelGGL((gather_sum_kernel<T, false, false>), grid, block, 0, s,                                        \
                       static_cast<const T *>(grad_expert_buffer), expert_indices, static_cast<const T *>(nullptr),   \
                       dispatch_map, expert_offsets, static_cast<T *>(grad_input), num_tokens, dim, top_k, num_experts)
  if (dtype == CAIFX_F32) {
    CAIFX_GO(float);
  } else if (dtype == CAIFX_F16) {
    CAIFX_GO(f16_t);
  } else {
    CAIFX_GO(bf16_t);
  }
#undef CAIFX_GO
  return launch_status();
}

}  // extern "C"
