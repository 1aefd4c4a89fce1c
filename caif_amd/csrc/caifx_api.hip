// extern "C" entry points of the dequant-GEMM seam: argument validation and kernel choice.
#include "caifx_internal.hpp"


#include <atomic>

using namespace caifx;

// Scratch of caifx_qlinear_forward_static: part of the device image, so every GPU the library is loaded on has
// its own copy at its own address.  In host code `static_scratch` is only a handle for hipGetSymbolAddress, not a
// device address; the address is looked up once per device and only that address is ever handed to a launch.
static __device__ __align__(256) unsigned char static_scratch[CAIFX_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::atomic<void *> static_scratch_ptr[kMaxDevices];

// Address of the current device's copy (nullptr on failure).  Two threads racing on a device's first call both
// look the same address up and store the same value.
void *static_scratch_on_current_device()
{
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void *p = static_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p) return p;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(static_scratch)) != hipSuccess || !p) return nullptr;
  static_scratch_ptr[dev].store(p, std::memory_order_release);
  return p;
}

bool float_kind(int w_kind) { return w_kind == CAIFX_W_F32 || w_kind == CAIFX_W_F16 || w_kind == CAIFX_W_BF16; }
// float storage in the 16-bit compute type itself: the weight needs no conversion and runs on the 16-bit matrix cores
bool same_16bit(int w_kind, int compute_dtype)
{
  return (w_kind == CAIFX_W_BF16 && compute_dtype == CAIFX_BF16) || (w_kind == CAIFX_W_F16 && compute_dtype == CAIFX_F16);
}

int validate_weight(int64_t N, int64_t K, int w_kind, const void *scales, int64_t scale_period, int group_size)
{
  (void)N;
  (void)K;
  if (w_kind == CAIFX_W_INT4_GROUP) {
    if (group_size <= 0 || !scales) return CAIFX_ERR_INVALID_ARGUMENT;
    if (!aligned_to(scales, 2)) return CAIFX_ERR_MISALIGNED;
  } else if (w_kind == CAIFX_W_INT8) {
    if (scales) {
      if (scale_period <= 0) return CAIFX_ERR_INVALID_ARGUMENT;
      if (!aligned_to(scales, 4)) return CAIFX_ERR_MISALIGNED;
    }
  } else if (!float_kind(w_kind)) {
    return CAIFX_ERR_INVALID_ARGUMENT;
  }
  return CAIFX_OK;
}

int validate_common(int64_t M, int64_t N, int64_t K, const void *x, int x_dtype, int compute_dtype, void *y,
                    int y_dtype)
{
  if (M < 0 || N <= 0 || K <= 0) return CAIFX_ERR_INVALID_ARGUMENT;
  if (!valid_dtype(x_dtype) || !valid_dtype(compute_dtype) || !valid_dtype(y_dtype)) return CAIFX_ERR_INVALID_ARGUMENT;
  if (M > 0 && (!x || !y)) return CAIFX_ERR_INVALID_ARGUMENT;
  if (!aligned_to(x, dtype_size(x_dtype)) || !aligned_to(y, dtype_size(y_dtype))) return CAIFX_ERR_MISALIGNED;
  return CAIFX_OK;
}

GemmArgs make_args(int64_t M, int64_t N, int64_t K, const void *x, int x_dtype, int compute_dtype, const void *wq,
                   int w_kind, const void *scales, int64_t scale_period, int group_size, void *y, int y_dtype,
                   void *workspace, size_t workspace_bytes)
{
  GemmArgs a{};
  a.M = M;
  a.N = N;
  a.K = K;
  a.x = x;
  a.y = y;
  a.x_dtype = x_dtype;
  a.y_dtype = y_dtype;
  a.compute_dtype = compute_dtype;
  a.w.q = wq;
  a.w.scales = float_kind(w_kind) ? nullptr : scales;
  a.w.kind = w_kind;
  a.w.group_size = group_size;
  a.w.scale_period = (w_kind == CAIFX_W_INT8 && scales) ? scale_period : 1;
  a.workspace = workspace;
  a.workspace_bytes = workspace_bytes;
  return a;
}

}  // namespace

extern "C" {

const char *caifx_status_string(int status)
{
  switch (status) {
    case CAIFX_OK: return "ok";
    case CAIFX_ERR_INVALID_ARGUMENT: return "invalid argument";
    case CAIFX_ERR_UNSUPPORTED: return "unsupported combination";
    case CAIFX_ERR_WORKSPACE_TOO_SMALL: return "workspace too small";
    case CAIFX_ERR_LAUNCH_FAILED: return "kernel launch failed";
    case CAIFX_ERR_MISALIGNED: return "misaligned pointer";
    case CAIFX_ERR_SCRATCH_EXCEEDED: return "problem needs more scratch than the library's static buffer holds";
    default: return "unknown status";
  }
}

int caifx_version(void) { return 1000; }

size_t caifx_qlinear_workspace_bytes(int64_t M, int64_t N, int64_t K, int x_dtype, int compute_dtype, int w_kind,
                                     int backward)
{
  GemmArgs a{};
  a.M = M;
  a.N = N;
  a.K = K;
  a.x_dtype = x_dtype;
  a.compute_dtype = compute_dtype;
  a.w.kind = w_kind;
  const size_t f32_bytes = mfma_f32_workspace_bytes(a, backward != 0);
  // float storage runs on the fp32 matrix-core kernel unless it is stored in the 16-bit compute type itself
  if (float_kind(w_kind) && !same_16bit(w_kind, compute_dtype)) return f32_bytes;
  size_t bytes = mfma_workspace_bytes(a, backward != 0);
  if (float_kind(w_kind)) return f32_bytes > bytes ? f32_bytes : bytes;
  const size_t decode_bytes = backward ? dxrows_workspace_bytes(a) : mblock_workspace_bytes(a);
  if (decode_bytes > bytes) bytes = decode_bytes;
  return f32_bytes > bytes ? f32_bytes : bytes;
}

// `addend` (optional): the matrix-core GEMM adds it in its store; every other path runs as usual and is
// followed by the element-wise Add in place, which rounds in the same two places
static int finish_add(int st, const void *addend, void *y, int y_dtype, int64_t n, caifx_stream_t stream)
{
  if (st != CAIFX_OK || !addend) return st;
  return caifx_add(y, addend, y, n, y_dtype, stream);
}

static int forward_impl(int64_t M, int64_t N, int64_t K, const void *x, int x_dtype, int compute_dtype,
                        const void *wq, int w_kind, const void *scales, int64_t scale_period, int group_size,
                        void *y, int y_dtype, const void *addend, void *workspace, size_t workspace_bytes,
                        caifx_stream_t stream)
{
  int st = validate_common(M, N, K, x, x_dtype, compute_dtype, y, y_dtype);
  if (st != CAIFX_OK) return st;
  if (!wq) return CAIFX_ERR_INVALID_ARGUMENT;
  st = validate_weight(N, K, w_kind, scales, scale_period, group_size);
  if (st != CAIFX_OK) return st;
  if (addend && (addend == y || !aligned_to(addend, dtype_size(y_dtype)))) return CAIFX_ERR_INVALID_ARGUMENT;
  if (M == 0) return CAIFX_OK;
  GemmArgs a = make_args(M, N, K, x, x_dtype, compute_dtype, wq, w_kind, scales, scale_period, group_size, y,
                         y_dtype, workspace, workspace_bytes);
  hipStream_t s = as_stream(stream);
  if (float_kind(w_kind)) {
    // float storage: stored in the 16-bit compute type -> the tiled kernel on the 16-bit matrix cores; every other
    // cell the fp32 matrix-core kernel, else the shape-agnostic one
    if (same_16bit(w_kind, compute_dtype)) {
      a.addend = addend;
      st = mfma_forward(a, s);
      if (st != CAIFX_ERR_UNSUPPORTED) return st;       // added in the store
      a.addend = nullptr;
    }
    st = mfma_f32_forward(a, s);
    if (st == CAIFX_ERR_UNSUPPORTED) st = generic_forward(a, s);
    return finish_add(st, addend, y, y_dtype, M * N, stream);
  }
  // one or two rows: stream each weight row linearly and reduce per row; from three rows on the
  // matrix-core tiling (cost independent of M) is faster; both fall through when a shape does not fit
  st = CAIFX_ERR_UNSUPPORTED;
  // fp32 compute.  int8 storage with up to 32 rows: the row-block decode kernel on the integer matrix core (digit
  // planes of the fp32 activations); otherwise from two rows on the fp32 matrix-core kernel (40-43 us at
  // K = N = 4096 whatever M <= 32); the VALU decode kernel below takes 40-46 us for one row
  if (compute_dtype == CAIFX_F32) {
    if (M <= 32 && w_kind == CAIFX_W_INT8) {
      st = mblock_forward(a, s);
      if (st != CAIFX_ERR_UNSUPPORTED) return finish_add(st, addend, y, y_dtype, M * N, stream);
    }
    if (M > 1) {
      st = mfma_f32_forward(a, s);
      if (st != CAIFX_ERR_UNSUPPORTED) return finish_add(st, addend, y, y_dtype, M * N, stream);
    }
    st = CAIFX_ERR_UNSUPPORTED;
  }
  if (M <= 2) st = rowlin_forward(a, s);
  if (st == CAIFX_ERR_UNSUPPORTED && M <= 16) {
    st = mblock_forward(a, s);
    if (st == CAIFX_ERR_UNSUPPORTED && M <= 4) st = rowlin_forward(a, s);
    if (st == CAIFX_ERR_UNSUPPORTED) st = skinny_forward(a, s);
  }
  if (M > 16 && M <= 32) {
    // 17..32 rows: the decode kernel with two tiles of 16 rows reads the weight once; without the workspace its
    // reduction slices need, two launches of the 16-row form (2 x 14-17 us at K = 4096, N = 4096..14336) still
    // beat the tiled GEMM, whose shortest launch is one tile's reduction (43 us int4, 68 us int8 at K = 4096)
    st = mblock_forward(a, s);
    if (st == CAIFX_ERR_UNSUPPORTED) {
      GemmArgs c = a;
      c.M = 16;
      st = mblock_forward(c, s);
      if (st == CAIFX_OK) {
        c.M = M - 16;
        c.x = static_cast<const char *>(x) + 16 * K * static_cast<int64_t>(dtype_size(x_dtype));
        c.y = static_cast<char *>(y) + 16 * N * static_cast<int64_t>(dtype_size(y_dtype));
        st = mblock_forward(c, s);
      }
    }
  }
  if (st == CAIFX_ERR_UNSUPPORTED) {
    a.addend = addend;
    st = mfma_forward(a, s);
    if (st != CAIFX_ERR_UNSUPPORTED) return st;       // added in the store
    a.addend = nullptr;
    st = generic_forward(a, s);
  }
  return finish_add(st, addend, y, y_dtype, M * N, stream);
}

int caifx_qlinear_forward(int64_t M, int64_t N, int64_t K, const void *x, int x_dtype, int compute_dtype,
                          const void *wq, int w_kind, const void *scales, int64_t scale_period, int group_size,
                          void *y, int y_dtype, void *workspace, size_t workspace_bytes, caifx_stream_t stream)
{
  return forward_impl(M, N, K, x, x_dtype, compute_dtype, wq, w_kind, scales, scale_period, group_size, y, y_dtype,
                      nullptr, workspace, workspace_bytes, stream);
}

int caifx_static_scratch_prepare(void)
{
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return CAIFX_ERR_LAUNCH_FAILED;
  void *p = nullptr;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(static_scratch)) != hipSuccess || !p) return CAIFX_ERR_LAUNCH_FAILED;
  static_scratch_ptr[dev].store(p, std::memory_order_release);       // also replaces an address from before a device reset
  return CAIFX_OK;
}

int caifx_qlinear_forward_static(int64_t M, int64_t N, int64_t K, const void *x, int x_dtype, int compute_dtype,
                                 const void *wq, int w_kind, const void *scales, int64_t scale_period, int group_size,
                                 void *y, int y_dtype, caifx_stream_t stream)
{
  const size_t need = (M > 0 && N > 0 && K > 0 && valid_dtype(x_dtype) && valid_dtype(compute_dtype))
                          ? caifx_qlinear_workspace_bytes(M, N, K, x_dtype, compute_dtype, w_kind, 0)
                          : 0;
  if (need > CAIFX_STATIC_SCRATCH_BYTES) return CAIFX_ERR_SCRATCH_EXCEEDED;
  void *ws = nullptr;
  if (need > 0) {
    ws = static_scratch_on_current_device();
    if (!ws) return CAIFX_ERR_LAUNCH_FAILED;
  }
  return forward_impl(M, N, K, x, x_dtype, compute_dtype, wq, w_kind, scales, scale_period, group_size, y, y_dtype,
                      nullptr, ws, need, stream);
}

int caifx_qlinear_forward_add(int64_t M, int64_t N, int64_t K, const void *x, int x_dtype, int compute_dtype,
                              const void *wq, int w_kind, const void *scales, int64_t scale_period, int group_size,
                              void *y, int y_dtype, const void *addend, void *workspace, size_t workspace_bytes,
                              caifx_stream_t stream)
{
  if (M > 0 && !addend) return CAIFX_ERR_INVALID_ARGUMENT;
  return forward_impl(M, N, K, x, x_dtype, compute_dtype, wq, w_kind, scales, scale_period, group_size, y, y_dtype,
                      addend, workspace, workspace_bytes, stream);
}

static int backward_impl(int64_t M, int64_t N, int64_t K, const void *dy, int dy_dtype, int compute_dtype,
                         const void *wq, int w_kind, const void *scales, int64_t scale_period, int group_size,
                         void *dx, int dx_dtype, const void *addend, void *workspace, size_t workspace_bytes,
                         caifx_stream_t stream)
{
  int st = validate_common(M, N, K, dy, dy_dtype, compute_dtype, dx, dx_dtype);
  if (st != CAIFX_OK) return st;
  if (!wq) return CAIFX_ERR_INVALID_ARGUMENT;
  st = validate_weight(N, K, w_kind, scales, scale_period, group_size);
  if (st != CAIFX_OK) return st;
  if (addend && (addend == dx || !aligned_to(addend, dtype_size(dx_dtype)))) return CAIFX_ERR_INVALID_ARGUMENT;
  if (M == 0) return CAIFX_OK;
  GemmArgs a = make_args(M, N, K, dy, dy_dtype, compute_dtype, wq, w_kind, scales, scale_period, group_size,
                         dx, dx_dtype, workspace, workspace_bytes);
  hipStream_t s = as_stream(stream);
  // up to 16 rows of int8 codes (scale vectors through residue classes of the rows, one scale, none) or of int4
  // codes in groups of 128 or more: one pass over the weight, whatever the compute type (16-bit compute types on
  // the 16-bit matrix cores)
  const bool few_rows_first = M <= 16 && (w_kind == CAIFX_W_INT8 || w_kind == CAIFX_W_INT4_GROUP);
  if (few_rows_first) {
    st = dxrows_backward(a, s);
    if (st != CAIFX_ERR_UNSUPPORTED) return finish_add(st, addend, dx, dx_dtype, M * K, stream);
  }
  if (same_16bit(w_kind, compute_dtype)) {
    a.addend = addend;
    st = mfma_backward(a, s);
    if (st != CAIFX_ERR_UNSUPPORTED) return st;         // added in the store
    a.addend = nullptr;
  }
  if (compute_dtype == CAIFX_F32 || float_kind(w_kind)) {
    st = mfma_f32_backward(a, s);
    if (st != CAIFX_ERR_UNSUPPORTED) return finish_add(st, addend, dx, dx_dtype, M * K, stream);
    if (float_kind(w_kind)) return finish_add(generic_backward(a, s), addend, dx, dx_dtype, M * K, stream);
  }
  a.addend = addend;
  st = mfma_backward(a, s);
  if (st != CAIFX_ERR_UNSUPPORTED) return st;         // added in the store
  a.addend = nullptr;
  return finish_add(generic_backward(a, s), addend, dx, dx_dtype, M * K, stream);
}

int caifx_qlinear_backward_input(int64_t M, int64_t N, int64_t K, const void *dy, int dy_dtype, int compute_dtype,
                                 const void *wq, int w_kind, const void *scales, int64_t scale_period,
                                 int group_size, void *dx, int dx_dtype, void *workspace, size_t workspace_bytes,
                                 caifx_stream_t stream)
{
  return backward_impl(M, N, K, dy, dy_dtype, compute_dtype, wq, w_kind, scales, scale_period, group_size, dx,
                       dx_dtype, nullptr, workspace, workspace_bytes, stream);
}

int caifx_qlinear_backward_input_add(int64_t M, int64_t N, int64_t K, const void *dy, int dy_dtype, int compute_dtype,
                                     const void *wq, int w_kind, const void *scales, int64_t scale_period,
                                     int group_size, void *dx, int dx_dtype, const void *addend, void *workspace,
                                     size_t workspace_bytes, caifx_stream_t stream)
{
  if (M > 0 && !addend) return CAIFX_ERR_INVALID_ARGUMENT;
  return backward_impl(M, N, K, dy, dy_dtype, compute_dtype, wq, w_kind, scales, scale_period, group_size, dx,
                       dx_dtype, addend, workspace, workspace_bytes, stream);
}

size_t caifx_qlinear_grouped_workspace_bytes(int num_experts, int64_t total_rows, int64_t N, int64_t K, int x_dtype,
                                             int compute_dtype, int w_kind, int backward)
{
  GemmArgs a{};
  a.M = total_rows;
  a.N = N;
  a.K = K;
  a.x_dtype = x_dtype;
  a.compute_dtype = compute_dtype;
  a.w.kind = w_kind;
  a.num_experts = num_experts;
  a.offsets = reinterpret_cast<const int32_t *>(uintptr_t{1});   // marks the grouped form for the size query
  return mfma_workspace_bytes(a, backward != 0);
}

static int grouped(bool backward, int num_experts, const int32_t *offsets, int64_t total_rows, int64_t N, int64_t K,
                   const void *x, int x_dtype, int compute_dtype, const void *const *wq_ptrs, int w_kind,
                   const void *const *scales_ptrs, int64_t scale_period, int group_size, void *y, int y_dtype,
                   const void *addend, void *workspace, size_t workspace_bytes, caifx_stream_t stream)
{
  int st = validate_common(total_rows, N, K, x, x_dtype, compute_dtype, y, y_dtype);
  if (st != CAIFX_OK) return st;
  if (num_experts < 0) return CAIFX_ERR_INVALID_ARGUMENT;
  if (num_experts == 0 || total_rows == 0) return CAIFX_OK;
  if (!offsets || !wq_ptrs) return CAIFX_ERR_INVALID_ARGUMENT;
  if (w_kind == CAIFX_W_INT4_GROUP) {
    if (group_size <= 0 || !scales_ptrs) return CAIFX_ERR_INVALID_ARGUMENT;
  } else if (w_kind == CAIFX_W_INT8) {
    if (scales_ptrs && scale_period <= 0) return CAIFX_ERR_INVALID_ARGUMENT;
  } else if (float_kind(w_kind)) {
    scales_ptrs = nullptr;
  } else {
    return CAIFX_ERR_INVALID_ARGUMENT;
  }
  GemmArgs a = make_args(total_rows, N, K, x, x_dtype, compute_dtype, nullptr, w_kind, nullptr, scale_period,
                         group_size, y, y_dtype, workspace, workspace_bytes);
  a.w.scale_period = (w_kind == CAIFX_W_INT8 && scales_ptrs) ? scale_period : 1;
  a.offsets = offsets;
  a.wq_ptrs = wq_ptrs;
  a.scales_ptrs = scales_ptrs;
  a.num_experts = num_experts;
  if (addend && (addend == y || !aligned_to(addend, dtype_size(y_dtype)))) return CAIFX_ERR_INVALID_ARGUMENT;
  hipStream_t s = as_stream(stream);
  if (same_16bit(w_kind, compute_dtype)) {
    a.addend = addend;
    st = backward ? mfma_backward(a, s) : mfma_forward(a, s);
    if (st != CAIFX_ERR_UNSUPPORTED) return st;
    a.addend = nullptr;
  }
  if ((compute_dtype == CAIFX_F32 || float_kind(w_kind)) && !addend) {
    st = backward ? mfma_f32_backward(a, s) : mfma_f32_forward(a, s);
    if (st != CAIFX_ERR_UNSUPPORTED) return st;
  }
  if (float_kind(w_kind)) {
    if (addend) return CAIFX_ERR_UNSUPPORTED;
    return backward ? generic_backward(a, s) : generic_forward(a, s);
  }
  if (!backward && !addend) {
    // few rows per expert (MoE decode): memory bound on the touched experts' weights
    st = mblock_grouped_forward(a, s);
    if (st != CAIFX_ERR_UNSUPPORTED) return st;
  }
  a.addend = addend;
  st = backward ? mfma_backward(a, s) : mfma_forward(a, s);
  if (st != CAIFX_ERR_UNSUPPORTED) return st;
  // the shape-agnostic kernels have no fused add, and rows past offsets[E] must stay untouched, which a
  // plain element-wise pass over the buffer would not respect
  if (addend) return CAIFX_ERR_UNSUPPORTED;
  return backward ? generic_backward(a, s) : generic_forward(a, s);
}

int caifx_qlinear_grouped_tile_stamps(void *stamps, int64_t tiles)
{
  if (tiles < 0 || (stamps && !aligned_to(stamps, 8))) return CAIFX_ERR_INVALID_ARGUMENT;
  mfma_grouped_tile_stamps(stamps, tiles);
  return CAIFX_OK;
}

int caifx_qlinear_grouped_forward(int num_experts, const int32_t *offsets, int64_t total_rows, int64_t N, int64_t K,
                                  const void *x, int x_dtype, int compute_dtype, const void *const *wq_ptrs,
                                  int w_kind, const void *const *scales_ptrs, int64_t scale_period, int group_size,
                                  void *y, int y_dtype, void *workspace, size_t workspace_bytes,
                                  caifx_stream_t stream)
{
  return grouped(false, num_experts, offsets, total_rows, N, K, x, x_dtype, compute_dtype, wq_ptrs, w_kind,
                 scales_ptrs, scale_period, group_size, y, y_dtype, nullptr, workspace, workspace_bytes, stream);
}

int caifx_qlinear_grouped_backward_input(int num_experts, const int32_t *offsets, int64_t total_rows, int64_t N,
                                         int64_t K, const void *dy, int dy_dtype, int compute_dtype,
                                         const void *const *wq_ptrs, int w_kind, const void *const *scales_ptrs,
                                         int64_t scale_period, int group_size, void *dx, int dx_dtype,
                                         void *workspace, size_t workspace_bytes, caifx_stream_t stream)
{
  return grouped(true, num_experts, offsets, total_rows, N, K, dy, dy_dtype, compute_dtype, wq_ptrs, w_kind,
                 scales_ptrs, scale_period, group_size, dx, dx_dtype, nullptr, workspace, workspace_bytes, stream);
}

int caifx_qlinear_grouped_backward_input_add(int num_experts, const int32_t *offsets, int64_t total_rows, int64_t N,
                                             int64_t K, const void *dy, int dy_dtype, int compute_dtype,
                                             const void *const *wq_ptrs, int w_kind, const void *const *scales_ptrs,
                                             int64_t scale_period, int group_size, void *dx, int dx_dtype,
                                             const void *addend, void *workspace, size_t workspace_bytes,
                                             caifx_stream_t stream)
{
  if (total_rows > 0 && num_experts > 0 && !addend) return CAIFX_ERR_INVALID_ARGUMENT;
  return grouped(true, num_experts, offsets, total_rows, N, K, dy, dy_dtype, compute_dtype, wq_ptrs, w_kind,
                 scales_ptrs, scale_period, group_size, dx, dx_dtype, addend, workspace, workspace_bytes, stream);
}

// Shared checks of the two gated-expert launches: 16-bit results, every tensor of the result's shape present,
// aligned to its element type and distinct from the results.
static int swiglu_grouped(bool backward, int num_experts, const int32_t *offsets, int64_t total_rows, int64_t N, int64_t K,
                          const void *x, int x_dtype, int compute_dtype, const void *const *wq_ptrs, int w_kind,
                          const void *const *scales_ptrs, int64_t scale_period, int group_size, const void *gate,
                          const void *up, void *y, void *y2, int y_dtype, caifx_stream_t stream)
{
  int st = validate_common(total_rows, N, K, x, x_dtype, compute_dtype, y, y_dtype);
  if (st != CAIFX_OK) return st;
  if (num_experts < 0) return CAIFX_ERR_INVALID_ARGUMENT;
  if (num_experts == 0 || total_rows == 0) return CAIFX_OK;
  if (!offsets || !wq_ptrs || !gate || !y2 || (backward && !up)) return CAIFX_ERR_INVALID_ARGUMENT;
  if (y_dtype != CAIFX_F16 && y_dtype != CAIFX_BF16) return CAIFX_ERR_INVALID_ARGUMENT;
  if (w_kind == CAIFX_W_INT4_GROUP) {
    if (group_size <= 0 || !scales_ptrs) return CAIFX_ERR_INVALID_ARGUMENT;
  } else if (w_kind == CAIFX_W_INT8) {
    if (scales_ptrs && scale_period <= 0) return CAIFX_ERR_INVALID_ARGUMENT;
  } else if (float_kind(w_kind)) {
    return CAIFX_ERR_UNSUPPORTED;        // the gated stores exist in the quantised kernels only
  } else {
    return CAIFX_ERR_INVALID_ARGUMENT;
  }
  if (y == y2 || gate == y || gate == y2 || (backward && (up == y || up == y2)) || x == y || x == y2)
    return CAIFX_ERR_INVALID_ARGUMENT;
  if (!aligned_to(gate, 2) || !aligned_to(y2, 2) || (backward && !aligned_to(up, 2))) return CAIFX_ERR_MISALIGNED;
  GemmArgs a = make_args(total_rows, N, K, x, x_dtype, compute_dtype, nullptr, w_kind, nullptr, scale_period,
                         group_size, y, y_dtype, nullptr, 0);
  a.w.scale_period = (w_kind == CAIFX_W_INT8 && scales_ptrs) ? scale_period : 1;
  a.offsets = offsets;
  a.wq_ptrs = wq_ptrs;
  a.scales_ptrs = scales_ptrs;
  a.num_experts = num_experts;
  a.epilogue = backward ? 2 : 1;
  a.e1 = gate;
  a.e2 = up;
  a.y2 = y2;
  hipStream_t s = as_stream(stream);
  return backward ? mfma_backward(a, s) : mfma_forward(a, s);
}

int caifx_qlinear_grouped_forward_swiglu(int num_experts, const int32_t *offsets, int64_t total_rows, int64_t N, int64_t K,
                                         const void *x, int x_dtype, int compute_dtype, const void *const *wq_ptrs,
                                         int w_kind, const void *const *scales_ptrs, int64_t scale_period,
                                         int group_size, const void *gate, void *up, void *hidden, int out_dtype,
                                         caifx_stream_t stream)
{
  return swiglu_grouped(false, num_experts, offsets, total_rows, N, K, x, x_dtype, compute_dtype, wq_ptrs, w_kind,
                        scales_ptrs, scale_period, group_size, gate, nullptr, up, hidden, out_dtype, stream);
}

int caifx_qlinear_grouped_backward_input_swiglu(int num_experts, const int32_t *offsets, int64_t total_rows, int64_t N,
                                                int64_t K, const void *dy, int dy_dtype, int compute_dtype,
                                                const void *const *wq_ptrs, int w_kind,
                                                const void *const *scales_ptrs, int64_t scale_period, int group_size,
                                                const void *gate, const void *up, void *grad_gate, void *grad_up,
                                                int out_dtype, caifx_stream_t stream)
{
  return swiglu_grouped(true, num_experts, offsets, total_rows, N, K, dy, dy_dtype, compute_dtype, wq_ptrs, w_kind,
                        scales_ptrs, scale_period, group_size, gate, up, grad_gate, grad_up, out_dtype, stream);
}

}  // extern "C"
