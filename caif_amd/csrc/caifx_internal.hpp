// Argument blocks and entry points shared by the dequant-GEMM translation units.
#pragma once

#include "caifx_common.hpp"

namespace caifx {

// One frozen weight as stored: codes + scales + how a scale is found for flat index f.
struct QWeight {
  const void *q;          // int8[N*K] or packed int4[(N*K+1)/2]
  const void *scales;     // int8: fp32[scale_period] or null; int4: fp16[ceil(N*K/group_size)]
  int kind;               // caifx_weight_kind
  int group_size;         // int4 only
  int64_t scale_period;   // int8 only: scale index = f % scale_period
};

// One dequant-GEMM problem.  Forward: x [M,K], y [M,N].  Backward: x = dY [M,N], y = dX [M,K].
// Grouped: offsets != null, rows of expert e are [offsets[e], offsets[e+1]), weight pointers
// come from wq_ptrs/scales_ptrs, and M is an upper bound on rows.
struct GemmArgs {
  int64_t M, N, K;
  const void *x;
  void *y;
  int x_dtype, y_dtype, compute_dtype;
  QWeight w;
  const int32_t *offsets;
  const void *const *wq_ptrs;
  const void *const *scales_ptrs;
  int num_experts;
  void *workspace;
  size_t workspace_bytes;
  // optional: y = T(float(T(acc)) + float(addend)), addend [M, columns of y] of y_dtype (may alias y)
  const void *addend;
  // optional gated-expert epilogue of the matrix-core kernel (0 = none, 1 = forward, 2 = backward; see
  // EPI_* in caifx_gemm.hip): e1 = gate, e2 = up (backward only), y2 = second result, all [M, columns of y]
  int epilogue;
  const void *e1, *e2;
  void *y2;
};

int generic_forward(const GemmArgs &a, hipStream_t s);
int generic_backward(const GemmArgs &a, hipStream_t s);

// M <= 16 decode path (memory bound).  Returns CAIFX_ERR_UNSUPPORTED when the shape is outside
// its tiling assumptions so that the caller can fall back.
int skinny_forward(const GemmArgs &a, hipStream_t s);
// M <= 4 decode path that streams each weight row linearly (the fastest access pattern).
int rowlin_forward(const GemmArgs &a, hipStream_t s);
// M <= 16 decode path on the matrix cores: activation rows are the A operand, so the cost per
// weight byte does not grow with M.
int mblock_forward(const GemmArgs &a, hipStream_t s);
// The same over token-sorted expert segments (forward), for launches with at most 16 rows per expert on average:
// an expert's weight is streamed once per 16 rows of its segment.
int mblock_grouped_forward(const GemmArgs &a, hipStream_t s);
// Workspace of mblock_forward when the reduction is longer than one workgroup covers (K > 4096), else 0.
size_t mblock_workspace_bytes(const GemmArgs &a);

// Input gradient for M <= 16 rows of dY with int8 codes (scale vectors through residue classes of the rows, one
// scale, or none) or int4 codes in groups of 128 or more, on the fp32 matrix core.  Needs the workspace
// dxrows_workspace_bytes reports when that is not 0; CAIFX_ERR_UNSUPPORTED otherwise.
int dxrows_backward(const GemmArgs &a, hipStream_t s);
size_t dxrows_workspace_bytes(const GemmArgs &a);

// Large-M MFMA path (compute bound), forward and input gradient, plain and grouped.  mfma_forward picks between
// the forward kernels (mfma_regw_forward where it applies, else mfma_tiled_forward).
int mfma_forward(const GemmArgs &a, hipStream_t s);
int mfma_tiled_forward(const GemmArgs &a, hipStream_t s);
int mfma_backward(const GemmArgs &a, hipStream_t s);
size_t mfma_workspace_bytes(const GemmArgs &a, bool backward);
// Measurement only: grouped launches of the matrix-core GEMM issued after this call record, per tile of their own
// numbering (expert by expert, row tile by row tile, column tile last), four 64-bit words {expert, rows in the
// tile, start, end} with the times in ticks of the 100 MHz wall clock, into buf (device memory for `tiles` tiles);
// a null buf switches the recording off.  Process-wide.
void mfma_grouped_tile_stamps(void *buf, int64_t tiles);
// Forward for packed int4 weights and 16-bit activations of the compute type with enough 128 x 256 tiles to fill
// the chip: the weight goes from global memory straight into matrix-core operand registers.
// CAIFX_ERR_UNSUPPORTED for everything else.
int mfma_regw_forward(const GemmArgs &a, hipStream_t s);

// fp32 compute type on the matrix cores (v_mfma_f32_32x32x2_f32), forward and input gradient, any M, plain
// and grouped.  CAIFX_ERR_UNSUPPORTED for an addend, reductions that are not a multiple of 32,
// int4 groups below 16 or not a power of two, int8 scale vectors shorter than 32 or not a multiple of 4 long.
int mfma_f32_forward(const GemmArgs &a, hipStream_t s);
int mfma_f32_backward(const GemmArgs &a, hipStream_t s);
size_t mfma_f32_workspace_bytes(const GemmArgs &a, bool backward);

// y[i] = T(partial[0][i] + partial[1][i] + ...) in that order for i < n, T = y_dtype, then the optional addend
// with the roundings of a cast and an Add: the second launch of a reduction shared among workgroups.
int splitk_reduce(const float *partial, int parts, int64_t n, void *y, int y_dtype, const void *addend, hipStream_t s);

}  // namespace caifx
