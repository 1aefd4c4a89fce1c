/*
 * caifx.h -- C ABI of the MI355X (gfx950) frozen quantized-linear kernels.
 *
 * This is the seam at which CAIF's C++ host code (CAIF_Ops quantise entry
 * points, CAIF_DeviceFrozenLinear, CAIF_DeviceMoEFrozenExpert) meets device
 * code.  Every entry point below replaces either one launcher declared in the
 * reference's include/caif/caif_cuda_kernels_quant.cuh or one vendor GEMM call
 * inside the frozen layers; the reference interface it replaces is cited as
 * file:line relative to the reference checkout (cppaif/caif).
 *
 * Conventions
 *  - Plain C: raw device pointers, element counts (not bytes), enums as int.
 *  - `stream` is a hipStream_t passed as void*; NULL is the default stream.
 *    All work is enqueued on it; no entry point synchronises the host, and
 *    none allocates or frees memory: scratch comes in through `workspace`.
 *  - Return value: CAIFX_OK (0) or a caifx_status error code.  The reference
 *    throws CAIF_Exception where these return non-zero; the C++ host layer
 *    maps a non-zero status back to THROW_CAIFE.
 *  - Like the reference launchers, an empty problem (n <= 0, rows <= 0, ...)
 *    is a successful no-op.
 *  - Weight layout is the reference's, untouched: W is logically [N,K]
 *    row-major (N = OutputDim, K = InputDim), flat index f = n*K + k
 *    (src/caif_device_frozen_linear.cpp:345).  int8 holds one code per byte;
 *    int4 holds two codes per byte, even f in the low nibble, two's complement
 *    (src/caif_cuda_kernels_quant.cu:205-237).
 */
#ifndef CAIFX_H
#define CAIFX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *caifx_stream_t;            /* hipStream_t */

#if defined(__GNUC__)
#define CAIFX_API __attribute__((visibility("default")))
#else
#define CAIFX_API
#endif

enum caifx_status {
  CAIFX_OK = 0,
  CAIFX_ERR_INVALID_ARGUMENT = 1,        /* null pointer, negative size, bad enum, group_size == 0 ... */
  CAIFX_ERR_UNSUPPORTED = 2,             /* a combination this build has no kernel for */
  CAIFX_ERR_WORKSPACE_TOO_SMALL = 3,
  CAIFX_ERR_LAUNCH_FAILED = 4,           /* hipGetLastError() != hipSuccess after a launch */
  CAIFX_ERR_MISALIGNED = 5,              /* pointer not aligned to its element type */
  CAIFX_ERR_SCRATCH_EXCEEDED = 6         /* the problem needs more scratch than the library's static buffer holds */
};

/* Float element types (CAIF_DataType::Float32 / Float16 / BFloat16). */
enum caifx_dtype { CAIFX_F32 = 0, CAIFX_F16 = 1, CAIFX_BF16 = 2 };

/* Stored weight kinds of a frozen linear.
 *  CAIFX_W_INT8:       one int8 code per element; W[n,k] = code * scales[(n*K+k) % scale_period].
 *                      scale_period 1 is CAIF_Ops::QuantScheme_e::PerTensor_e; scale_period N is
 *                      what PerChannel_e means once the layer reads the buffer as [N,K]
 *                      (src/caif_device_frozen_linear.cpp:356-361 with
 *                      src/caif_cuda_kernels_quant.cu:561-574).  scales == NULL is the
 *                      "int8 without scales" branch, a plain widening cast (:373-375).
 *  CAIFX_W_INT4_GROUP: packed nibbles; W[n,k] = code * fp16 scales[(n*K+k) / group_size]
 *                      (src/caif_cuda_kernels_quant.cu:233-235).
 *  CAIFX_W_F32 / CAIFX_W_F16 / CAIFX_W_BF16: the weight stored undequantised in that float type, W[n,k] =
 *                      element n*K+k cast to the compute type (the float-storage cells of the layer grid:
 *                      src/caif_device_frozen_linear.cpp:301-318 uses the buffer as it is when storage and
 *                      compute types agree, otherwise Weight().To(target)); scales, scale_period and group_size
 *                      are ignored.  These cells run on the fp32 matrix-core kernel (operands rounded to a
 *                      16-bit compute type first, fp32 products and sums), not on the fast paths of the quantised kinds. */
enum caifx_weight_kind { CAIFX_W_INT8 = 0, CAIFX_W_INT4_GROUP = 1, CAIFX_W_F32 = 2, CAIFX_W_F16 = 3, CAIFX_W_BF16 = 4 };

CAIFX_API const char *caifx_status_string(int status);
/* ABI version of this header: major*1000 + minor. */
CAIFX_API int caifx_version(void);

/* ------------------------------------------------------------------------- */
/* Seam 1: kernel launchers (include/caif/caif_cuda_kernels_quant.cuh)        */
/* ------------------------------------------------------------------------- */

/* launch_convert_fp32_to_fp16  (caif_cuda_kernels_quant.cuh:47-50)  RNE */
CAIFX_API int caifx_convert_fp32_to_fp16(const float *input, void *output, int64_t n, caifx_stream_t stream);
/* launch_convert_fp16_to_fp32  (caif_cuda_kernels_quant.cuh:56-59) */
CAIFX_API int caifx_convert_fp16_to_fp32(const void *input, float *output, int64_t n, caifx_stream_t stream);
/* launch_convert_fp32_to_bf16  (caif_cuda_kernels_quant.cuh:68-71)  RNE, NaN stays NaN */
CAIFX_API int caifx_convert_fp32_to_bf16(const float *input, void *output, int64_t n, caifx_stream_t stream);
/* launch_convert_bf16_to_fp32  (caif_cuda_kernels_quant.cuh:80-83) */
CAIFX_API int caifx_convert_bf16_to_fp32(const void *input, float *output, int64_t n, caifx_stream_t stream);
/* launch_convert_fp32_to_int8  (caif_cuda_kernels_quant.cuh:96-99)  clamp to +-127, then RNE */
CAIFX_API int caifx_convert_fp32_to_int8(const float *input, void *output, int64_t n, caifx_stream_t stream);
/* launch_convert_int8_to_fp32  (caif_cuda_kernels_quant.cuh:108-111) */
CAIFX_API int caifx_convert_int8_to_fp32(const void *input, float *output, int64_t n, caifx_stream_t stream);

/* launch_quantize_int8_per_tensor  (caif_cuda_kernels_quant.cuh:131-135)
 * output int8[n], scale float[1].  scale = max|x|/127 (1.0 for all-zero input). */
CAIFX_API int caifx_quantize_int8_per_tensor(const float *input, void *output, void *scale, int64_t n,
                                   caifx_stream_t stream);
/* launch_dequantize_int8_per_tensor  (caif_cuda_kernels_quant.cuh:143-147) */
CAIFX_API int caifx_dequantize_int8_per_tensor(const void *input, float *output, const void *scale, int64_t n,
                                     caifx_stream_t stream);
/* launch_quantize_int8_per_channel  (caif_cuda_kernels_quant.cuh:161-166)
 * input [rows,cols] row-major, output int8[rows*cols], scales float[cols]. */
CAIFX_API int caifx_quantize_int8_per_channel(const float *input, void *output, void *scales, int rows, int cols,
                                    caifx_stream_t stream);
/* launch_dequantize_int8_per_channel  (caif_cuda_kernels_quant.cuh:174-179) */
CAIFX_API int caifx_dequantize_int8_per_channel(const void *input, float *output, const void *scales, int rows,
                                      int cols, caifx_stream_t stream);
/* launch_quantize_to_int4  (caif_cuda_kernels_quant.cuh:219-224)
 * packed_output uint8[(n+1)/2], scales_output fp16[ceil(n/group_size)].
 * group_size must be even when there is more than one group: with an odd size
 * neighbouring groups share a byte and the reference's result is a data race. */
CAIFX_API int caifx_quantize_to_int4(const float *input, void *packed_output, void *scales_output,
                           int64_t num_elements, int group_size, caifx_stream_t stream);
/* launch_dequantize_int4  (caif_cuda_kernels_quant.cuh:199-204) */
CAIFX_API int caifx_dequantize_int4(const void *packed_data, const void *scales, float *output,
                          int64_t num_elements, int group_size, caifx_stream_t stream);

/* ------------------------------------------------------------------------- */
/* Seam 2: the dequantise + GEMM pairs inside the frozen layers, fused        */
/* ------------------------------------------------------------------------- */

/* Forward of CAIF_DeviceFrozenLinear::ForwardImpl
 * (src/caif_device_frozen_linear.cpp:412-509): replaces ConvertToComputeDtype()
 * + input.To(ComputeT) + cublasGemmEx / CAIF_Ops::MatMulTransposeB.
 *   Y[M,N] = cast<compute>(X)[M,K] * cast<compute>(dequant(W))[N,K]^T, fp32 accumulate.
 * x: [M,K] of x_dtype.  y: [M,N] of y_dtype; CAIFX_F32 is the layer's own
 * output type (:442), F16/BF16 fold the caller's following `.To(StorageT)` cast
 * (src/caif_device_moe_frozen_expert.cpp:119-126) into the store and give the
 * same bits as writing fp32 and casting.
 * compute_dtype is the layer's ComputeT.  No dense copy of W is ever written.
 * With up to 32 rows and a 16-bit compute type the memory-bound kernels skip the rounding of code * scale
 * to the compute type for int8 and for int4 with groups of 128 or more (the products with x are formed
 * exactly instead): results then differ from the formula above by that rounding, about 2e-3 of max|y|.
 * In the int8 kernels of that class a NaN or an infinity among the activations of a row turns every result of
 * that row into NaN (the formula above gives NaN or an infinity in each of them). */
CAIFX_API int caifx_qlinear_forward(int64_t M, int64_t N, int64_t K,
                          const void *x, int x_dtype, int compute_dtype,
                          const void *wq, int w_kind, const void *scales, int64_t scale_period,
                          int group_size,
                          void *y, int y_dtype,
                          void *workspace, size_t workspace_bytes, caifx_stream_t stream);

/* Input gradient of CAIF_DeviceFrozenLinear::BackwardImpl
 * (src/caif_device_frozen_linear.cpp:549-645): replaces ConvertToComputeDtype()
 * + grad.To(ComputeT) + cublasGemmEx / CAIF_Ops::MatMul.
 *   dX[M,K] = cast<compute>(dY)[M,N] * cast<compute>(dequant(W))[N,K], fp32 accumulate.
 * With up to 16 rows and int8 codes (any scale vector that leaves at most 64 residue classes of rows with
 * equal scales along k, each of 256 rows or more; one scale; none) or int4 codes in groups of 128 or more, the
 * weight is streamed once through the matrix cores (the 16-bit ones for a 16-bit compute type, the fp32 one
 * for fp32).  For int8 codes the scale is applied outside the products: like the forward's memory-bound kernels
 * this skips the rounding of code * scale to a 16-bit compute type (about 2e-3 of max|dX| for bf16; for the
 * fp32 compute type the difference is fp32 rounding, 1e-7).  int4 codes with a 16-bit compute type meet their
 * scale before the product, rounded once to the compute type: the reference's operand. */
CAIFX_API int caifx_qlinear_backward_input(int64_t M, int64_t N, int64_t K,
                                 const void *dy, int dy_dtype, int compute_dtype,
                                 const void *wq, int w_kind, const void *scales, int64_t scale_period,
                                 int group_size,
                                 void *dx, int dx_dtype,
                                 void *workspace, size_t workspace_bytes, caifx_stream_t stream);

/* The two calls above followed by the caller's cast to its tensor dtype and an element-wise Add, as
 * CAIF_DeviceLoRAAdapter composes the frozen base with the low-rank branch
 * (src/caif_device_lora_adapter.cpp:186-198 forward: base_out.To(StorageT) + lora_out;
 * :264-276 backward: grad_base.To(StorageT) + d_input_lora):
 *   y = T(float(T(acc)) + float(addend)),  T = y_dtype, addend [M,N] (forward) / [M,K] (backward) of y_dtype.
 * The roundings are those of the cast and of the Add, so the bits equal the three-launch sequence.  The
 * large-M kernels add in their store (the fp32 result and its cast copy never touch memory); other shapes
 * run the plain call and the Add.  addend must not alias the output. */
CAIFX_API int caifx_qlinear_forward_add(int64_t M, int64_t N, int64_t K,
                              const void *x, int x_dtype, int compute_dtype,
                              const void *wq, int w_kind, const void *scales, int64_t scale_period,
                              int group_size,
                              void *y, int y_dtype, const void *addend,
                              void *workspace, size_t workspace_bytes, caifx_stream_t stream);
CAIFX_API int caifx_qlinear_backward_input_add(int64_t M, int64_t N, int64_t K,
                                     const void *dy, int dy_dtype, int compute_dtype,
                                     const void *wq, int w_kind, const void *scales, int64_t scale_period,
                                     int group_size,
                                     void *dx, int dx_dtype, const void *addend,
                                     void *workspace, size_t workspace_bytes, caifx_stream_t stream);

/* Bytes of workspace the calls above can use for this problem (may be 0).
 * backward != 0 asks for caifx_qlinear_backward_input.  Nonzero for 16-bit compute types when the result has
 * fewer 128 x 128 tiles than the chip has compute units: up to 8 workgroups then share a tile's reduction through
 * fp32 partial tiles in the workspace (16-byte aligned) and a second launch adds them in a fixed order (results do
 * not depend on scheduling).  The fp32 compute type does the same for up to 128 rows.  The forward with up to
 * 32 rows cuts a reduction longer than one workgroup covers into slices whose sums meet there (K > 4096 with up
 * to 16 rows, K > 2048 with 17..32 rows or with int8 codes and N small enough that the activations' preparation
 * outweighs a workgroup's share of the weight), and the input gradient with up to 16 rows splits
 * the weight's rows among workgroups the same way.  With a smaller or null
 * workspace the calls run without that sharing, slower, and the sums are formed in a different order, so
 * the last bits of a result differ between a call with and a call without the workspace.  In two places the
 * workspace also selects between the two accuracy classes of caifx_qlinear_forward's comment: the input gradient
 * with up to 16 rows and the forward with up to 16 rows and K > 4096 run, without it, on kernels that round
 * code * scale to the 16-bit compute type as the reference does, and with it on the few-row kernels that multiply
 * unrounded codes (about 2e-3 of max|out| apart; both within the 1e-2 bound; the few-row input gradient of packed
 * int4 with a 16-bit compute type multiplies the rounded weight either way). */
CAIFX_API size_t caifx_qlinear_workspace_bytes(int64_t M, int64_t N, int64_t K, int x_dtype, int compute_dtype,
                                     int w_kind, int backward);

/* caifx_qlinear_forward for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc) and so have no workspace to pass: the fp32 partial tiles of a
 * shared reduction go to a buffer of CAIFX_STATIC_SCRATCH_BYTES that is part of the library's device image (one
 * copy per GPU, held until the process ends) instead of the caller's workspace.  It has no counterpart in the
 * reference, whose layers allocate freely.  Same arguments, kernels and results (bit for bit) as
 * caifx_qlinear_forward called with a workspace of caifx_qlinear_workspace_bytes(..., backward = 0) bytes.
 * A problem for which that size exceeds CAIFX_STATIC_SCRATCH_BYTES returns CAIFX_ERR_SCRATCH_EXCEEDED and
 * launches nothing (use caifx_qlinear_forward then; with a null workspace it runs without sharing).
 * The call itself allocates and frees nothing.  Every call on one GPU uses that GPU's one buffer: calls on
 * different streams of the same GPU that may overlap race on it; calls on one stream are ordered and need no
 * clearing in between (every partial tile is written in full before it is read).
 * The buffer's address on a GPU is looked up (hipGetSymbolAddress) on the first call there and kept for the life
 * of the process.  A caller that captures the call into a HIP graph should have that lookup done before the
 * capture begins, by an earlier call or by caifx_static_scratch_prepare() with that GPU current (which also
 * refreshes the address after a hipDeviceReset). */
#define CAIFX_STATIC_SCRATCH_BYTES (8u << 20)
CAIFX_API int caifx_static_scratch_prepare(void);
CAIFX_API int caifx_qlinear_forward_static(int64_t M, int64_t N, int64_t K,
                                 const void *x, int x_dtype, int compute_dtype,
                                 const void *wq, int w_kind, const void *scales, int64_t scale_period,
                                 int group_size,
                                 void *y, int y_dtype, caifx_stream_t stream);

/* Measurement only, no counterpart in the reference (whose per-expert loop, src/caif_device_moe_layer.cpp:534-557,
 * can simply be timed expert by expert on the host): grouped launches of the matrix-core GEMM issued after this
 * call record four 64-bit words per tile (128 rows x 128 columns, or x 256 for the int8 forward kernel that keeps
 * the weight out of LDS) - {expert, rows of the segment inside the tile (low 32 bits; from bit 32 up, when not 0,
 * how many workgroups of that kernel share a compute unit instead of two), start, end}, times in ticks of the
 * GPU's 100 MHz wall clock - into `stamps` (device memory for `tiles` tiles, 32 bytes each; sizing for 128 x 128
 * tiles covers both; tiles are numbered expert by expert, row tile by row tile, column tile last; clear it before
 * a launch, words of tiles that do not exist stay as they are).  stamps = NULL switches the recording off.
 * Process-wide state; not meant for timed runs (one more store per workgroup). */
CAIFX_API int caifx_qlinear_grouped_tile_stamps(void *stamps, int64_t tiles);

/* Measurement only, no counterpart in the reference: `iters` rounds of sixteen v_mfma_f32_32x32x16_bf16 per wave on
 * every compute unit (eight waves each) over the caller's operand values and nothing else - no loads, no stores,
 * no unpacking.  a_ops / b_ops: device buffers of 512 * 4 * 8 bf16 values each (16-byte aligned), e.g. a slice of
 * the activations and of the dequantised weight a benchmark runs on.  The matrix pipes' clock follows the power
 * the operand bit patterns draw, so this is the ceiling a GEMM on those values is priced against beside the
 * published peak.  *flops (host, optional) receives the floating-point operations of the launch; sink (device,
 * optional) 512 floats that keep the compiler from dropping the loop. */
CAIFX_API int caifx_probe_mfma_bf16(const void *a_ops, const void *b_ops, int64_t iters, void *sink, int64_t *flops,
                                    caifx_stream_t stream);

/* The per-expert loop of CAIF_DeviceMoELayer over frozen experts
 * (src/caif_device_moe_layer.cpp:534-557 forward, :754-778 backward) as ONE
 * launch: expert e owns rows [offsets[e], offsets[e+1]) of the token-sorted
 * buffer that MoEDispatchGPU packs (src/caif_cuda_kernels_moe.cu:616-647,
 * offsets from src/caif_ops_device.cpp:4910-4919) and its own frozen weight.
 *   forward : y[r,:] = x[r,:] * W_e^T      x [total_rows,K], y [total_rows,N]
 *   backward: dx[r,:] = dy[r,:] * W_e      dy [total_rows,N], dx [total_rows,K]
 * offsets: device int32[E+1], non-decreasing, offsets[E] <= total_rows (rows
 * past offsets[E] are left untouched; offsets that break this are cut to
 * 0 <= lo <= hi <= total_rows per expert on the device: rows are lost, nothing
 * outside the buffers is touched).  wq_ptrs / scales_ptrs: device arrays of
 * E device pointers (one frozen linear per expert, each its own allocation as
 * in the reference, 16-byte aligned); every expert shares N, K, kind, scale_period, group_size.
 * Forward with total_rows <= 16 * num_experts (MoE decode: a few rows per expert), K <= 4096 and a 16-bit
 * compute type runs the 16-row decode kernel over the segments: an expert's weight is streamed once per 16
 * rows of its segment and an expert without rows costs nothing; the results carry that kernel's rounding
 * (the weight is not rounded to the compute type, see caifx_qlinear_forward), a segment of 3..16 rows gets
 * the bits of caifx_qlinear_forward on its rows. */
CAIFX_API int caifx_qlinear_grouped_forward(int num_experts, const int32_t *offsets, int64_t total_rows,
                                  int64_t N, int64_t K,
                                  const void *x, int x_dtype, int compute_dtype,
                                  const void *const *wq_ptrs, int w_kind,
                                  const void *const *scales_ptrs, int64_t scale_period, int group_size,
                                  void *y, int y_dtype,
                                  void *workspace, size_t workspace_bytes, caifx_stream_t stream);
CAIFX_API int caifx_qlinear_grouped_backward_input(int num_experts, const int32_t *offsets, int64_t total_rows,
                                         int64_t N, int64_t K,
                                         const void *dy, int dy_dtype, int compute_dtype,
                                         const void *const *wq_ptrs, int w_kind,
                                         const void *const *scales_ptrs, int64_t scale_period,
                                         int group_size,
                                         void *dx, int dx_dtype,
                                         void *workspace, size_t workspace_bytes, caifx_stream_t stream);
/* caifx_qlinear_grouped_backward_input with the sum of CAIF_DeviceMoEFrozenExpert::BackwardImpl folded into
 * its store (src/caif_device_moe_frozen_expert.cpp:291-316: grad_input = gi_up.To(StorageT) +
 * gi_gate.To(StorageT)): dx[r,:] = T(float(T(dy[r,:] * W_e)) + float(addend[r,:])) for the rows of the segments;
 * addend [total_rows,K] of dx_dtype, not aliasing dx.  CAIFX_ERR_UNSUPPORTED for shapes the matrix-core kernel
 * does not take (the caller then uses the plain call and caifx_add). */
CAIFX_API int caifx_qlinear_grouped_backward_input_add(int num_experts, const int32_t *offsets, int64_t total_rows,
                                             int64_t N, int64_t K,
                                             const void *dy, int dy_dtype, int compute_dtype,
                                             const void *const *wq_ptrs, int w_kind,
                                             const void *const *scales_ptrs, int64_t scale_period,
                                             int group_size,
                                             void *dx, int dx_dtype, const void *addend,
                                             void *workspace, size_t workspace_bytes, caifx_stream_t stream);
/* The up projection of CAIF_DeviceMoEFrozenExpert::ForwardImpl with the expert's gating folded into its store
 * (src/caif_device_moe_frozen_expert.cpp:119-153: up_out.To(StorageT); SiLU(gate); Multiply): for the rows of
 * the segments up[r,:] = T(x[r,:] * W_e^T) and hidden[r,:] = T(T(silu(gate[r,:])) * up[r,:]), with the cast
 * points of the three separate launches (the result equals caifx_qlinear_grouped_forward followed by
 * caifx_silu_mul bit for bit).  gate, up, hidden: [total_rows,N] of out_dtype (CAIFX_F16 or CAIFX_BF16),
 * pairwise distinct.  CAIFX_ERR_UNSUPPORTED for shapes the matrix-core kernel does not take or results that
 * are not 16-byte aligned with N % 8 == 0 (the caller then uses the separate calls).  This form and the one
 * below save a launch and, in the backward, the grad-of-hidden buffer; at 64 experts x 24576 rows (2048 <-> 1408)
 * an expert pass built on them measures 1-2 % slower than one built on the separate launches, whose
 * element-wise pass runs at full occupancy. */
CAIFX_API int caifx_qlinear_grouped_forward_swiglu(int num_experts, const int32_t *offsets, int64_t total_rows,
                                         int64_t N, int64_t K,
                                         const void *x, int x_dtype, int compute_dtype,
                                         const void *const *wq_ptrs, int w_kind,
                                         const void *const *scales_ptrs, int64_t scale_period, int group_size,
                                         const void *gate, void *up, void *hidden, int out_dtype,
                                         caifx_stream_t stream);
/* The input gradient of the down projection in CAIF_DeviceMoEFrozenExpert::BackwardImpl with the gating's
 * backward folded into its store (src/caif_device_moe_frozen_expert.cpp:252-290): with h = T(dy[r,:] * W_e)
 * (never written), grad_up[r,:] = T(h * T(silu(gate[r,:]))) and grad_gate[r,:] = T(silu'(gate[r,:]) * T(h * up[r,:]))
 * (equal to caifx_qlinear_grouped_backward_input followed by caifx_swiglu_backward bit for bit).  gate, up,
 * grad_gate, grad_up: [total_rows,K] of out_dtype (16-bit), pairwise distinct.  CAIFX_ERR_UNSUPPORTED as above. */
CAIFX_API int caifx_qlinear_grouped_backward_input_swiglu(int num_experts, const int32_t *offsets, int64_t total_rows,
                                                int64_t N, int64_t K,
                                                const void *dy, int dy_dtype, int compute_dtype,
                                                const void *const *wq_ptrs, int w_kind,
                                                const void *const *scales_ptrs, int64_t scale_period,
                                                int group_size,
                                                const void *gate, const void *up, void *grad_gate, void *grad_up,
                                                int out_dtype, caifx_stream_t stream);
CAIFX_API size_t caifx_qlinear_grouped_workspace_bytes(int num_experts, int64_t total_rows, int64_t N, int64_t K,
                                             int x_dtype, int compute_dtype, int w_kind, int backward);

/* ------------------------------------------------------------------------- */
/* Element-wise ops between the expert GEMMs (CAIF_DeviceMoEFrozenExpert)     */
/* ------------------------------------------------------------------------- */

/* CAIF_Ops::SiLU -> swish_forward_kernel (src/caif_cuda_kernels_activations.cu:499-532):
 * out = T(x / (1 + expf(-x))), fp32 math, one rounding to `dtype`. */
CAIFX_API int caifx_silu(const void *input, void *output, int64_t n, int dtype, caifx_stream_t stream);
/* CAIF_Ops::SiLUBackward -> swish_backward_kernel (src/caif_cuda_kernels_activations.cu:539-582):
 * s = 1/(1+expf(-x)); grad_input = T(g * s * (1 + x * (1 - s))). */
CAIFX_API int caifx_silu_backward(const void *input, const void *grad_output, void *grad_input, int64_t n,
                        int dtype, caifx_stream_t stream);
/* CAIF_Ops::Multiply (src/caif_cuda_kernels_elementwise.cu:247-269): out = T(float(a) * float(b)). */
CAIFX_API int caifx_multiply(const void *a, const void *b, void *output, int64_t n, int dtype,
                   caifx_stream_t stream);
/* CAIF_Ops::Add (src/caif_cuda_kernels_elementwise.cu:42-64): out = T(float(a) + float(b)). */
CAIFX_API int caifx_add(const void *a, const void *b, void *output, int64_t n, int dtype, caifx_stream_t stream);
/* SiLU followed by Multiply as CAIF_DeviceMoEFrozenExpert::ForwardImpl chains them
 * (src/caif_device_moe_frozen_expert.cpp:148-153): hidden = T(float(T(silu(gate))) * float(up)).
 * The intermediate rounding of silu(gate) to T is kept, so the bits equal the two-op sequence. */
CAIFX_API int caifx_silu_multiply(const void *gate, const void *up, void *hidden, int64_t n, int dtype,
                        caifx_stream_t stream);
/* The element-wise part of CAIF_DeviceMoEFrozenExpert::BackwardImpl for the gated expert
 * (src/caif_device_moe_frozen_expert.cpp:266-289: SiLU, Multiply, Multiply, SiLUBackward) in one pass:
 *   grad_up   = T(float(grad_hidden) * float(T(silu(gate))))
 *   grad_gate = T(silu_backward(gate, T(float(grad_hidden) * float(up))))
 * Every intermediate is rounded to T where the four kernels round, so the bits equal the four-op
 * sequence.  The outputs must not alias the inputs. */
CAIFX_API int caifx_swiglu_backward(const void *gate, const void *up, const void *grad_hidden, void *grad_gate,
                          void *grad_up, int64_t n, int dtype, caifx_stream_t stream);

/* ---------------------------------------------------------------------------
 * MoE token routing around the grouped dequant-GEMMs: the dispatch map, the gather into the
 * token-sorted expert buffer, the weighted combine, and their backward passes.
 * Shapes: expert_indices / dispatch_map / expert_weights [num_tokens, top_k] (indices and map
 * int32, weights of `dtype`), expert_offsets int32 [num_experts + 1], token tensors
 * [num_tokens, dim], expert buffer [offsets[num_experts], dim], all row-major on the device.
 * An assignment whose expert index is outside [0, num_experts) or whose map entry is -1 (dropped
 * by the capacity limit) moves no data, as in the reference kernels.
 * ------------------------------------------------------------------------- */

/* CAIF_Ops::MoEBuildDispatchMapDevice (src/caif_ops_device.cpp:4876-4960), which copies the indices
 * to the host, loops there and copies map and offsets back.  Here everything stays on the device:
 *   count_e = number of assignments (t,k) with index e; capacity_per_expert > 0 clamps it;
 *   expert_offsets[e+1] = expert_offsets[e] + count_e;
 *   dispatch_map[t,k] = number of assignments to the same expert that come earlier in token-major,
 *   k-minor order, or -1 when that number is >= the clamped count (dropped).
 * expert_offsets[num_experts] is the reference's return value (total assigned rows); callers that
 * need it on the host read it back themselves.
 * workspace: caifx_moe_dispatch_map_workspace_bytes(num_tokens, top_k, num_experts) bytes. */
CAIFX_API size_t caifx_moe_dispatch_map_workspace_bytes(int64_t num_tokens, int top_k, int num_experts);
CAIFX_API int caifx_moe_build_dispatch_map(const int32_t *expert_indices, int64_t num_tokens, int top_k, int num_experts,
                                 int capacity_per_expert, int32_t *dispatch_map, int32_t *expert_offsets,
                                 void *workspace, size_t workspace_bytes, caifx_stream_t stream);

/* launch_moe_dispatch (include/caif/caif_cuda_kernels_moe.cuh:297-305, src/caif_cuda_kernels_moe.cu:616-647):
 * expert_buffer[offsets[e(t,k)] + map[t,k]] = input[t]  (row copy, bit exact). */
CAIFX_API int caifx_moe_dispatch(const void *input, const int32_t *expert_indices, const int32_t *dispatch_map,
                       const int32_t *expert_offsets, void *expert_buffer, int64_t num_tokens, int64_t dim,
                       int top_k, int num_experts, int dtype, caifx_stream_t stream);

/* launch_moe_combine (caif_cuda_kernels_moe.cuh:317-326, caif_cuda_kernels_moe.cu:705-745):
 * output[t,d] = T( sum over k in order of float(w[t,k]) * float(buffer[row(t,k), d]) ), fp32
 * accumulation with one fused multiply-add per k, one rounding to T. */
CAIFX_API int caifx_moe_combine(const void *expert_buffer, const int32_t *expert_indices, const void *expert_weights,
                      const int32_t *dispatch_map, const int32_t *expert_offsets, void *output,
                      int64_t num_tokens, int64_t dim, int top_k, int num_experts, int dtype,
                      caifx_stream_t stream);

/* launch_moe_combine_backward_grad_expert (caif_cuda_kernels_moe.cuh:333-342, caif_cuda_kernels_moe.cu:816-848):
 * grad_expert_buffer[row(t,k), d] = T( float(w[t,k]) * float(grad_output[t,d]) ).  Rows no assignment
 * maps to are left untouched, as in the reference. */
CAIFX_API int caifx_moe_combine_backward_grad_expert(const void *grad_output, const int32_t *expert_indices,
                                           const void *expert_weights, const int32_t *dispatch_map,
                                           const int32_t *expert_offsets, void *grad_expert_buffer,
                                           int64_t num_tokens, int64_t dim, int top_k, int num_experts, int dtype,
                                           caifx_stream_t stream);

/* launch_moe_combine_backward_grad_weights (caif_cuda_kernels_moe.cuh:349-358, caif_cuda_kernels_moe.cu:915-990):
 * grad_weights[t,k] = T( sum over d of float(grad_output[t,d]) * float(buffer[row(t,k), d]) ), fp32
 * accumulation; 0 for an assignment that moved no data.  The order of the additions is fixed but not the
 * reference's block reduction, so parity is to fp32 rounding (1e-5 of the largest value), not bitwise. */
CAIFX_API int caifx_moe_combine_backward_grad_weights(const void *grad_output, const void *expert_buffer,
                                            const int32_t *expert_indices, const int32_t *dispatch_map,
                                            const int32_t *expert_offsets, void *grad_weights,
                                            int64_t num_tokens, int64_t dim, int top_k, int num_experts, int dtype,
                                            caifx_stream_t stream);

/* launch_moe_dispatch_backward (caif_cuda_kernels_moe.cuh:365-373, caif_cuda_kernels_moe.cu:1040-1071):
 * grad_input[t,d] = T( sum over k in order of float(grad_expert_buffer[row(t,k), d]) ), fp32 sum. */
CAIFX_API int caifx_moe_dispatch_backward(const void *grad_expert_buffer, const int32_t *expert_indices,
                                const int32_t *dispatch_map, const int32_t *expert_offsets, void *grad_input,
                                int64_t num_tokens, int64_t dim, int top_k, int num_experts, int dtype,
                                caifx_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* CAIFX_H */
