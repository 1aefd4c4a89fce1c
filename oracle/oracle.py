"""ctypes front end of the CPU oracle (oracle/caif_oracle.c).

TEST INFRASTRUCTURE ONLY: tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg are the only importers.  The shipped package (caif_amd/) never
imports this module; its kernels run on the GPU or fail.

Arrays cross the boundary as C-contiguous numpy arrays.  16-bit floats are
carried as uint16 bit patterns; "values" arrays are float32 holding numbers that
are exactly representable in the dtype they stand for.

The layer-level compositions at the bottom restate the reference's host code
(which op is called on what, and where a tensor is rounded to its dtype); each
cites the reference file:line it follows.
"""
import ctypes
import os
import subprocess

import numpy as np

F32, F16, BF16 = 0, 1, 2            # dtype codes (same as include/caifx.h)
W_INT8, W_INT4_GROUP, W_F32, W_F16, W_BF16 = 0, 1, 2, 3, 4         # weight kinds (same as include/caifx.h)

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libcaif_oracle.so")


def build(force=False):
    """Compile the oracle with gcc (seconds)."""
    if force or not os.path.exists(_SO) or \
            os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "caif_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libcaif_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _declare(_lib)
    return _lib


_i64, _i32, _u32 = ctypes.c_int64, ctypes.c_int32, ctypes.c_uint32
_p = ctypes.c_void_p


def max_threads():
    """OpenMP threads the oracle's parallel loops use."""
    L = lib()
    L.orc_max_threads.restype = ctypes.c_int
    return int(L.orc_max_threads())


def _declare(L):
    L.orc_f32_to_bf16.restype = ctypes.c_uint16
    L.orc_f32_to_bf16.argtypes = [ctypes.c_float]
    L.orc_f32_to_f16.restype = ctypes.c_uint16
    L.orc_f32_to_f16.argtypes = [ctypes.c_float]
    L.orc_bf16_to_f32.restype = ctypes.c_float
    L.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
    L.orc_f16_to_f32.restype = ctypes.c_float
    L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
    for name in ("orc_convert_fp32_to_fp16", "orc_convert_fp16_to_fp32", "orc_convert_fp32_to_bf16",
                 "orc_convert_bf16_to_fp32", "orc_convert_fp32_to_int8", "orc_convert_int8_to_fp32"):
        getattr(L, name).restype = None
        getattr(L, name).argtypes = [_p, _p, _i64]
    L.orc_round_to_dtype.restype = None
    L.orc_round_to_dtype.argtypes = [_p, _i64, ctypes.c_int]
    L.orc_quantize_int8_per_tensor.restype = None
    L.orc_quantize_int8_per_tensor.argtypes = [_p, _p, _p, _i64]
    L.orc_dequantize_int8_per_tensor.restype = None
    L.orc_dequantize_int8_per_tensor.argtypes = [_p, _p, _p, _i64]
    L.orc_quantize_int8_per_channel.restype = None
    L.orc_quantize_int8_per_channel.argtypes = [_p, _p, _p, ctypes.c_int, ctypes.c_int]
    L.orc_dequantize_int8_per_channel.restype = None
    L.orc_dequantize_int8_per_channel.argtypes = [_p, _p, _p, ctypes.c_int, ctypes.c_int]
    L.orc_quantize_to_int4.restype = None
    L.orc_quantize_to_int4.argtypes = [_p, _p, _p, _i64, ctypes.c_int]
    L.orc_dequantize_int4.restype = None
    L.orc_dequantize_int4.argtypes = [_p, _p, _p, _i64, ctypes.c_int]
    L.orc_frozen_weight_compute.restype = None
    L.orc_frozen_weight_compute.argtypes = [_p, ctypes.c_int, _p, _i64, _i64, _i64, ctypes.c_int,
                                            ctypes.c_int, _p]
    L.orc_gemm_nt.restype = None
    L.orc_gemm_nt.argtypes = [_i64, _i64, _i64, _p, _p, _p]
    L.orc_gemm_nn.restype = None
    L.orc_gemm_nn.argtypes = [_i64, _i64, _i64, _p, _p, _p]
    L.orc_silu.restype = None
    L.orc_silu.argtypes = [_p, _p, _i64, ctypes.c_int]
    L.orc_silu_backward.restype = None
    L.orc_silu_backward.argtypes = [_p, _p, _p, _i64, ctypes.c_int]
    L.orc_multiply.restype = None
    L.orc_multiply.argtypes = [_p, _p, _p, _i64, ctypes.c_int]
    L.orc_add.restype = None
    L.orc_add.argtypes = [_p, _p, _p, _i64, ctypes.c_int]
    L.orc_moe_build_dispatch_map.restype = _u32
    L.orc_moe_build_dispatch_map.argtypes = [_p, _u32, _u32, _u32, _u32, _p, _p]


def _ptr(a):
    return a.ctypes.data_as(_p) if a is not None else None


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


# --------------------------------------------------------------------------- casts
def f32_to_bf16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_convert_fp32_to_bf16(_ptr(x), _ptr(out), x.size)
    return out


def bf16_bits_to_f32(b):
    b = _c(b, np.uint16)
    out = np.empty(b.shape, np.float32)
    lib().orc_convert_bf16_to_fp32(_ptr(b), _ptr(out), b.size)
    return out


def f32_to_f16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_convert_fp32_to_fp16(_ptr(x), _ptr(out), x.size)
    return out


def f16_bits_to_f32(b):
    b = _c(b, np.uint16)
    out = np.empty(b.shape, np.float32)
    lib().orc_convert_fp16_to_fp32(_ptr(b), _ptr(out), b.size)
    return out


def convert_fp32_to_int8(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.int8)
    lib().orc_convert_fp32_to_int8(_ptr(x), _ptr(out), x.size)
    return out


def convert_int8_to_fp32(q):
    q = _c(q, np.int8)
    out = np.empty(q.shape, np.float32)
    lib().orc_convert_int8_to_fp32(_ptr(q), _ptr(out), q.size)
    return out


def round_to_dtype(x, dtype):
    """Values of `x` after a cast to `dtype` (float32 array of representable values)."""
    out = _c(x, np.float32).copy()
    lib().orc_round_to_dtype(_ptr(out), out.size, dtype)
    return out


# --------------------------------------------------------------------------- quantise
def quantize_int8_per_tensor(x):
    x = _c(x, np.float32)
    q = np.zeros(x.shape, np.int8)
    s = np.zeros(1, np.float32)
    lib().orc_quantize_int8_per_tensor(_ptr(x), _ptr(q), _ptr(s), x.size)
    return q, s


def dequantize_int8_per_tensor(q, s):
    q = _c(q, np.int8)
    s = _c(s, np.float32)
    out = np.zeros(q.shape, np.float32)
    lib().orc_dequantize_int8_per_tensor(_ptr(q), _ptr(out), _ptr(s), q.size)
    return out


def quantize_int8_per_channel(x):
    x = _c(x, np.float32)
    assert x.ndim == 2
    rows, cols = x.shape
    q = np.zeros(x.shape, np.int8)
    s = np.zeros(cols, np.float32)
    lib().orc_quantize_int8_per_channel(_ptr(x), _ptr(q), _ptr(s), rows, cols)
    return q, s


def dequantize_int8_per_channel(q, s):
    q = _c(q, np.int8)
    s = _c(s, np.float32)
    rows, cols = q.shape
    out = np.zeros(q.shape, np.float32)
    lib().orc_dequantize_int8_per_channel(_ptr(q), _ptr(out), _ptr(s), rows, cols)
    return out


def quantize_to_int4(x, group_size):
    x = _c(x, np.float32).reshape(-1)
    n = x.size
    packed = np.zeros((n + 1) // 2, np.uint8)
    scales = np.zeros((n + group_size - 1) // group_size, np.uint16)
    lib().orc_quantize_to_int4(_ptr(x), _ptr(packed), _ptr(scales), n, group_size)
    return packed, scales


def dequantize_int4(packed, scales_f16_bits, n, group_size):
    packed = _c(packed, np.uint8)
    scales = _c(scales_f16_bits, np.uint16)
    out = np.zeros(n, np.float32)
    lib().orc_dequantize_int4(_ptr(packed), _ptr(scales), _ptr(out), n, group_size)
    return out


# --------------------------------------------------------------------------- frozen linear
def frozen_weight_compute(wq, w_kind, scales, N, K, scale_period, group_size, compute_dtype):
    """W[N,K] in the compute dtype, as ConvertToComputeDtype materialises it
    (src/caif_device_frozen_linear.cpp:289-378)."""
    if w_kind == W_F32:
        wq, scales = _c(wq, np.float32), None
    elif w_kind in (W_F16, W_BF16):           # the 16-bit patterns of the stored elements
        wq, scales = _c(wq, np.uint16), None
    elif w_kind == W_INT4_GROUP:
        wq = _c(wq, np.uint8)
        scales = _c(scales, np.uint16)
    else:
        wq = _c(wq, np.int8)
        scales = None if scales is None else _c(scales, np.float32)
    out = np.empty((N, K), np.float32)
    lib().orc_frozen_weight_compute(_ptr(wq), w_kind, _ptr(scales), N, K, scale_period, group_size,
                                    compute_dtype, _ptr(out))
    return out


def gemm_nt(x, w):
    x = _c(x, np.float32)
    w = _c(w, np.float32)
    M, K = x.shape
    N = w.shape[0]
    y = np.empty((M, N), np.float32)
    lib().orc_gemm_nt(M, N, K, _ptr(x), _ptr(w), _ptr(y))
    return y


def gemm_nn(dy, w):
    dy = _c(dy, np.float32)
    w = _c(w, np.float32)
    M, N = dy.shape
    K = w.shape[1]
    dx = np.empty((M, K), np.float32)
    lib().orc_gemm_nn(M, N, K, _ptr(dy), _ptr(w), _ptr(dx))
    return dx


class FrozenWeight:
    """Stored weight of one CAIF_DeviceFrozenLinear: codes + scales + scheme."""

    def __init__(self, wq, w_kind, scales, N, K, scale_period=1, group_size=128):
        self.wq, self.w_kind, self.scales = wq, w_kind, scales
        self.N, self.K, self.scale_period, self.group_size = N, K, scale_period, group_size
        self._cache = {}

    def compute_weight(self, compute_dtype):
        if compute_dtype not in self._cache:
            self._cache[compute_dtype] = frozen_weight_compute(
                self.wq, self.w_kind, self.scales, self.N, self.K, self.scale_period,
                self.group_size, compute_dtype)
        return self._cache[compute_dtype]


def frozen_linear_forward(x_values, fw, compute_dtype):
    """CAIF_DeviceFrozenLinear::ForwardImpl (src/caif_device_frozen_linear.cpp:382-524):
    input flattened to [n,K] and cast to the compute dtype (:459,:466), weight
    materialised in the compute dtype (:412-427), GEMM with fp32 output (:442)."""
    x = round_to_dtype(np.asarray(x_values, np.float32).reshape(-1, fw.K), compute_dtype)
    return gemm_nt(x, fw.compute_weight(compute_dtype))


def frozen_linear_backward(dy_values, fw, compute_dtype):
    """CAIF_DeviceFrozenLinear::BackwardImpl (src/caif_device_frozen_linear.cpp:528-660):
    dX[n,K] = dY[n,N] * W[N,K], dY cast to the compute dtype (:595,:602), fp32 output (:580)."""
    dy = round_to_dtype(np.asarray(dy_values, np.float32).reshape(-1, fw.N), compute_dtype)
    return gemm_nn(dy, fw.compute_weight(compute_dtype))


# --------------------------------------------------------------------------- element-wise
def _ew2(fn, a, b, dtype):
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    out = np.empty(a.shape, np.float32)
    fn(_ptr(a), _ptr(b), _ptr(out), a.size, dtype)
    return out


def silu(x, dtype):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.float32)
    lib().orc_silu(_ptr(x), _ptr(out), x.size, dtype)
    return out


def silu_backward(x, grad_out, dtype):
    return _ew2(lib().orc_silu_backward, x, grad_out, dtype)


def multiply(a, b, dtype):
    return _ew2(lib().orc_multiply, a, b, dtype)


def add(a, b, dtype):
    return _ew2(lib().orc_add, a, b, dtype)


# --------------------------------------------------------------------------- MoE frozen expert
def moe_frozen_expert_forward(x_values, gate, up, down, compute_dtype, storage_dtype):
    """CAIF_DeviceMoEFrozenExpert::ForwardImpl, gated branch
    (src/caif_device_moe_frozen_expert.cpp:92-179).  Each frozen linear returns
    fp32 and is cast to the storage dtype (:117-126, :131-141, :171-176);
    hidden = SiLU(gate_out) * up_out, both element-wise ops rounding to the
    storage dtype (:148-153).  Returns (out, cache) where cache holds what the
    training forward keeps for backward (:154-169)."""
    x = round_to_dtype(x_values, storage_dtype)
    up_out = round_to_dtype(frozen_linear_forward(x, up, compute_dtype), storage_dtype)
    gate_out = round_to_dtype(frozen_linear_forward(x, gate, compute_dtype), storage_dtype)
    gate_act = silu(gate_out, storage_dtype)
    hidden = multiply(gate_act, up_out, storage_dtype)
    out = round_to_dtype(frozen_linear_forward(hidden, down, compute_dtype), storage_dtype)
    return out, {"gate_out": gate_out, "up_out": up_out, "hidden": hidden}


def moe_frozen_expert_backward(grad_values, cache, gate, up, down, compute_dtype, storage_dtype):
    """CAIF_DeviceMoEFrozenExpert::BackwardImpl, gated branch
    (src/caif_device_moe_frozen_expert.cpp:231-317)."""
    g = round_to_dtype(grad_values, storage_dtype)
    grad_hidden = round_to_dtype(frozen_linear_backward(g, down, compute_dtype), storage_dtype)
    gate_act = silu(cache["gate_out"], storage_dtype)                       # :275-278
    grad_up = multiply(grad_hidden, gate_act, storage_dtype)                # :280-281
    grad_gate_act = multiply(grad_hidden, cache["up_out"], storage_dtype)   # :283-286
    grad_gate = silu_backward(cache["gate_out"], grad_gate_act, storage_dtype)  # :288-289
    gi_up = round_to_dtype(frozen_linear_backward(grad_up, up, compute_dtype), storage_dtype)
    gi_gate = round_to_dtype(frozen_linear_backward(grad_gate, gate, compute_dtype), storage_dtype)
    return add(gi_up, gi_gate, storage_dtype)                               # :314-315


# --------------------------------------------------------------------------- MoE segment map
def moe_build_dispatch_map(indices, num_experts, capacity_per_expert=0):
    """CAIF_Ops::MoEBuildDispatchMapDevice (src/caif_ops_device.cpp:4876-4960)."""
    idx = _c(indices, np.int32)
    T, top_k = idx.shape
    dmap = np.empty((T, top_k), np.int32)
    offsets = np.empty(num_experts + 1, np.int32)
    total = lib().orc_moe_build_dispatch_map(_ptr(idx), T, num_experts, top_k, capacity_per_expert,
                                             _ptr(dmap), _ptr(offsets))
    return dmap, offsets, int(total)


def _routed_rows(indices, dmap, offsets, num_experts):
    """Row of the expert buffer each assignment (t,k) maps to, -1 where it moves no data
    (expert index out of range or map entry -1), as the reference kernels test it
    (src/caif_cuda_kernels_moe.cu:640-645)."""
    idx = np.asarray(indices, np.int64)
    pos = np.asarray(dmap, np.int64)
    ok = (idx >= 0) & (idx < num_experts) & (pos >= 0)
    rows = np.where(ok, np.asarray(offsets, np.int64)[np.clip(idx, 0, num_experts - 1)] + pos, -1)
    return rows


def moe_dispatch(x_values, indices, dmap, offsets, num_experts, total_rows, dtype):
    """moe_dispatch_kernel (src/caif_cuda_kernels_moe.cu:616-647): buffer[row(t,k)] = input[t]; rows no
    assignment maps to keep their previous content (zeros here)."""
    x = round_to_dtype(np.asarray(x_values, np.float32), dtype)
    rows = _routed_rows(indices, dmap, offsets, num_experts)
    buf = np.zeros((total_rows, x.shape[1]), np.float32)
    T, top_k = rows.shape
    for t in range(T):
        for k in range(top_k):
            if rows[t, k] >= 0:
                buf[rows[t, k]] = x[t]
    return buf


def moe_combine(buffer_values, indices, weights, dmap, offsets, num_experts, dtype):
    """moe_combine_kernel (src/caif_cuda_kernels_moe.cu:705-745): per (t,d) an fp32 sum over k in order,
    sum += float(w) * float(buf) (one fused multiply-add, nvcc's default contraction), one rounding to T."""
    buf = round_to_dtype(np.asarray(buffer_values, np.float32), dtype)
    w = round_to_dtype(np.asarray(weights, np.float32), dtype)
    rows = _routed_rows(indices, dmap, offsets, num_experts)
    T, top_k = rows.shape
    out = np.zeros((T, buf.shape[1]), np.float32)
    for t in range(T):
        acc = np.zeros(buf.shape[1], np.float64)        # exact product + one fp32 rounding per step = fmaf
        acc32 = np.zeros(buf.shape[1], np.float32)
        for k in range(top_k):
            if rows[t, k] >= 0:
                acc = np.float64(w[t, k]) * buf[rows[t, k]].astype(np.float64) + acc32.astype(np.float64)
                acc32 = acc.astype(np.float32)
        out[t] = acc32
    return round_to_dtype(out, dtype)


def moe_combine_backward_grad_expert(grad_values, indices, weights, dmap, offsets, num_experts, total_rows, dtype):
    """moe_combine_backward_grad_expert_kernel (src/caif_cuda_kernels_moe.cu:816-848):
    grad_buffer[row(t,k)] = T(float(w[t,k]) * float(grad_output[t])); other rows untouched (zeros here)."""
    g = round_to_dtype(np.asarray(grad_values, np.float32), dtype)
    w = round_to_dtype(np.asarray(weights, np.float32), dtype)
    rows = _routed_rows(indices, dmap, offsets, num_experts)
    out = np.zeros((total_rows, g.shape[1]), np.float32)
    T, top_k = rows.shape
    for t in range(T):
        for k in range(top_k):
            if rows[t, k] >= 0:
                out[rows[t, k]] = round_to_dtype((w[t, k] * g[t]).astype(np.float32), dtype)
    return out


def moe_combine_backward_grad_weights(grad_values, buffer_values, indices, dmap, offsets, num_experts, dtype):
    """moe_combine_backward_grad_weights_block_kernel (src/caif_cuda_kernels_moe.cu:915-990):
    grad_weights[t,k] = T(sum_d float(grad_output[t,d]) * float(buffer[row(t,k),d])); 0 where the
    assignment moved no data.  Accumulated in fp64 here (the reference's block-reduction order is not
    part of its contract)."""
    g = round_to_dtype(np.asarray(grad_values, np.float32), dtype).astype(np.float64)
    buf = round_to_dtype(np.asarray(buffer_values, np.float32), dtype).astype(np.float64)
    rows = _routed_rows(indices, dmap, offsets, num_experts)
    T, top_k = rows.shape
    out = np.zeros((T, top_k), np.float64)
    for t in range(T):
        for k in range(top_k):
            if rows[t, k] >= 0:
                out[t, k] = float(np.dot(g[t], buf[rows[t, k]]))
    return round_to_dtype(out.astype(np.float32), dtype)


def moe_dispatch_backward(grad_buffer_values, indices, dmap, offsets, num_experts, dtype):
    """moe_dispatch_backward_kernel (src/caif_cuda_kernels_moe.cu:1040-1071): grad_input[t] =
    T(sum over k in order of float(grad_buffer[row(t,k)])), fp32 additions."""
    gb = round_to_dtype(np.asarray(grad_buffer_values, np.float32), dtype)
    rows = _routed_rows(indices, dmap, offsets, num_experts)
    T, top_k = rows.shape
    out = np.zeros((T, gb.shape[1]), np.float32)
    for t in range(T):
        acc = np.zeros(gb.shape[1], np.float32)
        for k in range(top_k):
            if rows[t, k] >= 0:
                acc = (acc + gb[rows[t, k]]).astype(np.float32)
        out[t] = acc
    return round_to_dtype(out, dtype)


# --------------------------------------------------------------------------- LoRA around a frozen base
def lora_forward(x_values, fw, lora_a, lora_b, alpha, compute_dtype, storage_dtype):
    """CAIF_DeviceLoRAAdapter::ForwardImpl (src/caif_device_lora_adapter.cpp:119-203):
    base_out = base(x) (fp32, cast to the storage dtype, :189-198); lora_hidden = x A^T and
    lora_out = lora_hidden B^T are stored in the storage dtype (:161-173); lora_out is scaled by
    alpha/rank in place (:175-177) and added element-wise (:187-198).  A is [rank, in], B is
    [out, rank].  Returns (output, lora_hidden)."""
    x = round_to_dtype(np.asarray(x_values, np.float32), storage_dtype)
    rank = lora_a.shape[0]
    base = round_to_dtype(frozen_linear_forward(x, fw, compute_dtype), storage_dtype)
    a = round_to_dtype(lora_a, storage_dtype)
    b = round_to_dtype(lora_b, storage_dtype)
    hidden = round_to_dtype(gemm_nt(x, a), storage_dtype)
    out = round_to_dtype(gemm_nt(hidden, b), storage_dtype)
    out = round_to_dtype(out * np.float32(alpha / rank), storage_dtype)
    return add(base, out, storage_dtype), hidden


def lora_backward_input(grad_values, fw, lora_a, lora_b, alpha, compute_dtype, storage_dtype):
    """Input gradient of CAIF_DeviceLoRAAdapter::BackwardImpl (src/caif_device_lora_adapter.cpp:
    205-281): d_lora_scaled = g * alpha/rank (:228-232); d_lora_hidden = d_lora_scaled B (:241-243);
    d_input_lora = d_lora_hidden A (:250-252); grad_base = base.Backward(g) (:255), cast to the
    storage dtype and added (:267-276)."""
    g = round_to_dtype(np.asarray(grad_values, np.float32), storage_dtype)
    rank = lora_a.shape[0]
    a = round_to_dtype(lora_a, storage_dtype)
    b = round_to_dtype(lora_b, storage_dtype)
    gs = round_to_dtype(g * np.float32(alpha / rank), storage_dtype)
    d_hidden = round_to_dtype(gemm_nn(gs, b), storage_dtype)
    d_in = round_to_dtype(gemm_nn(d_hidden, a), storage_dtype)
    base = round_to_dtype(frozen_linear_backward(g, fw, compute_dtype), storage_dtype)
    return add(base, d_in, storage_dtype)
