"""Thin callers of the C ABI for torch-owned device buffers (tests and bench.py plumbing).

torch supplies device memory and the current HIP stream; every computation is a
call into libcaifx.so.  Function names follow the reference's CAIF_Ops entry
points (src/caif_ops.cpp:504-680); argument meaning is the same.
"""
import torch

from . import capi
from .capi import F32, F16, BF16, W_INT8, W_INT4_GROUP, W_F32, W_F16, W_BF16

TORCH_DTYPE = {F32: torch.float32, F16: torch.float16, BF16: torch.bfloat16}
CODE_OF = {v: k for k, v in TORCH_DTYPE.items()}


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return 0 if t is None else t.data_ptr()


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            # CAIF_Ops quantise entry points throw for Host_e tensors (src/caif_ops.cpp:514-517)
            raise RuntimeError("host backend not supported")
        if t is not None and not t.is_contiguous():
            raise RuntimeError("tensor must be contiguous")


# ------------------------------------------------------------------ CAIF_Ops::Quantize* / Dequantize*
def quantize_int8(x, per_channel):
    """CAIF_Ops::QuantizeInt8 (src/caif_ops_device.cpp:1517-1573).  Returns (codes, scales)."""
    _need_cuda(x)
    if x.dtype != torch.float32:
        raise RuntimeError("QuantizeInt8: input must be fp32")
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    if not per_channel:
        s = torch.empty(1, dtype=torch.float32, device=x.device)
        capi.call("caifx_quantize_int8_per_tensor", _ptr(x), _ptr(q), _ptr(s), x.numel(), _stream())
        return q, s
    if x.dim() != 2:
        raise RuntimeError("QuantizeInt8 PerChannel: input must be 2D")
    rows, cols = x.shape
    s = torch.empty(cols, dtype=torch.float32, device=x.device)
    capi.call("caifx_quantize_int8_per_channel", _ptr(x), _ptr(q), _ptr(s), rows, cols, _stream())
    return q, s


def dequantize_int8(q, scales, per_channel):
    """CAIF_Ops::DequantizeInt8 (src/caif_ops_device.cpp:1584-1640)."""
    _need_cuda(q, scales)
    out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    if not per_channel:
        if scales.numel() != 1:
            raise RuntimeError("DequantizeInt8 PerTensor: scales must have 1 element")
        capi.call("caifx_dequantize_int8_per_tensor", _ptr(q), _ptr(out), _ptr(scales), q.numel(), _stream())
        return out
    if q.dim() != 2:
        raise RuntimeError("DequantizeInt8 PerChannel: input must be 2D")
    rows, cols = q.shape
    if scales.numel() != cols:
        raise RuntimeError("DequantizeInt8 PerChannel: scales length must equal cols")
    capi.call("caifx_dequantize_int8_per_channel", _ptr(q), _ptr(out), _ptr(scales), rows, cols, _stream())
    return out


def quantize_int4_per_group(x, group_size):
    """CAIF_Ops::QuantizeInt4PerGroup (src/caif_ops_device.cpp:1651-1687).  Returns (packed, fp16 scales)."""
    _need_cuda(x)
    if x.dtype != torch.float32:
        raise RuntimeError("QuantizeInt4PerGroup: input must be fp32")
    if group_size == 0:
        raise RuntimeError("QuantizeInt4PerGroup: group_size must be > 0")
    n = x.numel()
    packed = torch.empty((n + 1) // 2, dtype=torch.uint8, device=x.device)
    scales = torch.empty((n + group_size - 1) // group_size, dtype=torch.float16, device=x.device)
    capi.call("caifx_quantize_to_int4", _ptr(x), _ptr(packed), _ptr(scales), n, group_size, _stream())
    return packed, scales


def dequantize_int4_per_group(packed, scales, n, group_size):
    """CAIF_Ops::DequantizeInt4PerGroup (src/caif_ops_device.cpp:1698-1734)."""
    _need_cuda(packed, scales)
    if group_size == 0:
        raise RuntimeError("DequantizeInt4PerGroup: group_size must be > 0")
    if scales.numel() != (n + group_size - 1) // group_size:
        raise RuntimeError("DequantizeInt4PerGroup: scales length must equal num_groups")
    out = torch.empty(n, dtype=torch.float32, device=packed.device)
    capi.call("caifx_dequantize_int4", _ptr(packed), _ptr(scales), _ptr(out), n, group_size, _stream())
    return out


_CASTS = {
    (torch.float32, torch.float16): "caifx_convert_fp32_to_fp16",
    (torch.float16, torch.float32): "caifx_convert_fp16_to_fp32",
    (torch.float32, torch.bfloat16): "caifx_convert_fp32_to_bf16",
    (torch.bfloat16, torch.float32): "caifx_convert_bf16_to_fp32",
    (torch.float32, torch.int8): "caifx_convert_fp32_to_int8",
    (torch.int8, torch.float32): "caifx_convert_int8_to_fp32",
}


def convert(x, dtype):
    """The cast kernels behind CAIF_DeviceTensor::To (src/caif_device_tensor.cpp:604-706)."""
    _need_cuda(x)
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    capi.call(_CASTS[(x.dtype, dtype)], _ptr(x), _ptr(out), x.numel(), _stream())
    return out


# ------------------------------------------------------------------ frozen linear
class FrozenWeight:
    """Device storage of one CAIF_DeviceFrozenLinear: codes, scales and the scale scheme."""

    def __init__(self, wq, w_kind, scales, N, K, scale_period=1, group_size=128):
        self.wq, self.w_kind, self.scales = wq, w_kind, scales
        self.N, self.K, self.scale_period, self.group_size = N, K, scale_period, group_size


def _workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


def qlinear_forward(x, fw, compute_dtype, y_dtype=F32, out=None, workspace=None, addend=None):
    """caifx_qlinear_forward on x [..., K]; returns y [M, N].  With `addend` [M, N] of y_dtype:
    caifx_qlinear_forward_add, y = T(float(T(x W^T)) + float(addend))."""
    _need_cuda(x)
    M = x.numel() // fw.K
    y = out if out is not None else torch.empty((M, fw.N), dtype=TORCH_DTYPE[y_dtype], device=x.device)
    xd = CODE_OF[x.dtype]
    if workspace is None:
        workspace = _workspace(capi.lib().caifx_qlinear_workspace_bytes(M, fw.N, fw.K, xd, compute_dtype,
                                                                       fw.w_kind, 0), x.device)
    if addend is not None:
        assert addend.dtype == y.dtype and addend.numel() == y.numel()
        capi.call("caifx_qlinear_forward_add", M, fw.N, fw.K, _ptr(x), xd, compute_dtype, _ptr(fw.wq), fw.w_kind,
                  _ptr(fw.scales), fw.scale_period, fw.group_size, _ptr(y), y_dtype, _ptr(addend), _ptr(workspace),
                  workspace.numel(), _stream())
        return y
    capi.call("caifx_qlinear_forward", M, fw.N, fw.K, _ptr(x), xd, compute_dtype, _ptr(fw.wq), fw.w_kind,
              _ptr(fw.scales), fw.scale_period, fw.group_size, _ptr(y), y_dtype, _ptr(workspace),
              workspace.numel(), _stream())
    return y


def probe_mfma_bf16(a_values, b_values, iters):
    """caifx_probe_mfma_bf16: launches the matrix-pipe-only loop on the first 16384 bf16 values of each tensor;
    returns the floating-point operations of the launch (time it with events around the call)."""
    import ctypes
    _need_cuda(a_values)
    a = a_values.reshape(-1)[:16384].to(torch.bfloat16).contiguous()
    b = b_values.reshape(-1)[:16384].to(torch.bfloat16).contiguous()
    assert a.numel() == 16384 and b.numel() == 16384
    sink = torch.empty(512, dtype=torch.float32, device=a.device)
    flops = ctypes.c_int64(0)
    capi.call("caifx_probe_mfma_bf16", _ptr(a), _ptr(b), int(iters), _ptr(sink), ctypes.byref(flops), _stream())
    return flops.value, (a, b, sink)


def qlinear_backward_input(dy, fw, compute_dtype, dx_dtype=F32, out=None, workspace=None, addend=None):
    """caifx_qlinear_backward_input on dy [..., N]; returns dx [M, K] (plus `addend` [M, K], see qlinear_forward)."""
    _need_cuda(dy)
    M = dy.numel() // fw.N
    dx = out if out is not None else torch.empty((M, fw.K), dtype=TORCH_DTYPE[dx_dtype], device=dy.device)
    yd = CODE_OF[dy.dtype]
    if workspace is None:
        workspace = _workspace(capi.lib().caifx_qlinear_workspace_bytes(M, fw.N, fw.K, yd, compute_dtype,
                                                                       fw.w_kind, 1), dy.device)
    if addend is not None:
        assert addend.dtype == dx.dtype and addend.numel() == dx.numel()
        capi.call("caifx_qlinear_backward_input_add", M, fw.N, fw.K, _ptr(dy), yd, compute_dtype, _ptr(fw.wq),
                  fw.w_kind, _ptr(fw.scales), fw.scale_period, fw.group_size, _ptr(dx), dx_dtype, _ptr(addend),
                  _ptr(workspace), workspace.numel(), _stream())
        return dx
    capi.call("caifx_qlinear_backward_input", M, fw.N, fw.K, _ptr(dy), yd, compute_dtype, _ptr(fw.wq),
              fw.w_kind, _ptr(fw.scales), fw.scale_period, fw.group_size, _ptr(dx), dx_dtype,
              _ptr(workspace), workspace.numel(), _stream())
    return dx


class GroupedFrozenWeights:
    """E frozen linears of one shape (one per expert), addressed through device pointer arrays."""

    def __init__(self, weights):
        w0 = weights[0]
        self.weights = weights
        self.N, self.K, self.w_kind = w0.N, w0.K, w0.w_kind
        self.scale_period, self.group_size = w0.scale_period, w0.group_size
        dev = w0.wq.device
        self.wq_ptrs = torch.tensor([w.wq.data_ptr() for w in weights], dtype=torch.int64, device=dev)
        self.scales_ptrs = None
        if w0.scales is not None:
            self.scales_ptrs = torch.tensor([w.scales.data_ptr() for w in weights], dtype=torch.int64, device=dev)


def _check_grouped(x, in_dim, rows, offsets, E, results, out_dim, out_dtype):
    """The C ABI sees raw pointers: sizes and dtypes are checked here, before anything is launched."""
    if x.numel() != rows * in_dim:
        raise ValueError(f"input has {x.numel()} elements, not a multiple of the reduction length {in_dim}")
    if offsets.dtype != torch.int32 or offsets.numel() != E + 1:
        raise ValueError(f"offsets must be int32 [{E + 1}]")
    for t in results:
        _need_cuda(t)
        if t.dtype != out_dtype or t.numel() != rows * out_dim:
            raise ValueError(f"result / gating tensors must be {out_dtype} with {rows} x {out_dim} elements")


def _grouped(name, backward, x, offsets, gw, compute_dtype, out_dtype, out, workspace, addend=None):
    _need_cuda(x, offsets)
    in_dim = gw.N if backward else gw.K
    out_dim = gw.K if backward else gw.N
    rows = x.numel() // in_dim
    y = out if out is not None else torch.zeros((rows, out_dim), dtype=TORCH_DTYPE[out_dtype], device=x.device)
    xd = CODE_OF[x.dtype]
    E = len(gw.weights)
    _check_grouped(x, in_dim, rows, offsets, E, (y,), out_dim, TORCH_DTYPE[out_dtype])
    if workspace is None:
        workspace = _workspace(capi.lib().caifx_qlinear_grouped_workspace_bytes(
            E, rows, gw.N, gw.K, xd, compute_dtype, gw.w_kind, int(backward)), x.device)
    if addend is not None:
        assert addend.dtype == y.dtype and addend.numel() == y.numel()
        capi.call(name + "_add", E, _ptr(offsets), rows, gw.N, gw.K, _ptr(x), xd, compute_dtype, _ptr(gw.wq_ptrs),
                  gw.w_kind, _ptr(gw.scales_ptrs), gw.scale_period, gw.group_size, _ptr(y), out_dtype, _ptr(addend),
                  _ptr(workspace), workspace.numel(), _stream())
        return y
    capi.call(name, E, _ptr(offsets), rows, gw.N, gw.K, _ptr(x), xd, compute_dtype, _ptr(gw.wq_ptrs), gw.w_kind,
              _ptr(gw.scales_ptrs), gw.scale_period, gw.group_size, _ptr(y), out_dtype, _ptr(workspace),
              workspace.numel(), _stream())
    return y


def qlinear_grouped_forward(x, offsets, gw, compute_dtype, y_dtype=F32, out=None, workspace=None):
    return _grouped("caifx_qlinear_grouped_forward", False, x, offsets, gw, compute_dtype, y_dtype, out, workspace)


def qlinear_grouped_backward_input(dy, offsets, gw, compute_dtype, dx_dtype=F32, out=None, workspace=None,
                                   addend=None):
    return _grouped("caifx_qlinear_grouped_backward_input", True, dy, offsets, gw, compute_dtype, dx_dtype, out,
                    workspace, addend)


def qlinear_grouped_forward_swiglu(x, offsets, gw_up, gate, compute_dtype, out=None):
    """Up projection with the gating in its store: returns (up, hidden), both of gate's dtype and shape."""
    _need_cuda(x, offsets, gate)
    rows = x.numel() // gw_up.K
    up, hidden = out if out is not None else (torch.zeros_like(gate), torch.zeros_like(gate))
    _check_grouped(x, gw_up.K, rows, offsets, len(gw_up.weights), (gate, up, hidden), gw_up.N, gate.dtype)
    capi.call("caifx_qlinear_grouped_forward_swiglu", len(gw_up.weights), _ptr(offsets), rows, gw_up.N, gw_up.K, _ptr(x),
              CODE_OF[x.dtype], compute_dtype, _ptr(gw_up.wq_ptrs), gw_up.w_kind, _ptr(gw_up.scales_ptrs),
              gw_up.scale_period, gw_up.group_size, _ptr(gate), _ptr(up), _ptr(hidden), CODE_OF[gate.dtype], _stream())
    return up, hidden


def qlinear_grouped_backward_input_swiglu(dy, offsets, gw_down, gate, up, compute_dtype, out=None):
    """Input gradient of the down projection with the gating's backward in its store: returns (grad_gate, grad_up)."""
    _need_cuda(dy, offsets, gate, up)
    rows = dy.numel() // gw_down.N
    grad_gate, grad_up = out if out is not None else (torch.zeros_like(gate), torch.zeros_like(gate))
    _check_grouped(dy, gw_down.N, rows, offsets, len(gw_down.weights), (gate, up, grad_gate, grad_up), gw_down.K, gate.dtype)
    capi.call("caifx_qlinear_grouped_backward_input_swiglu", len(gw_down.weights), _ptr(offsets), rows, gw_down.N, gw_down.K,
              _ptr(dy), CODE_OF[dy.dtype], compute_dtype, _ptr(gw_down.wq_ptrs), gw_down.w_kind, _ptr(gw_down.scales_ptrs),
              gw_down.scale_period, gw_down.group_size, _ptr(gate), _ptr(up), _ptr(grad_gate), _ptr(grad_up),
              CODE_OF[gate.dtype], _stream())
    return grad_gate, grad_up


# ------------------------------------------------------------------ element-wise
def _ew(name, n_in, a, b=None, out=None):
    _need_cuda(a, b, out)
    if out is None:
        out = torch.empty_like(a)
    elif out.dtype != a.dtype or out.numel() != a.numel() or not out.is_contiguous():
        raise ValueError("out must be a contiguous tensor of the input's dtype and size")
    dt = CODE_OF[a.dtype]
    if n_in == 1:
        capi.call(name, _ptr(a), _ptr(out), a.numel(), dt, _stream())
    else:
        capi.call(name, _ptr(a), _ptr(b), _ptr(out), a.numel(), dt, _stream())
    return out


def silu(x):
    return _ew("caifx_silu", 1, x)


def silu_backward(x, grad_out):
    return _ew("caifx_silu_backward", 2, x, grad_out)


def multiply(a, b):
    return _ew("caifx_multiply", 2, a, b)


def add(a, b):
    return _ew("caifx_add", 2, a, b)


def silu_multiply(gate, up, out=None):
    return _ew("caifx_silu_multiply", 2, gate, up, out)


def swiglu_backward(gate, up, grad_hidden, out_gate=None, out_up=None):
    """(grad_gate, grad_up) of hidden = silu(gate) * up in one pass, bit-identical to
    multiply(grad_hidden, silu(gate)) and silu_backward(gate, multiply(grad_hidden, up))."""
    _need_cuda(gate, up, grad_hidden)
    assert gate.shape == up.shape == grad_hidden.shape and gate.dtype == up.dtype == grad_hidden.dtype
    grad_gate = torch.empty_like(gate) if out_gate is None else out_gate
    grad_up = torch.empty_like(gate) if out_up is None else out_up
    capi.call("caifx_swiglu_backward", _ptr(gate), _ptr(up), _ptr(grad_hidden), _ptr(grad_gate), _ptr(grad_up),
              gate.numel(), CODE_OF[gate.dtype], _stream())
    return grad_gate, grad_up


# ------------------------------------------------------------------ MoE token routing
def moe_build_dispatch_map(expert_indices, num_experts, capacity_per_expert=0):
    """(dispatch_map [T, top_k] int32, expert_offsets [E+1] int32), built on the device without a host
    round trip; expert_offsets[-1] is the number of assigned rows."""
    _need_cuda(expert_indices)
    assert expert_indices.dtype == torch.int32 and expert_indices.dim() == 2
    T_, top_k = expert_indices.shape
    dmap = torch.empty_like(expert_indices)
    offsets = torch.empty(num_experts + 1, dtype=torch.int32, device=expert_indices.device)
    nb = capi.lib().caifx_moe_dispatch_map_workspace_bytes(T_, top_k, num_experts)
    ws = torch.empty(max(nb, 4 * num_experts), dtype=torch.uint8, device=expert_indices.device)
    capi.call("caifx_moe_build_dispatch_map", _ptr(expert_indices), T_, top_k, num_experts, capacity_per_expert,
              _ptr(dmap), _ptr(offsets), _ptr(ws), ws.numel(), _stream())
    return dmap, offsets


def moe_dispatch(x, expert_indices, dispatch_map, expert_offsets, total_rows, out=None):
    _need_cuda(x, expert_indices, dispatch_map, expert_offsets)
    T_, dim = x.shape
    top_k = expert_indices.shape[1]
    buf = out if out is not None else torch.zeros((total_rows, dim), dtype=x.dtype, device=x.device)
    capi.call("caifx_moe_dispatch", _ptr(x), _ptr(expert_indices), _ptr(dispatch_map), _ptr(expert_offsets), _ptr(buf),
              T_, dim, top_k, expert_offsets.numel() - 1, CODE_OF[x.dtype], _stream())
    return buf


def moe_combine(expert_buffer, expert_indices, expert_weights, dispatch_map, expert_offsets, out=None):
    _need_cuda(expert_buffer, expert_indices, expert_weights, dispatch_map, expert_offsets)
    T_, top_k = expert_indices.shape
    dim = expert_buffer.shape[1]
    y = out if out is not None else torch.empty((T_, dim), dtype=expert_buffer.dtype, device=expert_buffer.device)
    capi.call("caifx_moe_combine", _ptr(expert_buffer), _ptr(expert_indices), _ptr(expert_weights), _ptr(dispatch_map),
              _ptr(expert_offsets), _ptr(y), T_, dim, top_k, expert_offsets.numel() - 1, CODE_OF[expert_buffer.dtype],
              _stream())
    return y


def moe_combine_backward_grad_expert(grad_output, expert_indices, expert_weights, dispatch_map, expert_offsets,
                                     total_rows, out=None):
    _need_cuda(grad_output, expert_indices, expert_weights, dispatch_map, expert_offsets)
    T_, dim = grad_output.shape
    top_k = expert_indices.shape[1]
    gb = out if out is not None else torch.zeros((total_rows, dim), dtype=grad_output.dtype, device=grad_output.device)
    capi.call("caifx_moe_combine_backward_grad_expert", _ptr(grad_output), _ptr(expert_indices), _ptr(expert_weights),
              _ptr(dispatch_map), _ptr(expert_offsets), _ptr(gb), T_, dim, top_k, expert_offsets.numel() - 1,
              CODE_OF[grad_output.dtype], _stream())
    return gb


def moe_dispatch_backward(grad_expert_buffer, expert_indices, dispatch_map, expert_offsets, out=None):
    _need_cuda(grad_expert_buffer, expert_indices, dispatch_map, expert_offsets)
    T_, top_k = expert_indices.shape
    dim = grad_expert_buffer.shape[1]
    gi = out if out is not None else torch.empty((T_, dim), dtype=grad_expert_buffer.dtype,
                                                 device=grad_expert_buffer.device)
    capi.call("caifx_moe_dispatch_backward", _ptr(grad_expert_buffer), _ptr(expert_indices), _ptr(dispatch_map),
              _ptr(expert_offsets), _ptr(gi), T_, dim, top_k, expert_offsets.numel() - 1,
              CODE_OF[grad_expert_buffer.dtype], _stream())
    return gi


def moe_combine_backward_grad_weights(grad_output, expert_buffer, expert_indices, dispatch_map, expert_offsets):
    _need_cuda(grad_output, expert_buffer, expert_indices, dispatch_map, expert_offsets)
    T_, top_k = expert_indices.shape
    dim = grad_output.shape[1]
    gw = torch.empty((T_, top_k), dtype=grad_output.dtype, device=grad_output.device)
    capi.call("caifx_moe_combine_backward_grad_weights", _ptr(grad_output), _ptr(expert_buffer), _ptr(expert_indices),
              _ptr(dispatch_map), _ptr(expert_offsets), _ptr(gw), T_, dim, top_k, expert_offsets.numel() - 1,
              CODE_OF[grad_output.dtype], _stream())
    return gw
