"""ctypes bindings of include/caifx.h (one Python function per C entry point).

Pointers are passed as integers (``tensor.data_ptr()``), streams as the integer
handle of a HIP stream (``torch.cuda.current_stream().cuda_stream``).  Every
wrapper raises ``CaifxError`` on a non-zero status, which is how the C++ host
layer turns the same codes back into the reference's exceptions.
"""
import ctypes
import os
import subprocess

F32, F16, BF16 = 0, 1, 2
W_INT8, W_INT4_GROUP, W_F32, W_F16, W_BF16 = 0, 1, 2, 3, 4

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libcaifx.so")
CSRC = os.path.join(_HERE, "csrc")

EXPORTS = [
    "caifx_status_string", "caifx_version",
    "caifx_convert_fp32_to_fp16", "caifx_convert_fp16_to_fp32", "caifx_convert_fp32_to_bf16",
    "caifx_convert_bf16_to_fp32", "caifx_convert_fp32_to_int8", "caifx_convert_int8_to_fp32",
    "caifx_quantize_int8_per_tensor", "caifx_dequantize_int8_per_tensor",
    "caifx_quantize_int8_per_channel", "caifx_dequantize_int8_per_channel",
    "caifx_quantize_to_int4", "caifx_dequantize_int4",
    "caifx_qlinear_forward", "caifx_qlinear_backward_input", "caifx_qlinear_workspace_bytes",
    "caifx_qlinear_forward_static", "caifx_static_scratch_prepare", "caifx_probe_mfma_bf16", "caifx_qlinear_grouped_tile_stamps",
    "caifx_qlinear_forward_add", "caifx_qlinear_backward_input_add", "caifx_qlinear_grouped_backward_input_add",
    "caifx_qlinear_grouped_forward", "caifx_qlinear_grouped_backward_input",
    "caifx_qlinear_grouped_workspace_bytes", "caifx_qlinear_grouped_forward_swiglu",
    "caifx_qlinear_grouped_backward_input_swiglu",
    "caifx_silu", "caifx_silu_backward", "caifx_multiply", "caifx_add", "caifx_silu_multiply",
    "caifx_swiglu_backward",
    "caifx_moe_dispatch_map_workspace_bytes", "caifx_moe_build_dispatch_map", "caifx_moe_dispatch",
    "caifx_moe_combine", "caifx_moe_combine_backward_grad_expert", "caifx_moe_combine_backward_grad_weights",
    "caifx_moe_dispatch_backward",
]


class CaifxError(RuntimeError):
    def __init__(self, status, what):
        self.status = status
        super().__init__(f"{what}: caifx status {status} ({status_string(status)})")


def build(jobs=8):
    """Compile every HIP source for gfx950 into caif_amd/lib/libcaifx.so (always recompiles)."""
    subprocess.check_call(["make", "-C", CSRC, "-B", f"-j{jobs}", "all"],
                          stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    return LIB_PATH


_lib = None
_i64, _int, _p, _sz = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t


def lib():
    """The loaded library.  Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(hipcc, gfx950).  caif_amd has no CPU or PyTorch fallback.")
        L = ctypes.CDLL(LIB_PATH)
        L.caifx_status_string.restype = ctypes.c_char_p
        L.caifx_status_string.argtypes = [_int]
        L.caifx_version.restype = _int
        for name in ("caifx_convert_fp32_to_fp16", "caifx_convert_fp16_to_fp32", "caifx_convert_fp32_to_bf16",
                     "caifx_convert_bf16_to_fp32", "caifx_convert_fp32_to_int8", "caifx_convert_int8_to_fp32"):
            getattr(L, name).argtypes = [_p, _p, _i64, _p]
        L.caifx_quantize_int8_per_tensor.argtypes = [_p, _p, _p, _i64, _p]
        L.caifx_dequantize_int8_per_tensor.argtypes = [_p, _p, _p, _i64, _p]
        L.caifx_quantize_int8_per_channel.argtypes = [_p, _p, _p, _int, _int, _p]
        L.caifx_dequantize_int8_per_channel.argtypes = [_p, _p, _p, _int, _int, _p]
        L.caifx_quantize_to_int4.argtypes = [_p, _p, _p, _i64, _int, _p]
        L.caifx_dequantize_int4.argtypes = [_p, _p, _p, _i64, _int, _p]
        gemm = [_i64, _i64, _i64, _p, _int, _int, _p, _int, _p, _i64, _int, _p, _int, _p, _sz, _p]
        L.caifx_qlinear_forward.argtypes = gemm
        L.caifx_qlinear_backward_input.argtypes = gemm
        L.caifx_qlinear_forward_static.argtypes = gemm[:13] + [_p]      # no workspace pair
        L.caifx_qlinear_grouped_tile_stamps.argtypes = [_p, _i64]
        L.caifx_static_scratch_prepare.argtypes = []
        L.caifx_probe_mfma_bf16.argtypes = [_p, _p, _i64, _p, ctypes.POINTER(ctypes.c_int64), _p]
        gemm_add = gemm[:13] + [_p] + gemm[13:]                     # addend after (y, y_dtype)
        L.caifx_qlinear_forward_add.argtypes = gemm_add
        L.caifx_qlinear_backward_input_add.argtypes = gemm_add
        L.caifx_qlinear_workspace_bytes.restype = _sz
        L.caifx_qlinear_workspace_bytes.argtypes = [_i64, _i64, _i64, _int, _int, _int, _int]
        grouped = [_int, _p, _i64, _i64, _i64, _p, _int, _int, _p, _int, _p, _i64, _int, _p, _int, _p, _sz, _p]
        L.caifx_qlinear_grouped_forward.argtypes = grouped
        L.caifx_qlinear_grouped_backward_input.argtypes = grouped
        L.caifx_qlinear_grouped_backward_input_add.argtypes = grouped[:15] + [_p] + grouped[15:]
        L.caifx_qlinear_grouped_forward_swiglu.argtypes = grouped[:13] + [_p, _p, _p, _int, _p]
        L.caifx_qlinear_grouped_backward_input_swiglu.argtypes = grouped[:13] + [_p, _p, _p, _p, _int, _p]
        L.caifx_qlinear_grouped_workspace_bytes.restype = _sz
        L.caifx_qlinear_grouped_workspace_bytes.argtypes = [_int, _i64, _i64, _i64, _int, _int, _int, _int]
        L.caifx_silu.argtypes = [_p, _p, _i64, _int, _p]
        L.caifx_silu_backward.argtypes = [_p, _p, _p, _i64, _int, _p]
        L.caifx_multiply.argtypes = [_p, _p, _p, _i64, _int, _p]
        L.caifx_add.argtypes = [_p, _p, _p, _i64, _int, _p]
        L.caifx_silu_multiply.argtypes = [_p, _p, _p, _i64, _int, _p]
        L.caifx_swiglu_backward.argtypes = [_p, _p, _p, _p, _p, _i64, _int, _p]
        L.caifx_moe_dispatch_map_workspace_bytes.restype = _sz
        L.caifx_moe_dispatch_map_workspace_bytes.argtypes = [_i64, _int, _int]
        L.caifx_moe_build_dispatch_map.argtypes = [_p, _i64, _int, _int, _int, _p, _p, _p, _sz, _p]
        L.caifx_moe_dispatch.argtypes = [_p, _p, _p, _p, _p, _i64, _i64, _int, _int, _int, _p]
        L.caifx_moe_combine.argtypes = [_p, _p, _p, _p, _p, _p, _i64, _i64, _int, _int, _int, _p]
        L.caifx_moe_combine_backward_grad_expert.argtypes = [_p, _p, _p, _p, _p, _p, _i64, _i64, _int, _int, _int, _p]
        L.caifx_moe_combine_backward_grad_weights.argtypes = [_p, _p, _p, _p, _p, _p, _i64, _i64, _int, _int, _int, _p]
        L.caifx_moe_dispatch_backward.argtypes = [_p, _p, _p, _p, _p, _i64, _i64, _int, _int, _int, _p]
        _lib = L
    return _lib


def status_string(status):
    return lib().caifx_status_string(int(status)).decode()


def check(status, what):
    if status != 0:
        raise CaifxError(status, what)


def call(name, *args):
    """Call entry point `name`; raise CaifxError unless it returns CAIFX_OK."""
    check(getattr(lib(), name)(*args), name)
