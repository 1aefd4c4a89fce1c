"""Shared plumbing of the GPU parity tests: numpy <-> device tensors and error metrics."""
import numpy as np
import torch

from caif_amd import torch_ops as T

TORCH_OF = {0: torch.float32, 1: torch.float16, 2: torch.bfloat16}


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def dev_as(values_f32, dtype_code):
    """Device tensor of the given float dtype holding `values_f32` (rounded by torch, RNE)."""
    return torch.from_numpy(np.ascontiguousarray(values_f32, dtype=np.float32)).cuda().to(TORCH_OF[dtype_code])


def host(t):
    return t.detach().float().cpu().numpy() if t.dtype in (torch.float16, torch.bfloat16) else t.detach().cpu().numpy()


def f16_bits(t):
    return t.detach().cpu().view(torch.int16).numpy().view(np.uint16)


def max_rel_err(got, want):
    """max |got - want| / max |want|: the normalisation the reference's own parity tests use
    (tests/test_device_frozen_linear.cpp:154-175)."""
    want = np.asarray(want, np.float64)
    got = np.asarray(got, np.float64)
    denom = np.abs(want).max()
    return float(np.abs(got - want).max() / (denom if denom > 0 else 1.0))


def make_weight(orc, rng, N, K, kind, group=128, std=0.02):
    """Quantise a random fp32 weight with the ORACLE and return (oracle FrozenWeight, device FrozenWeight)."""
    w = rng.normal(0, std, (N, K)).astype(np.float32)
    if kind == "int4":
        p, s = orc.quantize_to_int4(w, group)
        ow = orc.FrozenWeight(p, orc.W_INT4_GROUP, s, N, K, 1, group)
        dw = T.FrozenWeight(dev(p), T.W_INT4_GROUP, dev(s.view(np.float16)), N, K, 1, group)
    elif kind == "int8pc":
        q, s = orc.quantize_int8_per_channel(w.reshape(K, N))   # callers label the buffer [in, out]
        ow = orc.FrozenWeight(q.reshape(-1), orc.W_INT8, s, N, K, N, group)
        dw = T.FrozenWeight(dev(q.reshape(-1)), T.W_INT8, dev(s), N, K, N, group)
    elif kind == "int8pt":
        q, s = orc.quantize_int8_per_tensor(w)
        ow = orc.FrozenWeight(q.reshape(-1), orc.W_INT8, s, N, K, 1, group)
        dw = T.FrozenWeight(dev(q.reshape(-1)), T.W_INT8, dev(s), N, K, 1, group)
    else:   # int8 codes without scales
        q = rng.integers(-127, 128, N * K).astype(np.int8)
        ow = orc.FrozenWeight(q, orc.W_INT8, None, N, K, 1, group)
        dw = T.FrozenWeight(dev(q), T.W_INT8, None, N, K, 1, group)
    return ow, dw
