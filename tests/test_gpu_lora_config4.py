"""BASELINE config 4: a LoRA fine-tune step through a frozen int4 base (Llama-2-7B FFN shape,
K=4096, N=11008, group 128, M=4096 bf16 tokens, rank 16, alpha 32, B = 0).

The adapter's own small GEMMs belong to the caller (trainable weights, the reference runs them
through CAIF_Ops::MatMul*); here torch computes them.  What is under test is the frozen base that
the adapter calls into: forward with the output cast fused, the transposed input gradient, and the
reference's identities  B = 0  =>  LoRA(x) == base(x)  (tests/test_device_lora_adapter.cpp:371-443)
and  B = 0  =>  dX == base dX."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from caif_amd import torch_ops as T                                  # noqa: E402
from gpu_helpers import dev_as, host, make_weight, max_rel_err        # noqa: E402


def _lora_step(x, dy, dw, A, B, alpha):
    rank = A.shape[0]
    scale = alpha / rank
    base = T.qlinear_forward(x, dw, T.BF16, T.BF16)                          # base(x).To(bf16), fused
    hidden = (x.float() @ A.float().t()).to(torch.bfloat16)
    lora = (hidden.float() @ B.float().t()).to(torch.bfloat16)
    lora = (lora.float() * scale).to(torch.bfloat16)
    out = T.add(base, lora)
    gs = (dy.float() * scale).to(torch.bfloat16)
    d_hidden = (gs.float() @ B.float()).to(torch.bfloat16)
    d_in = (d_hidden.float() @ A.float()).to(torch.bfloat16)
    gbase = T.qlinear_backward_input(dy, dw, T.BF16, T.BF16)
    return out, T.add(gbase, d_in), base, gbase


def test_config4_full_size(orc):
    rng = np.random.default_rng(4)
    M, K, N, rank, alpha = 4096, 4096, 11008, 16, 32.0
    ow, dw = make_weight(orc, rng, N, K, "int4")
    x = dev_as(rng.normal(0, 1, (M, K)), 2)
    dy = dev_as(rng.normal(0, 1e-3, (M, N)), 2)
    A_h = rng.normal(0, 0.01, (rank, K)).astype(np.float32)
    A = dev_as(A_h, 2)
    B = torch.zeros(N, rank, dtype=torch.bfloat16, device="cuda")
    out, dx, base, gbase = _lora_step(x, dy, dw, A, B, alpha)
    # B = 0 identities, exact
    assert torch.equal(out, base)
    assert torch.equal(dx, gbase)
    # parity of sampled rows against the oracle's restatement of the adapter
    rows = np.sort(rng.choice(M, 12, replace=False))
    xo, dyo = host(x)[rows], host(dy)[rows]
    want_out, _ = orc.lora_forward(xo, ow, host(A), np.zeros((N, rank), np.float32), alpha, 2, 2)
    want_dx = orc.lora_backward_input(dyo, ow, host(A), np.zeros((N, rank), np.float32), alpha, 2, 2)
    e_out = max_rel_err(host(out)[rows], want_out)
    e_dx = max_rel_err(host(dx)[rows], want_dx)
    assert e_out <= 1e-2 and e_dx <= 1e-2, (e_out, e_dx)
    # dX of the base alone, fp32 output (the frozen layer's own contract), tight
    dx32 = host(T.qlinear_backward_input(dy, dw, T.BF16, T.F32))[rows]
    assert max_rel_err(dx32, orc.frozen_linear_backward(dyo, ow, 2)) <= 5e-5


def test_lora_with_nonzero_b_small(orc):
    rng = np.random.default_rng(5)
    M, K, N, rank, alpha = 160, 256, 384, 16, 32.0
    ow, dw = make_weight(orc, rng, N, K, "int4")
    x = dev_as(rng.normal(0, 1, (M, K)), 2)
    dy = dev_as(rng.normal(0, 1e-3, (M, N)), 2)
    A = dev_as(rng.normal(0, 0.01, (rank, K)), 2)
    B = dev_as(rng.normal(0, 0.01, (N, rank)), 2)
    out, dx, _, _ = _lora_step(x, dy, dw, A, B, alpha)
    want_out, _ = orc.lora_forward(host(x), ow, host(A), host(B), alpha, 2, 2)
    want_dx = orc.lora_backward_input(host(dy), ow, host(A), host(B), alpha, 2, 2)
    assert max_rel_err(host(out), want_out) <= 1e-2
    assert max_rel_err(host(dx), want_dx) <= 1e-2
