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


@pytest.mark.parametrize("M,K,N,kind", [(640, 4096, 1024, "int4"), (512, 1024, 4096, "int8pc"), (7, 512, 384, "int4"),
                                        (300, 256, 384, "int8pt")])
@pytest.mark.parametrize("dt", [T.BF16, T.F32, T.F16])
def test_fused_add_equals_cast_then_add(orc, M, K, N, kind, dt):
    # caifx_qlinear_forward_add / _backward_input_add fold the adapter's `base.To(StorageT)` and `Add` into the
    # GEMM's store (the large-M kernel) or run them after it (the other shapes: M = 7 takes a decode kernel):
    # either way the bits are those of the three launches
    rng = np.random.default_rng(M + N)
    ow, dw = make_weight(orc, rng, N, K, kind)
    x = dev_as(rng.normal(0, 1, (M, K)), 2)
    dy = dev_as(rng.normal(0, 1e-2, (M, N)), 2)
    add_y = dev_as(rng.normal(0, 1, (M, N)), dt)
    add_x = dev_as(rng.normal(0, 1e-2, (M, K)), dt)
    cd = T.F16 if dt == T.F16 else T.BF16
    if dt == T.F16:
        x, dy = x.to(torch.float16), dy.to(torch.float16)
    want_y = T.add(T.qlinear_forward(x, dw, cd, dt), add_y)
    want_dx = T.add(T.qlinear_backward_input(dy, dw, cd, dt), add_x)
    got_y = T.qlinear_forward(x, dw, cd, dt, addend=add_y)
    got_dx = T.qlinear_backward_input(dy, dw, cd, dt, addend=add_x)
    assert torch.equal(got_y, want_y) and torch.equal(got_dx, want_dx)


def test_lora_step_with_fused_adds(orc):
    # the adapter's forward and backward with the two Adds folded into the base GEMMs, against the oracle's
    # restatement of the unfused reference sequence
    rng = np.random.default_rng(55)
    M, K, N, rank, alpha = 384, 1024, 1536, 16, 32.0
    ow, dw = make_weight(orc, rng, N, K, "int4")
    x = dev_as(rng.normal(0, 1, (M, K)), 2)
    dy = dev_as(rng.normal(0, 1e-3, (M, N)), 2)
    A = dev_as(rng.normal(0, 0.01, (rank, K)), 2)
    B = dev_as(rng.normal(0, 0.01, (N, rank)), 2)
    scale = alpha / rank
    hidden = (x.float() @ A.float().t()).to(torch.bfloat16)
    lora = ((hidden.float() @ B.float().t()).to(torch.bfloat16).float() * scale).to(torch.bfloat16)
    out = T.qlinear_forward(x, dw, T.BF16, T.BF16, addend=lora)
    gs = (dy.float() * scale).to(torch.bfloat16)
    d_in = ((gs.float() @ B.float()).to(torch.bfloat16).float() @ A.float()).to(torch.bfloat16)
    dx = T.qlinear_backward_input(dy, dw, T.BF16, T.BF16, addend=d_in)
    ref_out, ref_dx, _, _ = _lora_step(x, dy, dw, A, B, alpha)
    assert torch.equal(out, ref_out) and torch.equal(dx, ref_dx)
    want_out, _ = orc.lora_forward(host(x), ow, host(A), host(B), alpha, 2, 2)
    want_dx = orc.lora_backward_input(host(dy), ow, host(A), host(B), alpha, 2, 2)
    assert max_rel_err(host(out), want_out) <= 1e-2
    assert max_rel_err(host(dx), want_dx) <= 1e-2


def test_fused_add_argument_errors():
    from caif_amd import capi
    x = torch.zeros(4, 64, device="cuda", dtype=torch.bfloat16)
    y = torch.zeros(4, 32, device="cuda")
    wq = torch.zeros(32 * 64, device="cuda", dtype=torch.int8)
    L = capi.lib()
    args = (4, 32, 64, x.data_ptr(), T.BF16, T.BF16, wq.data_ptr(), T.W_INT8, None, 1, 0, y.data_ptr(), T.F32)
    assert L.caifx_qlinear_forward_add(*args, None, None, 0, None) == 1          # no addend
    assert L.caifx_qlinear_forward_add(*args, y.data_ptr(), None, 0, None) == 1  # addend aliases the output
