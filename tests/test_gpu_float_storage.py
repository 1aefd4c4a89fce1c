"""GPU parity of the float-storage cells of the frozen linear (weight kept undequantised in fp32, fp16 or bf16;
src/caif_device_frozen_linear.cpp:301-318 and the .To(target) branch): forward and input gradient against the CPU
oracle for the nine (storage, compute) cells, plain and over expert segments.

Tolerances: the fp32 compute type is held to the north star's 1e-4; with a 16-bit compute type both operands
are rounded to it exactly as the oracle rounds them and the sums are fp32, so only the summation order differs."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from caif_amd import torch_ops as T                                  # noqa: E402
from gpu_helpers import TORCH_OF, dev, dev_as, host, max_rel_err      # noqa: E402

KIND = {0: T.W_F32, 1: T.W_F16, 2: T.W_BF16}


def _weight(orc, rng, N, K, sd):
    w = rng.normal(0, 0.05, (N, K)).astype(np.float32)
    wt = torch.from_numpy(w).cuda().to(TORCH_OF[sd]).contiguous()
    stored = wt.cpu().numpy() if sd == 0 else wt.cpu().view(torch.int16).numpy().view(np.uint16)
    okind = {0: orc.W_F32, 1: orc.W_F16, 2: orc.W_BF16}[sd]
    return orc.FrozenWeight(stored, okind, None, N, K), T.FrozenWeight(wt.reshape(-1), KIND[sd], None, N, K)


@pytest.mark.parametrize("sd", [0, 1, 2])
@pytest.mark.parametrize("cd", [0, 1, 2])
@pytest.mark.parametrize("M,N,K", [(2, 8, 16), (16, 48, 64), (200, 256, 512), (5, 33, 40), (130, 4096, 96)])
def test_float_storage_forward_backward(orc, sd, cd, M, N, K):
    rng = np.random.default_rng(100 * sd + 10 * cd + M)
    ow, dw = _weight(orc, rng, N, K, sd)
    x = dev_as(rng.normal(0, 1, (M, K)), 2 if cd == 2 else (1 if cd == 1 else 0))
    dy = dev_as(rng.normal(0, 1e-2, (M, N)), 2 if cd == 2 else (1 if cd == 1 else 0))
    bound = 1e-4 if cd == 0 else 2e-5
    y = host(T.qlinear_forward(x, dw, cd))
    assert max_rel_err(y, orc.frozen_linear_forward(host(x), ow, cd)) <= bound
    dx = host(T.qlinear_backward_input(dy, dw, cd))
    assert max_rel_err(dx, orc.frozen_linear_backward(host(dy), ow, cd)) <= bound


@pytest.mark.parametrize("sd", [1, 2])
@pytest.mark.parametrize("M,N,K", [(2048, 1024, 512),      # full 256-row tiles forward, 128-row tiles for the gradient
                                   (300, 1100, 1408),      # ragged rows and columns; the gradient reduces over 1100: other kernel
                                   (64, 2048, 2048)])      # few tiles: workgroups share each tile's reduction
def test_same_type_16bit_storage_on_the_16bit_matrix_cores(orc, sd, M, N, K):
    # weight stored in the compute type (bf16 / bf16, fp16 / fp16): the tiled kernel with the dequantisation compiled
    # out, src/caif_device_frozen_linear.cpp:301-318 (same-dtype view) + :465-509; fp32 and storage-type results,
    # and the fused Add of a LoRA-style branch
    rng = np.random.default_rng(1000 * sd + M)
    ow, dw = _weight(orc, rng, N, K, sd)
    x = dev_as(rng.normal(0, 1, (M, K)), sd)
    dy = dev_as(rng.normal(0, 1e-2, (M, N)), sd)
    sel = np.sort(rng.choice(M, min(M, 24), replace=False))
    y = T.qlinear_forward(x, dw, sd)
    assert max_rel_err(host(y)[sel], orc.frozen_linear_forward(host(x)[sel], ow, sd)) <= 2e-5
    dx = T.qlinear_backward_input(dy, dw, sd)
    assert max_rel_err(host(dx)[sel], orc.frozen_linear_backward(host(dy)[sel], ow, sd)) <= 2e-5
    y16 = T.qlinear_forward(x, dw, sd, sd)
    assert torch.equal(y16, y.to(TORCH_OF[sd]))
    add = dev_as(rng.normal(0, 1, (M, N)), sd)
    fused = T.qlinear_forward(x, dw, sd, sd, addend=add)
    assert torch.equal(fused, (y16.float() + add.float()).to(TORCH_OF[sd]))


def test_float_storage_fp32_is_the_dense_product(orc):
    # storage and compute both fp32: the layout pin of tests/test_device_frozen_linear.cpp:996-1072
    # (W is [output_dim, input_dim], y = x W^T) against torch's own GEMM
    rng = np.random.default_rng(7)
    M, N, K = 32, 64, 128
    w = torch.from_numpy(rng.normal(0, 0.05, (N, K)).astype(np.float32)).cuda()
    x = torch.from_numpy(rng.normal(0, 1, (M, K)).astype(np.float32)).cuda()
    y = T.qlinear_forward(x, T.FrozenWeight(w.reshape(-1), T.W_F32, None, N, K), T.F32)
    want = (x.double() @ w.double().T).float()
    assert max_rel_err(host(y), host(want)) <= 1e-5


@pytest.mark.parametrize("sd,cd", [(2, 2), (0, 0), (1, 2)])
def test_float_storage_over_expert_segments(orc, sd, cd):
    rng = np.random.default_rng(31 + sd)
    E, N, K = 5, 96, 64
    counts = np.array([40, 0, 3, 130, 17])
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    total = int(offsets[-1])
    pairs = [_weight(orc, rng, N, K, sd) for _ in range(E)]
    gw = T.GroupedFrozenWeights([p[1] for p in pairs])
    x = dev_as(rng.normal(0, 1, (total + 2, K)), 2)
    dy = dev_as(rng.normal(0, 1e-2, (total + 2, N)), 2)
    y = host(T.qlinear_grouped_forward(x, dev(offsets), gw, cd))
    dx = host(T.qlinear_grouped_backward_input(dy, dev(offsets), gw, cd))
    bound = 1e-4 if cd == 0 else 2e-5
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi == lo:
            continue
        assert max_rel_err(y[lo:hi], orc.frozen_linear_forward(host(x)[lo:hi], pairs[e][0], cd)) <= bound
        assert max_rel_err(dx[lo:hi], orc.frozen_linear_backward(host(dy)[lo:hi], pairs[e][0], cd)) <= bound
    assert not y[total:].any() and not dx[total:].any()


def test_float_storage_is_refused_by_the_gated_stores():
    E, N, K = 2, 64, 64
    w = [T.FrozenWeight(torch.zeros(N * K, dtype=torch.bfloat16, device="cuda"), T.W_BF16, None, N, K) for _ in range(E)]
    gw = T.GroupedFrozenWeights(w)
    x = torch.zeros(8, K, dtype=torch.bfloat16, device="cuda")
    gate = torch.zeros(8, N, dtype=torch.bfloat16, device="cuda")
    off = torch.tensor([0, 4, 8], dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="unsupported"):
        T.qlinear_grouped_forward_swiglu(x, off, gw, gate, T.BF16)
