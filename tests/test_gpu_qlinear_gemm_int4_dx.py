"""GPU parity of the int4 input-gradient GEMM at large shapes (whole and ragged row tiles, reductions of 4 to 172
steps, both compute types, every result type, the fused add) against the CPU oracle's restatement of
CAIF_DeviceFrozenLinear::BackwardImpl (src/caif_device_frozen_linear.cpp:528-660).  The operand tile the kernel
builds holds the oracle's dequantise-then-cast weight bit for bit, so what is measured is the fp32 summation
order only: the north star's 1e-2 is asserted, and a bound two hundred times tighter."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from caif_amd import torch_ops as T                                  # noqa: E402
from gpu_helpers import dev_as, host, make_weight, max_rel_err        # noqa: E402

TOL = 1e-2
TIGHT = 5e-5


def _backward(orc, rng, M, N, K, cd=2, yd=0, rows=16):
    ow, dw = make_weight(orc, rng, N, K, "int4", 128)
    dy = dev_as(rng.normal(0, 1e-3, (M, N)), cd)
    dx = host(T.qlinear_backward_input(dy, dw, cd, yd))
    sel = np.sort(rng.choice(M, min(rows, M), replace=False))
    sel[-1] = M - 1
    want = orc.frozen_linear_backward(host(dy)[sel], ow, cd)
    if yd != 0:
        want = orc.round_to_dtype(want, yd)
    return max_rel_err(dx[sel], want)


@pytest.mark.parametrize("M,N,K", [(2048, 256, 4096),        # four steps
                                   (2048, 448, 4096),        # seven steps: an odd count for the double-buffered loop
                                   (1024, 1024, 8192),       # 16 steps
                                   (2048, 4096, 4096),       # BASELINE configs[2] weight
                                   (4096, 2816, 2048)])      # 44 steps, other aspect ratio
def test_full_tiles(orc, M, N, K):
    err = _backward(orc, np.random.default_rng(M + N + K), M, N, K)
    assert err <= TOL and err <= TIGHT, (M, N, K, err)


@pytest.mark.parametrize("M", [4001, 16500])
def test_ragged_rows(orc, M):
    # the last row tile has 33 / 116 rows; columns always come in whole tiles (K % 256 == 0)
    K = 4096 if M == 4001 else 512
    err = _backward(orc, np.random.default_rng(M), M, 768, K)
    assert err <= TOL and err <= TIGHT, (M, err)


@pytest.mark.parametrize("cd", [1, 2])
@pytest.mark.parametrize("yd", [0, 1, 2])
def test_compute_and_result_types(orc, cd, yd):
    err = _backward(orc, np.random.default_rng(10 * cd + yd), 2048, 1024, 4096, cd=cd, yd=yd)
    bound = TIGHT if yd == 0 else (1e-3 if yd == 1 else 8e-3)
    assert err <= bound, (cd, yd, err)


@pytest.mark.parametrize("yd", [0, 2])
def test_fused_add_equals_cast_then_add(orc, yd):
    rng = np.random.default_rng(177 + yd)
    M, N, K = 2048, 768, 4096
    ow, dw = make_weight(orc, rng, N, K, "int4", 128)
    dy = dev_as(rng.normal(0, 1e-3, (M, N)), 2)
    add = dev_as(rng.normal(0, 1e-3, (M, K)), yd)
    fused = T.qlinear_backward_input(dy, dw, 2, yd, addend=add)
    plain = T.qlinear_backward_input(dy, dw, 2, yd)
    want = (plain.float() + add.float()).to(plain.dtype)
    assert torch.equal(fused, want)


def test_one_hot_rows_return_single_weight_rows(orc):
    # dY = e_n: row m of dX is row n of the dequantised weight, exactly; every n of a step, every wave's rows
    rng = np.random.default_rng(15)
    M, N, K = 2048, 512, 4096
    ow, dw = make_weight(orc, rng, N, K, "int4", 128)
    ns = rng.choice(N, M, replace=True)
    ns[:N] = np.arange(N)
    dy = np.zeros((M, N), np.float32)
    dy[np.arange(M), ns] = 1.0
    dx = host(T.qlinear_backward_input(dev_as(dy, 2), dw, 2))
    wd = np.asarray(ow.compute_weight(2)).reshape(N, K)
    assert np.array_equal(dx, wd[ns])


def test_adjoint_with_the_forward(orc):
    # <X W^T, dY> == <X, dY W> at full size (BASELINE configs[3]'s linear), both through the int4 kernels
    rng = np.random.default_rng(16)
    M, N, K = 4096, 11008, 4096
    ow, dw = make_weight(orc, rng, N, K, "int4", 128)
    x = dev_as(rng.normal(0, 1, (M, K)), 2)
    dy = dev_as(rng.normal(0, 1e-3, (M, N)), 2)
    y = T.qlinear_forward(x, dw, 2)
    dx = T.qlinear_backward_input(dy, dw, 2)
    lhs = (y.double() * dy.double()).sum().item()
    rhs = (x.double() * dx.double()).sum().item()
    assert abs(lhs - rhs) <= 1e-4 * max(abs(lhs), abs(rhs))
