"""GPU parity of the large-M matrix-core dequant-GEMMs (forward and input gradient) against the
CPU oracle.  Tolerances: the north star's 1e-2 (bf16/fp16 compute, fp32 accumulate) relative to
max|ref|; the weights fed to the matrix cores are bit-identical to the oracle's, so the measured
error is the fp32 summation order only and a much tighter bound is asserted as well."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from caif_amd import torch_ops as T                                  # noqa: E402
from gpu_helpers import dev_as, host, make_weight, max_rel_err        # noqa: E402

TOL = 1e-2
TIGHT = 5e-5


def _both(orc, rng, M, N, K, kind, cd=2, xd=2, group=128, rows=None):
    ow, dw = make_weight(orc, rng, N, K, kind, group)
    x = dev_as(rng.normal(0, 1, (M, K)), xd)
    dy = dev_as(rng.normal(0, 1e-3, (M, N)), xd)
    y = host(T.qlinear_forward(x, dw, cd))
    dx = host(T.qlinear_backward_input(dy, dw, cd))
    sel = np.arange(M) if rows is None else rows
    e1 = max_rel_err(y[sel], orc.frozen_linear_forward(host(x)[sel], ow, cd))
    e2 = max_rel_err(dx[sel], orc.frozen_linear_backward(host(dy)[sel], ow, cd))
    assert e1 <= TOL and e2 <= TOL, (M, N, K, kind, e1, e2)
    assert e1 <= TIGHT and e2 <= TIGHT, (M, N, K, kind, e1, e2)


@pytest.mark.parametrize("kind", ["int4", "int8pc", "int8pt", "int8raw"])
def test_single_tile_and_multi_tile(orc, kind):
    rng = np.random.default_rng(3)
    _both(orc, rng, 128, 128, 64, kind)
    _both(orc, rng, 256, 384, 512, kind)


@pytest.mark.parametrize("M,N,K", [(17, 64, 64), (130, 200 * 0 + 192, 160), (300, 320, 1408), (129, 1408, 2048),
                                   (64, 2048, 1408), (1000, 448, 96)])
@pytest.mark.parametrize("kind", ["int4", "int8pc"])
def test_ragged_tiles(orc, M, N, K, kind):
    # rows, columns and (for dX) output columns that do not fill the 128x128 tile
    _both(orc, np.random.default_rng(M + N + K), M, N, K, kind, group=32)


@pytest.mark.parametrize("cd,xd", [(2, 0), (1, 1), (1, 0)])
@pytest.mark.parametrize("kind", ["int4", "int8pc"])
def test_dtype_mixes(orc, kind, cd, xd):
    _both(orc, np.random.default_rng(cd + 5 * xd), 192, 256, 256, kind, cd=cd, xd=xd)


def test_int8_scale_period_not_multiple_of_four(orc):
    # scale period 66 (N=66): the quad fetch of scales is not available, per-element lookup is used
    _both(orc, np.random.default_rng(9), 140, 66 * 0 + 64, 128, "int8pc")
    ow, dw = make_weight(orc, np.random.default_rng(10), 66, 128, "int8pc")
    x = dev_as(np.random.default_rng(11).normal(0, 1, (200, 128)), 2)
    y = host(T.qlinear_forward(x, dw, 2))
    assert max_rel_err(y, orc.frozen_linear_forward(host(x), ow, 2)) <= TIGHT


@pytest.mark.parametrize("group", [32, 64, 256])
def test_int4_group_sizes(orc, group):
    _both(orc, np.random.default_rng(group), 160, 256, 512, "int4", group=group)


@pytest.mark.parametrize("N", [4096, 11008])
def test_config3_prefill_shapes_sampled_rows(orc, N):
    # BASELINE config 3 at full size; the oracle checks 16 sampled rows (it is O(M N K) on the CPU)
    rng = np.random.default_rng(N)
    rows = np.sort(rng.choice(2048, 16, replace=False))
    _both(orc, rng, 2048, N, 4096, "int4", rows=rows)


def test_fused_output_cast(orc):
    rng = np.random.default_rng(12)
    ow, dw = make_weight(orc, rng, 256, 256, "int8pc")
    x = dev_as(rng.normal(0, 1, (200, 256)), 2)
    for yd in (1, 2):
        y = host(T.qlinear_forward(x, dw, 2, yd))
        y32 = host(T.qlinear_forward(x, dw, 2, 0))
        assert np.array_equal(y, orc.round_to_dtype(y32, yd))


def test_linearity_and_adjoint_at_full_size(orc):
    # size-independent properties at BASELINE config 4's shape: f(a x1 + x2) vs a f(x1) + f(x2) is only
    # approximate in bf16, so use exact ones: a zero row gives a zero row, a row scaled by 2 doubles,
    # and <Y, dY> == <X, dX>
    import torch
    rng = np.random.default_rng(13)
    N, K, M = 11008, 4096, 512
    ow, dw = make_weight(orc, rng, N, K, "int4")
    x = dev_as(rng.normal(0, 1, (M, K)), 2)
    x[7] = 0
    x[9] = x[8] * 2
    dy = dev_as(rng.normal(0, 1e-3, (M, N)), 2)
    y = T.qlinear_forward(x, dw, 2)
    dx = T.qlinear_backward_input(dy, dw, 2)
    assert not y[7].any()
    assert torch.equal(y[9], y[8] * 2)
    lhs = (y.double() * dy.double()).sum().item()
    rhs = (x.double() * dx.double()).sum().item()
    assert abs(lhs - rhs) <= 1e-4 * max(abs(lhs), abs(rhs))


@pytest.mark.parametrize("M,N,K", [(40, 640, 2048),      # 5 tiles, 32 steps: 4 parts of 8 forward; dX (16 tiles, 10 steps) unsplit
                                   (130, 1280, 1536),    # 20 tiles, 24 steps: 3 parts of 8
                                   (100, 4096, 4096),    # 32 tiles, 64 steps: 8 parts, forward and dX
                                   (64, 1100, 1088)])    # ragged columns; 17 steps do not divide evenly (2 parts: 9 + 8)
@pytest.mark.parametrize("kind", ["int4", "int8pc", "int8pt"])
def test_shared_reduction_of_few_tiles(orc, M, N, K, kind):
    # few tiles: several workgroups share a tile's reduction through fp32 partial tiles in the caller's workspace;
    # same operands as the plain launch, so the tight bound holds; without a workspace the plain launch runs
    import torch
    rng = np.random.default_rng(M + N + K)
    _both(orc, rng, M, N, K, kind, group=64)
    ow, dw = make_weight(orc, rng, N, K, kind, 64)
    x = dev_as(rng.normal(0, 1, (M, K)), 2)
    add = dev_as(rng.normal(0, 1, (M, N)), 2)
    none = torch.empty(1, dtype=torch.uint8, device="cuda")          # too small: no sharing
    y_split = T.qlinear_forward(x, dw, T.BF16, T.BF16, addend=add)
    y_plain = T.qlinear_forward(x, dw, T.BF16, T.BF16, addend=add, workspace=none)
    base = orc.round_to_dtype(orc.frozen_linear_forward(host(x), ow, 2), 2)
    want = orc.add(base, host(add), 2)
    # bf16 results: the fp32 sums differ in their last bits, which can move the cast's rounding by one ulp of
    # the GEMM result (up to 2^-7 relative to it) before the Add, whose own rounding can then move by one ulp too
    for got in (y_split, y_plain):
        assert np.all(np.abs(host(got) - want) <= 2.0 ** -6 * np.maximum(np.maximum(np.abs(want), np.abs(base)), 1e-2))
