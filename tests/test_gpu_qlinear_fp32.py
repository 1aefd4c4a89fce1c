"""GPU parity of the fp32 compute type (ComputeT = float of CAIF_DeviceFrozenLinear, the reference's Accuracy_e
matmul mode) on the fp32 matrix-core kernel: forward (src/caif_device_frozen_linear.cpp:382-524) and input gradient
(:528-660) against the oracle, which accumulates in fp64.  Tolerance: 1e-4 of max|ref| (the north star's fp32
bar); what is measured is ~1e-6."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from caif_amd import torch_ops as T                                  # noqa: E402
from gpu_helpers import dev_as, host, make_weight, max_rel_err        # noqa: E402

TOL = 1e-4


@pytest.mark.parametrize("kind,group", [("int8pc", 128), ("int8pt", 128), ("int8raw", 128), ("int4", 128), ("int4", 32),
                                        ("int4", 16)])
@pytest.mark.parametrize("M,N,K", [(5, 192, 256),       # 32-row tiles, one partial row tile
                                   (70, 160, 96),       # N and K below a column tile; K % 128 != 0 (input gradient)
                                   (300, 416, 512),     # several row tiles, N % 128 != 0
                                   (33, 100, 64),       # N % 32 != 0: the input gradient takes the shape-agnostic kernel
                                   (100, 256, 512),     # 32 x 32 split tiles, four row tiles (the last one partial)
                                   (70, 384, 2048)])    # ... with two workgroups sharing each tile's reduction (forward)
def test_fp32_compute_forward_and_input_gradient(orc, kind, group, M, N, K):
    rng = np.random.default_rng(M * 1000 + N + K + group)
    if kind == "int4" and (N * K) % group:
        pytest.skip("whole groups only")
    ow, dw = make_weight(orc, rng, N, K, kind, group, std=0.02 if kind != "int8raw" else 1.0)
    for xdt in (0, 2, 1):
        x = dev_as(rng.normal(0, 1, (M, K)), xdt)
        dy = dev_as(rng.normal(0, 1e-3, (M, N)), xdt)
        y = host(T.qlinear_forward(x, dw, T.F32))
        dx = host(T.qlinear_backward_input(dy, dw, T.F32))
        assert max_rel_err(y, orc.frozen_linear_forward(host(x), ow, orc.F32)) <= TOL, (kind, xdt)
        assert max_rel_err(dx, orc.frozen_linear_backward(host(dy), ow, orc.F32)) <= TOL, (kind, xdt)


def test_fp32_compute_one_hot_reads_single_weights(orc):
    # a one-hot activation row returns one weight column (forward) / one weight row (input gradient) exactly:
    # pins the operand layout, the scale index (period N with K mod N != 0) and the tile edges
    rng = np.random.default_rng(8)
    N, K, M = 224, 160, 40
    for kind in ("int8pc", "int4"):
        ow, dw = make_weight(orc, rng, N, K, kind, 32)
        x = np.zeros((M, K), np.float32)
        ks = rng.integers(0, K, M)
        x[np.arange(M), ks] = 1.0
        y = host(T.qlinear_forward(dev_as(x, 0), dw, T.F32))
        want = orc.frozen_linear_forward(x, ow, orc.F32)
        assert np.array_equal(y, want.astype(np.float32)), kind
        dy = np.zeros((M, N), np.float32)
        ns = rng.integers(0, N, M)
        dy[np.arange(M), ns] = 1.0
        dx = host(T.qlinear_backward_input(dev_as(dy, 0), dw, T.F32))
        wantb = orc.frozen_linear_backward(dy, ow, orc.F32)
        assert np.array_equal(dx, wantb.astype(np.float32)), kind


def test_fp32_compute_config0_shape_and_large_m(orc):
    # the baseline's first configuration (K = N = 4096, fp32 X[16, 4096], int8 per-channel) and a 2048-row problem on
    # 128-row tiles, the latter on sampled rows
    rng = np.random.default_rng(21)
    N = K = 4096
    ow, dw = make_weight(orc, rng, N, K, "int8pc")
    x = dev_as(rng.normal(0, 1, (16, K)), 0)
    dy = dev_as(rng.normal(0, 1e-3, (16, N)), 0)
    assert max_rel_err(host(T.qlinear_forward(x, dw, T.F32)), orc.frozen_linear_forward(host(x), ow, orc.F32)) <= TOL
    assert max_rel_err(host(T.qlinear_backward_input(dy, dw, T.F32)), orc.frozen_linear_backward(host(dy), ow, orc.F32)) <= TOL
    M = 2048
    xb = dev_as(rng.normal(0, 1, (M, K)), 0)
    dyb = dev_as(rng.normal(0, 1e-3, (M, N)), 0)
    rows = np.sort(rng.choice(M, 24, replace=False))
    y = host(T.qlinear_forward(xb, dw, T.F32))[rows]
    dx = host(T.qlinear_backward_input(dyb, dw, T.F32))[rows]
    assert max_rel_err(y, orc.frozen_linear_forward(host(xb)[rows], ow, orc.F32)) <= TOL
    assert max_rel_err(dx, orc.frozen_linear_backward(host(dyb)[rows], ow, orc.F32)) <= TOL
    # bf16 results round the fp32 result once
    yb = T.qlinear_forward(xb, dw, T.F32, y_dtype=T.BF16)
    import torch
    assert torch.equal(yb[rows], T.qlinear_forward(xb, dw, T.F32)[rows].to(torch.bfloat16))


@pytest.mark.parametrize("kind,group", [("int8pc", 128), ("int8pt", 128), ("int4", 32)])
@pytest.mark.parametrize("counts", [[130, 0, 1, 257, 64, 5],        # mean below 128 rows: 32-row tiles
                                    [300, 129, 0, 256, 128, 200]])  # mean above: 128-row tiles, partial last tiles
def test_fp32_compute_grouped_segments(orc, kind, group, counts):
    # the MoE wrapper's ComputeT = float cells: expert segments on the fp32 matrix-core kernel; rows past the
    # last segment are not written
    from gpu_helpers import dev
    from caif_amd import torch_ops as TT
    import torch
    rng = np.random.default_rng(sum(counts) + group)
    E, N, K = len(counts), 192, 256
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    total = int(offsets[-1])
    pairs = [make_weight(orc, rng, N, K, kind, group) for _ in range(E)]
    gw = TT.GroupedFrozenWeights([p[1] for p in pairs])
    x = dev_as(rng.normal(0, 1, (total + 3, K)), 0)
    dy = dev_as(rng.normal(0, 1e-2, (total + 3, N)), 0)
    y = torch.full((total + 3, N), 7.0, device="cuda")
    dx = torch.full((total + 3, K), 5.0, device="cuda")
    TT.qlinear_grouped_forward(x, dev(offsets), gw, TT.F32, TT.F32, out=y)
    TT.qlinear_grouped_backward_input(dy, dev(offsets), gw, TT.F32, TT.F32, out=dx)
    yh, dxh, xh, dyh = host(y), host(dx), host(x), host(dy)
    for e in range(E):
        lo, hi = offsets[e], offsets[e + 1]
        if hi == lo:
            continue
        assert max_rel_err(yh[lo:hi], orc.frozen_linear_forward(xh[lo:hi], pairs[e][0], orc.F32)) <= TOL, (kind, e)
        assert max_rel_err(dxh[lo:hi], orc.frozen_linear_backward(dyh[lo:hi], pairs[e][0], orc.F32)) <= TOL, (kind, e)
    assert np.all(yh[total:] == 7.0) and np.all(dxh[total:] == 5.0)
