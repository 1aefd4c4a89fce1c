"""GPU parity of forward and input-gradient dequant-GEMMs over awkward shapes, every compute
dtype and BASELINE config 1 (fp32 plumbing case), against the CPU oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from caif_amd import torch_ops as T                                  # noqa: E402
from gpu_helpers import dev_as, host, make_weight, max_rel_err        # noqa: E402

TOL = {0: 1e-4, 1: 1e-2, 2: 1e-2}


def _fwd_bwd(orc, rng, M, N, K, kind, cd, xd, group=128):
    ow, dw = make_weight(orc, rng, N, K, kind, group)
    x = dev_as(rng.normal(0, 1, (M, K)), xd)
    dy = dev_as(rng.normal(0, 1e-3, (M, N)), xd)
    y = host(T.qlinear_forward(x, dw, cd))
    dx = host(T.qlinear_backward_input(dy, dw, cd))
    e1 = max_rel_err(y, orc.frozen_linear_forward(host(x), ow, cd))
    e2 = max_rel_err(dx, orc.frozen_linear_backward(host(dy), ow, cd))
    assert e1 <= TOL[cd] and e2 <= TOL[cd], (M, N, K, kind, cd, xd, e1, e2)
    return y, dx, x, dy


@pytest.mark.parametrize("kind", ["int4", "int8pc", "int8pt", "int8raw"])
@pytest.mark.parametrize("cd", [0, 1, 2])
def test_reference_unit_test_shape(orc, kind, cd):
    # K=16, N=8, M=2: the shape of tests/test_device_frozen_linear.cpp:43-46
    _fwd_bwd(orc, np.random.default_rng(71 + cd), 2, 8, 16, kind, cd, xd=0, group=16)


@pytest.mark.parametrize("M,N,K,group", [(1, 1, 2, 2), (3, 5, 6, 2), (17, 33, 70, 10), (5, 7, 24, 24),
                                         (40, 130, 258, 6)])
@pytest.mark.parametrize("kind", ["int4", "int8pc"])
def test_odd_shapes(orc, M, N, K, group, kind):
    for cd in (0, 2):
        _fwd_bwd(orc, np.random.default_rng(M * N + K), M, N, K, kind, cd, xd=cd, group=group)


def test_config1_fp32_plumbing(orc):
    # BASELINE config 1: K=N=4096, M=16, int8 per-channel, fp32 activations, dY ~ N(0, 1e-3)
    rng = np.random.default_rng(1)
    y, dx, x, dy = _fwd_bwd(orc, rng, 16, 4096, 4096, "int8pc", 0, 0)
    assert y.shape == (16, 4096) and dx.shape == (16, 4096)


def test_adjoint_identity_on_gpu(orc):
    # <Y, dY> == <X, dX> for the same stored weight ties dX's transposed access to the forward's
    rng = np.random.default_rng(2)
    for kind in ("int4", "int8pc"):
        ow, dw = make_weight(orc, rng, 96, 160, kind, 32)
        x = dev_as(rng.normal(0, 1, (9, 160)), 2)
        dy = dev_as(rng.normal(0, 1, (9, 96)), 2)
        y = host(T.qlinear_forward(x, dw, 2)).astype(np.float64)
        dx = host(T.qlinear_backward_input(dy, dw, 2)).astype(np.float64)
        lhs, rhs = (y * host(dy)).sum(), (host(x) * dx).sum()
        assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), abs(rhs))


def test_argument_errors():
    from caif_amd import capi
    import torch
    L = capi.lib()
    x = torch.zeros(4, 16, device="cuda")
    y = torch.zeros(4, 8, device="cuda")
    w = torch.zeros(8 * 16, dtype=torch.int8, device="cuda")
    s = torch.ones(8, device="cuda")
    args = lambda **kw: [kw.get("M", 4), kw.get("N", 8), kw.get("K", 16), kw.get("x", x.data_ptr()), kw.get("xd", 0),
                         kw.get("cd", 0), kw.get("w", w.data_ptr()), kw.get("kind", 0), s.data_ptr(),
                         kw.get("period", 8), kw.get("group", 128), y.data_ptr(), 0, None, 0, None]
    assert L.caifx_qlinear_forward(*args()) == 0
    assert L.caifx_qlinear_forward(*args(M=0)) == 0                  # empty batch: no-op
    assert L.caifx_qlinear_forward(*args(N=0)) == 1
    assert L.caifx_qlinear_forward(*args(x=None)) == 1
    assert L.caifx_qlinear_forward(*args(w=None)) == 1
    assert L.caifx_qlinear_forward(*args(cd=7)) == 1
    assert L.caifx_qlinear_forward(*args(kind=5)) == 1
    assert L.caifx_qlinear_forward(*args(period=0)) == 1
    assert L.caifx_qlinear_forward(*args(kind=1, group=0)) == 1
    assert L.caifx_qlinear_forward(*args(x=x.data_ptr() + 2)) == 5   # misaligned fp32 pointer
    torch.cuda.synchronize()


@pytest.mark.parametrize("seed", range(8))
def test_seeded_random_shapes_cross_every_kernel_boundary(orc, seed):
    # forward and input gradient on shapes drawn around the row counts, reduction lengths and widths at which the
    # dispatcher changes kernels (1/2 rows row-streaming, 3..16 and 17..32 row blocks in one or more reduction slices,
    # the few-row input gradient, tiled GEMM with and without a shared reduction, the shape-agnostic floor for K not a
    # multiple of 64), with every weight kind and compute type
    rng = np.random.default_rng(9000 + seed)
    Ms = [1, 2, 3, 4, 8, 15, 16, 17, 24, 31, 32, 33, 48, 64, 100]
    Ns = [16, 24, 40, 64, 200, 512, 777, 1000, 1536, 2050]
    Ks = [64, 96, 128, 256, 384, 512, 1024, 1280, 2048, 2176, 4096, 4224, 5120]
    for _ in range(8):
        M, N, K = (int(rng.choice(v)) for v in (Ms, Ns, Ks))
        kind = str(rng.choice(["int4", "int8pc", "int8pt", "int8raw"]))
        cd = int(rng.choice([0, 1, 2]))
        xd = int(rng.choice([0, cd]))            # the compute type or fp32 activations
        group = int(rng.choice([32, 128])) if K % 128 == 0 else 32
        _fwd_bwd(orc, rng, M, N, K, kind, cd, xd, group=group)
