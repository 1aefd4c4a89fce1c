"""caifx_qlinear_forward_static: the forward for callers that cannot allocate, whose shared-reduction
partial tiles live in a buffer inside the library's device image.  It must return the bits of
caifx_qlinear_forward called with a caller workspace (same kernels, same order of additions), on
two calls in a row with the second one smaller (the buffer keeps the first call's contents), it
must not allocate, and it must refuse problems whose partial tiles do not fit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from caif_amd import capi, torch_ops as T                            # noqa: E402
from gpu_helpers import dev_as, host, make_weight, max_rel_err        # noqa: E402

SCRATCH_BYTES = 8 << 20
ERR_SCRATCH_EXCEEDED = 6


def _static(x, fw, cd, y_dtype=T.F32):
    M = x.numel() // fw.K
    y = torch.full((M, fw.N), float("nan"), dtype=T.TORCH_DTYPE[y_dtype], device=x.device)
    before = torch.cuda.memory_allocated()
    st = capi.lib().caifx_qlinear_forward_static(M, fw.N, fw.K, x.data_ptr(), T.CODE_OF[x.dtype], cd, fw.wq.data_ptr(),
                                                 fw.w_kind, 0 if fw.scales is None else fw.scales.data_ptr(),
                                                 fw.scale_period, fw.group_size, y.data_ptr(), y_dtype,
                                                 torch.cuda.current_stream().cuda_stream)
    assert torch.cuda.memory_allocated() == before
    return st, y


def _need(M, fw, xd, cd):
    return capi.lib().caifx_qlinear_workspace_bytes(M, fw.N, fw.K, xd, cd, fw.w_kind, 0)


@pytest.mark.parametrize("kind,cd,xd", [("int4", 2, 2), ("int8pc", 2, 2), ("int8pc", 0, 0)])
def test_two_calls_second_smaller_match_the_workspace_form(orc, kind, cd, xd):
    rng = np.random.default_rng(41)
    N = K = 2048
    ow, dw = make_weight(orc, rng, N, K, kind)
    # 16-bit compute shares a tile's reduction from 33 rows on, the fp32 compute type up to 128 rows
    sizes = (128, 48) if cd != 0 else (64, 16)
    for M in sizes:
        assert 0 < _need(M, dw, xd, cd) <= SCRATCH_BYTES, "the case must exercise the scratch buffer"
        x = dev_as(rng.normal(0, 1, (M, K)), xd)
        st, y = _static(x, dw, cd)
        assert st == 0, capi.status_string(st)
        want = T.qlinear_forward(x, dw, cd)          # allocates a workspace of the queried size
        torch.cuda.synchronize()
        assert torch.equal(y, want), (kind, cd, M)
        tol = 1e-4 if cd == 0 else 1e-2
        assert max_rel_err(host(y), orc.frozen_linear_forward(host(x), ow, cd)) <= tol


@pytest.mark.parametrize("kind", ["int4", "int8pc"])
def test_long_reduction_slices_meet_in_the_static_buffer(orc, kind):
    # K > 4096 with up to 16 rows, K > 2048 with 17..32: the decode kernel's slices of the reduction use the same buffer
    rng = np.random.default_rng(47)
    N, K = 1024, 8192
    ow, dw = make_weight(orc, rng, N, K, kind)
    for M in (16, 24, 5, 32):
        assert 0 < _need(M, dw, 2, 2) <= SCRATCH_BYTES
        x = dev_as(rng.normal(0, 1, (M, K)), 2)
        st, y = _static(x, dw, 2)
        assert st == 0, capi.status_string(st)
        want = T.qlinear_forward(x, dw, 2)
        torch.cuda.synchronize()
        assert torch.equal(y, want), (kind, M)
        assert max_rel_err(host(y), orc.frozen_linear_forward(host(x), ow, 2)) <= 1e-2


def test_shapes_without_scratch_run_and_oversized_ones_are_refused(orc):
    rng = np.random.default_rng(43)
    ow, dw = make_weight(orc, rng, 4096, 4096, "int4")
    # one row (the decode kernel ignores the scratch) and 1024 rows (enough tiles: nothing is shared)
    assert _need(1024, dw, 2, 2) == 0
    for M in (1, 1024):
        x = dev_as(rng.normal(0, 1, (M, 4096)), 2)
        st, y = _static(x, dw, 2)
        assert st == 0 and torch.equal(y, T.qlinear_forward(x, dw, 2)), M
    # 128 rows x 4096 columns in 8 parts: 16 MiB of partial tiles, more than the buffer holds
    x = dev_as(rng.normal(0, 1, (128, 4096)), 2)
    assert _need(128, dw, 2, 2) > SCRATCH_BYTES
    st, y = _static(x, dw, 2)
    assert st == ERR_SCRATCH_EXCEEDED
    assert "scratch" in capi.status_string(st)
    assert bool(torch.isnan(y).all()), "a refused call must not launch anything"
