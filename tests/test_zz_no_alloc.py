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


def _call_static(x, fw, cd, y, y_dtype):
    M = x.numel() // fw.K
    return capi.lib().caifx_qlinear_forward_static(M, fw.N, fw.K, x.data_ptr(), T.CODE_OF[x.dtype], cd, fw.wq.data_ptr(),
                                                   fw.w_kind, 0 if fw.scales is None else fw.scales.data_ptr(),
                                                   fw.scale_period, fw.group_size, y.data_ptr(), y_dtype,
                                                   torch.cuda.current_stream().cuda_stream)


def _static(x, fw, cd, y_dtype=T.F32):
    """Two identical calls.  Torch's allocator must see nothing on either; the driver's free-memory figure, which
    would show a hipMalloc inside the library, is compared across the second one (the first launch of a kernel makes
    the runtime load its code object onto the GPU, which that figure also sees)."""
    M = x.numel() // fw.K
    y = torch.full((M, fw.N), float("nan"), dtype=T.TORCH_DTYPE[y_dtype], device=x.device)
    before = torch.cuda.memory_allocated()
    first = _call_static(x, fw, cd, y, y_dtype)
    torch.cuda.synchronize()
    kept = y.clone()
    y.fill_(float("nan"))
    torch.cuda.synchronize()
    before2 = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]
    st = _call_static(x, fw, cd, y, y_dtype)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.cuda.memory_allocated() == before2 and before2 - before == kept.numel() * kept.element_size()
    assert st == first
    if st == 0:
        assert torch.equal(y, kept)
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


def test_float_storage_in_the_compute_type_uses_the_static_buffer(orc):
    # bf16 weight, bf16 compute: the tiled kernel's shared reduction; the size query counts only what that cell uses
    rng = np.random.default_rng(53)
    N = K = 2048
    w = torch.from_numpy(rng.normal(0, 0.05, (N, K)).astype(np.float32)).cuda().to(torch.bfloat16).contiguous()
    dw = T.FrozenWeight(w.reshape(-1), T.W_BF16, None, N, K)
    for M in (128, 48):
        need = _need(M, dw, 2, 2)
        assert 0 < need <= SCRATCH_BYTES
        x = dev_as(rng.normal(0, 1, (M, K)), 2)
        st, y = _static(x, dw, 2)
        assert st == 0, capi.status_string(st)
        assert torch.equal(y, T.qlinear_forward(x, dw, 2))
        ref = x.float() @ w.float().T
        assert max_rel_err(host(y), host(ref)) <= 2e-5
    # fp32 storage with a 16-bit compute type runs on the fp32 matrix-core kernel: the query reports that kernel's need only
    w32 = T.FrozenWeight(w.float().reshape(-1), T.W_F32, None, N, K)
    assert _need(128, w32, 2, 2) <= SCRATCH_BYTES
    st, y = _static(dev_as(rng.normal(0, 1, (128, K)), 2), w32, 2)
    assert st == 0, capi.status_string(st)


def test_prepare_then_capture_into_a_graph(orc):
    # the address lookup happens before the capture; the captured call replays with the bits of the eager call
    rng = np.random.default_rng(59)
    N = K = 2048
    ow, dw = make_weight(orc, rng, N, K, "int4")
    assert capi.lib().caifx_static_scratch_prepare() == 0
    x = dev_as(rng.normal(0, 1, (64, K)), 2)
    y = torch.empty(64, N, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            st = capi.lib().caifx_qlinear_forward_static(64, N, K, x.data_ptr(), T.BF16, T.BF16, dw.wq.data_ptr(), dw.w_kind,
                                                         dw.scales.data_ptr(), dw.scale_period, dw.group_size, y.data_ptr(),
                                                         T.F32, side.cuda_stream)
    assert st == 0
    torch.cuda.synchronize()
    for rep in range(3):
        x.copy_(dev_as(rng.normal(0, 1, (64, K)), 2))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, T.qlinear_forward(x, dw, 2)), rep
