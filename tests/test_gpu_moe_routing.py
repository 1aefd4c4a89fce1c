"""GPU parity of the MoE routing kernels (dispatch map, dispatch, combine, their backward passes) against
the CPU oracle, through the C ABI.  Integer results and row copies are bit exact; the weighted sums are one
fused multiply-add per k in fp32 in both, so they are bit exact too."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from caif_amd import torch_ops as T                                  # noqa: E402
from gpu_helpers import dev, dev_as, host                             # noqa: E402


def _case(rng, Tk, top_k, E, bad=0):
    idx = rng.integers(0, E, (Tk, top_k)).astype(np.int32)
    for _ in range(bad):
        idx[rng.integers(0, Tk), rng.integers(0, top_k)] = rng.choice([-1, E, E + 7])
    return idx


@pytest.mark.parametrize("Tk,top_k,E,cap", [(1, 1, 1, 0), (37, 3, 5, 0), (300, 6, 64, 0), (257, 2, 70, 0),
                                            (128, 4, 8, 9), (64, 1, 3, 5), (4096, 6, 64, 0), (1000, 8, 130, 40),
                                            # past what one workgroup's LDS holds: the launches over a workspace
                                            (16384, 8, 64, 0), (3000, 6, 200, 50), (9000, 4, 64, 500)])
def test_dispatch_map_matches_reference_order(orc, Tk, top_k, E, cap):
    rng = np.random.default_rng(Tk + top_k + E)
    idx = _case(rng, Tk, top_k, E, bad=3 if Tk > 10 else 0)
    want_map, want_off, total = orc.moe_build_dispatch_map(idx, E, cap)
    dmap, offsets = T.moe_build_dispatch_map(dev(idx), E, cap)
    assert np.array_equal(offsets.cpu().numpy(), want_off)
    assert np.array_equal(dmap.cpu().numpy(), want_map)
    assert int(offsets[-1]) == total


def test_dispatch_map_empty_batch(orc):
    idx = torch.empty((0, 2), dtype=torch.int32, device="cuda")
    dmap, offsets = T.moe_build_dispatch_map(idx, 4)
    assert offsets.cpu().tolist() == [0, 0, 0, 0, 0] and dmap.numel() == 0


@pytest.mark.parametrize("dtype", [0, 1, 2])
@pytest.mark.parametrize("Tk,top_k,E,dim,cap", [(37, 3, 5, 24, 0), (300, 6, 16, 2048, 0), (90, 2, 4, 37, 11)])
def test_dispatch_combine_and_backward(orc, dtype, Tk, top_k, E, dim, cap):
    rng = np.random.default_rng(Tk * 3 + dim + dtype)
    idx = _case(rng, Tk, top_k, E, bad=2)
    dmap_h, off_h, total = orc.moe_build_dispatch_map(idx, E, cap)
    idx_d = dev(idx)
    dmap, offsets = T.moe_build_dispatch_map(idx_d, E, cap)
    x = dev_as(rng.normal(0, 1, (Tk, dim)), dtype)
    w = dev_as(rng.random((Tk, top_k)), dtype)
    buf = T.moe_dispatch(x, idx_d, dmap, offsets, total)
    assert np.array_equal(host(buf), orc.moe_dispatch(host(x), idx, dmap_h, off_h, E, total, dtype))
    eb = dev_as(rng.normal(0, 1, (total, dim)), dtype)               # stand-in for the expert outputs
    out = T.moe_combine(eb, idx_d, w, dmap, offsets)
    assert np.array_equal(host(out), orc.moe_combine(host(eb), idx, host(w), dmap_h, off_h, E, dtype))
    go = dev_as(rng.normal(0, 1e-2, (Tk, dim)), dtype)
    gb = T.moe_combine_backward_grad_expert(go, idx_d, w, dmap, offsets, total)
    assert np.array_equal(host(gb), orc.moe_combine_backward_grad_expert(host(go), idx, host(w), dmap_h, off_h, E,
                                                                          total, dtype))
    gw = host(T.moe_combine_backward_grad_weights(go, eb, idx_d, dmap, offsets))
    want_gw = orc.moe_combine_backward_grad_weights(host(go), host(eb), idx, dmap_h, off_h, E, dtype)
    # fp32 accumulation in a different (fixed) order than the oracle's fp64 dot: equal to fp32 rounding,
    # plus one unit in the last place of the 16-bit result types
    tol = {0: 1e-5, 1: 2e-3, 2: 1.6e-2}[dtype] * max(np.abs(want_gw).max(), 1e-30)
    assert np.abs(gw - want_gw).max() <= tol and not gw[dmap_h < 0].any()
    gi = T.moe_dispatch_backward(gb, idx_d, dmap, offsets)
    assert np.array_equal(host(gi), orc.moe_dispatch_backward(host(gb), idx, dmap_h, off_h, E, dtype))


def test_full_size_round_trip_properties():
    # BASELINE configs[4] sizes: 4096 tokens, top-6 of 64 experts, dim 2048, bf16.  Size-independent checks:
    # the map is a bijection onto [0, offsets[E]); dispatch followed by combine with weights that sum to one
    # returns every token to bf16 rounding; dispatch_backward of a dispatched tensor is top_k times the token.
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7)
    Tk, top_k, E, dim = 4096, 6, 64, 2048
    idx = torch.randint(0, E, (Tk, top_k), device="cuda", generator=gen, dtype=torch.int32)
    dmap, offsets = T.moe_build_dispatch_map(idx, E)
    total = int(offsets[-1])
    assert total == Tk * top_k
    rows = (offsets[idx.long()] + dmap).flatten().long()
    assert torch.equal(torch.sort(rows).values, torch.arange(total, device="cuda"))
    x = torch.empty(Tk, dim, device="cuda").normal_(0, 1, generator=gen).to(torch.bfloat16)
    buf = T.moe_dispatch(x, idx, dmap, offsets, total)
    assert torch.equal(buf[rows], x.repeat_interleave(top_k, dim=0))
    w = torch.full((Tk, top_k), 1.0 / 8, device="cuda").to(torch.bfloat16)     # exact in bf16; 6/8 of the token
    out = T.moe_combine(buf, idx, w, dmap, offsets)
    assert torch.equal(out, (x.float() * 0.75).to(torch.bfloat16))
    gi = T.moe_dispatch_backward(buf, idx, dmap, offsets)
    assert torch.equal(gi, (x.float() * top_k).to(torch.bfloat16))


def test_argument_errors():
    from caif_amd import capi
    L = capi.lib()
    idx = torch.zeros((4, 2), dtype=torch.int32, device="cuda")
    m = torch.zeros_like(idx)
    off = torch.zeros(4, dtype=torch.int32, device="cuda")
    ws = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    assert L.caifx_moe_build_dispatch_map(idx.data_ptr(), 4, 2, 3, 0, m.data_ptr(), off.data_ptr(), ws.data_ptr(), 4096, None) == 0
    assert L.caifx_moe_build_dispatch_map(idx.data_ptr(), 4, 2, 0, 0, m.data_ptr(), off.data_ptr(), ws.data_ptr(), 4096, None) == 1
    assert L.caifx_moe_build_dispatch_map(idx.data_ptr(), 4, 2, 3, 0, m.data_ptr(), off.data_ptr(), ws.data_ptr(), 8, None) == 3
    assert L.caifx_moe_build_dispatch_map(None, 4, 2, 3, 0, m.data_ptr(), off.data_ptr(), ws.data_ptr(), 4096, None) == 1
    x = torch.zeros((4, 8), device="cuda")
    buf = torch.zeros((8, 8), device="cuda")
    assert L.caifx_moe_dispatch(x.data_ptr(), idx.data_ptr(), m.data_ptr(), off.data_ptr(), buf.data_ptr(), 4, 8, 2, 3, 0, None) == 0
    assert L.caifx_moe_dispatch(None, idx.data_ptr(), m.data_ptr(), off.data_ptr(), buf.data_ptr(), 4, 8, 2, 3, 0, None) == 1
    assert L.caifx_moe_dispatch(x.data_ptr(), idx.data_ptr(), m.data_ptr(), off.data_ptr(), buf.data_ptr(), 4, 8, 2, 3, 9, None) == 1
    assert L.caifx_moe_dispatch(x.data_ptr(), idx.data_ptr(), m.data_ptr(), off.data_ptr(), buf.data_ptr(), 0, 8, 2, 3, 0, None) == 0
    torch.cuda.synchronize()
