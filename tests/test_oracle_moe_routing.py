"""Pins for the oracle's MoE routing restatements (dispatch, combine and their backward passes), none of
which retypes the oracle's own loops: scatter/gather written with numpy fancy indexing from the map
definition, identities that hold for any correct implementation (adjointness of dispatch / dispatch
backward and of combine / combine backward, identity experts with weights summing to one), a hand example,
and capacity drops."""
import numpy as np
import pytest


def _route(rng, T, top_k, E):
    return rng.integers(0, E, (T, top_k)).astype(np.int32)


def test_hand_example(orc):
    # 3 tokens, top-2, 2 experts: arrival order (t,k) = (0,0)e1 (0,1)e0 (1,0)e1 (1,1)e1 (2,0)e0 (2,1)e1
    idx = np.array([[1, 0], [1, 1], [0, 1]], np.int32)
    dmap, offsets, total = orc.moe_build_dispatch_map(idx, 2)
    assert offsets.tolist() == [0, 2, 6] and total == 6
    assert dmap.tolist() == [[0, 0], [1, 2], [1, 3]]
    x = np.array([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0]], np.float32)
    buf = orc.moe_dispatch(x, idx, dmap, offsets, 2, total, 0)
    # expert 0 rows: token 0, token 2; expert 1 rows: token 0, 1, 1, 2
    assert buf.tolist() == [[1, 10], [3, 30], [1, 10], [2, 20], [2, 20], [3, 30]]
    w = np.array([[0.25, 0.75], [0.5, 0.5], [1.0, 2.0]], np.float32)
    out = orc.moe_combine(buf, idx, w, dmap, offsets, 2, 0)
    assert np.array_equal(out, x * w.sum(1, keepdims=True))


@pytest.mark.parametrize("dtype", [0, 2])
def test_scatter_gather_against_fancy_indexing(orc, dtype):
    rng = np.random.default_rng(3)
    T, top_k, E, dim = 37, 3, 5, 24
    idx = _route(rng, T, top_k, E)
    dmap, offsets, total = orc.moe_build_dispatch_map(idx, E)
    rows = (offsets[idx] + dmap).astype(np.int64)                    # no drops here
    assert sorted(rows.ravel().tolist()) == list(range(total))      # a permutation of the buffer rows
    x = orc.round_to_dtype(rng.normal(0, 1, (T, dim)), dtype)
    buf = orc.moe_dispatch(x, idx, dmap, offsets, E, total, dtype)
    want = np.zeros_like(buf)
    want[rows.ravel()] = np.repeat(x, top_k, axis=0)
    assert np.array_equal(buf, want)
    g = orc.round_to_dtype(rng.normal(0, 1, (total, dim)), dtype)
    gi = orc.moe_dispatch_backward(g, idx, dmap, offsets, E, dtype)
    ref = g[rows].astype(np.float64).sum(1)
    assert np.abs(gi - ref).max() <= (1e-6 if dtype == 0 else 2e-2) * np.abs(ref).max()


def test_adjoint_identities(orc):
    # <dispatch(x), g> = <x, dispatch_backward(g)>  and  <combine(b), g> = <b, combine_backward(g)>, fp32
    rng = np.random.default_rng(4)
    T, top_k, E, dim = 29, 4, 6, 16
    idx = _route(rng, T, top_k, E)
    dmap, offsets, total = orc.moe_build_dispatch_map(idx, E)
    x = rng.normal(0, 1, (T, dim)).astype(np.float32)
    g = rng.normal(0, 1, (total, dim)).astype(np.float32)
    lhs = (orc.moe_dispatch(x, idx, dmap, offsets, E, total, 0).astype(np.float64) * g).sum()
    rhs = (x.astype(np.float64) * orc.moe_dispatch_backward(g, idx, dmap, offsets, E, 0)).sum()
    assert abs(lhs - rhs) <= 1e-5 * abs(lhs)
    w = rng.random((T, top_k)).astype(np.float32)
    b = rng.normal(0, 1, (total, dim)).astype(np.float32)
    go = rng.normal(0, 1, (T, dim)).astype(np.float32)
    lhs = (orc.moe_combine(b, idx, w, dmap, offsets, E, 0).astype(np.float64) * go).sum()
    rhs = (b.astype(np.float64) * orc.moe_combine_backward_grad_expert(go, idx, w, dmap, offsets, E, total, 0)).sum()
    assert abs(lhs - rhs) <= 1e-5 * abs(lhs)


def test_grad_weights_is_the_derivative_of_combine(orc):
    # combine is linear in the weights: <combine(b; w + h e_tk) - combine(b; w), g> = h * grad_weights[t,k]
    rng = np.random.default_rng(8)
    T, top_k, E, dim = 9, 3, 4, 12
    idx = _route(rng, T, top_k, E)
    dmap, offsets, total = orc.moe_build_dispatch_map(idx, E)
    b = rng.normal(0, 1, (total, dim)).astype(np.float32)
    go = rng.normal(0, 1, (T, dim)).astype(np.float32)
    gw = orc.moe_combine_backward_grad_weights(go, b, idx, dmap, offsets, E, 0)
    rows = offsets[idx] + dmap
    want = np.einsum("td,tkd->tk", go.astype(np.float64), b[rows].astype(np.float64))
    assert np.abs(gw - want).max() <= 1e-6 * np.abs(want).max()


def test_identity_experts_return_the_tokens(orc):
    # dispatch, do nothing, combine with weights that sum to one: every token comes back (fp32, up to the
    # rounding of the weighted sum)
    rng = np.random.default_rng(5)
    T, top_k, E, dim = 50, 6, 8, 8
    idx = _route(rng, T, top_k, E)
    dmap, offsets, total = orc.moe_build_dispatch_map(idx, E)
    x = rng.normal(0, 1, (T, dim)).astype(np.float32)
    w = rng.random((T, top_k)).astype(np.float32)
    w /= w.sum(1, keepdims=True)
    out = orc.moe_combine(orc.moe_dispatch(x, idx, dmap, offsets, E, total, 0), idx, w, dmap, offsets, E, 0)
    assert np.abs(out - x).max() <= 1e-6 * np.abs(x).max()


def test_capacity_drops_move_no_data(orc):
    rng = np.random.default_rng(6)
    T, top_k, E, dim, cap = 40, 2, 3, 4, 7
    idx = _route(rng, T, top_k, E)
    idx[5, 1] = -1                                                   # an invalid expert id moves nothing either
    dmap, offsets, total = orc.moe_build_dispatch_map(idx, E, cap)
    assert total == int(offsets[-1]) <= E * cap and (np.diff(offsets) <= cap).all()
    assert dmap[5, 1] == -1 and (dmap < cap).all()
    x = rng.normal(0, 1, (T, dim)).astype(np.float32)
    buf = orc.moe_dispatch(x, idx, dmap, offsets, E, total, 0)
    kept = dmap >= 0
    assert kept.sum() == total
    w = np.ones((T, top_k), np.float32)
    out = orc.moe_combine(buf, idx, w, dmap, offsets, E, 0)
    assert np.allclose(out, x * kept.sum(1, keepdims=True), rtol=1e-6)
