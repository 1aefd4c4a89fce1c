"""Pins the oracle's frozen-linear, expert and segment-map restatements.

What fixes them without running the reference: the layout pin of the
reference's own test (W is [out,in] row-major, tests/test_device_frozen_linear.cpp:
996-1072), textbook GEMM in numpy float64, one-hot probes that read single
columns of the materialised weight, the adjoint identity <Y,dY> = <X,dX> that
ties the dX access pattern and scale indexing to the forward's, and brute force
on tiny inputs for the integer map.
"""
import numpy as np
import pytest


def _w(orc, rng, N, K, kind, group=8):
    w = rng.normal(0, 0.02, (N, K)).astype(np.float32)
    if kind == "int4":
        p, s = orc.quantize_to_int4(w, group)
        return orc.FrozenWeight(p, orc.W_INT4_GROUP, s, N, K, 1, group), w
    if kind == "int8pc":
        # callers hand the quantiser an [in,out]-labelled view of the same buffer: cols = N
        q, s = orc.quantize_int8_per_channel(w.reshape(K, N))
        return orc.FrozenWeight(q.reshape(-1), orc.W_INT8, s, N, K, N, group), w
    q, s = orc.quantize_int8_per_tensor(w)
    return orc.FrozenWeight(q.reshape(-1), orc.W_INT8, s, N, K, 1, group), w


@pytest.mark.parametrize("kind", ["int4", "int8pc", "int8pt"])
@pytest.mark.parametrize("cd", [0, 1, 2])
def test_weight_materialisation_index_maps(orc, kind, cd):
    # N=6, K=16: K % N != 0, so the per-channel scale index (n*K+k) % N differs from both n and k
    rng = np.random.default_rng(1)
    N, K = 6, 16
    fw, _ = _w(orc, rng, N, K, kind)
    W = fw.compute_weight(cd)
    for n in range(N):
        for k in range(K):
            f = n * K + k
            if kind == "int4":
                nib = (int(fw.wq[f // 2]) >> (4 * (f & 1))) & 0xF
                qv = nib - 16 if nib >= 8 else nib
                sc = float(fw.scales[f // 8:f // 8 + 1].view(np.float16)[0])
                want = np.float32(qv) * np.float32(sc)
            elif kind == "int8pc":
                want = np.float32(fw.wq[f]) * fw.scales[f % N]
            else:
                want = np.float32(fw.wq[f]) * fw.scales[0]
            want = orc.round_to_dtype(np.array([want], np.float32), cd)[0]
            assert W[n, k] == want


def test_int8_without_scales_is_plain_cast(orc):
    q = np.arange(-12, 12).astype(np.int8)
    fw = orc.FrozenWeight(q, orc.W_INT8, None, 4, 6)
    assert np.array_equal(fw.compute_weight(2), q.astype(np.float32).reshape(4, 6))


@pytest.mark.parametrize("kind", ["int4", "int8pc", "int8pt"])
def test_forward_is_x_times_w_transposed(orc, kind):
    rng = np.random.default_rng(2)
    M, N, K = 5, 12, 32
    fw, _ = _w(orc, rng, N, K, kind)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    for cd in (orc.F32, orc.BF16, orc.F16):
        y = orc.frozen_linear_forward(x, fw, cd)
        W = fw.compute_weight(cd).astype(np.float64)
        xr = orc.round_to_dtype(x, cd).astype(np.float64)
        want = xr @ W.T
        assert y.shape == (M, N)
        assert np.abs(y - want).max() <= 1e-6 * np.abs(want).max()
        # one-hot row reads one column of W: layout pin [out,in] row-major
        e = np.zeros((1, K), np.float32)
        e[0, 7] = 1.0
        assert np.array_equal(orc.frozen_linear_forward(e, fw, cd)[0], fw.compute_weight(cd)[:, 7])


@pytest.mark.parametrize("kind", ["int4", "int8pc"])
def test_backward_adjoint_identity(orc, kind):
    rng = np.random.default_rng(3)
    M, N, K = 7, 10, 24                                  # K % N != 0
    fw, _ = _w(orc, rng, N, K, kind)
    cd = orc.BF16
    x = orc.round_to_dtype(rng.normal(0, 1, (M, K)), cd)
    dy = orc.round_to_dtype(rng.normal(0, 1, (M, N)), cd)
    y = orc.frozen_linear_forward(x, fw, cd).astype(np.float64)
    dx = orc.frozen_linear_backward(dy, fw, cd).astype(np.float64)
    lhs, rhs = (y * dy).sum(), (x * dx).sum()
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), abs(rhs), 1e-3)
    want = dy.astype(np.float64) @ fw.compute_weight(cd).astype(np.float64)
    assert np.abs(dx - want).max() <= 1e-6 * np.abs(want).max()
    # one-hot dY row reads one row of W
    e = np.zeros((1, N), np.float32)
    e[0, 3] = 1.0
    assert np.array_equal(orc.frozen_linear_backward(e, fw, cd)[0], fw.compute_weight(cd)[3])


def test_leading_dims_are_flattened(orc):
    rng = np.random.default_rng(4)
    fw, _ = _w(orc, rng, 8, 16, "int4")
    x = rng.normal(0, 1, (2, 3, 16)).astype(np.float32)
    y3 = orc.frozen_linear_forward(x, fw, orc.BF16)
    y0 = orc.frozen_linear_forward(x[1, 2:3], fw, orc.BF16)
    assert y3.shape == (6, 8) and np.array_equal(y3[5], y0[0])


def test_quantised_forward_close_to_dense(orc):
    # the reference's own accuracy bars: int8 <= 2e-2..4e-2, int4 <= 1.5e-1 of max|ref|
    # (tests/test_device_frozen_linear.cpp:1103-1206), K=16, N=8, M=2
    rng = np.random.default_rng(71)
    N, K, M = 8, 16, 2
    for kind, tol in (("int8pt", 2e-2), ("int8pc", 3e-2), ("int4", 1.5e-1)):
        fw, w = _w(orc, rng, N, K, kind, group=16)
        x = rng.uniform(-1, 1, (M, K)).astype(np.float32)
        ref = x.astype(np.float64) @ w.astype(np.float64).T
        y = orc.frozen_linear_forward(x, fw, orc.F32)
        assert np.abs(y - ref).max() / np.abs(ref).max() <= tol


# ----------------------------------------------------------------------------- element-wise + expert
def test_silu_closed_form(orc):
    x = np.linspace(-12, 12, 4001).astype(np.float32)
    s = orc.silu(x, orc.F32).astype(np.float64)
    xd = x.astype(np.float64)
    want = xd / (1 + np.exp(-xd))
    assert np.abs(s - want).max() <= 4e-7 * np.abs(want).max() + 1e-9
    g = np.ones_like(x)
    gb = orc.silu_backward(x, g, orc.F32).astype(np.float64)
    sig = 1 / (1 + np.exp(-xd))
    assert np.abs(gb - sig * (1 + xd * (1 - sig))).max() <= 1e-6
    # finite-difference cross-check of the derivative formula
    h = 1e-4
    fd = ((xd + h) / (1 + np.exp(-(xd + h))) - (xd - h) / (1 + np.exp(-(xd - h)))) / (2 * h)
    assert np.abs(gb - fd).max() <= 1e-5
    # rounding to the tensor dtype happens once, at the end
    sb = orc.silu(x, orc.BF16)
    assert np.array_equal(sb, orc.round_to_dtype(orc.silu(x, orc.F32), orc.BF16))


def test_expert_matches_float64_swiglu(orc):
    rng = np.random.default_rng(5)
    T, D, H = 6, 32, 48
    gate, _ = _w(orc, rng, H, D, "int8pc")
    up, _ = _w(orc, rng, H, D, "int8pc")
    down, _ = _w(orc, rng, D, H, "int8pc")
    x = rng.normal(0, 1, (T, D)).astype(np.float32)
    out, cache = orc.moe_frozen_expert_forward(x, gate, up, down, orc.F32, orc.F32)
    Wg, Wu, Wd = (l.compute_weight(orc.F32).astype(np.float64) for l in (gate, up, down))
    xd = x.astype(np.float64)
    g, u = xd @ Wg.T, xd @ Wu.T
    want = ((g / (1 + np.exp(-g))) * u) @ Wd.T
    assert np.abs(out - want).max() <= 1e-5 * np.abs(want).max()
    # backward against a finite difference of the float64 forward
    gy = rng.normal(0, 1, (T, D)).astype(np.float32)
    dx = orc.moe_frozen_expert_backward(gy, cache, gate, up, down, orc.F32, orc.F32)

    def loss(xx):
        gg, uu = xx @ Wg.T, xx @ Wu.T
        return ((((gg / (1 + np.exp(-gg))) * uu) @ Wd.T) * gy).sum()
    for (t, d) in [(0, 0), (3, 17), (5, 31)]:
        xp, xm = xd.copy(), xd.copy()
        xp[t, d] += 1e-4
        xm[t, d] -= 1e-4
        fd = (loss(xp) - loss(xm)) / 2e-4
        assert abs(dx[t, d] - fd) <= 1e-4 * max(1.0, abs(fd))
    # bf16 storage: every intermediate is a bf16 value
    out_b, cache_b = orc.moe_frozen_expert_forward(x, gate, up, down, orc.BF16, orc.BF16)
    for a in (out_b, cache_b["gate_out"], cache_b["up_out"], cache_b["hidden"]):
        assert np.array_equal(a, orc.round_to_dtype(a, orc.BF16))
    assert np.abs(out_b - want).max() <= 3e-2 * np.abs(want).max()


# ----------------------------------------------------------------------------- segment map
def test_dispatch_map_hand_example(orc):
    # T=3, top_k=2, E=3.  arrivals in token-major, k-minor order:
    # (0,0)->e2 pos0, (0,1)->e0 pos0, (1,0)->e2 pos1, (1,1)->e2 pos2, (2,0)->e0 pos1, (2,1)->e7 ignored
    idx = np.array([[2, 0], [2, 2], [0, 7]], np.int32)
    dmap, off, total = orc.moe_build_dispatch_map(idx, 3)
    assert off.tolist() == [0, 2, 2, 5] and total == 5
    assert dmap.tolist() == [[0, 0], [1, 2], [1, -1]]
    # capacity 2: expert 2 keeps its first two arrivals, the third is dropped
    dmap, off, total = orc.moe_build_dispatch_map(idx, 3, capacity_per_expert=2)
    assert off.tolist() == [0, 2, 2, 4] and total == 4
    assert dmap.tolist() == [[0, 0], [1, -1], [1, -1]]


def test_dispatch_map_is_a_bijection_onto_segments(orc):
    rng = np.random.default_rng(6)
    T, k, E = 257, 6, 64
    idx = rng.integers(0, E, (T, k)).astype(np.int32)
    dmap, off, total = orc.moe_build_dispatch_map(idx, E)
    assert total == T * k and off[0] == 0 and np.all(np.diff(off) == np.bincount(idx.ravel(), minlength=E))
    rows = off[idx] + dmap
    assert sorted(rows.ravel().tolist()) == list(range(T * k))
    # arrival order inside a segment is token-major
    flat_e = idx.ravel()
    for e in range(E):
        assert np.array_equal(dmap.ravel()[flat_e == e], np.arange((flat_e == e).sum()))


# --------------------------------------------------------------------------- LoRA wrapper around the frozen base
def _lora_case(orc, seed, kind, M=7, N=24, K=32, rank=4):
    rng = np.random.default_rng(seed)
    fw, _ = _w(orc, rng, N, K, kind)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    g = rng.normal(0, 1e-3, (M, N)).astype(np.float32)
    a = rng.normal(0, 0.01, (rank, K)).astype(np.float32)
    b = rng.normal(0, 0.01, (N, rank)).astype(np.float32)
    return fw, x, g, a, b


@pytest.mark.parametrize("kind", ["int4", "int8pc"])
def test_lora_forward_and_input_gradient_against_float64_composition(orc, kind):
    # out = x W^T + (alpha/rank) (x A^T) B^T and dX = g W + (alpha/rank) (g B) A
    # (src/caif_device_lora_adapter.cpp:161-198, 228-276), written here with numpy float64 matmuls on the
    # materialised weight.  With fp32 storage and compute the oracle's intermediate casts are identities, so it
    # must agree to fp32 rounding; with bf16 it must agree to the size of its seven bf16 roundings.
    alpha, rank = 32.0, 4
    fw, x, g, a, b = _lora_case(orc, 31, kind)
    W = fw.compute_weight(0).astype(np.float64)
    x64, g64, a64, b64 = (v.astype(np.float64) for v in (x, g, a, b))
    want_y = x64 @ W.T + (alpha / rank) * (x64 @ a64.T) @ b64.T
    want_dx = g64 @ W + (alpha / rank) * (g64 @ b64) @ a64
    y, hidden = orc.lora_forward(x, fw, a, b, alpha, 0, 0)
    dx = orc.lora_backward_input(g, fw, a, b, alpha, 0, 0)
    assert np.abs(y - want_y).max() <= 1e-5 * np.abs(want_y).max()
    assert np.abs(hidden - x64 @ a64.T).max() <= 1e-5 * np.abs(x64 @ a64.T).max()
    assert np.abs(dx - want_dx).max() <= 1e-5 * np.abs(want_dx).max()
    # a swapped operand or a dropped alpha/rank would be off by far more than this
    wrong_y = x64 @ W.T + (x64 @ a64.T) @ b64.T
    assert np.abs(y - wrong_y).max() > 1e-3 * np.abs(want_y).max()
    # bf16 storage and compute: the same quantities, each intermediate rounded to 8 bits of mantissa
    xb = orc.round_to_dtype(x, 2)
    gb = orc.round_to_dtype(g, 2)
    yb, _ = orc.lora_forward(xb, fw, a, b, alpha, 2, 2)
    dxb = orc.lora_backward_input(gb, fw, a, b, alpha, 2, 2)
    Wb = fw.compute_weight(2).astype(np.float64)
    ab, bb = orc.round_to_dtype(a, 2).astype(np.float64), orc.round_to_dtype(b, 2).astype(np.float64)
    want_yb = xb.astype(np.float64) @ Wb.T + (alpha / rank) * (xb.astype(np.float64) @ ab.T) @ bb.T
    want_dxb = gb.astype(np.float64) @ Wb + (alpha / rank) * (gb.astype(np.float64) @ bb) @ ab
    assert np.abs(yb - want_yb).max() <= 2e-2 * np.abs(want_yb).max()
    assert np.abs(dxb - want_dxb).max() <= 2e-2 * np.abs(want_dxb).max()


@pytest.mark.parametrize("sd", [0, 1, 2])
def test_lora_with_zero_b_is_the_base_layer(orc, sd):
    # B = 0 is how every adapter starts (tests/test_device_lora_adapter.cpp:371-443): the low-rank branch adds an
    # exact zero, so output and input gradient are the base layer's, cast to the storage dtype
    fw, x, g, a, b = _lora_case(orc, 32, "int4")
    b[:] = 0.0
    cd = sd
    y, _ = orc.lora_forward(x, fw, a, b, 32.0, cd, sd)
    dx = orc.lora_backward_input(g, fw, a, b, 32.0, cd, sd)
    xs, gs = orc.round_to_dtype(x, sd), orc.round_to_dtype(g, sd)
    assert np.array_equal(y, orc.round_to_dtype(orc.frozen_linear_forward(xs, fw, cd), sd))
    assert np.array_equal(dx, orc.round_to_dtype(orc.frozen_linear_backward(gs, fw, cd), sd))
