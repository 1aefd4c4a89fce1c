"""Seeded sweep over shapes on both sides of every kernel choice (rows 1 ... 8225, columns 64 ... 3072, reduction
128 ... 4096, int8 per-channel / per-tensor and int4, both 16-bit compute types, fp32 and bf16 results; expert counts on
both sides of 64 with empty, one-row and multi-tile segments): forward (src/caif_device_frozen_linear.cpp:382-524) and
input gradient (:528-660), plain and over expert segments (src/caif_device_moe_layer.cpp:534-557, :754-778), a handful of
rows of every case against the CPU oracle at the north star's 1e-2.  The per-kernel files assert the tighter bounds; this
one is about the shapes between their cases."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from caif_amd import torch_ops as T                                  # noqa: E402
from gpu_helpers import dev, dev_as, host, make_weight, max_rel_err   # noqa: E402

TOL = 1e-2


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_plain_shapes(orc, seed):
    rng = np.random.default_rng(seed)
    kinds = ["int8pc", "int8pc", "int8pt", "int4"]
    for n in range(60):
        kind = kinds[n % len(kinds)]
        N = int(rng.choice([64, 96, 160, 256, 352, 512, 640, 1000, 1056, 1408, 1536, 2048, 2112, 3072]))
        K = int(rng.choice([128, 256, 384, 512, 640, 768, 1024, 1408, 1536, 2048, 2560, 4096]))
        if kind == "int4":
            N, K = (N + 7) // 8 * 8, max(256, K // 256 * 256)
        M = int(rng.choice([1, 2, 3, 5, 16, 17, 32, 33, 64, 100, 128, 300, 1024, 2048 + 5, 4096, 8192 + 33]))
        cd, yd = int(rng.choice([1, 2])), int(rng.choice([0, 2]))
        ow, dw = make_weight(orc, rng, N, K, kind)
        x = dev_as(rng.normal(0, 1, (M, K)), cd)
        dy = dev_as(rng.normal(0, 1, (M, N)), cd)
        y = host(T.qlinear_forward(x, dw, cd, yd))
        dx = host(T.qlinear_backward_input(dy, dw, cd, yd))
        sel = np.unique(np.concatenate([rng.choice(M, min(6, M), replace=False), [0, M - 1]]))
        want_y = orc.frozen_linear_forward(host(x)[sel], ow, cd)
        want_dx = orc.frozen_linear_backward(host(dy)[sel], ow, cd)
        if yd != 0:
            want_y, want_dx = orc.round_to_dtype(want_y, yd), orc.round_to_dtype(want_dx, yd)
        what = (seed, n, kind, M, N, K, cd, yd)
        assert np.isfinite(y).all() and np.isfinite(dx).all(), what
        assert max_rel_err(y[sel], want_y) <= TOL, what
        assert max_rel_err(dx[sel], want_dx) <= TOL, what


@pytest.mark.parametrize("seed", [21, 22])
def test_expert_segments(orc, seed):
    rng = np.random.default_rng(seed)
    for n in range(40):
        kind = ["int8pc", "int8pt", "int4", "int8pc"][n % 4]
        E = int(rng.choice([1, 2, 7, 33, 63, 64, 65, 70, 100]))
        N = int(rng.choice([128, 256, 512, 640, 1408]))
        K = int(rng.choice([128, 256, 384, 512, 1024]))
        if kind == "int4":
            K = max(256, K // 256 * 256)
        mean = int(rng.choice([0, 1, 3, 20, 100, 300]))
        counts = rng.poisson(mean, E) if mean else rng.integers(0, 2, E)
        if rng.random() < 0.3:
            counts[rng.integers(0, E)] += int(rng.choice([129, 257, 1000]))
        if counts.sum() == 0:
            counts[0] = 1
        offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
        total, pad = int(offsets[-1]), int(rng.choice([0, 3]))
        pairs = [make_weight(orc, rng, N, K, kind) for _ in range(E)]
        gw = T.GroupedFrozenWeights([p[1] for p in pairs])
        x = dev_as(rng.normal(0, 1, (total + pad, K)), 2)
        dy = dev_as(rng.normal(0, 1, (total + pad, N)), 2)
        y = torch.full((total + pad, N), 7.0, device="cuda")
        dx = torch.full((total + pad, K), 7.0, device="cuda")
        T.qlinear_grouped_forward(x, dev(offsets), gw, 2, out=y)
        T.qlinear_grouped_backward_input(dy, dev(offsets), gw, 2, out=dx)
        y, dx, xh, dyh = host(y), host(dx), host(x), host(dy)
        what = (seed, n, kind, E, N, K, total)
        assert (y[total:] == 7.0).all() and (dx[total:] == 7.0).all(), what          # rows past offsets[E] untouched
        assert np.isfinite(y).all() and np.isfinite(dx).all(), what
        for e in rng.choice(E, min(E, 6), replace=False):
            lo, hi = int(offsets[e]), int(offsets[e + 1])
            if hi == lo:
                continue
            sel = np.unique(np.concatenate([rng.choice(hi - lo, min(4, hi - lo), replace=False), [0, hi - lo - 1]])) + lo
            assert max_rel_err(y[sel], orc.frozen_linear_forward(xh[sel], pairs[e][0], 2)) <= TOL, (what, int(e))
            assert max_rel_err(dx[sel], orc.frozen_linear_backward(dyh[sel], pairs[e][0], 2)) <= TOL, (what, int(e))
