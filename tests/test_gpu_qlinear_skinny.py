"""GPU parity of the decode-regime dequant-GEMM (M <= 16) against the CPU oracle.

Tolerance (north star): max relative error <= 1e-2 for bf16/fp16 compute with fp32
accumulation, <= 1e-4 for the fp32 path; both relative to max|ref| as the reference's own
parity tests normalise.  The asserts are tighter than the contract:
  * int4 with group sizes below 128, and int8 with two activation rows on the row-streaming kernel,
    feed the matrix cores weights that are bit-identical to the oracle's, so only the summation
    order differs (~1e-6);
  * int4 with group size 128 (or a multiple) is scaled after the per-group accumulation, and int8
    with up to 32 activation rows (two launches of the 16-row kernel from 17 on) folds the scales into the activations and multiplies the integer
    codes exactly on the integer matrix core: both skip the reference's rounding of code*scale to
    the compute dtype; the difference is that rounding, <= 2^-9 per weight with random sign, about
    2e-3 of max|ref| after the sum over K (2e-4 for fp16 compute).
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from caif_amd import torch_ops as T                                  # noqa: E402
from gpu_helpers import dev, dev_as, host, make_weight, max_rel_err   # noqa: E402

TOL_16 = 1e-2      # contract
TOL_32 = 1e-4      # contract
TIGHT_16 = 2e-5    # what identical operands + fp32 accumulation actually give
TIGHT_POST = 4e-3  # post-scaled int4: bf16 rounding of the weights is not applied


def _check(orc, rng, M, N, K, kind, cd, xd, group=128, yd=0):
    ow, dw = make_weight(orc, rng, N, K, kind, group)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    xt = dev_as(x, xd)
    y = host(T.qlinear_forward(xt, dw, cd, yd))
    want = orc.frozen_linear_forward(host(xt), ow, cd)
    if yd != 0:
        want = orc.round_to_dtype(want, yd)
    err = max_rel_err(y, want)
    bound = TOL_32 if cd == 0 else TOL_16
    assert err <= bound, (M, N, K, kind, cd, xd, err)
    if cd != 0 and yd == 0:
        post = (kind == "int4" and group % 128 == 0) or (kind.startswith("int8") and M <= 32)
        assert err <= (TIGHT_POST if post else TIGHT_16), (M, N, K, kind, cd, xd, err)
    return err


@pytest.mark.parametrize("kind", ["int4", "int8pc", "int8pt", "int8raw"])
@pytest.mark.parametrize("M", [1, 4, 16])
def test_decode_shapes_bf16(orc, kind, M):
    # BASELINE config 2 geometry at reduced N (the oracle GEMM is O(M N K) on the CPU)
    _check(orc, np.random.default_rng(M), M, 1792, 4096, kind, cd=2, xd=2)


@pytest.mark.parametrize("kind", ["int4", "int8pc"])
def test_decode_full_width_m1(orc, kind):
    _check(orc, np.random.default_rng(17), 1, 14336, 4096, kind, cd=2, xd=2)


@pytest.mark.parametrize("kind", ["int4", "int8pc"])
def test_decode_full_width_two_row_tiles(orc, kind):
    # the decode geometry at its full width with 32 rows: two tiles, two reduction slices, 7 residue classes (int8)
    _check(orc, np.random.default_rng(18), 32, 14336, 4096, kind, cd=2, xd=2)


@pytest.mark.parametrize("kind", ["int4", "int8pc", "int8pt"])
@pytest.mark.parametrize("N,K,M", [(4096, 14336, 1), (4096, 14336, 16), (1024, 8192, 4), (528, 11008, 9), (640, 4224, 24),
                                   (2048, 8192, 1), (1024, 11264, 1), (1536, 5120, 1), (512, 16384, 1), (1027, 9216, 1)])
def test_reductions_longer_than_one_workgroup_covers(orc, kind, N, K, M):
    # the FFN down projection (N = 4096, K = 14336) and other K > 4096: the 16-row decode kernel cuts the
    # reduction into slices of 4096 (the last one shorter) whose sums meet in the workspace; with one activation
    # row the row-streaming kernels split a weight row among the waves of a workgroup (int8: 2 or 4 slices of up
    # to 4 KiB, the last one shorter or empty; int4: 7 or 8 chunks per wave)
    rng = np.random.default_rng(N + K + M)
    _check(orc, rng, M, N, K, kind, cd=2, xd=2)


def test_long_reduction_without_a_workspace_takes_the_fallback(orc):
    rng = np.random.default_rng(8)
    N, K, M = 256, 8192, 5
    ow, dw = make_weight(orc, rng, N, K, "int8pc")
    xt = dev_as(rng.normal(0, 1, (M, K)), 2)
    want = orc.frozen_linear_forward(host(xt), ow, 2)
    import torch
    none = torch.empty(0, dtype=torch.uint8, device="cuda")
    y = host(T.qlinear_forward(xt, dw, 2, 0, workspace=none))
    assert max_rel_err(y, want) <= TOL_16


@pytest.mark.parametrize("cd,xd", [(2, 0), (2, 1), (1, 1), (1, 2), (1, 0)])
@pytest.mark.parametrize("kind", ["int4", "int8pc"])
def test_dtype_mixes(orc, kind, cd, xd):
    _check(orc, np.random.default_rng(cd * 3 + xd), 3, 256, 1024, kind, cd, xd)


@pytest.mark.parametrize("N,K,M", [(16, 128, 1), (24, 256, 2), (1000, 384, 5), (4096, 4096, 16), (48, 8192, 7),
                                   (1408, 2048, 13), (2048, 1408, 16)])
def test_ragged_and_wave_count_variants(orc, N, K, M):
    rng = np.random.default_rng(N + K + M)
    _check(orc, rng, M, N, K, "int4", 2, 2)
    _check(orc, rng, M, N, K, "int8pc", 2, 2)


@pytest.mark.parametrize("N,K", [(4097, 4096), (2049, 2048), (1793, 4096), (6145, 1024), (8193, 4096)])
@pytest.mark.parametrize("M", [1, 2])
def test_row_streaming_tails(orc, N, K, M):
    # one and two activation rows stream whole weight rows through a small ring per wave; these row
    # counts leave a last wave with a single row (fewer rows than the ring holds), waves with no rows
    # at all inside the last workgroup, and residue classes of unequal size for the per-channel scales
    rng = np.random.default_rng(N + K + M)
    for kind in ("int4", "int8pc", "int8pt"):
        _check(orc, rng, M, N, K, kind, 2, 2)


@pytest.mark.parametrize("N,K,M", [(1536, 1024, 6), (14336, 4096, 4), (14336, 4096, 16), (200, 4096, 3), (2050, 640, 11)])
def test_residue_classes_and_masked_row_blocks(orc, N, K, M):
    # 3 <= M <= 16 runs on the matrix cores in blocks of 16 weight rows: N = 200 and 2050 leave a
    # partly masked last block; int8 per-channel scales (period N) split the rows into
    # N / gcd(K mod N, N) residue classes: 3 for (1536, 1024), 7 for the full decode shape
    rng = np.random.default_rng(N * 7 + K + M)
    _check(orc, rng, M, N, K, "int4", 2, 2)
    _check(orc, rng, M, N, K, "int8pc", 2, 2)
    _check(orc, rng, M, N, K, "int8pt", 1, 0)


@pytest.mark.parametrize("group", [32, 64, 256, 512])
def test_int4_group_sizes(orc, group):
    _check(orc, np.random.default_rng(group), 2, 128, 1024, "int4", 2, 2, group=group)


@pytest.mark.parametrize("yd", [1, 2])
def test_fused_output_cast_equals_cast_of_fp32(orc, yd):
    _check(orc, np.random.default_rng(yd), 4, 512, 1024, "int8pc", 2, 2, yd=yd)


def test_m1_equals_row0_of_m16(orc):
    rng = np.random.default_rng(5)
    ow, dw = make_weight(orc, rng, 512, 2048, "int4")
    x = dev_as(rng.normal(0, 1, (16, 2048)), 2)
    y16 = host(T.qlinear_forward(x, dw, 2))
    y1 = host(T.qlinear_forward(x[:1].contiguous(), dw, 2))
    y4 = host(T.qlinear_forward(x[:4].contiguous(), dw, 2))
    # different M take different kernels (summation order differs), so equal up to fp32 rounding
    assert np.abs(y16[0] - y1[0]).max() <= 1e-5 * np.abs(y16).max()
    assert np.abs(y16[:4] - y4).max() <= 1e-5 * np.abs(y16).max()


def test_one_hot_reads_a_weight_column_exactly(orc):
    # X = e_j  =>  Y[0, n] = W[n, j] (a single non-zero product).  Paths that round each weight to the
    # compute dtype return that rounded weight bit for bit; post-scaled int4 (group 128) returns the
    # unrounded fp32 code*scale bit for bit; int8 on the integer matrix core passes the scale through
    # three 7-bit digits, so code*scale comes back exact to 2^-21.  Which int8 kernel a shape takes
    # depends on the rows per scale-residue class, so int8 accepts either of its two answers.
    rng = np.random.default_rng(6)

    def int8_ok(y, ow, j):
        return np.array_equal(y, ow.compute_weight(2)[:, j]) or np.allclose(y, ow.compute_weight(0)[:, j], rtol=1e-6, atol=0)

    for kind, group, N, how in (("int4", 128, 320, "fp32"), ("int4", 64, 320, "bf16"), ("int8pc", 128, 320, "int8"),
                                ("int8pt", 128, 320, "int8"), ("int8pc", 128, 2048, "int8")):
        ow, dw = make_weight(orc, rng, N, 1024, kind, group)
        for j in (0, 1, 4, 127, 128, 777, 1023):
            e = np.zeros((1, 1024), np.float32)
            e[0, j] = 1.0
            y = host(T.qlinear_forward(dev_as(e, 2), dw, 2))
            if how == "int8":
                assert int8_ok(y[0], ow, j), (kind, group, N, j)
            else:
                assert np.array_equal(y[0], ow.compute_weight(0 if how == "fp32" else 2)[:, j]), (kind, group, N, j)
        if kind.startswith("int8"):
            for rows in (2, 5):
                e = np.zeros((rows, 1024), np.float32)
                e[0, 5] = e[rows - 1, 900] = 1.0
                y = host(T.qlinear_forward(dev_as(e, 2), dw, 2))
                assert int8_ok(y[0], ow, 5) and int8_ok(y[rows - 1], ow, 900), (kind, N, rows)
                if rows > 2:
                    assert not y[1:rows - 1].any(), (kind, N, rows)


@pytest.mark.parametrize("kind", ["int4", "int8pc", "int8pt"])
@pytest.mark.parametrize("M", [17, 24, 32])
def test_two_row_blocks_of_the_decode_kernel(orc, kind, M):
    # 17..32 rows: two tiles of 16 activation rows share one pass over the weight (same accuracy class as
    # M <= 16); a workgroup then reaches 2048 of the reduction, so K = 1024 is one slice, K = 4096 two and
    # K = 5120 three with a short last one, meeting in the workspace.  Rows 16 onwards are the second tile.
    _check(orc, np.random.default_rng(700 + M), M, 1536, 1024, kind, 2, 2)
    _check(orc, np.random.default_rng(701 + M), M, 200, 4096, kind, 1, 1, yd=2)
    _check(orc, np.random.default_rng(702 + M), M, 1792, 4096, kind, 2, 0)
    _check(orc, np.random.default_rng(703 + M), M, 272, 5120, kind, 2, 2, yd=1)


@pytest.mark.parametrize("kind", ["int4", "int8pc"])
def test_two_row_blocks_without_a_workspace_run_16_rows_at_a_time(orc, kind):
    # without room for the slices' partial sums the same rows go through two launches of the 16-row form;
    # both forms are of one accuracy class and agree to fp32 summation order
    rng = np.random.default_rng(12)
    N, K, M = 528, 4096, 27
    ow, dw = make_weight(orc, rng, N, K, kind)
    xt = dev_as(rng.normal(0, 1, (M, K)), 2)
    want = orc.frozen_linear_forward(host(xt), ow, 2)
    import torch
    none = torch.empty(0, dtype=torch.uint8, device="cuda")
    y0 = host(T.qlinear_forward(xt, dw, 2, 0, workspace=none))
    y1 = host(T.qlinear_forward(xt, dw, 2, 0))
    assert max_rel_err(y0, want) <= TIGHT_POST
    assert max_rel_err(y1, want) <= TIGHT_POST
    assert np.abs(y0 - y1).max() <= 2e-4 * np.abs(want).max()


@pytest.mark.parametrize("M", [17, 32])
@pytest.mark.parametrize("xd", [0, 2])
def test_two_row_blocks_fp32_compute(orc, M, xd):
    # fp32 compute type with int8 codes: digit planes of the unrounded activations, 1e-4 contract
    _check(orc, np.random.default_rng(750 + M + xd), M, 1024, 4096, "int8pc", 0, xd)
    _check(orc, np.random.default_rng(751 + M + xd), M, 336, 1152, "int8pt", 0, xd)


@pytest.mark.parametrize("cd,xd", [(2, 0), (2, 1), (1, 0), (1, 2)])
@pytest.mark.parametrize("K", [1024, 4096])
@pytest.mark.parametrize("kind", ["int8pc", "int8pt"])
def test_one_row_int8_casts_the_activations_to_the_compute_dtype(orc, kind, K, cd, xd):
    # one activation row with int8 codes takes the integer-matrix-core kernel, which works on fp32 activations: when
    # the caller's activations are of another type than the compute type they must pass through it first, as the
    # layer's input.To(ComputeT) does (src/caif_device_frozen_linear.cpp:459).  fp32 activations that are not
    # bf16 values make the difference visible: without the cast the error against the oracle is ~4e-3 here.
    rng = np.random.default_rng(cd * 7 + xd + K)
    ow, dw = make_weight(orc, rng, 2048, K, kind)
    x = rng.normal(0, 1, (1, K)).astype(np.float32)
    xt = dev_as(x, xd)
    y = host(T.qlinear_forward(xt, dw, cd))
    want = orc.frozen_linear_forward(host(xt), ow, cd)
    assert max_rel_err(y, want) <= TIGHT_POST
    # and an M = 1 call equals row 0 of an M = 16 call of the same accuracy class to fp32 rounding
    x16 = dev_as(np.concatenate([x, rng.normal(0, 1, (15, K)).astype(np.float32)]), xd)
    y16 = host(T.qlinear_forward(x16, dw, cd))
    assert np.abs(y16[0] - y[0]).max() <= 2e-4 * np.abs(y16[0]).max()


@pytest.mark.parametrize("kind", ["int8pc", "int8pt", "int4"])
@pytest.mark.parametrize("M", [1, 2, 4, 16, 24, 32])
def test_non_finite_activations_are_not_masked(orc, kind, M):
    # A NaN or an infinity in an activation row reaches every output of that row in the reference (dequantise +
    # GEMM: every output multiplies every activation, and 0 * inf is NaN too).  The integer-matrix-core kernels
    # split activations into digits, which has no meaning for such values: they must still answer non-finite for
    # exactly those rows, and leave the other rows alone.
    rng = np.random.default_rng(900 + M)
    N, K = 1792, 4096
    ow, dw = make_weight(orc, rng, N, K, kind)
    for bad_value in (np.nan, np.inf, -np.inf):
        x = rng.normal(0, 1, (M, K)).astype(np.float32)
        bad_row = M - 1
        x[bad_row, 1234] = bad_value
        xt = dev_as(x, 2)
        y = host(T.qlinear_forward(xt, dw, 2))
        want = orc.frozen_linear_forward(host(xt), ow, 2)
        assert not np.isfinite(want[bad_row]).any(), "the oracle's own answer for the poisoned row"
        assert not np.isfinite(y[bad_row]).any(), (kind, M, bad_value)
        good = [m for m in range(M) if m != bad_row]
        if good:
            assert np.isfinite(y[good]).all(), (kind, M, bad_value)
            assert max_rel_err(y[good], want[good]) <= TIGHT_POST, (kind, M, bad_value)


@pytest.mark.parametrize("kind", ["int4", "int8pc"])
@pytest.mark.parametrize("M", [1, 4, 16, 32])
def test_post_scaled_kernels_on_correlated_inputs(orc, kind, M):
    # The memory-bound kernels skip the reference's rounding of code*scale to bf16.  On N(0,1) activations those
    # rounding differences add up like a random walk (about 2e-3 of max|ref|).  Correlated inputs are the worst
    # case for that argument: all-positive activations against constant codes make every difference push the
    # same way.  Cases: |N(0,1)| activations; alternating-sign constant activations; a weight whose every group
    # holds one repeated code (so every product in a group shares one rounding difference); all-ones
    # activations against that weight.  The contract's 1e-2 must hold on each; the worst value is recorded in the
    # assertion message of the bound below.
    rng = np.random.default_rng(77 + M)
    N, K = 1792, 4096
    cases = {}
    w_rand = rng.normal(0, 0.02, (N, K)).astype(np.float32)
    # constant code per 128-k group: each group's value is drawn once, so code*scale repeats 128 times
    w_const = np.repeat(rng.normal(0, 0.02, (N, K // 128)).astype(np.float32), 128, axis=1)
    x_abs = np.abs(rng.normal(0, 1, (M, K))).astype(np.float32)
    x_alt = np.tile(np.array([1.0, -1.0], np.float32), (M, K // 2)) * 0.7311
    x_one = np.ones((M, K), np.float32)
    for wname, w in (("random", w_rand), ("constant-per-group", w_const)):
        if kind == "int4":
            p, s = orc.quantize_to_int4(w, 128)
            ow = orc.FrozenWeight(p, orc.W_INT4_GROUP, s, N, K, 1, 128)
            dw = T.FrozenWeight(dev(p), T.W_INT4_GROUP, dev(s.view(np.float16)), N, K, 1, 128)
        else:
            q, s = orc.quantize_int8_per_channel(w.reshape(K, N))
            ow = orc.FrozenWeight(q.reshape(-1), orc.W_INT8, s, N, K, N, 128)
            dw = T.FrozenWeight(dev(q.reshape(-1)), T.W_INT8, dev(s), N, K, N, 128)
        for xname, x in (("abs-normal", x_abs), ("alternating", x_alt), ("ones", x_one)):
            xt = dev_as(x, 2)
            y = host(T.qlinear_forward(xt, dw, 2))
            want = orc.frozen_linear_forward(host(xt), ow, 2)
            cases[(wname, xname)] = max_rel_err(y, want)
    worst = max(cases.values())
    print(f"post-scaled {kind} M={M}: " + ", ".join(f"{w}/{x}={e:.2e}" for (w, x), e in cases.items()))
    assert worst <= TOL_16, cases


# ---------------------------------------------------------------- input gradient for a few rows

def _check_dx(orc, rng, M, N, K, kind, cd, xd, yd=0, workspace=None):
    ow, dw = make_weight(orc, rng, N, K, kind)
    dy = dev_as(rng.normal(0, 1e-3, (M, N)).astype(np.float32), xd)
    dx = host(T.qlinear_backward_input(dy, dw, cd, yd, workspace=workspace))
    want = orc.frozen_linear_backward(host(dy), ow, cd)
    if yd != 0:
        want = orc.round_to_dtype(want, yd)
    err = max_rel_err(dx, want)
    assert err <= (TOL_32 if cd == 0 else TOL_16), (M, N, K, kind, cd, xd, err)
    return err


@pytest.mark.parametrize("kind", ["int8pc", "int8pt", "int8raw", "int4"])
@pytest.mark.parametrize("M", [1, 5, 16])
def test_input_gradient_few_rows_fp32(orc, kind, M):
    # dX = dY W for up to 16 rows streams the weight once through the fp32 matrix core: int8 codes when the scale
    # of W[n][k] does not depend on n (square per-channel weight: K mod N = 0; one scale; none), int4 codes in
    # groups of 128 or more (the scale of a row and group rides on the gradient).  Shapes: BASELINE
    # config 1 (4096 x 4096), a row count that is no multiple of a wave's 16 rows (N = 1000), a single column slab
    # (K = 128), fewer rows than one workgroup pass (N = 40).
    rng = np.random.default_rng(300 + M)
    for N, K in ((4096, 4096), (1000, 1024), (3000, 128), (40, 256)):
        if kind == "int8pc" and K % N != 0:
            continue
        assert _check_dx(orc, rng, M, N, K, kind, 0, 0) <= 2e-6, (N, K)


@pytest.mark.parametrize("cd,xd,yd", [(2, 2, 0), (2, 0, 2), (1, 1, 1), (1, 0, 0), (0, 2, 0), (0, 1, 2)])
def test_input_gradient_few_rows_dtype_mixes(orc, cd, xd, yd):
    # 16-bit compute types: dY is rounded to the compute type first (the layer's cast of its input); the weight is
    # not (post-scaled class, like the decode forward)
    rng = np.random.default_rng(cd * 9 + xd * 3 + yd)
    for kind, N, K in (("int8pc", 512, 1024), ("int8pt", 777, 384), ("int4", 640, 1280)):
        err = _check_dx(orc, rng, 7, N, K, kind, cd, xd, yd)
        if cd != 0 and yd == 0:
            assert err <= TIGHT_POST


@pytest.mark.parametrize("cd", [1, 2])
def test_input_gradient_few_rows_int4_multiplies_the_rounded_weight(orc, cd):
    # 16-bit compute types run the few-row kernel on the 16-bit matrix cores; int4 codes meet their scale before the
    # product, rounded once to the compute type, so the operands are the oracle's and only the order of the fp32 sums
    # differs.  N = 1000 leaves a last stage with 8 of 16 rows; M = 1 and a gradient given in fp32.
    rng = np.random.default_rng(90 + cd)
    for M, N, K, xd in ((16, 4096, 4096, cd), (7, 640, 1280, cd), (3, 1000, 1024, 0), (1, 2048, 256, cd)):
        assert _check_dx(orc, rng, M, N, K, "int4", cd, xd) <= TIGHT_16, (M, N, K)


def test_input_gradient_few_rows_other_paths(orc):
    # per-channel scales whose index depends on the weight row in too many ways (205 residue classes), int4 groups
    # below 128, more than 16 rows and a call without a workspace go to the tiled kernels; all must agree with the oracle
    import torch
    rng = np.random.default_rng(31)
    _check_dx(orc, rng, 8, 2050, 640, "int8pc", 0, 0)
    ow, dw = make_weight(orc, rng, 512, 1024, "int4", 64)
    dy = dev_as(rng.normal(0, 1e-3, (8, 512)), 2)
    assert max_rel_err(host(T.qlinear_backward_input(dy, dw, 2)), orc.frozen_linear_backward(host(dy), ow, 2)) <= TIGHT_16
    _check_dx(orc, rng, 17, 512, 512, "int8pc", 0, 0)
    none = torch.empty(0, dtype=torch.uint8, device="cuda")
    _check_dx(orc, rng, 16, 2048, 2048, "int8pc", 0, 0, workspace=none)
    _check_dx(orc, rng, 3, 40, 128, "int8pt", 0, 0, workspace=none)     # one workgroup: no workspace needed


@pytest.mark.parametrize("N,K,M", [(1536, 1024, 16), (14336, 4096, 4), (14336, 4096, 16), (3584, 1024, 9)])
def test_input_gradient_few_rows_residue_classes(orc, N, K, M):
    # one scale per output feature with K mod N != 0: the scale of W[n][k] depends on n, but rows with equal
    # n mod V (V = 3, 7, 7, 7 here) share their scales along k; a workgroup stays inside one class.  (14336, 4096) is
    # BASELINE configs[1]'s up projection at full width, with 4 rows and with all 16.
    rng = np.random.default_rng(N + K + M)
    assert _check_dx(orc, rng, M, N, K, "int8pc", 0, 0) <= 2e-6
    assert _check_dx(orc, rng, M, N, K, "int8pc", 2, 2) <= TIGHT_POST


def test_input_gradient_few_rows_is_the_adjoint_of_the_forward(orc):
    # <dY, X W^T> = <dY W, X> with both sides from the device kernels (fp32 compute)
    rng = np.random.default_rng(32)
    N, K, M = 1024, 1024, 16
    ow, dw = make_weight(orc, rng, N, K, "int8pc")
    x = dev_as(rng.normal(0, 1, (M, K)).astype(np.float32), 0)
    dy = dev_as(rng.normal(0, 1, (M, N)).astype(np.float32), 0)
    y = host(T.qlinear_forward(x, dw, 0)).astype(np.float64)
    dx = host(T.qlinear_backward_input(dy, dw, 0)).astype(np.float64)
    lhs = (host(dy).astype(np.float64) * y).sum()
    rhs = (dx * host(x).astype(np.float64)).sum()
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), abs(rhs))


def test_input_gradient_few_rows_keeps_non_finite_gradients_in_their_row(orc):
    rng = np.random.default_rng(33)
    N, K, M = 512, 512, 6
    ow, dw = make_weight(orc, rng, N, K, "int8pt")
    for bad in (np.nan, np.inf):
        dy = rng.normal(0, 1e-3, (M, N)).astype(np.float32)
        dy[2, 77] = bad
        dx = host(T.qlinear_backward_input(dev_as(dy, 0), dw, 0))
        want = orc.frozen_linear_backward(dy, ow, 0)
        assert not np.isfinite(want[2]).any() and not np.isfinite(dx[2]).any()
        assert np.array_equal(np.isfinite(dx), np.isfinite(want))
        good = [m for m in range(M) if m != 2]
        assert max_rel_err(dx[good], want[good]) <= TOL_32


@pytest.mark.parametrize("yd", [1, 2])
def test_fused_add_on_the_few_row_paths_equals_the_two_launches(orc, yd):
    # the LoRA composition base.To(T) + branch on the decode kernels (two row tiles forward, few-row input gradient):
    # the fused entry points must give the bits of the plain call followed by the element-wise Add
    import torch
    rng = np.random.default_rng(60 + yd)
    N, K = 512, 4096
    ow, dw = make_weight(orc, rng, N, K, "int8pt")
    x = dev_as(rng.normal(0, 1, (24, K)), 2)
    add_y = dev_as(rng.normal(0, 1, (24, N)), yd)
    fused = T.qlinear_forward(x, dw, 2, yd, addend=add_y)
    plain = T.add(T.qlinear_forward(x, dw, 2, yd), add_y)
    assert torch.equal(fused, plain)
    dy = dev_as(rng.normal(0, 1e-2, (9, N)), 2)
    add_x = dev_as(rng.normal(0, 1e-2, (9, K)), yd)
    fused = T.qlinear_backward_input(dy, dw, 2, yd, addend=add_x)
    plain = T.add(T.qlinear_backward_input(dy, dw, 2, yd), add_x)
    assert torch.equal(fused, plain)
    want = orc.round_to_dtype(orc.frozen_linear_backward(host(dy), ow, 2), yd) + host(add_x)
    assert max_rel_err(host(fused), want) <= TOL_16
