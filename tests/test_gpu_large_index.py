"""GPU parity at the largest sizes: a weight of more than 2^31 elements (N = 270336, K = 8192), so that every
kernel's flat index n*K + k, byte offsets and scale indices pass 2^31 on the high rows.  The CPU oracle would need
minutes and tens of GB for this, so the check is a size-independent property: the last rows of the big weight,
taken as a weight of their own, give the reference (torch fp32 matmul on the dequantised slice; int8 codes and
int4 code * scale products are formed independently of the library with torch ops)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from caif_amd import torch_ops as T                                  # noqa: E402

N, K, R = 270336, 8192, 4096           # N*K = 2.2e9 > 2^31; R = rows checked at the top end


def _rel(got, want):
    return float((got.double() - want.double()).abs().max() / want.double().abs().max())


def _int8_weight(gen, scale):
    q = torch.randint(-127, 128, (N * K,), device="cuda", dtype=torch.int8, generator=gen)
    s = torch.tensor([scale], device="cuda") if scale else None
    dense_top = q[-R * K:].view(R, K).float() * (scale if scale else 1.0)
    return T.FrozenWeight(q, T.W_INT8, s, N, K, 1), dense_top


def _int4_weight(gen):
    p = torch.randint(0, 256, (N * K // 2,), device="cuda", dtype=torch.uint8, generator=gen)
    s = (torch.rand(N * K // 128, device="cuda", generator=gen) * 0.01 + 0.001).to(torch.float16)
    pt = p[-R * K // 2:].to(torch.int16)
    lo, hi = pt & 15, pt >> 4
    codes = torch.stack([lo, hi], dim=1).reshape(-1)
    codes = torch.where(codes >= 8, codes - 16, codes).float()
    dense_top = (codes * s[-R * K // 128:].float().repeat_interleave(128)).view(R, K)
    return T.FrozenWeight(p, T.W_INT4_GROUP, s, N, K, 1, 128), dense_top


@pytest.mark.parametrize("kind", ["int8raw", "int8pt", "int4"])
def test_flat_indices_beyond_2_31(kind):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    fw, dense_top = _int4_weight(gen) if kind == "int4" else _int8_weight(gen, 0.0 if kind == "int8raw" else 0.0123)
    w_bf16 = dense_top.to(torch.bfloat16).float()                  # what the reference feeds its GEMM
    for M in (1, 2, 16, 24, 64):                                    # row-streaming, row-block, two row blocks, tiled GEMM
        x = torch.randn(M, K, device="cuda", generator=gen).to(torch.bfloat16)
        y = T.qlinear_forward(x, fw, T.BF16)
        want = x.float() @ w_bf16.t()
        # up to 32 rows the kernels skip the bf16 rounding of code*scale (exact for bare int8 codes)
        tol = 2e-5 if (M > 32 or kind == "int8raw") else 4e-3
        assert _rel(y[:, -R:], want) <= tol, (kind, M)
    # input gradient: dY is zero outside the top rows, so only they contribute, but every row is visited
    for M in (8, 64):
        dy = torch.zeros(M, N, device="cuda", dtype=torch.bfloat16)
        dy[:, -R:] = torch.randn(M, R, device="cuda", generator=gen).to(torch.bfloat16)
        dx = T.qlinear_backward_input(dy, fw, T.BF16)
        # up to 16 rows take the few-row kernel, which skips the bf16 rounding of code*scale as well
        tol = 4e-3 if (M <= 16 and kind != "int8raw") else 2e-5
        assert _rel(dx, dy[:, -R:].float() @ w_bf16) <= tol, (kind, M)
    # fp32 compute type on the same weight
    x = torch.randn(16, K, device="cuda", generator=gen)
    assert _rel(T.qlinear_forward(x, fw, T.F32)[:, -R:], x @ dense_top.t()) <= 1e-4, kind
    for M in (16, 40):                                              # few-row kernel, tiled kernel
        dy = torch.zeros(M, N, device="cuda")
        dy[:, -R:] = torch.randn(M, R, device="cuda", generator=gen)
        assert _rel(T.qlinear_backward_input(dy, fw, T.F32), dy[:, -R:] @ dense_top) <= 1e-4, (kind, M)


def test_quantisers_beyond_2_31_elements():
    # codes and scales of 2^31 + 2^21 elements against the reference's arithmetic restated with torch ops
    # (IEEE fp32 division for max/127, max/7 and 1/scale, one rounding for x * inv, clamp, round half to even;
    # src/caif_cuda_kernels_quant.cu:258-362,384-444,502-559); bit-exact, as at the small sizes the oracle covers
    rows, cols = 262400, 8192
    n = rows * cols
    gen = torch.Generator(device="cuda")
    gen.manual_seed(9)
    x = torch.randn(n, device="cuda", generator=gen)
    x[-5] = 7.5                                                      # the maximum sits beyond 2^31
    # torch divides by a Python scalar through its reciprocal; tensor / tensor is the IEEE division the kernels use
    c127, c7, one = (torch.tensor(v, device="cuda") for v in (127.0, 7.0, 1.0))
    # per tensor
    q, s = T.quantize_int8(x, per_channel=False)
    scale = x.abs().max() / c127
    assert torch.equal(s, scale.reshape(1))
    want = (x * (one / scale)).clamp_(-127.0, 127.0).round_().to(torch.int8)
    assert torch.equal(q, want)
    del q, want
    # per channel: scale[c] over the rows of column c
    x2 = x.view(rows, cols)
    q, s = T.quantize_int8(x2, per_channel=True)
    scale = x2.abs().amax(dim=0) / c127
    assert torch.equal(s, scale)
    want = (x2 * (one / scale)).clamp_(-127.0, 127.0).round_().to(torch.int8)
    assert torch.equal(q, want)
    back = T.dequantize_int8(q, s, per_channel=True)
    assert torch.equal(back, q.float() * s)
    del q, want, back
    # int4, groups of 128 along the flat index
    p, s16 = T.quantize_int4_per_group(x, 128)
    g = x.view(-1, 128)
    s32 = g.abs().amax(dim=1) / c7
    assert torch.equal(s16, s32.to(torch.float16))
    codes = (g * (one / s32).unsqueeze(1)).clamp_(-7.0, 7.0).round_().to(torch.int16).view(-1) & 15
    want = (codes[0::2] | (codes[1::2] << 4)).to(torch.uint8)
    assert torch.equal(p, want)
    del codes, want, g
    back = T.dequantize_int4_per_group(p, s16, n, 128)
    lo, hi = (p & 15).to(torch.int16), (p >> 4).to(torch.int16)
    c = torch.stack([lo, hi], dim=1).reshape(-1)
    c = torch.where(c >= 8, c - 16, c).float()
    assert torch.equal(back, c * s16.float().repeat_interleave(128))
