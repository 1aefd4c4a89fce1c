"""GPU parity of the quantise / pack / cast launchers against the CPU oracle: bit-exact."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from caif_amd import torch_ops as T            # noqa: E402
from gpu_helpers import dev, host, f16_bits     # noqa: E402


def _inputs(rng, n, std=0.02):
    x = rng.normal(0, std, n).astype(np.float32)
    x[rng.integers(0, n, max(1, n // 50))] = 0.0
    return x


@pytest.mark.parametrize("n", [1, 7, 1024, 4099, 1 << 20])
def test_int8_per_tensor_bit_exact(orc, n):
    x = _inputs(np.random.default_rng(n), n)
    q, s = T.quantize_int8(dev(x), per_channel=False)
    qo, so = orc.quantize_int8_per_tensor(x)
    assert np.array_equal(host(s).view(np.uint32), so.view(np.uint32))
    assert np.array_equal(host(q), qo)
    d = T.dequantize_int8(q, s, per_channel=False)
    assert np.array_equal(host(d).view(np.uint32), orc.dequantize_int8_per_tensor(qo, so).view(np.uint32))


@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (32, 64), (37, 64), (70, 12), (257, 129), (1024, 1408), (4096, 4096)])
def test_int8_per_channel_bit_exact(orc, shape):
    rng = np.random.default_rng(shape[0] * 7 + shape[1])
    x = _inputs(rng, shape[0] * shape[1]).reshape(shape)
    if shape[1] > 4:
        x[:, 3] = 0.0                                           # an all-zero column: scale 1.0
    q, s = T.quantize_int8(dev(x), per_channel=True)
    qo, so = orc.quantize_int8_per_channel(x)
    assert np.array_equal(host(s).view(np.uint32), so.view(np.uint32))
    assert np.array_equal(host(q), qo)
    d = T.dequantize_int8(q, s, per_channel=True)
    assert np.array_equal(host(d).view(np.uint32), orc.dequantize_int8_per_channel(qo, so).view(np.uint32))


def test_quantisers_on_buffers_that_are_not_16_byte_aligned(orc):
    # views one element into a buffer: the kernels fall back from 16-byte to element accesses, same bits
    rng = np.random.default_rng(5)
    n, rows, cols = 4099, 37, 64
    x = _inputs(rng, n)
    buf = dev(np.concatenate([[0.0], x]).astype(np.float32))
    q, s = T.quantize_int8(buf[1:], per_channel=False)
    qo, so = orc.quantize_int8_per_tensor(x)
    assert np.array_equal(host(s).view(np.uint32), so.view(np.uint32)) and np.array_equal(host(q), qo)
    m = x[: rows * cols].reshape(rows, cols)
    q, s = T.quantize_int8(buf[1 : 1 + rows * cols].view(rows, cols), per_channel=True)
    qo, so = orc.quantize_int8_per_channel(m)
    assert np.array_equal(host(s).view(np.uint32), so.view(np.uint32)) and np.array_equal(host(q), qo)
    p, s = T.quantize_int4_per_group(buf[1 : 1 + 4096], 128)
    po, so = orc.quantize_to_int4(x[:4096], 128)
    assert np.array_equal(f16_bits(s), so) and np.array_equal(host(p), po)


@pytest.mark.parametrize("n,group", [(4, 4), (5, 2), (512, 128), (128 * 37 + 77, 128), (1000, 24), (4096, 32),
                                      (2049, 64), (1 << 20, 128), (300, 512), (96, 6)])
def test_int4_bit_exact(orc, n, group):
    rng = np.random.default_rng(n + group)
    x = _inputs(rng, n)
    x[: min(group, n)] = 0.0                                    # an all-zero group: scale 0
    p, s = T.quantize_int4_per_group(dev(x), group)
    po, so = orc.quantize_to_int4(x, group)
    assert np.array_equal(f16_bits(s), so)
    assert np.array_equal(host(p), po)
    d = T.dequantize_int4_per_group(p, s, n, group)
    assert np.array_equal(host(d).view(np.uint32), orc.dequantize_int4(po, so, n, group).view(np.uint32))


def test_quantisers_at_the_decode_weight_bit_exact(orc):
    """BASELINE configs[1]'s weight at its real size against the oracle, bit for bit: per-channel int8 on the
    [4096, 14336] buffer the reference labels [in, out] (src/caif_cuda_kernels_quant.cu:488-558; 14336 column
    maxima, seven residue classes of column phase per 16-byte lane) and int4 with groups of 128 on its 58,720,256
    elements (:281-330; 458,752 groups)."""
    rng = np.random.default_rng(14336)
    K, N = 4096, 14336
    w = rng.normal(0, 0.02, (K, N)).astype(np.float32)
    w[rng.integers(0, K, 2000), rng.integers(0, N, 2000)] = 0.0
    wd = dev(w)
    q, s = T.quantize_int8(wd, per_channel=True)
    qo, so = orc.quantize_int8_per_channel(w)
    assert np.array_equal(host(s).view(np.uint32), so.view(np.uint32))
    assert np.array_equal(host(q), qo)
    del q, s, qo, so
    p, s4 = T.quantize_int4_per_group(wd.reshape(-1), 128)
    po, so4 = orc.quantize_to_int4(w.reshape(-1), 128)
    assert np.array_equal(f16_bits(s4), so4)
    assert np.array_equal(host(p), po)


def test_int4_decodes_code_minus_eight(orc):
    rng = np.random.default_rng(3)
    packed = rng.integers(0, 256, 4096, dtype=np.uint8)         # every nibble value incl. 0x8
    scales = rng.uniform(1e-3, 1.0, 64).astype(np.float16)
    d = T.dequantize_int4_per_group(dev(packed), dev(scales), 8192, 128)
    want = orc.dequantize_int4(packed, scales.view(np.uint16), 8192, 128)
    assert np.array_equal(host(d).view(np.uint32), want.view(np.uint32))


def test_golden_kat_on_gpu(orc):
    import json, os
    kat = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "quant_kat.json")))
    for case in kat["int8_per_tensor"]:
        q, s = T.quantize_int8(dev(np.array(case["x"], np.float32)), per_channel=False)
        assert host(s)[0] == np.float32(case["scale"]) and host(q).tolist() == case["q"], case["why"]
    for case in kat["int8_per_channel"]:
        x = np.array(case["x"], np.float32).reshape(case["rows"], case["cols"])
        q, s = T.quantize_int8(dev(x), per_channel=True)
        assert host(s).tolist() == case["scales"] and host(q).reshape(-1).tolist() == case["q"], case["why"]
    for case in kat["int4_group"]:
        p, s = T.quantize_int4_per_group(dev(np.array(case["x"], np.float32)), case["group"])
        assert f16_bits(s).tolist() == case["scales_f16"] and host(p).tolist() == case["packed"], case["why"]
    for case in kat["int4_decode"]:
        d = T.dequantize_int4_per_group(dev(np.array(case["packed"], np.uint8)),
                                        dev(np.array(case["scales_f16"], np.uint16).view(np.float16)),
                                        case["n"], case["group"])
        assert host(d).tolist() == case["out"], case["why"]


def test_casts_bit_exact(orc):
    rng = np.random.default_rng(4)
    u = rng.integers(0, 2**32, size=1 << 18, dtype=np.uint64).astype(np.uint32)
    x = u.view(np.float32)
    x = x[~np.isnan(x)]
    xd = dev(x)
    assert np.array_equal(f16_bits(T.convert(xd, torch.bfloat16)), orc.f32_to_bf16_bits(x))
    assert np.array_equal(f16_bits(T.convert(xd, torch.float16)), orc.f32_to_f16_bits(x))
    bits = np.arange(65536, dtype=np.uint16)
    keep = ~np.isnan(bits.view(np.float16))
    hb = dev(bits[keep].view(np.float16))
    assert np.array_equal(host(T.convert(hb, torch.float32)).view(np.uint32),
                          orc.f16_bits_to_f32(bits[keep]).view(np.uint32))
    bb = torch.from_numpy(bits.view(np.int16).copy()).cuda().view(torch.bfloat16)
    got = host(T.convert(bb, torch.float32)).view(np.uint32)
    assert np.array_equal(got, bits.astype(np.uint32) << 16)
    y = rng.uniform(-200, 200, 5000).astype(np.float32)
    y[:6] = [0.5, 1.5, 2.5, -2.5, 126.5, -127.5]
    assert np.array_equal(host(T.convert(dev(y), torch.int8)), orc.convert_fp32_to_int8(y))
    q = np.arange(-128, 128).astype(np.int8)
    assert np.array_equal(host(T.convert(dev(q), torch.float32)), q.astype(np.float32))


def test_zero_input_exact(orc):
    z = dev(np.zeros((8, 16), np.float32))
    q, s = T.quantize_int8(z, per_channel=False)
    assert host(s)[0] == 1.0 and not host(q).any()
    q, s = T.quantize_int8(z, per_channel=True)
    assert np.all(host(s) == 1.0) and not host(q).any()
    p, sc = T.quantize_int4_per_group(z, 128)
    assert not host(p).any() and not f16_bits(sc).any()
    assert not host(T.dequantize_int4_per_group(p, sc, 128, 128)).any()


def test_error_contracts():
    # wrong dtype / rank / scales length / group 0 / host tensors: tests/test_quantize_ops.cpp:302-402
    x = dev(np.zeros((4, 8), np.float32))
    with pytest.raises(RuntimeError):
        T.quantize_int8(x.half(), per_channel=False)
    with pytest.raises(RuntimeError):
        T.quantize_int8(x.reshape(-1), per_channel=True)
    with pytest.raises(RuntimeError):
        T.quantize_int4_per_group(x, 0)
    with pytest.raises(RuntimeError, match="host backend not supported"):
        T.quantize_int8(x.cpu(), per_channel=False)
    p, s = T.quantize_int4_per_group(x, 8)
    with pytest.raises(RuntimeError):
        T.dequantize_int4_per_group(p, s[:2], 32, 8)
    from caif_amd import capi
    L = capi.lib()
    assert L.caifx_quantize_to_int4(x.data_ptr(), p.data_ptr(), s.data_ptr(), 32, 0, None) == 1
    assert L.caifx_quantize_to_int4(x.data_ptr(), p.data_ptr(), s.data_ptr(), 32, 3, None) == 1
    assert L.caifx_quantize_to_int4(None, None, None, 0, 8, None) == 0       # empty problem: no-op
