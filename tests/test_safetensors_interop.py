"""The host layer's SafeTensors writer and reader against an independent implementation of the format.

`tests/cpp/bin/test_safetensors_quantized` (built by __graft_entry__.build()) writes and dumps files;
the `safetensors` Python package (the format's own library) reads and writes the same files, so a
mistake in the length prefix, the header text, the offsets or the byte order fails here even if the
C++ writer and reader agree with each other.  The package does not know the "I4" tag (it is the
reference's own, include/caif/caif_serialization_constants.h:219), so the packed-int4 entry is
checked at the level of the format's definition: 8-byte little-endian header length, JSON header,
payload bytes at the stated offsets.  No GPU is involved.
"""
import json
import os
import struct
import subprocess

import numpy as np
import pytest
import torch
from safetensors import safe_open
from safetensors.torch import load_file, save_file

EXE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "bin", "test_safetensors_quantized")

FIXED = [("layer.0.weight", torch.int8, (3, 4), 1, 1), ("bytes", torch.uint8, (5,), 2, 1), ("half", torch.float16, (2, 2), 3, 2),
         ("single", torch.float32, (3,), 4, 4), ("brain", torch.bfloat16, (4,), 5, 2), ("ints", torch.int32, (2,), 6, 4)]


def _run(*args):
    if not os.path.exists(EXE):
        pytest.fail(f"{EXE} is missing: run `python -c 'import __graft_entry__ as g; g.build()'`")
    p = subprocess.run([EXE, *args], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stdout[-2000:] + p.stderr[-2000:]
    return p.stdout


def _fixed_bytes(dtype, shape, seed, esize):
    n = int(np.prod(shape)) * esize
    out = bytearray(n)
    for i in range(n):
        v = (17 * i + seed) % 251
        if dtype.is_floating_point and i % esize == esize - 1:
            v &= 0x3F
        out[i] = v
    return bytes(out)


def _raw(t):
    return t.contiguous().view(torch.uint8).numpy().tobytes() if t.dtype != torch.uint8 else t.numpy().tobytes()


def test_file_written_by_the_host_layer_loads_in_the_safetensors_package(tmp_path):
    path = str(tmp_path / "from_cpp.safetensors")
    _run("--write", path)
    got = load_file(path)
    assert sorted(got) == sorted(name for name, *_ in FIXED)
    for name, dtype, shape, seed, esize in FIXED:
        assert got[name].dtype == dtype and tuple(got[name].shape) == shape, name
        assert _raw(got[name]) == _fixed_bytes(dtype, shape, seed, esize), name
    with safe_open(path, framework="pt") as f:
        assert f.metadata() == {"format": "pt", "note": 'quote " backslash \\ tab \t'}


def test_file_written_by_the_safetensors_package_is_read_by_the_host_layer(tmp_path):
    path = str(tmp_path / "from_python.safetensors")
    g = torch.Generator().manual_seed(5)
    tensors = {
        "model.layers.0.mlp.up_proj.weight": torch.randint(-127, 128, (6, 8), generator=g, dtype=torch.int8),
        "model.layers.0.mlp.up_proj.scales": torch.rand(6, generator=g, dtype=torch.float32),
        "packed": torch.randint(0, 256, (7,), generator=g, dtype=torch.uint8),
        "h": torch.randn(3, 2, generator=g).to(torch.float16),
        "b": torch.randn(5, generator=g).to(torch.bfloat16),
        "i": torch.tensor([-5, 70000], dtype=torch.int32),
    }
    meta = {"format": "pt", "up_proj.int8_scheme": "per_channel", "odd": 'a"b\\c'}
    save_file(tensors, path, metadata=meta)
    lines = _run("--read", path).splitlines()
    seen, seen_meta = {}, {}
    for line in lines:
        parts = line.split("|")
        if parts[0] == "meta":
            seen_meta[parts[1]] = "|".join(parts[2:])
        else:
            seen[parts[0]] = parts[1:]
    tag = {torch.int8: "I8", torch.float32: "F32", torch.uint8: "U8", torch.float16: "F16", torch.bfloat16: "BF16", torch.int32: "I32"}
    assert sorted(seen) == sorted(tensors)
    for name, t in tensors.items():
        dtype, shape, hexbytes = seen[name]
        assert dtype == tag[t.dtype] and shape == ",".join(str(d) for d in t.shape), name
        assert bytes.fromhex(hexbytes) == _raw(t), name
    assert seen_meta == meta


def test_packed_int4_entry_follows_the_format_definition(tmp_path):
    path = str(tmp_path / "quantized.safetensors")
    _run("--write-quantized", path)
    blob = open(path, "rb").read()
    (hlen,) = struct.unpack("<Q", blob[:8])
    assert hlen % 8 == 0 and 8 + hlen <= len(blob)
    header = json.loads(blob[8:8 + hlen].decode("utf-8"))
    meta = header.pop("__metadata__")
    assert meta == {"ffn.group_size": "128", "ffn.int8_scheme": "per_channel"}
    odd = 'blk "q"\\w\n'
    assert header["ffn.weight"] == {"dtype": "I8", "shape": [3, 4], "data_offsets": [0, 12]}
    assert header[odd] == {"dtype": "I4", "shape": [3, 5], "data_offsets": [12, 20]}          # ceil(15 / 2) bytes
    assert header["ffn.scales"] == {"dtype": "F16", "shape": [2], "data_offsets": [20, 24]}
    assert header["t.scales"] == {"dtype": "F32", "shape": [1], "data_offsets": [24, 28]}
    data = blob[8 + hlen:]
    assert len(data) == 28
    assert np.frombuffer(data[0:12], np.int8).tolist() == [-127, -1, 0, 1, 2, 3, 4, 5, 6, 7, 8, 127]
    packed = np.frombuffer(data[12:20], np.uint8)
    lo, hi = packed & 0xF, packed >> 4                                                       # low nibble = even flat index
    codes = np.stack([lo, hi], 1).reshape(-1)[:15].astype(np.int8)
    codes = np.where(codes >= 8, codes - 16, codes)
    assert codes.tolist() == [1, 2, 3, 4, 5, 6, 7, -8, -7, -6, -5, -4, -3, -2, -1] and int(hi[-1]) == 0
    assert np.frombuffer(data[20:24], np.float16).tolist() == [1.0, np.float16(0.1).item()]
    assert np.frombuffer(data[24:28], np.float32).tolist() == [0.015625]
