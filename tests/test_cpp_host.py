"""Runs the C++ host-layer test programs (tests/cpp/*.cpp, built by __graft_entry__.build()).

The programs exercise the reference-named classes (CAIF_Ops, CAIF_DeviceFrozenLinear,
CAIF_DeviceFrozenLinearFactory, CAIF_DeviceMoEFrozenExpert, CAIF_SafeTensorsFormat) over the C ABI.  Without a GPU only the
checks that need no device run (`--cpu`); with one, everything."""
import os
import subprocess

import pytest

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "bin")
PROGRAMS = ["test_quantize_ops", "test_device_frozen_linear", "test_device_moe_frozen_expert", "test_moe_routing",
            "test_safetensors_quantized"]


def _run(name, args):
    exe = os.path.join(BIN, name)
    if not os.path.exists(exe):
        pytest.fail(f"{exe} is missing: run `python -c 'import __graft_entry__ as g; g.build()'`")
    p = subprocess.run([exe] + args, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stdout[-4000:] + p.stderr[-2000:]
    assert "[FAIL]" not in p.stdout
    return p.stdout


@pytest.mark.parametrize("name", PROGRAMS)
def test_host_contracts_without_device(name):
    out = _run(name, ["--cpu"])
    assert "[PASS]" in out


@pytest.mark.gpu
@pytest.mark.parametrize("name", PROGRAMS)
def test_host_layer_on_gpu(name):
    out = _run(name, [])
    assert "[SKIP]" not in out and out.count("[PASS]") >= 8
