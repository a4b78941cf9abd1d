"""The reference's OWN layer driver (src/timing_layers.c, compiled unchanged into
oracle/_ref/ref_timing_layers and linked against libftnn_hip.so instead of the reference's
CPU objects) run in its self-test mode: for its 12 test shapes it calls tnns_conv, computes
its fp32 direct convolution and abort()s on a mismatch (src/timing_layers.c:142-165)."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "oracle", "_ref", "ref_timing_layers")


@pytest.mark.parametrize("net", ["tnn", "tbn", "btn", "bnn"])
def test_reference_driver_self_test_passes_on_the_hip_library(net, tmp_path):
    if not os.path.exists(DRIVER):
        pytest.skip("NOT RUN: oracle/_ref/ref_timing_layers is absent (it is compiled from the reference tree, which "
                    "this machine lacks, and travels as a built file); tests/test_gpu_harness.py runs the same 12 "
                    "shapes through the repository's own driver")
    os.makedirs(tmp_path / "out" / "measurements")
    print("case reference driver", net, flush=True)
    r = subprocess.run([DRIVER, "final", net, "test"], cwd=str(tmp_path), capture_output=True, text=True,
                       timeout=280)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "SHAPE 11" in r.stdout
    csv = [f for f in os.listdir(tmp_path / "out" / "measurements") if f.endswith(".csv")]
    assert len(csv) == 1
    lines = open(tmp_path / "out" / "measurements" / csv[0]).read().strip().splitlines()
    assert lines[0] == "TNNs-type, Version, Shape-type, Shape, Runtime" and len(lines) == 13
