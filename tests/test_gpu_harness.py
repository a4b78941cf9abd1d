"""The repository's own timing drivers (harness/ftnn_timing_layers, harness/ftnn_timing_gemm): the command line,
constants and CSV files of the reference's drivers (src/timing_layers.c:46-48,83-94,209,226-261;
src/timing_gemm.c:25-46,73-81,90-97) on device-resident tensors.  Every mode runs through the C ABI of the library;
the self-test mode checks each layer against a plain fp32 direct convolution and aborts on a mismatch.  The
reference's own drivers, linked against the same library, run beside them in every mode where their build is
present."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LAYERS = os.path.join(ROOT, "harness", "ftnn_timing_layers")
GEMM = os.path.join(ROOT, "harness", "ftnn_timing_gemm")
REF_LAYERS = os.path.join(ROOT, "oracle", "_ref", "ref_timing_layers")
REF_GEMM = os.path.join(ROOT, "oracle", "_ref", "ref_timing_gemm")

LAYER_HEADER = ["TNNs-type", "Version", "Shape-type", "Shape", "Runtime"]
EXTRA = ["Device-ms", "GMAC", "GMAC/s", "Engine", "Roofline-frac"]


def run(cmd, cwd, timeout=280):
    print("case", " ".join(os.path.basename(c) if os.sep in c else c for c in cmd), flush=True)
    r = subprocess.run(cmd, cwd=str(cwd), capture_output=True, text=True, timeout=timeout)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    return r.stdout


def read_csv(folder):
    files = [f for f in os.listdir(folder) if f.endswith(".csv")]
    assert len(files) == 1, files
    rows = [[c.strip() for c in l.split(",")] for l in open(os.path.join(folder, files[0])).read().strip().splitlines()]
    return rows[0], rows[1:]


def test_drivers_are_built():
    """built by __graft_entry__.build() beside their sources; a missing driver is a failure, not a skip"""
    assert os.access(LAYERS, os.X_OK) and os.access(GEMM, os.X_OK)


@pytest.mark.parametrize("net", ["tnn", "tbn", "btn", "bnn"])
def test_self_test_mode(net, tmp_path):
    out = run([LAYERS, "hip", net, "test"], tmp_path)
    assert "SHAPE 11" in out
    header, rows = read_csv(tmp_path / "out" / "measurements")
    assert header == LAYER_HEADER + EXTRA and len(rows) == 12
    for i, r in enumerate(rows):
        assert r[:4] == [net.upper(), "hip", "TEST", str(i)] and float(r[4]) > 0 and float(r[5]) > 0


@pytest.mark.parametrize("net", ["tnn", "btn"])
def test_layer_mode(net, tmp_path):
    run([LAYERS, "hip", net, "layer"], tmp_path)
    header, rows = read_csv(tmp_path / "out" / "measurements")
    assert header == LAYER_HEADER + EXTRA and len(rows) == 17      # include/timing/shapes_layers.h
    for i, r in enumerate(rows):
        assert r[:4] == [net.upper(), "hip", "LAYER", str(i)]
        wall_s, dev_ms, gmac, rate, engine, frac = float(r[4]), float(r[5]), float(r[6]), float(r[7]), r[8], float(r[9])
        assert 0 < dev_ms * 1e-3 <= wall_s * 1.05 and gmac > 0 and engine in ("valu", "mfma_f4") and 0 < frac < 1
        if gmac >= 1.0:   # below that the printed digits of GMAC and Device-ms round too coarsely to compare
            assert abs(rate - gmac / (dev_ms * 1e-3)) <= 0.02 * rate
    assert abs(float(rows[11][6]) - 59.19) < 0.01                 # the 1024-channel 56 x 56 layer at batch 8


def test_e2e_mode(tmp_path):
    run([LAYERS, "hip", "tnn", "e2e"], tmp_path)
    header, rows = read_csv(tmp_path / "out" / "measurements")
    assert header == LAYER_HEADER + EXTRA and len(rows) == 7       # include/timing/shapes_e2e.h:407-410
    gmac = [float(r[6]) for r in rows]
    assert abs(gmac[0] - 50.5) < 0.1 and abs(gmac[6] - 349.8) < 0.1   # ResNet-18 and ResNet-152 at batch 8
    for i, r in enumerate(rows):
        assert r[:4] == ["TNN", "hip", "E2E", str(i)] and 0 < float(r[5]) < 50.0


def test_gemm_sweep(tmp_path):
    out = run([GEMM, "hip"], tmp_path)
    header, rows = read_csv(tmp_path / "out" / "measurements" / "gemm")
    assert header == ["m", "n", "p", "Runtime", "Type", "Device-ms", "GMAC/s", "Engine", "Roofline-frac"]
    assert [int(r[0]) for r in rows] == [32, 64, 128, 256, 512, 1024, 2048, 4096]
    for r in rows:
        assert r[0] == r[1] and int(r[2]) == 8 * int(r[0]) and r[4] == "hip" and float(r[3]) > 0 and 0 < float(r[8]) < 1
    assert rows[-1][7] == "mfma_f4" and "4096" in out


def test_bad_command_lines_are_refused(tmp_path):
    for cmd in ([LAYERS], [LAYERS, "hip", "xnn", "layer"], [LAYERS, "hip", "tnn", "all"], [GEMM]):
        r = subprocess.run(cmd, cwd=str(tmp_path), capture_output=True, text=True, timeout=60)
        assert r.returncode != 0 and ("Usage" in r.stdout or "Invalid" in r.stdout)


# ---- the reference's own drivers on the same library, in the modes its self-test does not cover ----

def _need(path):
    if not os.path.exists(path):
        pytest.skip("NOT RUN: %s is absent (it is compiled from the reference tree, which this machine lacks, "
                    "and travels as a built file)" % os.path.relpath(path, ROOT))


@pytest.mark.parametrize("mode,count", [("layer", 17), ("e2e", 7)])
def test_reference_layer_driver_other_modes(mode, count, tmp_path):
    _need(REF_LAYERS)
    os.makedirs(tmp_path / "out" / "measurements")
    run([REF_LAYERS, "final", "tnn", mode], tmp_path, timeout=560)
    header, rows = read_csv(tmp_path / "out" / "measurements")
    assert header == LAYER_HEADER and len(rows) == count
    assert all(r[:3] == ["TNN", "final", mode.upper()] and float(r[4]) > 0 for r in rows)


def test_reference_gemm_driver(tmp_path):
    _need(REF_GEMM)
    os.makedirs(tmp_path / "out" / "measurements" / "gemm")
    run([REF_GEMM, "final"], tmp_path, timeout=560)
    header, rows = read_csv(tmp_path / "out" / "measurements" / "gemm")
    assert header == ["m", "n", "p", "Runtime", "Type"] and [int(r[0]) for r in rows] == [32, 64, 128, 256, 512, 1024, 2048, 4096]


# ---- the same drivers with the reference's operand packers (bitpacking2, ternarize_opt_avx2, binarize_opt_avx2) taken
# from the library as well: the reference's utils.c compiled with those three names renamed (oracle/Makefile) ----
REF_LAYERS_DEVPACK = REF_LAYERS + "_devpack"
REF_GEMM_DEVPACK = REF_GEMM + "_devpack"


@pytest.mark.parametrize("net", ["tnn", "tbn", "btn", "bnn"])
def test_reference_self_test_with_the_librarys_weight_packers(net, tmp_path):
    """the driver packs its weights with the library's ternarize_opt_avx2 / binarize_opt_avx2, runs tnns_conv on them and
    abort()s unless the result equals its fp32 direct convolution (src/timing_layers.c:127-165)"""
    _need(REF_LAYERS_DEVPACK)
    os.makedirs(tmp_path / "out" / "measurements")
    out = run([REF_LAYERS_DEVPACK, "final", net, "test"], tmp_path)
    assert "SHAPE 11" in out


def test_reference_gemm_driver_with_the_librarys_bitpacking2(tmp_path):
    """the sweep up to 4096 x 4096 x 32768 with both operands of every size packed by the library's bitpacking2 (the
    reference's scalar packer takes seconds on the largest); wall time of both forms is printed"""
    import time
    _need(REF_GEMM_DEVPACK)
    os.makedirs(tmp_path / "out" / "measurements" / "gemm")
    t0 = time.perf_counter()
    run([REF_GEMM_DEVPACK, "final"], tmp_path, timeout=560)
    dt = time.perf_counter() - t0
    header, rows = read_csv(tmp_path / "out" / "measurements" / "gemm")
    assert header == ["m", "n", "p", "Runtime", "Type"] and [int(r[0]) for r in rows] == [32, 64, 128, 256, 512, 1024, 2048, 4096]
    print("reference GEMM driver with the library's bitpacking2: %.2f s of wall time" % dt)
