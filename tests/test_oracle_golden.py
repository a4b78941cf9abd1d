"""The oracle against the golden vectors written by the compiled reference
(tests/golden/make_golden.py).  CPU only."""
import glob
import hashlib
import json
import os

import numpy as np
import pytest

from fastertnn_amd import synth, TNN, act_is_ternary, weight_is_ternary
from oracle.ftnn_oracle import out_dim, cpack
from tests.cases import make_layer

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
MANIFEST = json.load(open(os.path.join(GOLDEN, "manifest.json")))
FULL = sorted(glob.glob(os.path.join(GOLDEN, "full_*_shape*.npz")))


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def oracle_layer(oracle, typ, x, thr, w, wthr, shape, alpha):
    c, ih, iw, kn, kw, kh, pad, stride = [int(v) for v in shape]
    n = x.shape[0]
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    qw = oracle.pack_weights(w, wthr, wt)
    rows = oracle.quantize_im2row(x, thr, kh, kw, pad, stride, at)
    oh, ow = out_dim(ih, pad, kh, stride), out_dim(iw, pad, kw, stride)
    y = oracle.mm(typ, rows, qw, n, oh, ow, kn, cpack(c) * kh * kw, alpha, c * kh * kw)
    yc = oracle.conv(typ, x, thr, qw, kn, kh, kw, pad, stride, alpha)
    assert yc.tobytes() == y.tobytes()
    return qw, rows, y


@pytest.mark.parametrize("path", FULL, ids=[os.path.basename(p)[5:-4] for p in FULL])
def test_full_vectors(oracle, path):
    g = np.load(path)
    qw, rows, y = oracle_layer(oracle, int(g["type"]), g["x"], g["thr"], g["w"], g["wthr"], g["shape"],
                               float(g["alpha"]))
    assert np.array_equal(qw, g["qw"])
    assert np.array_equal(rows, g["rows"])
    assert y.tobytes() == g["y"].tobytes()


@pytest.mark.parametrize("case", MANIFEST["layers"], ids=[c["name"] for c in MANIFEST["layers"]])
def test_manifest_layers(oracle, case):
    L = make_layer(case["type"], tuple(case["shape"]), case["batch"], case["seed"], case["alpha"])
    assert sha(L["x"]) == case["x"] and sha(L["w"]) == case["w"], "seeded inputs changed"
    qw, rows, y = oracle_layer(oracle, case["type"], L["x"], L["thr"], L["w"], L["wthr"], case["shape"],
                               case["alpha"])
    assert sha(qw) == case["qw"]
    assert sha(rows) == case["rows"]
    assert sha(y) == case["y"]


@pytest.mark.parametrize("case", MANIFEST["gemms"], ids=[c["name"] for c in MANIFEST["gemms"]])
def test_manifest_gemms(oracle, case):
    m, n, p = case["m"], case["n"], case["p"]
    a = synth.ternary(case["seed_a"], (m, p))
    b = synth.ternary(case["seed_b"], (n, p))
    assert sha(a) == case["a"], "seeded inputs changed"
    ap, bp = oracle.pack_gemm_operand(a), oracle.pack_gemm_operand(b)
    assert sha(ap) == case["ap"] and sha(bp) == case["bp"]
    assert sha(oracle.mm(TNN, ap, bp, m, 1, 1, n, p // 64, 0.5)) == case["y_alpha05"]
    assert sha(oracle.gemm(ap, bp, m, n, p // 64)) == case["y_alpha1"]


def test_full_gemm_vector(oracle):
    g = np.load(os.path.join(GOLDEN, "full_gemm_32.npz"))
    ap, bp = oracle.pack_gemm_operand(g["a"]), oracle.pack_gemm_operand(g["b"])
    assert np.array_equal(ap, g["ap"]) and np.array_equal(bp, g["bp"])
    assert oracle.mm(TNN, ap, bp, 32, 1, 1, 32, 4, 0.5).reshape(32, 32).tobytes() == g["y05"].tobytes()
    assert oracle.gemm(ap, bp, 32, 32, 4).tobytes() == g["y1"].tobytes()
