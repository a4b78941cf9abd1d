"""HIP library against the golden vectors of the compiled reference (no oracle involved)."""
import glob
import hashlib
import json
import os

import numpy as np
import pytest

from fastertnn_amd import synth, TNN, act_is_ternary, weight_is_ternary
from tests.cases import make_layer

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
MANIFEST = json.load(open(os.path.join(GOLDEN, "manifest.json")))
FULL = sorted(glob.glob(os.path.join(GOLDEN, "full_*_shape*.npz")))


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def hip_layer(hip, typ, x, thr, w, wthr, shape, alpha):
    c, ih, iw, kn, kw, kh, pad, stride = [int(v) for v in shape]
    n = x.shape[0]
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    qw = hip.pack_weights(_dev(w), _dev(wthr), wt)
    rows = hip.quantize_im2row(_dev(x), _dev(thr), kh, kw, pad, stride, at)
    oh, ow = hip.out_dim(ih, pad, kh, stride), hip.out_dim(iw, pad, kw, stride)
    y = hip.mm(typ, rows, qw, n, oh, ow, kn, ((c + 63) // 64) * kh * kw, alpha, c * kh * kw)
    yc = hip.conv(typ, _dev(x), _dev(thr), qw, kn, kh, kw, pad, stride, alpha)
    y = y.cpu().numpy()
    assert yc.cpu().numpy().tobytes() == y.tobytes()
    return qw.cpu().numpy(), rows.cpu().numpy(), y


@pytest.mark.parametrize("path", FULL, ids=[os.path.basename(p)[5:-4] for p in FULL])
def test_full_vectors(hip, path):
    g = np.load(path)
    print("case", os.path.basename(path), flush=True)
    qw, rows, y = hip_layer(hip, int(g["type"]), g["x"], g["thr"], g["w"], g["wthr"], g["shape"], float(g["alpha"]))
    assert np.array_equal(qw, g["qw"])
    assert np.array_equal(rows, g["rows"])
    assert y.tobytes() == g["y"].tobytes()
    # the reference's host-memory entry point on the same vectors
    c, ih, iw, kn, kw, kh, pad, stride = [int(v) for v in g["shape"]]
    yh = hip.host_conv(int(g["type"]), g["x"], g["thr"], g["qw"], kn, kh, kw, pad, stride, float(g["alpha"]))
    assert yh.tobytes() == g["y"].tobytes()


@pytest.mark.parametrize("case", MANIFEST["layers"], ids=[c["name"] for c in MANIFEST["layers"]])
def test_manifest_layers(hip, case):
    print("case", case["name"], flush=True)
    L = make_layer(case["type"], tuple(case["shape"]), case["batch"], case["seed"], case["alpha"])
    assert sha(L["x"]) == case["x"] and sha(L["w"]) == case["w"], "seeded inputs changed"
    qw, rows, y = hip_layer(hip, case["type"], L["x"], L["thr"], L["w"], L["wthr"], case["shape"], case["alpha"])
    assert sha(qw) == case["qw"]
    assert sha(rows) == case["rows"]
    assert sha(y) == case["y"]


@pytest.mark.parametrize("case", MANIFEST["gemms"], ids=[c["name"] for c in MANIFEST["gemms"]])
def test_manifest_gemms(hip, case):
    print("case", case["name"], flush=True)
    m, n, p = case["m"], case["n"], case["p"]
    a = synth.ternary(case["seed_a"], (m, p))
    b = synth.ternary(case["seed_b"], (n, p))
    ap, bp = hip.pack_gemm_operand(_dev(a)), hip.pack_gemm_operand(_dev(b))
    assert sha(ap.cpu().numpy()) == case["ap"] and sha(bp.cpu().numpy()) == case["bp"]
    assert sha(hip.mm(TNN, ap, bp, m, 1, 1, n, p // 64, 0.5).cpu().numpy()) == case["y_alpha05"]
    # tnns_gemm (alpha fixed to 1), both ownership branches (src/tnns/tnns_cpu_mm_p2.c:126-132)
    aph, bph = ap.cpu().numpy(), bp.cpu().numpy()
    assert sha(hip.host_gemm(aph, bph, m, n, p // 64)) == case["y_alpha1"]
    into = np.full((m, n), -7.0, np.float32)
    hip.host_gemm(aph, bph, m, n, p // 64, into=into)
    assert sha(into) == case["y_alpha1"]
