#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ from the COMPILED REFERENCE.

Run in the build container, where `make -C oracle ref` has compiled the
reference's own "final" CPU path from /root/reference into oracle/_ref:

    python tests/golden/make_golden.py

Inputs come from the seeded generators in fastertnn_amd/synth.py (tests/cases.py:
make_layer); every expected output here is produced by the reference's functions
(ternarize_opt_avx2 / binarize_opt_avx2 / bitpacking2, t2r_p2_opt / b2r, mm_*,
tnns_conv), never by the oracle or the HIP library.

Two kinds of fixtures:
  full_*.npz     inputs and expected outputs in full, for tiny cases
  manifest.json  SHA-256 of every buffer (inputs, packed weights, packed rows,
                 fp32 output) for the reference's 12 self-test shapes x 4 types and
                 the benchmark configurations that a CPU finishes in seconds
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from fastertnn_amd import synth, TNN, TBN, BTN, BNN, TYPE_NAMES, act_is_ternary, weight_is_ternary  # noqa: E402
from oracle.ftnn_oracle import Reference, out_dim, cpack  # noqa: E402
from tests.cases import REF_TEST_SHAPES, EXTRA_SHAPES, ALL_TYPES, make_layer  # noqa: E402

# benchmark configurations small enough for the CPU (C, IH, IW, KN, KW, KH, pad, stride), batch
BENCH_LAYERS = {
    "cfg2_tnn_conv": (TNN, (256, 56, 56, 256, 3, 3, 1, 1), 1),
    "cfg3_tbn_conv": (TBN, (128, 28, 28, 128, 3, 3, 1, 1), 8),
    "cfg3_btn_conv": (BTN, (128, 28, 28, 128, 3, 3, 1, 1), 8),
    "stem_7x7_s2": (TNN, (3, 64, 64, 64, 7, 7, 3, 2), 2),
    "proj_1x1_s2": (TNN, (64, 28, 28, 128, 1, 1, 0, 2), 2),
    "fc_512_1000": (TNN, (512, 1, 1, 1000, 1, 1, 0, 1), 32),
}


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def run_reference(ref, L):
    typ = L["type"]
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    qw = ref.pack_weights(L["w"], L["wthr"], wt)
    rows = ref.quantize_im2row(L["x"], L["thr"], L["kh"], L["kw"], L["pad"], L["stride"], at)
    oh = out_dim(L["ih"], L["pad"], L["kh"], L["stride"])
    ow = out_dim(L["iw"], L["pad"], L["kw"], L["stride"])
    k = cpack(L["c"]) * L["kh"] * L["kw"]
    y = ref.mm(typ, rows, qw, L["batch"], oh, ow, L["kn"], k, L["alpha"], L["c"] * L["kh"] * L["kw"])
    y2 = ref.conv(typ, L["x"], L["thr"], qw, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"])
    assert y.tobytes() == y2.tobytes(), "reference mm_* and tnns_conv disagree"
    return qw, rows, y.reshape(L["batch"], L["kn"], oh, ow)


def main():
    ref = Reference()
    manifest = {"layers": [], "gemms": []}

    # ---- full dumps: tiny layers, all four types
    for typ in ALL_TYPES:
        for si, batch in ((0, 2), (1, 2), (2, 1), (10, 4)):
            L = make_layer(typ, REF_TEST_SHAPES[si], batch, seed=7000 + 10 * si + typ)
            qw, rows, y = run_reference(ref, L)
            name = "full_%s_shape%d_b%d" % (TYPE_NAMES[typ], si, batch)
            np.savez_compressed(os.path.join(HERE, name + ".npz"), type=np.int32(typ),
                                shape=np.array(L["shape"], np.int32), alpha=np.float32(L["alpha"]),
                                x=L["x"], thr=L["thr"], w=L["w"], wthr=L["wthr"], qw=qw, rows=rows, y=y)

    # ---- manifest: reference self-test shapes, edge shapes, benchmark layers
    cases = []
    for typ in ALL_TYPES:
        for si, shape in enumerate(REF_TEST_SHAPES + EXTRA_SHAPES):
            cases.append(("%s_shape%d_b8" % (TYPE_NAMES[typ], si), typ, shape, 8, 9000 + 31 * si + typ))
    for name, (typ, shape, batch) in BENCH_LAYERS.items():
        cases.append((name, typ, shape, batch, 9900 + len(cases)))
    for name, typ, shape, batch, seed in cases:
        L = make_layer(typ, shape, batch, seed)
        qw, rows, y = run_reference(ref, L)
        manifest["layers"].append({"name": name, "type": typ, "shape": list(shape), "batch": batch,
                                   "seed": seed, "alpha": L["alpha"], "x": sha(L["x"]), "w": sha(L["w"]),
                                   "qw": sha(qw), "rows": sha(rows), "y": sha(y)})
        print(name, "ok", flush=True)

    # ---- GEMM operands (bitpacking2 + mm_tnn, alpha 0.5 and the alpha=1 of tnns_gemm)
    for name, m, n, p in (("gemm_32", 32, 32, 256), ("gemm_cfg1", 256, 256, 4096), ("gemm_ragged", 37, 21, 768)):
        a = synth.ternary(4242 + m, (m, p))
        b = synth.ternary(4243 + n, (n, p))
        ap, bp = ref.pack_gemm_operand(a), ref.pack_gemm_operand(b)
        y05 = ref.mm(TNN, ap, bp, m, 1, 1, n, p // 64, 0.5)
        y1 = ref.mm(TNN, ap, bp, m, 1, 1, n, p // 64, 1.0)
        assert np.array_equal(y1.reshape(m, n), a @ b.T)
        manifest["gemms"].append({"name": name, "m": m, "n": n, "p": p, "seed_a": 4242 + m, "seed_b": 4243 + n,
                                  "a": sha(a), "ap": sha(ap), "bp": sha(bp), "y_alpha05": sha(y05),
                                  "y_alpha1": sha(y1)})
        if name == "gemm_32":
            np.savez_compressed(os.path.join(HERE, "full_gemm_32.npz"), a=a, b=b, ap=ap, bp=bp,
                                y05=y05.reshape(m, n), y1=y1.reshape(m, n))
        print(name, "ok", flush=True)

    with open(os.path.join(HERE, "manifest.json"), "w") as f:
        json.dump(manifest, f, indent=1)


if __name__ == "__main__":
    main()
