"""The oracle against the compiled reference (oracle/_ref/libref_final.so), buffer by
buffer.  Runs wherever that library is present; the same comparison is frozen in
tests/golden/ for machines without it.  CPU only."""
import numpy as np
import pytest

from fastertnn_amd import synth, TNN, TBN, BTN, BNN, TYPE_NAMES, act_is_ternary, weight_is_ternary
from oracle.ftnn_oracle import out_dim, cpack
from tests.cases import ALL_TYPES, EXTRA_SHAPES, REF_TEST_SHAPES, make_layer

SHAPES = REF_TEST_SHAPES + EXTRA_SHAPES


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
@pytest.mark.parametrize("si", range(len(SHAPES)))
def test_every_buffer_matches(oracle, reference, typ, si):
    for batch in (8, 1):
        L = make_layer(typ, SHAPES[si], batch, seed=300 + 7 * si + typ)
        at, wt = act_is_ternary(typ), weight_is_ternary(typ)
        qw_o = oracle.pack_weights(L["w"], L["wthr"], wt)
        qw_r = reference.pack_weights(L["w"], L["wthr"], wt)
        assert np.array_equal(qw_o, qw_r), "packed weights"
        a_o = oracle.quantize_im2row(L["x"], L["thr"], L["kh"], L["kw"], L["pad"], L["stride"], at)
        a_r = reference.quantize_im2row(L["x"], L["thr"], L["kh"], L["kw"], L["pad"], L["stride"], at)
        assert np.array_equal(a_o, a_r), "packed activations"
        oh, ow = out_dim(L["ih"], L["pad"], L["kh"], L["stride"]), out_dim(L["iw"], L["pad"], L["kw"], L["stride"])
        k, ku = cpack(L["c"]) * L["kh"] * L["kw"], L["c"] * L["kh"] * L["kw"]
        y_o = oracle.mm(typ, a_o, qw_o, batch, oh, ow, L["kn"], k, L["alpha"], ku)
        y_r = reference.mm(typ, a_r, qw_r, batch, oh, ow, L["kn"], k, L["alpha"], ku)
        assert y_o.tobytes() == y_r.tobytes(), "GEMM output"
        yc_r = reference.conv(typ, L["x"], L["thr"], qw_r, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"])
        assert yc_r.tobytes() == y_o.tobytes(), "tnns_conv output"


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
def test_reference_self_test_protocol(oracle, reference, typ):
    """src/timing_layers.c:142-165: inputs already in {-1,0,1}/{-1,1}, thresholds 0.5/0.0,
    compared with the reference's fp32 direct convolution (pad value +1 for binary inputs)"""
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    for si in (1, 5, 9):
        c, ih, iw, kn, kw, kh, pad, stride = REF_TEST_SHAPES[si]
        x = synth.ternary(si, (8, c, ih, iw)) if at else synth.binary(si, (8, c, ih, iw))
        w = synth.ternary(si + 50, (kn, c, kh, kw)) if wt else synth.binary(si + 50, (kn, c, kh, kw))
        thr = np.full(8, 0.5 if at else 0.0, np.float32)
        wthr = np.full(kn, 0.5 if wt else 0.0, np.float32)
        want = reference.direct_conv(x, w, pad, stride, 0.5, 0 if at else 1)
        got = oracle.conv(typ, x, thr, oracle.pack_weights(w, wthr, wt), kn, kh, kw, pad, stride, 0.5)
        assert np.array_equal(got, want)


def test_gemm_operands_and_tnns_gemm(oracle, reference):
    for (m, n, p) in [(32, 32, 256), (64, 48, 1024), (5, 7, 512)]:
        a, b = synth.ternary(1, (m, p)), synth.ternary(2, (n, p))
        ao, ar = oracle.pack_gemm_operand(a), reference.pack_gemm_operand(a)
        bo, br = oracle.pack_gemm_operand(b), reference.pack_gemm_operand(b)
        assert np.array_equal(ao, ar) and np.array_equal(bo, br)
        assert oracle.gemm(ao, bo, m, n, p // 64).tobytes() == reference.mm(TNN, ar, br, m, 1, 1, n, p // 64, 1.0).tobytes()


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
def test_independent_baseline_pipeline_agrees(oracle, reference_baseline, typ):
    """the reference's Packing-0 "baseline" build (ternarise -> img2row -> popcount GEMM -> PReLU as
    four passes, src/tnns/tnns_cpu_naive.c:255-292) shares no kernel code with the Packing-2 path;
    its layer output must equal the oracle's bit for bit"""
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    for si in (0, 1, 2, 4, 5, 6, 9, 10, 12, 13, 18, 20):
        L = make_layer(typ, SHAPES[si], 4, seed=900 + si)
        qw0 = reference_baseline.pack_weights(L["w"], L["wthr"], wt)
        try:
            want = reference_baseline.conv(typ, L["x"], L["thr"], qw0, L["kn"], L["kh"], L["kw"], L["pad"],
                                           L["stride"], L["alpha"])
        finally:
            reference_baseline.free_weights(qw0)
        got = oracle.conv(typ, L["x"], L["thr"], oracle.pack_weights(L["w"], L["wthr"], wt), L["kn"], L["kh"],
                          L["kw"], L["pad"], L["stride"], L["alpha"])
        assert got.tobytes() == want.tobytes(), SHAPES[si]
