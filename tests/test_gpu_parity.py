"""HIP library vs the oracle on identical seeded inputs, through the C ABI (bit-exact)."""
import numpy as np
import pytest

from fastertnn_amd import TNN, TBN, BTN, BNN, TYPE_NAMES, act_is_ternary, weight_is_ternary
from tests.cases import REF_TEST_SHAPES, EXTRA_SHAPES, ALL_TYPES, make_layer

pytestmark = pytest.mark.gpu


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _same_bits(got, want, what):
    got = np.ascontiguousarray(got).reshape(-1)
    want = np.ascontiguousarray(want).reshape(-1)
    assert got.dtype == want.dtype and got.size == want.size, what
    if got.tobytes() != want.tobytes():
        bad = np.flatnonzero(got.view("u%d" % got.itemsize) != want.view("u%d" % want.itemsize))
        raise AssertionError("%s: %d of %d elements differ, first at %s: got %s want %s" % (
            what, bad.size, got.size, bad[:4].tolist(), got[bad[:4]].tolist(), want[bad[:4]].tolist()))


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
@pytest.mark.parametrize("si", range(len(REF_TEST_SHAPES) + len(EXTRA_SHAPES)))
@pytest.mark.parametrize("batch", [8, 1])
def test_layer_device_api(hip, oracle, typ, si, batch):
    """every stage of one layer: weight pack, quantise+im2row, GEMM, fused conv"""
    shape = (REF_TEST_SHAPES + EXTRA_SHAPES)[si]
    L = make_layer(typ, shape, batch, seed=1000 + 17 * si + typ)
    print("case", TYPE_NAMES[typ], shape, "batch", batch, flush=True)
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    qw_o = oracle.pack_weights(L["w"], L["wthr"], wt)
    a_o = oracle.quantize_im2row(L["x"], L["thr"], L["kh"], L["kw"], L["pad"], L["stride"], at)
    oh = hip.out_dim(L["ih"], L["pad"], L["kh"], L["stride"])
    ow = hip.out_dim(L["iw"], L["pad"], L["kw"], L["stride"])
    k = ((L["c"] + 63) // 64) * L["kh"] * L["kw"]
    ku = L["c"] * L["kh"] * L["kw"]
    y_o = oracle.mm(typ, a_o, qw_o, batch, oh, ow, L["kn"], k, L["alpha"], ku)

    x_d, thr_d = _dev(L["x"]), _dev(L["thr"])
    qw_d = hip.pack_weights(_dev(L["w"]), _dev(L["wthr"]), wt)
    _same_bits(qw_d.cpu().numpy(), qw_o, "packed weights")
    a_d = hip.quantize_im2row(x_d, thr_d, L["kh"], L["kw"], L["pad"], L["stride"], at)
    _same_bits(a_d.cpu().numpy(), a_o, "packed activations")
    y_d = hip.mm(typ, a_d, qw_d, batch, oh, ow, L["kn"], k, L["alpha"], ku)
    _same_bits(y_d.cpu().numpy(), y_o, "GEMM output")
    yc_d = hip.conv(typ, x_d, thr_d, qw_d, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"])
    _same_bits(yc_d.cpu().numpy(), y_o, "conv output")
    prepared = hip.prepare_conv_weights(typ, qw_d, L["c"], L["kn"], L["kh"], L["kw"])
    yp_d = hip.conv_prepared(typ, x_d, thr_d, prepared, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"])
    _same_bits(yp_d.cpu().numpy(), y_o, "conv output, prepared weights")
    for eng in (hip.ENGINE_VALU, hip.ENGINE_MFMA_F4):   # the layer on each engine explicitly
        ye_d = hip.conv(typ, x_d, thr_d, qw_d, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"],
                        engine=eng)
        _same_bits(ye_d.cpu().numpy(), y_o, "conv output, engine %d" % eng)
