"""First layers with few input channels (C <= 8) on the fp4 engine: one kernel from fp32 input to result
(fastertnn_amd/csrc/stem_kernels.hip).  Every channel count (each has its own word layout: T = 64 / C taps per
word, the upper half of a word starting mid-tap when C does not divide 32), every type, windows whose taps do and
do not fill their last word, tiles that overhang the image, kernel counts that are no multiple of 32; fp32 results
and all hand-over forms; and the smaller tile and the two-kernel form that take over when the input patch of a tile exceeds the LDS."""
import numpy as np
import pytest

from fastertnn_amd import synth, TNN, TBN, BTN, BNN, TYPE_NAMES, act_is_ternary, weight_is_ternary
from tests.cases import ALL_TYPES, make_layer

pytestmark = pytest.mark.gpu

# (ih, iw, kn, kw, kh, pad, stride)
GEOMS = [(20, 23, 64, 3, 3, 1, 1), (37, 35, 70, 7, 7, 3, 2), (19, 19, 33, 5, 5, 0, 3), (9, 40, 130, 4, 2, 2, 1)]


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
@pytest.mark.parametrize("c", range(1, 9))
def test_first_layer_fp32_result(hip, oracle, typ, c):
    import torch
    for gi, (ih, iw, kn, kw, kh, pad, stride) in enumerate(GEOMS):
        shape = (c, ih, iw, kn, kw, kh, pad, stride)
        print("case", TYPE_NAMES[typ], shape, flush=True)
        L = make_layer(typ, shape, 3, seed=9000 + 100 * c + 10 * typ + gi)
        wt = weight_is_ternary(typ)
        qw = oracle.pack_weights(L["w"], L["wthr"], wt)
        for alpha in (0.5, -0.25):
            want = oracle.conv(typ, L["x"], L["thr"], qw, kn, kh, kw, pad, stride, alpha)
            got = hip.conv(typ, torch.from_numpy(L["x"]).cuda(), torch.from_numpy(L["thr"]).cuda(),
                           torch.from_numpy(qw).cuda(), kn, kh, kw, pad, stride, alpha, engine=hip.ENGINE_MFMA_F4)
            assert got.cpu().numpy().tobytes() == np.ascontiguousarray(want).tobytes(), (shape, alpha)


def _chain(hip, oracle, batch, specs, x, seed):
    """specs: (type, shape, threshold, alpha) per layer; returns (device result, oracle result)"""
    import torch
    layers, want = [], x
    for i, (typ, shape, thr, alpha) in enumerate(specs):
        c, ih, iw, kn, kw, kh, pad, stride = shape
        wt = weight_is_ternary(typ)
        w = synth.ternary(seed + i, (kn, c, kh, kw)) if wt else synth.binary(seed + i, (kn, c, kh, kw))
        qw = oracle.pack_weights(w, np.full(kn, 0.5 if wt else 0.0, np.float32), wt)
        layers.append(dict(type=typ, shape=shape, threshold=thr, alpha=alpha, qw=torch.from_numpy(qw).cuda()))
        want = oracle.conv(typ, want, np.full(batch, thr, np.float32), qw, kn, kh, kw, pad, stride, alpha)
    net = hip.Net(batch, layers)
    got = net.run(torch.from_numpy(x).cuda()).cpu().numpy()
    net.close()
    return got, np.ascontiguousarray(want)


@pytest.mark.parametrize("c", range(1, 9))
def test_first_layer_hand_over(hip, oracle, c):
    """a first layer followed by an fp4 layer of every activation kind: the ternary hand-over in its compare-free
    form (ordinary slope and threshold) and in its select form (negative slope, negative or huge threshold), the
    binary hand-over in both forms as well (thresholds on either side of zero, tiny, huge); 70 kernels leave padding lanes in the second word"""
    batch = 2
    x = synth.normal(500 + c, (batch, c, 21, 26))
    first = (c, 21, 26, 70, 3, 3, 1, 1)
    second = (70, 21, 26, 40, 3, 3, 1, 2)
    cases = [(TNN, 0.5, 0.5), (TNN, 0.5, -0.5), (TNN, -1.0, 0.5), (TNN, 1e13, 0.5), (TNN, 0.0, 0.0), (TNN, 2.0, 0.25),
             (TBN, 1.5, 1.0), (BTN, 0.5, 0.5), (BNN, -1.0, 0.25), (BTN, 0.0, 0.5), (BTN, 1e-30, 0.5), (BNN, 1e13, 0.5),
             (BTN, 0.25, -0.5), (BNN, -3.0, 0.0)]
    for first_typ in (TNN, BNN, TBN):
        for next_typ, next_thr, alpha in cases:
            print("case", c, TYPE_NAMES[first_typ], TYPE_NAMES[next_typ], next_thr, alpha, flush=True)
            first_thr = 0.5 if act_is_ternary(first_typ) else 0.0
            got, want = _chain(hip, oracle, batch,
                               [(first_typ, first, first_thr, alpha), (next_typ, second, next_thr, 0.5)], x, 700 + c)
            assert got.tobytes() == want.tobytes()


@pytest.mark.parametrize("stride,what", [(8, "16 x 8 tiles"), (12, "two-kernel form")])
def test_patches_larger_than_the_lds(hip, oracle, stride, what):
    """a 3x3 window at stride 8: the input patch of a 16 x 16 output tile is 123 x 123 pixels, beyond the LDS of a
    workgroup, and the layer runs on tiles of 16 x 8 pixels (two wavefronts); at stride 12 that patch is too large as
    well and the layer runs as nibble quantiser + per-pixel rows + 1x1 fp4 layer; same bits either way"""
    import torch
    for typ in ALL_TYPES:
        shape = (3, 75, 91, 64, 3, 3, 1, stride)
        print("case", what, TYPE_NAMES[typ], shape, flush=True)
        L = make_layer(typ, shape, 2, seed=77 + typ)
        qw = oracle.pack_weights(L["w"], L["wthr"], weight_is_ternary(typ))
        want = oracle.conv(typ, L["x"], L["thr"], qw, 64, 3, 3, 1, stride, 0.5)
        got = hip.conv(typ, torch.from_numpy(L["x"]).cuda(), torch.from_numpy(L["thr"]).cuda(),
                       torch.from_numpy(qw).cuda(), 64, 3, 3, 1, stride, 0.5, engine=hip.ENGINE_MFMA_F4)
        assert got.cpu().numpy().tobytes() == np.ascontiguousarray(want).tobytes()
