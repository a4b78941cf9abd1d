"""Seeded random conv shapes (channels, image, kernel, padding, stride, batch, type): the fused
device layer, the staged device path and the host entry point against the oracle, bit for bit.
Covers combinations the fixed shape tables do not: kernels wider than high, stride > kernel,
padding > kernel / 2, one-pixel outputs, C just around multiples of 64 and the few-channel
re-packing with every taps-per-word count."""
import numpy as np
import pytest

from fastertnn_amd import TYPE_NAMES, act_is_ternary, weight_is_ternary
from tests.cases import make_layer

pytestmark = pytest.mark.gpu


def random_shapes(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        c = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 11, 16, 21, 22, 31, 32, 33, 63, 64, 65, 100, 128, 129, 192, 200]))
        kh, kw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        pad = int(rng.integers(0, 4))
        stride = int(rng.integers(1, 4))
        ih, iw = int(rng.integers(1, 19)), int(rng.integers(1, 19))
        if ih + 2 * pad < kh or iw + 2 * pad < kw:
            continue
        kn = int(rng.choice([1, 2, 5, 8, 17, 31, 32, 33, 64, 70, 130]))
        typ = int(rng.integers(0, 4))
        batch = int(rng.integers(1, 6))
        out.append((typ, (c, ih, iw, kn, kw, kh, pad, stride), batch))
    return out


@pytest.mark.parametrize("chunk", range(6))
def test_random_layers(hip, oracle, chunk):
    import torch
    for k, (typ, shape, batch) in enumerate(random_shapes(1234 + chunk, 40)):
        print("case", chunk, k, TYPE_NAMES[typ], shape, "batch", batch, flush=True)
        L = make_layer(typ, shape, batch, seed=50000 + 100 * chunk + k)
        at, wt = act_is_ternary(typ), weight_is_ternary(typ)
        qw = oracle.pack_weights(L["w"], L["wthr"], wt)
        want = oracle.conv(typ, L["x"], L["thr"], qw, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"])
        x_d, thr_d, qw_d = (torch.from_numpy(np.ascontiguousarray(v)).cuda() for v in (L["x"], L["thr"], qw))
        got = hip.conv(typ, x_d, thr_d, qw_d, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"])
        assert got.cpu().numpy().tobytes() == want.tobytes(), "fused layer"
        for eng in (hip.ENGINE_VALU, hip.ENGINE_MFMA_F4):
            got = hip.conv(typ, x_d, thr_d, qw_d, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"],
                           engine=eng)
            assert got.cpu().numpy().tobytes() == want.tobytes(), "fused layer, engine %d" % eng
        rows = hip.quantize_im2row(x_d, thr_d, L["kh"], L["kw"], L["pad"], L["stride"], at)
        oh, ow = want.shape[2], want.shape[3]
        kk, ku = ((L["c"] + 63) // 64) * L["kh"] * L["kw"], L["c"] * L["kh"] * L["kw"]
        for eng in (hip.ENGINE_VALU, hip.ENGINE_MFMA_F4):
            got2 = hip.mm_engine(eng, typ, rows, qw_d, batch, oh, ow, L["kn"], kk, L["alpha"], ku)
            assert got2.cpu().numpy().tobytes() == want.tobytes(), "staged path, engine %d" % eng
        if k % 8 == 0:
            got3 = hip.host_conv(typ, L["x"], L["thr"], qw, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"])
            assert got3.tobytes() == want.tobytes(), "tnns_conv"
