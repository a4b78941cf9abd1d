"""Conv layers on the tile kernel with implicit im2row (the matrix-core GEMM kernel whose activation fragments are
gathered from the quantised input, for layers with many tiles and an fp32 result): forced onto small and ragged layers of
every type with both tile sizes (child processes: the switches are read once per process), and at a size that takes the
route by itself.  Every result bit for bit against the oracle."""
import os
import subprocess
import sys

import numpy as np
import pytest

from fastertnn_amd import TNN, TYPE_NAMES, weight_is_ternary
from tests.cases import ALL_TYPES, make_layer

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

_CHILD = r"""
import sys
import numpy as np, torch
sys.path.insert(0, sys.argv[1])
import fastertnn_amd.lib as hip
from fastertnn_amd import TYPE_NAMES, weight_is_ternary
from oracle.ftnn_oracle import Oracle
from tests.cases import make_layer
oracle = Oracle()
# (C, IH, IW, KN, KW, KH, pad, stride), batch: tiles that straddle images, ragged pixel and kernel counts, channel
# tails, strides, windows that are not square, 1 x 1, padding wider than one pixel, rows of 1 .. 50 words (padding words)
SHAPES = [((64, 12, 12, 64, 3, 3, 1, 1), 3), ((130, 17, 17, 70, 3, 3, 1, 2), 5), ((200, 6, 7, 33, 1, 1, 0, 1), 9),
          ((96, 9, 11, 257, 5, 3, 2, 1), 2), ((320, 15, 23, 320, 3, 3, 1, 2), 2), ((64, 30, 30, 300, 3, 3, 1, 1), 1),
          ((128, 8, 8, 130, 2, 2, 0, 2), 7), ((640, 5, 5, 40, 3, 3, 2, 1), 4)]
for typ in range(4):
    for shape, batch in SHAPES:
        L = make_layer(typ, shape, batch, seed=9100 + typ)
        print("case", TYPE_NAMES[typ], shape, batch, flush=True)
        wt = weight_is_ternary(typ)
        qw = oracle.pack_weights(L["w"], L["wthr"], wt)
        for alpha in (0.5, -0.25):
            want = oracle.conv(typ, L["x"], L["thr"], qw, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], alpha)
            y = torch.full(want.shape, float("nan"), device="cuda")
            hip.conv(typ, torch.from_numpy(L["x"]).cuda(), torch.from_numpy(L["thr"]).cuda(), torch.from_numpy(qw).cuda(),
                     L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], alpha, engine=hip.ENGINE_MFMA_F4, out=y)
            assert y.cpu().numpy().tobytes() == want.tobytes(), (typ, shape, alpha)
print("child ok")
"""


@pytest.mark.parametrize("tile", ["11", "22", "42", "44"])
def test_tile_route_forced_on_small_and_ragged_layers(tile):
    """tiles of 64 kernels x 64 pixels, 128 x 128, 256 x 128 and 256 x 256"""
    env = dict(os.environ, FTNN_CONV_TILES_FROM="1", FTNN_CONV_TILE_SHAPE=tile)
    print("case conv tile route forced, tile shape", tile, flush=True)
    r = subprocess.run([sys.executable, "-c", _CHILD, ROOT], env=env, capture_output=True, text=True, timeout=280)
    assert r.returncode == 0 and "child ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
@pytest.mark.parametrize("batch", [13, 8], ids=["160_tiles_of_128x128", "98_tiles_on_64x64"])
def test_layer_that_takes_the_tile_route_by_itself(hip, oracle, typ, batch):
    """128 channels, 28 x 28, 256 kernels, rows of 18 words: at batch 13 160 tiles of 128 x 128, at batch 8 98 of them,
    which run as tiles of 64 x 64"""
    import torch
    shape = (128, 28, 28, 256, 3, 3, 1, 1)
    assert hip.conv_scratch_bytes(typ, batch, 128, 28, 28, 256, 3, 3, 1, 1) > 0
    L = make_layer(typ, shape, batch, seed=9300 + typ)
    print("case", TYPE_NAMES[typ], shape, batch, flush=True)
    qw = oracle.pack_weights(L["w"], L["wthr"], weight_is_ternary(typ))
    want = oracle.conv(typ, L["x"], L["thr"], qw, L["kn"], 3, 3, 1, 1, 0.5)
    got = hip.conv(typ, torch.from_numpy(L["x"]).cuda(), torch.from_numpy(L["thr"]).cuda(), torch.from_numpy(qw).cuda(),
                   L["kn"], 3, 3, 1, 1, 0.5)
    assert got.cpu().numpy().tobytes() == want.tobytes()
    got = hip.host_conv(typ, L["x"], L["thr"], qw, L["kn"], 3, 3, 1, 1, 0.5)
    assert got.tobytes() == want.tobytes()


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
def test_single_layer_chain_takes_the_tile_route(hip, oracle, typ):
    """a chain of one large layer (fp32 in, fp32 out) goes through the same route from ftnn_net_run: 160 tiles of
    128 x 128 at batch 13, and at batch 50 the net's two half-batch chains with 225 tiles of 64 x 64 each"""
    import torch
    for shape, batch in (((128, 28, 28, 256, 3, 3, 1, 1), 13), ((256, 30, 30, 300, 3, 3, 1, 2), 50)):
        L = make_layer(typ, shape, batch, seed=9500 + typ)
        print("case", TYPE_NAMES[typ], shape, batch, flush=True)
        qw = oracle.pack_weights(L["w"], L["wthr"], weight_is_ternary(typ))
        thr = float(L["thr"][0])
        want = oracle.conv(typ, L["x"], np.full(batch, thr, np.float32), qw, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], 0.5)
        net = hip.Net(batch, [dict(type=typ, shape=shape, threshold=thr, alpha=0.5, qw=torch.from_numpy(qw).cuda())])
        got = net.run(torch.from_numpy(L["x"]).cuda()).cpu().numpy()
        net.close()
        assert got.tobytes() == np.ascontiguousarray(want).tobytes()
