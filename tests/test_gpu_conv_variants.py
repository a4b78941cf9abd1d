"""The fp4 layer kernels in the variants that the default choice never takes on test-sized layers: plain global
loads instead of buffer loads (the path of operands of 3.75 GiB and more: FTNN_CONV_NO_BUFFER_LOADS=1), with every
K split of the 64 x 64 kernel forced (FTNN_CONV_SPLIT=1|2|4) and on 32 x 32 tiles, fp32 results and both quantised
hand-overs, all four types.  The switches are read once per process, so each combination runs in a child process;
every result is compared bit for bit with the oracle."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

_CHILD = r"""
import sys
import numpy as np, torch
sys.path.insert(0, sys.argv[1])
import fastertnn_amd.lib as hip
from fastertnn_amd import synth, TYPE_NAMES, act_is_ternary, weight_is_ternary
from oracle.ftnn_oracle import Oracle
from tests.cases import make_layer
from tests.test_gpu_net import STACK, STACK2, STACK3, build, oracle_chain
oracle = Oracle()
# single layers with an fp32 result: 256 tiles of 64 x 64 (the 64 x 64 kernel, split as forced), 8 tiles (32 x 32
# tiles), ragged kernel counts and pixel counts, a strided window, and 1 x 1 layers of one and two K words on more
# than 150 tiles of 64 x 64 (a forced split of 2 or 4 must not leave a wavefront without a word of its own)
for typ in range(4):
    for shape, batch in (((64, 32, 32, 128, 3, 3, 1, 1), 8), ((130, 17, 17, 70, 3, 3, 1, 2), 21), ((64, 10, 10, 64, 3, 3, 1, 1), 2),
                         ((200, 6, 7, 33, 1, 1, 0, 1), 3), ((64, 40, 40, 64, 1, 1, 0, 1), 11), ((100, 24, 24, 96, 1, 1, 0, 2), 40)):
        L = make_layer(typ, shape, batch, seed=8000 + typ)
        print("case", TYPE_NAMES[typ], shape, batch, flush=True)
        wt = weight_is_ternary(typ)
        qw = oracle.pack_weights(L["w"], L["wthr"], wt)
        want = oracle.conv(typ, L["x"], L["thr"], qw, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], 0.5)
        got = hip.conv(typ, torch.from_numpy(L["x"]).cuda(), torch.from_numpy(L["thr"]).cuda(), torch.from_numpy(qw).cuda(),
                       L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], 0.5, engine=hip.ENGINE_MFMA_F4)
        assert got.cpu().numpy().tobytes() == want.tobytes(), (typ, shape)
# chains: every layer but the last hands its result over quantised (ternary and binary forms, ragged kernel counts)
for stack, batch in ((STACK, 3), (STACK2, 5), (STACK3, 9)):
    print("case chain of", len(stack), "layers, batch", batch, flush=True)
    net, host = build(hip, oracle, batch, stack)
    c, ih, iw = stack[0][1][:3]
    x = synth.normal(77, (batch, c, ih, iw))
    got = net.run(torch.from_numpy(x).cuda())
    assert got.cpu().numpy().tobytes() == oracle_chain(oracle, host, x).tobytes()
    net.close()
print("child ok")
"""


# ("on", "auto") is the default configuration, which every other suite covers
@pytest.mark.parametrize("buffer_loads,split", [("off", "auto"), ("off", "1"), ("off", "2"), ("off", "4"), ("on", "1"), ("on", "2"),
                                                ("on", "4")])
def test_layer_kernel_variants(split, buffer_loads):
    env = dict(os.environ)
    if buffer_loads == "off":
        env["FTNN_CONV_NO_BUFFER_LOADS"] = "1"
    if split != "auto":
        env["FTNN_CONV_SPLIT"] = split
    print("case layer kernels: buffer loads", buffer_loads, "split", split, flush=True)
    r = subprocess.run([sys.executable, "-c", _CHILD, ROOT], env=env, capture_output=True, text=True, timeout=280)
    assert r.returncode == 0 and "child ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


def test_bad_split_values_are_ignored():
    """FTNN_CONV_SPLIT accepts 1, 2 and 4; anything else (0 would divide by zero) leaves the library's own choice"""
    for bad in ("0", "3", "8", "-1", "x"):
        env = dict(os.environ, FTNN_CONV_SPLIT=bad)
        code = _CHILD.split("# chains:")[0] + 'print("child ok")\n'
        r = subprocess.run([sys.executable, "-c", code, ROOT], env=env, capture_output=True, text=True, timeout=280)
        assert r.returncode == 0 and "child ok" in r.stdout, bad + r.stdout[-1500:] + r.stderr[-1500:]
