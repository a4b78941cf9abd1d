"""The networks of the reference's e2e mode (include/timing/shapes_e2e.h via tests/golden/reference_shape_tables.json)
as device-resident layer chains (ftnn_net_*), against the same chain of tnns_conv calls on the CPU
(src/timing_layers.c:182-207): bit-identical final activations.  Four of the seven tables chain shape to shape
(ResNet-18, Darknet-19, Darknet-53, ResNet-152); the other three leave out their pooling layers, the reference's
driver re-reads a prefix of the previous buffer there, and a layer chain rejects them."""
import json
import os

import numpy as np
import pytest

from fastertnn_amd import synth, TNN, TBN, BTN, BNN, TYPE_NAMES, act_is_ternary, weight_is_ternary

pytestmark = pytest.mark.gpu

TABLES = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                                     "reference_shape_tables.json")))
NETS = {n["name"]: [tuple(r) for r in n["layers"]] for n in TABLES["e2e"]}
CHAINABLE = ["resnet18", "darknet19", "darknet53", "resnet152"]


def chainable(layers):
    c, h, w = layers[0][:3]
    for (cc, ih, iw, kn, kw, kh, p, s) in layers:
        if (cc, ih, iw) != (c, h, w):
            return False
        c, h, w = kn, (ih + 2 * p - kh) // s + 1, (iw + 2 * p - kw) // s + 1
    return True


def test_which_tables_chain():
    assert len(NETS) == 7 and [len(NETS[n]) for n in ("resnet18", "resnet152")] == [18, 152]
    assert sorted(n for n in NETS if chainable(NETS[n])) == sorted(CHAINABLE)


@pytest.mark.parametrize("name,typ", [("resnet18", TNN), ("darknet19", TBN), ("darknet19", BTN), ("darknet53", TNN),
                                      ("resnet152", TNN), ("resnet18", BNN)])
def test_reference_network_on_the_device(hip, oracle, name, typ):
    import torch
    from oracle.ftnn_oracle import Reference, aligned_copy
    if not Reference.available():
        pytest.skip("needs the compiled reference (oracle/_ref) as the CPU side of networks this size")
    ref = Reference()
    layers = NETS[name]
    batch = 1
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    thr = 0.5 if at else 0.0                       # src/timing_layers.c:100-107
    host, dev = [], []
    for i, (c, ih, iw, kn, kw, kh, p, s) in enumerate(layers):
        w = synth.ternary(900 + i, (kn, c, kh, kw)) if wt else synth.binary(900 + i, (kn, c, kh, kw))
        qw = ref.pack_weights(w, np.full(kn, 0.5 if wt else 0.0, np.float32), wt)
        host.append(qw)
        dev.append(dict(type=typ, shape=(c, ih, iw, kn, kw, kh, p, s), threshold=thr, alpha=0.5,
                        qw=torch.from_numpy(np.ascontiguousarray(qw)).cuda()))
    c, ih, iw = layers[0][:3]
    x = synth.normal(77, (batch, c, ih, iw))
    print("net", name, TYPE_NAMES[typ], len(layers), "layers", flush=True)
    want = x
    for (c, ih, iw, kn, kw, kh, p, s), qw in zip(layers, host):
        want = ref.conv(typ, aligned_copy(want), np.full(batch, thr, np.float32), qw, kn, kh, kw, p, s, 0.5)
    net = hip.Net(batch, dev)
    got = net.run(torch.from_numpy(x).cuda()).cpu().numpy()
    net.close()
    assert got.tobytes() == np.ascontiguousarray(want).tobytes()


def test_tables_that_do_not_chain_are_rejected(hip):
    import torch
    layers = NETS["vgg16"]
    qw = torch.zeros(16, dtype=torch.int64, device="cuda")
    dev = [dict(type=TNN, shape=tuple(r), threshold=0.5, alpha=0.5, qw=qw) for r in layers[:4]]
    assert not chainable(layers)
    with pytest.raises(hip.FtnnError, match="not the output"):
        hip.Net(1, dev)
