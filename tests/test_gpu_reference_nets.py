"""The networks of the reference's e2e mode (include/timing/shapes_e2e.h, kept as data in fastertnn_amd/data/reference_shape_tables.txt)
as device-resident layer chains (ftnn_net_*), against the same chain of tnns_conv calls on the CPU
(src/timing_layers.c:182-207): bit-identical final activations.  Four of the seven tables chain shape to shape
(ResNet-18, Darknet-19, Darknet-53, ResNet-152); the other three leave out their pooling layers, the reference's
driver re-reads a prefix of the previous buffer there (src/timing_layers.c:187-200); a layer chain rejects them unless
it is created with FTNN_NET_REREAD_PREFIX, and then does the same."""
import numpy as np
import pytest

from fastertnn_amd import shapes, synth, TNN, TBN, BTN, BNN, TYPE_NAMES, act_is_ternary, weight_is_ternary

pytestmark = pytest.mark.gpu

TABLES = shapes.reference_tables()
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


@pytest.mark.parametrize("name,typ,batch", [("resnet34", TNN, 1), ("vgg16", TNN, 2), ("vgg19", BTN, 1), ("vgg16", TBN, 1)])
def test_tables_without_pooling_reread_the_previous_buffer(hip, oracle, name, typ, batch):
    """the three tables that leave out their pooling layers, as the reference's driver runs them: where a row's
    input shape is not the previous output shape, the layer reads the leading floats of the previous output buffer
    (across images at batch 2)"""
    import torch
    from oracle.ftnn_oracle import Reference, aligned_copy
    if not Reference.available():
        pytest.skip("needs the compiled reference (oracle/_ref) as the CPU side of networks this size")
    ref = Reference()
    layers = NETS[name]
    assert not chainable(layers)
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    thr = 0.5 if at else 0.0
    host, dev = [], []
    for i, (c, ih, iw, kn, kw, kh, p, s) in enumerate(layers):
        w = synth.ternary(1900 + i, (kn, c, kh, kw)) if wt else synth.binary(1900 + i, (kn, c, kh, kw))
        qw = ref.pack_weights(w, np.full(kn, 0.5 if wt else 0.0, np.float32), wt)
        host.append(qw)
        dev.append(dict(type=typ, shape=(c, ih, iw, kn, kw, kh, p, s), threshold=thr, alpha=0.5,
                        qw=torch.from_numpy(np.ascontiguousarray(qw)).cuda()))
    c, ih, iw = layers[0][:3]
    x = synth.normal(78, (batch, c, ih, iw))
    print("net", name, TYPE_NAMES[typ], len(layers), "layers, batch", batch, flush=True)
    want, rereads = x, 0
    for (c, ih, iw, kn, kw, kh, p, s), qw in zip(layers, host):
        if want.shape[1:] != (c, ih, iw):      # what `test->input = test->output` amounts to under the new row
            want = np.ascontiguousarray(want).reshape(-1)[:batch * c * ih * iw].reshape(batch, c, ih, iw)
            rereads += 1
        want = ref.conv(typ, aligned_copy(want), np.full(batch, thr, np.float32), qw, kn, kh, kw, p, s, 0.5)
    assert rereads >= 1
    net = hip.Net(batch, dev, flags=hip.NET_REREAD_PREFIX)
    xd = torch.from_numpy(x).cuda()
    got = net.run(xd).cpu().numpy()
    assert got.tobytes() == np.ascontiguousarray(want).tobytes()
    s2 = torch.cuda.Stream()
    with torch.cuda.stream(s2):
        for rep in range(2):
            out = torch.full(net.out_shape, -1.0, device="cuda")
            net.run(xd, out=out, graph=True)
            s2.synchronize()
            assert out.cpu().numpy().tobytes() == got.tobytes(), rep
    net.close()


def test_a_reread_must_fit_the_previous_output(hip):
    import torch
    qw = torch.zeros(64 * 2 * 4, dtype=torch.int64, device="cuda")
    first = dict(type=TNN, shape=(64, 8, 8, 64, 1, 1, 0, 1), threshold=0.5, alpha=0.5, qw=qw)
    larger = dict(type=TNN, shape=(64, 9, 9, 64, 1, 1, 0, 1), threshold=0.5, alpha=0.5, qw=qw)
    with pytest.raises(hip.FtnnError, match="not the output"):
        hip.Net(2, [first, larger], flags=hip.NET_REREAD_PREFIX)


def test_tables_that_do_not_chain_are_rejected(hip):
    import torch
    layers = NETS["vgg16"]
    qw = torch.zeros(16, dtype=torch.int64, device="cuda")
    dev = [dict(type=TNN, shape=tuple(r), threshold=0.5, alpha=0.5, qw=qw) for r in layers[:4]]
    assert not chainable(layers)
    with pytest.raises(hip.FtnnError, match="not the output"):
        hip.Net(1, dev)
