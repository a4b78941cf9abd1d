"""The layer chain (ftnn_net_*): device-resident e2e mode of the reference's layer driver
(src/timing_layers.c:182-207).  Bit-exact against the oracle run layer by layer; HIP-graph
replays are checked one by one against the eager result with other work in between."""
import numpy as np
import pytest

from fastertnn_amd import synth, TNN, TBN, BTN, BNN, TYPE_NAMES, act_is_ternary, weight_is_ternary

pytestmark = pytest.mark.gpu

# (type, (C, IH, IW, KN, KW, KH, pad, stride)): a shrunk ResNet-like stack with every network type
STACK = [
    (TNN, (3, 40, 40, 64, 7, 7, 3, 2)),
    (TNN, (64, 20, 20, 64, 3, 3, 1, 2)),
    (TNN, (64, 10, 10, 64, 3, 3, 1, 1)),
    (TBN, (64, 10, 10, 128, 3, 3, 1, 2)),
    (BTN, (128, 5, 5, 128, 3, 3, 1, 1)),
    (BNN, (128, 5, 5, 192, 1, 1, 0, 1)),
    (TNN, (192, 5, 5, 100, 1, 1, 0, 1)),
]


# kernel counts that are no multiple of 64 or 32 (padding lanes in the handed-over operand), a few-channel layer
# in the middle (vector-ALU layer fed with fp32 by an fp4 layer, and feeding one), an fp4 layer first
STACK2 = [
    (TBN, (64, 12, 12, 70, 3, 3, 1, 1)),
    (TNN, (70, 12, 12, 130, 3, 3, 1, 1)),
    (BNN, (130, 12, 12, 16, 1, 1, 0, 1)),
    (BTN, (16, 12, 12, 33, 3, 3, 1, 2)),
    (TNN, (33, 6, 6, 200, 3, 3, 0, 1)),
    (TBN, (200, 4, 4, 10, 4, 4, 0, 1)),
]
# larger pixel counts: the unsplit and the two-way split fp4 kernels, wide vector-ALU tiles in the stem
STACK3 = [
    (TNN, (3, 64, 64, 64, 7, 7, 3, 2)),
    (TNN, (64, 32, 32, 64, 3, 3, 1, 1)),
    (BTN, (64, 32, 32, 128, 3, 3, 1, 2)),
    (TNN, (128, 16, 16, 32, 1, 1, 0, 1)),
]


def build(hip, oracle, batch, stack=None):
    import torch
    layers, host = [], []
    for i, (typ, shape) in enumerate(stack or STACK):
        c, ih, iw, kn, kw, kh, pad, stride = shape
        wt = weight_is_ternary(typ)
        w = synth.ternary(600 + i, (kn, c, kh, kw)) if wt else synth.binary(600 + i, (kn, c, kh, kw))
        wthr = np.full(kn, 0.5 if wt else 0.0, np.float32)
        qw = oracle.pack_weights(w, wthr, wt)
        thr = 0.5 if act_is_ternary(typ) else 0.0
        host.append((typ, shape, qw, thr))
        layers.append(dict(type=typ, shape=shape, threshold=thr, alpha=0.5, qw=torch.from_numpy(qw).cuda()))
    return hip.Net(batch, layers), host


def oracle_chain(oracle, host, x):
    for typ, (c, ih, iw, kn, kw, kh, pad, stride), qw, thr in host:
        x = oracle.conv(typ, x, np.full(x.shape[0], thr, np.float32), qw, kn, kh, kw, pad, stride, 0.5)
    return x


def test_chain_matches_the_oracle_layer_by_layer(hip, oracle):
    import torch
    batch = 3
    net, host = build(hip, oracle, batch)
    x = synth.normal(1, (batch, 3, 40, 40))
    want = oracle_chain(oracle, host, x)
    xd = torch.from_numpy(x).cuda()
    got = net.run(xd)
    assert got.cpu().numpy().tobytes() == want.tobytes()
    # HIP graph: several replays, with eager work and synchronisation in between, each checked
    s = torch.cuda.Stream()
    out = torch.empty_like(got)
    with torch.cuda.stream(s):
        for rep in range(4):
            out.fill_(-1.0)
            net.run(xd, out=out, graph=True)
            s.synchronize()
            assert out.cpu().numpy().tobytes() == want.tobytes(), "replay %d" % rep
            (torch.ones(1000, device="cuda") * rep).sum().item()
        # new input contents in the same buffer: the recorded graph must see them
        x2 = synth.normal(2, (batch, 3, 40, 40))
        xd.copy_(torch.from_numpy(x2).cuda())
        net.run(xd, out=out, graph=True)
        s.synchronize()
        assert out.cpu().numpy().tobytes() == oracle_chain(oracle, host, x2).tobytes()
        # a different output buffer forces a new recording
        out2 = torch.empty_like(out)
        net.run(xd, out=out2, graph=True)
        s.synchronize()
        assert torch.equal(out, out2)
    net.close()


@pytest.mark.parametrize("which", [2, 3])
def test_other_chains_match_the_oracle(hip, oracle, which):
    import torch
    stack, batch = (STACK2, 5) if which == 2 else (STACK3, 70)
    net, host = build(hip, oracle, batch, stack)
    c, ih, iw = stack[0][1][:3]
    x = synth.normal(10 + which, (batch, c, ih, iw))
    want = oracle_chain(oracle, host, x)
    xd = torch.from_numpy(x).cuda()
    got = net.run(xd)
    assert got.cpu().numpy().tobytes() == want.tobytes()
    s = torch.cuda.Stream()
    out = torch.empty_like(got)
    with torch.cuda.stream(s):
        for rep in range(2):
            out.fill_(-1.0)
            net.run(xd, out=out, graph=True)
            s.synchronize()
            assert out.cpu().numpy().tobytes() == want.tobytes(), "replay %d" % rep
    net.close()


@pytest.mark.parametrize("which,batch", [(1, 2), (1, 5), (2, 3), (3, 17)])
def test_batch_split_over_two_concurrent_chains(hip, oracle, monkeypatch, which, batch):
    """a net may run its batch as two chains side by side on two streams (by default from batch 16 on; forced
    here for small and odd batches): same bits as one chain and as the oracle, eager and as replayed graph, over
    repeated runs that reuse the parts' buffers"""
    import torch
    stack = {1: STACK, 2: STACK2, 3: STACK3}[which]
    c, ih, iw = stack[0][1][:3]
    x = synth.normal(40 + which, (batch, c, ih, iw))
    xd = torch.from_numpy(x).cuda()
    outs = {}
    for parts in ("1", "2"):
        monkeypatch.setenv("FTNN_NET_PARTS", parts)
        net, host = build(hip, oracle, batch, stack)
        s = torch.cuda.Stream()
        with torch.cuda.stream(s):
            for rep in range(3):
                for graph in (False, True):
                    out = torch.full(net.out_shape, -1.0, device="cuda")
                    net.run(xd, out=out, graph=graph)
                    s.synchronize()
                    outs.setdefault(parts, out.cpu().numpy())
                    assert out.cpu().numpy().tobytes() == outs[parts].tobytes(), (parts, rep, graph)
                    (torch.ones(1000, device="cuda") * rep).sum().item()
        net.close()
    want = oracle_chain(oracle, host, x)
    assert outs["1"].tobytes() == want.tobytes()
    assert outs["2"].tobytes() == want.tobytes()


def test_chain_rejects_mismatched_layers(hip, oracle):
    import torch
    qw = torch.zeros(64 * 2 * 4, dtype=torch.int64, device="cuda")
    good = dict(type=TNN, shape=(64, 8, 8, 64, 1, 1, 0, 1), threshold=0.5, alpha=0.5, qw=qw)
    bad = dict(type=TNN, shape=(32, 8, 8, 64, 1, 1, 0, 1), threshold=0.5, alpha=0.5, qw=qw)
    with pytest.raises(hip.FtnnError, match="not the output"):
        hip.Net(2, [good, bad])


def test_random_chains_match_the_oracle(hip, oracle):
    """seeded random chains of 2-5 layers: every type, thresholds and PReLU slopes of either sign, kernel
    counts around the 32- and 64-channel word boundaries, few-channel inputs -- the quantised hand-over between
    layers must not change a single output bit"""
    import torch
    rng = np.random.default_rng(2024)
    done = 0
    while done < 150:
        batch = int(rng.integers(1, 7))
        c = int(rng.choice([1, 3, 4, 8, 12, 32, 64, 70, 128, 192]))
        h, w = int(rng.integers(4, 30)), int(rng.integers(4, 30))
        x = synth.normal(int(rng.integers(1, 1 << 30)), (batch, c, h, w))
        layers, host = [], []
        for _ in range(int(rng.integers(2, 6))):
            typ = int(rng.integers(0, 4))
            kh, kw = int(rng.integers(1, 5)), int(rng.integers(1, 5))
            pad, stride = int(rng.integers(0, 3)), int(rng.integers(1, 3))
            if h + 2 * pad < kh or w + 2 * pad < kw:
                break
            kn = int(rng.choice([1, 5, 16, 33, 64, 65, 100, 128, 130, 200]))
            wt = weight_is_ternary(typ)
            seed = int(rng.integers(1, 1 << 30))
            wgt = synth.ternary(seed, (kn, c, kh, kw)) if wt else synth.binary(seed, (kn, c, kh, kw))
            qw = oracle.pack_weights(wgt, np.full(kn, 0.5 if wt else 0.0, np.float32), wt)
            thr = float(rng.choice([0.5, 0.0, 1.5, 3.0])) if act_is_ternary(typ) else float(rng.choice([0.0, 0.5, -1.0]))
            alpha = float(rng.choice([0.5, 0.25, 1.0, 0.0, -0.5]))
            host.append((typ, (c, h, w, kn, kw, kh, pad, stride), qw, thr, alpha))
            layers.append(dict(type=typ, shape=(c, h, w, kn, kw, kh, pad, stride), threshold=thr, alpha=alpha,
                               qw=torch.from_numpy(qw).cuda()))
            c, h, w = kn, (h + 2 * pad - kh) // stride + 1, (w + 2 * pad - kw) // stride + 1
        if len(layers) < 2:
            continue
        print("chain", done, [(TYPE_NAMES[t], s) for t, s, _, _, _ in host], "batch", batch, flush=True)
        want = x
        for typ, (_, _, _, kn, kw, kh, pad, stride), qw, thr, alpha in host:
            want = oracle.conv(typ, want, np.full(want.shape[0], thr, np.float32), qw, kn, kh, kw, pad, stride, alpha)
        net = hip.Net(batch, layers)
        got = net.run(torch.from_numpy(x).cuda()).cpu().numpy()
        net.close()
        assert got.tobytes() == np.ascontiguousarray(want).tobytes()
        done += 1


def test_resnet18_like_stack_at_batch_32(hip, oracle):
    """The end-to-end configuration at its stated size: batch 32, 3 x 224 x 224 fp32 N(0,1) input, the 19 layers of
    the ResNet-18-like TNN stack (thresholds 0.5, uniform ternary weights, PReLU 0.5), chained on the device with the
    quantised hand-over between layers.  Eager launches and HIP-graph replays give the same bits; sampled images are
    bit-exact against the oracle's layer-by-layer chain (images of a batch never meet, so a chain over a sub-batch
    is exact), and the whole batch against the reference's own tnns_conv chain where its compiled form is present
    (src/timing_layers.c:182-207)."""
    import torch
    from fastertnn_amd.shapes import RESNET18_LIKE
    from oracle.ftnn_oracle import Reference, aligned_copy
    batch = 32
    stack = [(TNN, row) for row in RESNET18_LIKE]
    net, host = build(hip, oracle, batch, stack)
    g = torch.Generator(device="cuda")
    g.manual_seed(6)
    xd = torch.randn((batch, 3, 224, 224), generator=g, device="cuda")
    got = net.run(xd)
    torch.cuda.synchronize()
    assert got.shape == (batch, 1000, 7, 7)   # the fully connected layer is the 1x1 layer of the reference's table, on 7 x 7 pixels
    s = torch.cuda.Stream()
    out = torch.empty_like(got)
    with torch.cuda.stream(s):
        for rep in range(3):
            out.fill_(-1.0)
            net.run(xd, out=out, graph=True)
            s.synchronize()
            assert torch.equal(out.view(torch.int32), got.view(torch.int32)), "replay %d" % rep
    net.close()
    imgs = [0, 13, 31]
    print("oracle chain on images", imgs, flush=True)
    want = oracle_chain(oracle, host, xd[imgs].cpu().numpy())
    assert got[imgs].cpu().numpy().tobytes() == np.ascontiguousarray(want).tobytes()
    if Reference.available():
        print("reference chain on the whole batch", flush=True)
        ref = Reference()
        xh = xd.cpu().numpy()
        for typ, (c, ih, iw, kn, kw, kh, pad, stride), qw, thr in host:
            xh = ref.conv(typ, xh, np.full(batch, thr, np.float32), aligned_copy(qw), kn, kh, kw, pad, stride, 0.5)
        assert got.cpu().numpy().tobytes() == np.ascontiguousarray(xh).tobytes()
