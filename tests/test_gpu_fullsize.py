"""Benchmark-size runs checked through size-independent properties, plus sampled rows
against the oracle."""
import numpy as np
import pytest

from fastertnn_amd import TNN, TBN, BTN, BNN, TYPE_NAMES, act_is_ternary, weight_is_ternary

pytestmark = pytest.mark.gpu


def test_large_tnn_gemm_properties(hip, oracle):
    """M = N = 8192, K = 32768 with B == A: the result is symmetric, its diagonal is the
    non-zero count of each row, an all-zero row gives +0.0, |acc| <= K, and sampled rows are
    bit-exact against the oracle"""
    import torch
    m, k = 8192, 32768
    g = torch.Generator(device="cuda")
    g.manual_seed(123)
    x = torch.randint(-1, 2, (m, k), generator=g, device="cuda", dtype=torch.int8)
    x[17] = 0
    nnz = (x != 0).sum(1).to(torch.float32)
    a = hip.pack_gemm_operand(x.float())
    del x
    y = hip.mm(TNN, a, a, m, 1, 1, m, k // 64, 1.0).view(m, m)
    assert torch.equal(y, y.t())
    assert torch.equal(torch.diagonal(y), nnz)
    assert float(y.abs().max()) <= k
    assert y[17].cpu().numpy().tobytes() == np.zeros(m, np.float32).tobytes()
    # alpha = 0.5 relates to alpha = 1 by halving the non-positive entries, exactly
    y05 = hip.mm(TNN, a, a, m, 1, 1, m, k // 64, 0.5).view(m, m)
    assert torch.equal(y05, torch.where(y <= 0, y * 0.5, y))
    # sampled rows against the oracle (rows from different workgroups and tile positions)
    rows = [0, 63, 64, 255, 256, 4097, 8191]
    ah = a.cpu().numpy().reshape(m, -1)
    sub = np.ascontiguousarray(ah[rows])
    want = oracle.mm(TNN, sub.reshape(-1), ah.reshape(-1), len(rows), 1, 1, m, k // 64, 0.5).reshape(len(rows), m)
    assert y05[rows].cpu().numpy().tobytes() == want.tobytes()


def test_large_tnn_gemm_on_every_engine(hip, oracle):
    """M = N = 8192, K = 32768 on independent uniform ternary operands, PReLU 0.5: the engine AUTO resolves to is
    the fp4 matrix-core one (512 K words through its LDS ring), and AUTO, fp4 and int8 give the vector-ALU
    engine's bits on every element; rows from different tiles and wavefronts are bit-exact against the oracle
    (src/tnns/mm_p2_final_tnn_avx2.c:384-387)"""
    import torch
    m = n = 8192
    k = 32768
    kw = k // 64
    ops = []
    for seed in (5, 6):
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        packed = torch.empty(m * k // 32, dtype=torch.int64, device="cuda")
        for r0 in range(0, m, 2048):   # 256 MiB of fp32 at a time
            x = torch.randint(-1, 2, (2048, k), generator=g, device="cuda", dtype=torch.int8).float()
            packed[r0 * k // 32:(r0 + 2048) * k // 32] = hip.pack_gemm_operand(x)
        ops.append(packed)
    a, b = ops
    assert hip.select_engine(TNN, m, 1, 1, n, kw) == hip.ENGINE_MFMA_F4
    need = max(hip.mm_scratch_bytes(e, TNN, m, 1, 1, n, kw) for e in (hip.ENGINE_MFMA_I8, hip.ENGINE_MFMA_F4))
    assert hip.mm_scratch_bytes(hip.ENGINE_AUTO, TNN, m, 1, 1, n, kw) == hip.mm_scratch_bytes(hip.ENGINE_MFMA_F4, TNN, m, 1, 1, n, kw)
    scratch = torch.empty(need, dtype=torch.uint8, device="cuda")
    ref = hip.mm_engine(hip.ENGINE_VALU, TNN, a, b, m, 1, 1, n, kw, 0.5)
    rows = [0, 31, 32, 127, 128, 255, 256, 4097, 6000, 8191]
    ah = a.view(m, 2 * kw)[rows].cpu().numpy()
    want = oracle.mm(TNN, np.ascontiguousarray(ah).reshape(-1), b.cpu().numpy(), len(rows), 1, 1, n, kw, 0.5)
    assert ref.view(m, n)[rows].cpu().numpy().tobytes() == np.ascontiguousarray(want).tobytes()
    for eng in (hip.ENGINE_AUTO, hip.ENGINE_MFMA_F4, hip.ENGINE_MFMA_I8):
        print("engine", eng, flush=True)
        y = torch.full((m, n, 1, 1), float("nan"), dtype=torch.float32, device="cuda")
        scratch.fill_(0x5a)
        hip.mm_engine(eng, TNN, a, b, m, 1, 1, n, kw, 0.5, out=y, scratch=scratch)
        assert torch.equal(y.view(torch.int32), ref.view(torch.int32)), "engine %d" % eng
        del y
    # a caller that keeps the weights expanded (ftnn_expand_rows once, ftnn_mm_expanded per call) gets the same bits
    for eng in (hip.ENGINE_MFMA_F4, hip.ENGINE_MFMA_I8):
        a_exp, b_exp = hip.expand_rows(eng, a, m, kw, True), hip.expand_rows(eng, b, n, kw, True)
        y = hip.mm_expanded(eng, TNN, a_exp, b_exp, m, 1, 1, n, kw, 0.5)
        assert torch.equal(y.view(torch.int32), ref.view(torch.int32)), "expanded, engine %d" % eng
        del a_exp, b_exp, y


@pytest.mark.parametrize("typ", [TNN, TBN, BTN, BNN], ids=lambda t: TYPE_NAMES[t])
def test_resnet_stage_layers_batch32(hip, oracle, typ):
    """the 3x3 stage layers of the batch-32 stack (C=64@56x56 ... C=512@7x7): the fused layer
    equals quantise+im2row followed by the GEMM, the packed rows round-trip through the
    decoder, and one image of the batch is bit-exact against the oracle"""
    import torch
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    g = torch.Generator(device="cuda")
    g.manual_seed(5 + typ)
    for (c, hw) in ((64, 56), (128, 28), (256, 14), (512, 7)):
        print("case", TYPE_NAMES[typ], c, hw, flush=True)
        x = torch.randn((32, c, hw, hw), generator=g, device="cuda")
        thr = torch.full((32,), 0.5 if at else 0.0, device="cuda")
        w = torch.randint(-1, 2, (c, c, 3, 3), generator=g, device="cuda", dtype=torch.int8).float()
        if not wt:
            w = torch.where(w == 0, torch.ones_like(w), w)
        wthr = torch.full((c,), 0.5 if wt else 0.0, device="cuda")
        qw = hip.pack_weights(w, wthr, wt)
        y = hip.conv(typ, x, thr, qw, c, 3, 3, 1, 1, 0.5)
        rows = hip.quantize_im2row(x, thr, 3, 3, 1, 1, at)
        y2 = hip.mm(typ, rows, qw, 32, hw, hw, c, ((c + 63) // 64) * 9, 0.5, c * 9)
        assert torch.equal(y, y2)
        # linear-algebra cross-check on the whole batch: fp32 conv of the quantised tensors
        if at:
            qx = (x > 0.5).float() - (x < -0.5).float()
            px = torch.nn.functional.pad(qx, (1, 1, 1, 1), value=0.0)
        else:
            qx = torch.where(x < 0.0, -1.0, 1.0)
            px = torch.nn.functional.pad(qx, (1, 1, 1, 1), value=1.0)
        qwf = ((w > 0.5).float() - (w < -0.5).float()) if wt else torch.where(w < 0.0, -1.0, 1.0)
        # unfold + fp32 matmul: sums of +-1 products stay far below 2^24, so fp32 is exact in any order
        cols = torch.nn.functional.unfold(px, kernel_size=3)                  # [32, C*9, hw*hw]
        ref = torch.matmul(qwf.reshape(c, -1), cols).reshape(32, c, hw, hw)
        ref = torch.where(ref >= 0, ref, ref * 0.5)
        assert torch.equal(y, ref)
        # one image against the oracle
        n = 7
        want = oracle.conv(typ, x[n:n + 1].cpu().numpy(), thr[n:n + 1].cpu().numpy(), qw.cpu().numpy(), c, 3, 3,
                           1, 1, 0.5)
        assert y[n:n + 1].cpu().numpy().tobytes() == want.tobytes()


def _rand_words(torch, count, seed):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return torch.randint(-2 ** 62, 2 ** 62, (count,), generator=g, device="cuda", dtype=torch.int64)


def test_row_major_result_beyond_2_32_elements(hip, oracle):
    """66000 x 65600 results (17 GB): offsets into the result need more than 32 bits.  All three engines agree
    on every element, and rows on either side of the 2^31- and 2^32-element marks are bit-exact against the oracle"""
    import torch
    m, n, kw = 66000, 65600, 4
    assert m * n > 2 ** 32
    a, b = _rand_words(torch, m * 2 * kw, 1), _rand_words(torch, n * 2 * kw, 2)
    ref = None
    for eng in (hip.ENGINE_VALU, hip.ENGINE_MFMA_F4, hip.ENGINE_MFMA_I8):
        print("engine", eng, flush=True)
        y = torch.full((m, n, 1, 1), float("nan"), dtype=torch.float32, device="cuda")
        hip.mm_engine(eng, TNN, a, b, m, 1, 1, n, kw, 0.5, out=y)
        if ref is None:
            ref = y
            rows = [0, 2 ** 31 // n, 2 ** 31 // n + 1, 2 ** 32 // n, 2 ** 32 // n + 1, m - 1]
            ah = a.view(m, 2 * kw)[rows].cpu().numpy()
            want = oracle.mm(TNN, np.ascontiguousarray(ah).reshape(-1), b.cpu().numpy(), len(rows), 1, 1, n, kw, 0.5)
            assert y.view(m, n)[rows].cpu().numpy().tobytes() == want.tobytes()
        else:
            assert torch.equal(y, ref), "engine %d" % eng
            del y


def test_nchw_results_beyond_2_32_elements(hip, oracle):
    """1050 images x 1000 kernels x 64 x 64 pixels (17 GB) from a 3x3 layer: both layer engines and the GEMM
    engines behind packed rows agree on every element; the first, the last and the images around the 2^31- and
    2^32-element marks are bit-exact against the oracle"""
    import torch
    n, c, hw, kn = 1050, 64, 64, 1000
    assert n * kn * hw * hw > 2 ** 32
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    x = torch.randn((n, c, hw, hw), generator=g, device="cuda")
    thr = torch.full((n,), 0.5, device="cuda")
    from fastertnn_amd import synth
    w = synth.ternary(9, (kn, c, 3, 3))
    qw_h = oracle.pack_weights(w, np.full(kn, 0.5, np.float32), True)
    qw = torch.from_numpy(qw_h).cuda()
    per_img = kn * hw * hw
    imgs = [0, 2 ** 31 // per_img, 2 ** 31 // per_img + 1, 2 ** 32 // per_img, 2 ** 32 // per_img + 1, n - 1]
    ref = None
    for eng in (hip.ENGINE_MFMA_F4, hip.ENGINE_VALU):
        print("layer engine", eng, flush=True)
        y = torch.full((n, kn, hw, hw), float("nan"), dtype=torch.float32, device="cuda")
        hip.conv(TNN, x, thr, qw, kn, 3, 3, 1, 1, 0.5, out=y, engine=eng)
        if ref is None:
            ref = y
            want = oracle.conv(TNN, x[imgs].cpu().numpy(), np.full(len(imgs), 0.5, np.float32), qw_h, kn, 3, 3, 1, 1, 0.5)
            assert y[imgs].cpu().numpy().tobytes() == np.ascontiguousarray(want).tobytes()
        else:
            assert torch.equal(y, ref), "layer engine %d" % eng
            del y
    rows = hip.quantize_im2row(x, thr, 3, 3, 1, 1, True)
    for eng in (hip.ENGINE_MFMA_F4, hip.ENGINE_MFMA_I8):
        print("gemm engine", eng, flush=True)
        y = torch.full((n, kn, hw, hw), float("nan"), dtype=torch.float32, device="cuda")
        hip.mm_engine(eng, TNN, rows, qw, n, hw, hw, kn, 9, 0.5, out=y)
        assert torch.equal(y, ref), "gemm engine %d" % eng
        del y


@pytest.mark.parametrize("typ", [TNN, TBN, BTN, BNN], ids=lambda t: TYPE_NAMES[t])
def test_large_layer_takes_the_gemm_route(hip, oracle, typ):
    """a 29.6 GMAC layer (batch 16, 512 -> 512 channels at 28 x 28, 392 tiles of 128 x 128): the fp4 engine runs it as quantise + im2row +
    expansion + the tiled GEMM kernel.  Same bits as the vector-ALU engine on every element, and as the oracle on
    one image"""
    import torch
    from fastertnn_amd import synth
    n, c, hw, kn = 16, 512, 28, 512
    assert ((n * hw * hw + 127) // 128) * ((kn + 127) // 128) >= 256
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    g = torch.Generator(device="cuda")
    g.manual_seed(31 + typ)
    x = torch.randn((n, c, hw, hw), generator=g, device="cuda")
    thr = torch.full((n,), 0.5 if at else 0.0, device="cuda")
    w = synth.ternary(40 + typ, (kn, c, 3, 3)) if wt else synth.binary(40 + typ, (kn, c, 3, 3))
    qw_h = oracle.pack_weights(w, np.full(kn, 0.5 if wt else 0.0, np.float32), wt)
    qw = torch.from_numpy(qw_h).cuda()
    got = hip.conv(typ, x, thr, qw, kn, 3, 3, 1, 1, 0.5, engine=hip.ENGINE_MFMA_F4)
    ref = hip.conv(typ, x, thr, qw, kn, 3, 3, 1, 1, 0.5, engine=hip.ENGINE_VALU)
    assert torch.equal(got, ref)
    want = oracle.conv(typ, x[5:6].cpu().numpy(), np.full(1, 0.5 if at else 0.0, np.float32), qw_h, kn, 3, 3, 1, 1, 0.5)
    assert got[5:6].cpu().numpy().tobytes() == np.ascontiguousarray(want).tobytes()
    # prepared weights take the same route
    prepared = hip.prepare_conv_weights(typ, qw, c, kn, 3, 3)
    got2 = hip.conv_prepared(typ, x, thr, prepared, kn, 3, 3, 1, 1, 0.5)
    assert torch.equal(got2, ref)
