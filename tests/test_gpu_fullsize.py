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
