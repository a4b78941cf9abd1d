"""Pins of the oracle that need neither the reference nor its vectors: what the
mathematics fixes.  Each check is chosen so that a plausible slip (wrong bit order,
swapped planes, transposed operand, wrong pad value, off-by-one in the im2row index,
non-strict compare) fails it.  CPU only."""
import numpy as np
import pytest
import torch

from fastertnn_amd import TNN, TBN, BTN, BNN, TYPE_NAMES, act_is_ternary, weight_is_ternary
from oracle.ftnn_oracle import out_dim, cpack, round4
from tests.cases import (ALL_TYPES, EXTRA_SHAPES, REF_TEST_SHAPES, decode_binary_rows, decode_ternary_rows,
                         make_layer)

SHAPES = REF_TEST_SHAPES[:10] + EXTRA_SHAPES


def quantize_np(x, thr, ternary):
    """closed form of the quantisers: strict compares (ternarize2row_avx2.c:443-449,
    binarize2row_avx2.c:19-21)"""
    t = np.asarray(thr, np.float32).reshape(-1, 1, 1, 1)
    if ternary:
        return (x > t).astype(np.float32) - (x < -t).astype(np.float32)
    return np.where(x < t, -1.0, 1.0).astype(np.float32)


def prelu(v, alpha):
    return np.where(v >= 0, v, alpha * v).astype(np.float32)


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
@pytest.mark.parametrize("si", range(len(SHAPES)))
def test_conv_equals_direct_convolution(oracle, typ, si):
    """layer == PReLU(conv2d(pad(quantise(x), pad_val), quantise(w))): the reference's own
    self-test (src/timing_layers.c:142-165), pad value +1 for binary activations"""
    shape = SHAPES[si]
    L = make_layer(typ, shape, 3, seed=500 + si)
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    qx = quantize_np(L["x"], L["thr"], at)
    qw = quantize_np(L["w"], L["wthr"], wt)
    pad = L["pad"]
    px = np.pad(qx, ((0, 0), (0, 0), (pad, pad), (pad, pad)), constant_values=0.0 if at else 1.0)
    want = torch.nn.functional.conv2d(torch.from_numpy(px), torch.from_numpy(qw), stride=L["stride"]).numpy()
    want = prelu(want, L["alpha"])
    packed = oracle.pack_weights(L["w"], L["wthr"], wt)
    got = oracle.conv(typ, L["x"], L["thr"], packed, L["kn"], L["kh"], L["kw"], pad, L["stride"], L["alpha"])
    assert np.array_equal(got, want)


@pytest.mark.parametrize("ternary", [True, False])
@pytest.mark.parametrize("si", range(len(SHAPES)))
def test_rows_decode_to_quantised_patches(oracle, ternary, si):
    """brute-force im2row: every lane of every packed row, decoded, equals the quantised
    input at (oh*s+kh-p, ow*s+kw-p, c); fill lanes are 0 (ternary) / +1 (binary)"""
    c, ih, iw, kn, kw, kh, pad, stride = SHAPES[si]
    typ = TNN if ternary else BNN
    L = make_layer(typ, SHAPES[si], 2, seed=800 + si)
    rows = oracle.quantize_im2row(L["x"], L["thr"], kh, kw, pad, stride, ternary)
    oh, ow = out_dim(ih, pad, kh, stride), out_dim(iw, pad, kw, stride)
    cp, kwords = cpack(c), round4(cpack(c) * kh * kw)
    dec = (decode_ternary_rows if ternary else decode_binary_rows)(rows, 2 * oh * ow, kwords)
    fill = 0 if ternary else 1
    q = quantize_np(L["x"], L["thr"], ternary)
    want = np.full((2, oh, ow, kwords * 64), fill, np.int8)
    for a in range(kh):
        for b in range(kw):
            for o in range(oh):
                for p in range(ow):
                    y, x = o * stride + a - pad, p * stride + b - pad
                    if 0 <= y < ih and 0 <= x < iw:
                        base = (a * kw + b) * cp * 64
                        want[:, o, p, base:base + c] = q[:, :, y, x]
    assert np.array_equal(dec.reshape(want.shape), want)


@pytest.mark.parametrize("ternary", [True, False])
def test_weight_rows_decode_to_quantised_weights(oracle, ternary):
    for (c, kh, kw, kn) in [(32, 3, 3, 5), (127, 3, 5, 3), (193, 1, 1, 7), (64, 2, 2, 2)]:
        L = make_layer(TNN if ternary else BNN, (c, 8, 8, kn, kw, kh, 0, 1), 1, seed=c)
        rows = oracle.pack_weights(L["w"], L["wthr"], ternary)
        cp, kwords = cpack(c), round4(cpack(c) * kh * kw)
        dec = (decode_ternary_rows if ternary else decode_binary_rows)(rows, kn, kwords)
        q = quantize_np(L["w"], L["wthr"], ternary)
        want = np.full((kn, kwords * 64), 0 if ternary else 1, np.int8)
        for a in range(kh):
            for b in range(kw):
                base = (a * kw + b) * cp * 64
                want[:, base:base + c] = q[:, :, a, b]
        assert np.array_equal(dec, want)


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
def test_gemm_equals_integer_matmul_of_decoded_operands(oracle, typ):
    """mm_* == decode(A) @ decode(B)^T over the padded lanes (BNN: real lanes only), in the
    NCHW output order of include/tnns/mm.h:30"""
    rng = np.random.default_rng(typ)
    n, oh, ow, kn, k = 2, 3, 5, 11, 6   # k not a multiple of 4: two pad words
    kwords, m = round4(k), 2 * 3 * 5
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)

    def operand(rows_n, ternary):
        s = rng.integers(0, 2 ** 63, size=(rows_n, kwords), dtype=np.int64)
        if not ternary:
            return s.reshape(-1), decode_binary_rows(s.reshape(-1), rows_n, kwords)
        z = rng.integers(0, 2 ** 63, size=(rows_n, kwords), dtype=np.int64)
        s &= ~z
        out = np.empty((rows_n, kwords // 4, 2, 4), np.int64)
        out[:, :, 0, :] = s.reshape(rows_n, kwords // 4, 4)
        out[:, :, 1, :] = z.reshape(rows_n, kwords // 4, 4)
        return out.reshape(-1), decode_ternary_rows(out.reshape(-1), rows_n, kwords)

    a, da = operand(m, at)
    b, db = operand(kn, wt)
    k_unpack = 64 * kwords - 37
    if typ == BNN:  # lanes past K_unpack must agree (both +1) for the formula to be a dot product
        am = a.view(np.uint64).reshape(m, kwords)
        bm = b.view(np.uint64).reshape(kn, kwords)
        am[:, -1] &= np.uint64((1 << 27) - 1)
        bm[:, -1] &= np.uint64((1 << 27) - 1)
        da, db = decode_binary_rows(a, m, kwords), decode_binary_rows(b, kn, kwords)
    acc = da.astype(np.int32) @ db.astype(np.int32).T
    if typ == BNN:
        acc -= 37
    want = prelu(acc.astype(np.float32), 0.5).reshape(n, oh * ow, kn).transpose(0, 2, 1).reshape(n, kn, oh, ow)
    y, raw = oracle.mm(typ, a, b, n, oh, ow, kn, k, 0.5, k_unpack, want_acc=True)
    assert np.array_equal(raw.reshape(n, kn, oh * ow).transpose(0, 2, 1).reshape(m, kn), acc)
    assert np.array_equal(y.reshape(want.shape), want)


def test_gemm_operand_packer_layout(oracle):
    """bitpacking2: lane j of row i is bit j%64 of word (j%256)/64 of group j/256, sign
    words first (src/utils.c:266-288)"""
    x = np.ones((3, 512), np.float32)
    x[1, 70] = -1.0
    x[2, 300] = 0.0
    p = oracle.pack_gemm_operand(x).view(np.uint64).reshape(3, 2, 2, 4)  # row, group, plane, word
    want = np.zeros_like(p)
    want[1, 0, 0, 1] = np.uint64(1) << np.uint64(6)
    want[2, 1, 1, 0] = np.uint64(1) << np.uint64(44)
    assert np.array_equal(p, want)
    with pytest.raises(ValueError):
        oracle.pack_gemm_operand(np.zeros((2, 128), np.float32))


def test_quantiser_boundaries(oracle):
    """strict compares at the thresholds; -0.0 and +0.0 binarise to +1 at threshold 0"""
    x = np.zeros((1, 64, 1, 1), np.float32)
    x[0, :8, 0, 0] = [0.5, -0.5, np.nextafter(np.float32(0.5), np.float32(1)), np.nextafter(np.float32(-0.5), np.float32(-1)), 0.0, -0.0, 3.0, -3.0]
    r = oracle.quantize_im2row(x, np.array([0.5], np.float32), 1, 1, 0, 1, True).view(np.uint64)
    sign, zero = int(r[0]), int(r[4])
    assert sign & 0xFF == 0b10001000            # only lanes 3 and 7 are negative
    assert zero & 0xFF == 0b00110011            # +-0.5 and +-0 are zero
    assert zero >> 8 == (1 << 56) - 1           # untouched lanes hold 0.0 -> zero
    rb = oracle.quantize_im2row(x, np.array([0.0], np.float32), 1, 1, 0, 1, False).view(np.uint64)
    assert int(rb[0]) == 0b10001010             # -0.5, just below -0.5, -3.0 ; +-0.0 are +1


def test_popcount_invariants(oracle):
    """|acc| <= non-zero products <= 64*Kw; acc == non-zero products (mod 2); an all-zero row
    gives +0.0; B == A puts the non-zero count on the diagonal"""
    from fastertnn_amd import synth
    m, p = 24, 768
    a = synth.ternary(77, (m, p))
    a[5] = 0.0
    ap = oracle.pack_gemm_operand(a)
    y, acc = oracle.mm(TNN, ap, ap, m, 1, 1, m, p // 64, 0.5, want_acc=True)
    acc = acc.reshape(m, m)
    nz = (a != 0).astype(np.int32)
    nzprod = nz @ nz.T
    assert np.all(np.abs(acc) <= nzprod)
    assert np.all((acc - nzprod) % 2 == 0)
    assert np.array_equal(np.diag(acc), nz.sum(1))
    assert np.array_equal(acc, acc.T)
    assert y.reshape(m, m)[5].tobytes() == np.zeros(m, np.float32).tobytes()
