"""The three GEMM engines (vector-ALU popcount, MFMA int8, MFMA fp4) give the same bits as the
oracle for all four network types, for GEMM-shaped (row-major) and conv-shaped (NCHW) outputs,
ragged tiles and K tails."""
import numpy as np
import pytest

from fastertnn_amd import TNN, TBN, BTN, BNN, TYPE_NAMES, act_is_ternary, weight_is_ternary
from tests.cases import ALL_TYPES, REF_TEST_SHAPES, EXTRA_SHAPES, make_layer

pytestmark = pytest.mark.gpu

LAYERS = [REF_TEST_SHAPES[i] for i in (1, 5, 6, 8, 9, 10)] + [EXTRA_SHAPES[0], EXTRA_SHAPES[3],
                                                            (64, 20, 20, 300, 3, 3, 1, 1)]


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
@pytest.mark.parametrize("si", range(len(LAYERS)))
def test_engines_on_layers(hip, oracle, typ, si):
    shape = LAYERS[si]
    batch = 3
    L = make_layer(typ, shape, batch, seed=4000 + 13 * si + typ)
    print("case", TYPE_NAMES[typ], shape, flush=True)
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    qw = oracle.pack_weights(L["w"], L["wthr"], wt)
    rows = oracle.quantize_im2row(L["x"], L["thr"], L["kh"], L["kw"], L["pad"], L["stride"], at)
    oh = hip.out_dim(L["ih"], L["pad"], L["kh"], L["stride"])
    ow = hip.out_dim(L["iw"], L["pad"], L["kw"], L["stride"])
    k, ku = ((L["c"] + 63) // 64) * L["kh"] * L["kw"], L["c"] * L["kh"] * L["kw"]
    for alpha in (0.5, -0.25):
        want = oracle.mm(typ, rows, qw, batch, oh, ow, L["kn"], k, alpha, ku)
        a_d, b_d = _dev(rows), _dev(qw)
        for eng in (hip.ENGINE_VALU, hip.ENGINE_MFMA_I8, hip.ENGINE_MFMA_F4, hip.ENGINE_AUTO):
            got = hip.mm_engine(eng, typ, a_d, b_d, batch, oh, ow, L["kn"], k, alpha, ku).cpu().numpy()
            assert got.tobytes() == want.tobytes(), "engine %d alpha %g" % (eng, alpha)


@pytest.mark.parametrize("mnp", [(300, 70, 768), (257, 513, 256), (1024, 1024, 2048), (33, 1000, 512)])
def test_engines_on_gemm_operands(hip, oracle, mnp):
    from fastertnn_amd import synth
    m, n, p = mnp
    a, b = synth.ternary(m, (m, p)), synth.ternary(n + 1, (n, p))
    ap, bp = oracle.pack_gemm_operand(a), oracle.pack_gemm_operand(b)
    want = oracle.mm(TNN, ap, bp, m, 1, 1, n, p // 64, 0.5)
    assert np.array_equal(oracle.gemm(ap, bp, m, n, p // 64), a @ b.T)
    a_d, b_d = _dev(ap), _dev(bp)
    for eng in (hip.ENGINE_VALU, hip.ENGINE_MFMA_I8, hip.ENGINE_MFMA_F4):
        got = hip.mm_engine(eng, TNN, a_d, b_d, m, 1, 1, n, p // 64, 0.5).cpu().numpy()
        assert got.tobytes() == want.tobytes(), "engine %d" % eng


@pytest.mark.parametrize("ternary", [True, False], ids=["ternary", "binary"])
@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (5, 3, 7, 7), (64, 64, 3, 3), (33, 65, 1, 1), (7, 130, 5, 2),
                                   (130, 127, 3, 3), (3, 200, 1, 7), (2, 64, 2, 3)])
def test_weight_packer_matches_the_oracle(hip, oracle, ternary, shape):
    """ftnn_pack_weights against the oracle's ternarize_opt / binarize_opt restatement (src/utils.c:468-521, 634-675),
    word for word: channel tails, tap counts that are no multiple of the four loaded together, padding words, and
    thresholds of either sign (a negative ternary threshold turns the channels past C into +1, as in the reference)"""
    from fastertnn_amd import synth
    kn, c, kh, kw = shape
    w = synth.normal(kn * 31 + c, (kn, c, kh, kw))
    for thr_value in (0.5, 0.0, -0.25):
        thr = np.full(kn, thr_value, np.float32)
        thr[::2] *= 0.5
        want = oracle.pack_weights(w, thr, ternary)
        got = hip.pack_weights(_dev(w), _dev(thr), ternary).cpu().numpy()
        assert got.tobytes() == np.ascontiguousarray(want).tobytes(), thr_value


@pytest.mark.parametrize("rows,cols", [(1, 256), (3, 1280), (70, 768), (257, 4096), (5, 256 * 9)])
def test_gemm_operand_packer_matches_bitpacking2(hip, oracle, rows, cols):
    """ftnn_pack_gemm_operand against the oracle's bitpacking2 (src/utils.c:257-291), word for word: one group of 256
    values, group counts that leave the last workgroup partly idle, several rows"""
    from fastertnn_amd import synth
    x = synth.ternary(rows * 7 + cols, (rows, cols))
    want = oracle.pack_gemm_operand(x)
    got = hip.pack_gemm_operand(_dev(x)).cpu().numpy()
    assert got.tobytes() == np.ascontiguousarray(want).tobytes()


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
@pytest.mark.parametrize("mnk", [(1, 64, 4), (5, 65, 8), (70, 100, 12), (200, 257, 36), (1000, 64, 4),
                                 (129, 1000, 8), (64, 63, 4), (300, 2048, 20)])
def test_row_major_gemm_all_types(hip, oracle, typ, mnk):
    """fully connected / GEMM-shaped results (OH = OW = 1) on random packed words, every type and
    engine; a BTN product of this shape runs as the TBN form with the operands exchanged and a
    transposed store, which ragged row and column counts on either side exercise"""
    m, n, kw = mnk
    rng = np.random.default_rng(1000 * typ + m + n + kw)
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    a = rng.integers(-2 ** 63, 2 ** 63, size=m * kw * (2 if at else 1), dtype=np.int64)
    b = rng.integers(-2 ** 63, 2 ** 63, size=n * kw * (2 if wt else 1), dtype=np.int64)
    ku = 64 * kw - 7
    a_d, b_d = _dev(a), _dev(b)
    for alpha in (0.5, -0.25):
        want = oracle.mm(typ, a, b, m, 1, 1, n, kw, alpha, ku)
        for eng in (hip.ENGINE_VALU, hip.ENGINE_MFMA_I8, hip.ENGINE_MFMA_F4, hip.ENGINE_AUTO):
            got = hip.mm_engine(eng, typ, a_d, b_d, m, 1, 1, n, kw, alpha, ku).cpu().numpy()
            assert got.tobytes() == want.tobytes(), "engine %d alpha %g" % (eng, alpha)


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
@pytest.mark.parametrize("shape", [(3333, 1, 1, 3100, 4), (5, 29, 29, 2700, 12)], ids=["row_major", "nchw"])
def test_matrix_core_engines_with_256x256_tiles(hip, oracle, typ, shape):
    """the matrix-core kernel works on 128 x 128 tiles while a problem has few of them and on 256 x 256
    tiles from 160 of those on; the cases above are all of the first kind, these are of the second
    (ragged in both directions, row-major and NCHW stores)"""
    n, oh, ow, kn, kw = shape
    m = n * oh * ow
    assert ((m + 255) // 256) * ((kn + 255) // 256) >= 160
    rng = np.random.default_rng(77 + typ + kw)
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    a = rng.integers(-2 ** 63, 2 ** 63, size=m * kw * (2 if at else 1), dtype=np.int64)
    b = rng.integers(-2 ** 63, 2 ** 63, size=kn * kw * (2 if wt else 1), dtype=np.int64)
    ku = 64 * kw - 3
    want = oracle.mm(typ, a, b, n, oh, ow, kn, kw, 0.5, ku)
    a_d, b_d = _dev(a), _dev(b)
    for eng in (hip.ENGINE_MFMA_I8, hip.ENGINE_MFMA_F4):
        got = hip.mm_engine(eng, typ, a_d, b_d, n, oh, ow, kn, kw, 0.5, ku).cpu().numpy()
        assert got.tobytes() == want.tobytes(), "engine %d" % eng


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
@pytest.mark.parametrize("shape", [(1500, 1, 1, 1480, 4), (3, 23, 23, 1500, 8)], ids=["row_major", "nchw"])
def test_matrix_core_engines_with_128x128_tiles(hip, oracle, typ, shape):
    """on plain fragments (the int8 engine, fp4 whole calls with few 256 x 256 tiles) the tile kernel works on
    64 x 64 tiles below 112 tiles of 128 x 128, as in the small cases above, and on 128 x 128 tiles from there
    up to 160 tiles of 256 x 256: these cases are of that middle kind"""
    n, oh, ow, kn, kw = shape
    m = n * oh * ow
    assert ((m + 127) // 128) * ((kn + 127) // 128) >= 112 and ((m + 255) // 256) * ((kn + 255) // 256) < 160
    rng = np.random.default_rng(91 + typ + kw)
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    a = rng.integers(-2 ** 63, 2 ** 63, size=m * kw * (2 if at else 1), dtype=np.int64)
    b = rng.integers(-2 ** 63, 2 ** 63, size=kn * kw * (2 if wt else 1), dtype=np.int64)
    ku = 64 * kw - 7
    want = oracle.mm(typ, a, b, n, oh, ow, kn, kw, -0.5, ku)
    a_d, b_d = _dev(a), _dev(b)
    for eng in (hip.ENGINE_MFMA_I8, hip.ENGINE_MFMA_F4):
        got = hip.mm_engine(eng, typ, a_d, b_d, n, oh, ow, kn, kw, -0.5, ku).cpu().numpy()
        assert got.tobytes() == want.tobytes(), "engine %d" % eng


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
def test_weights_kept_in_engine_form_serve_every_batch(hip, oracle, typ):
    """ftnn_expand_rows once for the weights, then ftnn_mm_expanded for activations of several sizes: few rows (128 x 128
    tiles), many rows (256 x 256 tiles), a conv-shaped result; the engine form of an operand must not depend on the
    other operand or on the tiling that a call picks.  Both matrix-core engines, ragged everywhere, K tail."""
    kn, kw = 2700, 8
    ku = 64 * kw - 5
    rng = np.random.default_rng(300 + typ)
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    b = rng.integers(-2 ** 63, 2 ** 63, size=kn * kw * (2 if wt else 1), dtype=np.int64)
    b_d = _dev(b)
    for eng in (hip.ENGINE_MFMA_I8, hip.ENGINE_MFMA_F4):
        b_exp = hip.expand_rows(eng, b_d, kn, kw, wt)
        for n, oh, ow in ((70, 1, 1), (3700, 1, 1), (3, 37, 35)):
            m = n * oh * ow
            print("case", TYPE_NAMES[typ], "engine", eng, "rows", m, flush=True)
            a = rng.integers(-2 ** 63, 2 ** 63, size=m * kw * (2 if at else 1), dtype=np.int64)
            want = oracle.mm(typ, a, b, n, oh, ow, kn, kw, -0.5, ku)
            a_exp = hip.expand_rows(eng, _dev(a), m, kw, at)
            got = hip.mm_expanded(eng, typ, a_exp, b_exp, n, oh, ow, kn, kw, -0.5, ku).cpu().numpy()
            assert got.tobytes() == want.tobytes(), "engine %d rows %d" % (eng, m)


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
@pytest.mark.parametrize("shape", [(4200, 1, 1, 1100, 4), (7, 30, 29, 1070, 8)], ids=["row_major", "nchw"])
def test_vector_alu_gemm_walks_large_grids_in_panels(hip, oracle, typ, shape):
    """grids of 32 x 32 workgroups and more are renumbered into panels of 32 row tiles (the last one narrower when the
    count is no multiple of 32): every tile must still be computed exactly once"""
    n, oh, ow, kn, kw = shape
    m = n * oh * ow
    rng = np.random.default_rng(5 + typ + kw)
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    a = rng.integers(-2 ** 63, 2 ** 63, size=m * kw * (2 if at else 1), dtype=np.int64)
    b = rng.integers(-2 ** 63, 2 ** 63, size=kn * kw * (2 if wt else 1), dtype=np.int64)
    ku = 64 * kw - 5
    want = oracle.mm(typ, a, b, n, oh, ow, kn, kw, 0.5, ku)
    import torch
    y = torch.full((n, kn, oh, ow), float("nan"), dtype=torch.float32, device="cuda")
    hip.mm_engine(hip.ENGINE_VALU, typ, _dev(a), _dev(b), n, oh, ow, kn, kw, 0.5, ku, out=y)
    assert y.cpu().numpy().tobytes() == want.tobytes()


# shapes (n, oh, ow, kn, words) that the vector-ALU GEMM runs with K split over the wavefronts of a workgroup: few tiles,
# rows of 16 words and more.  By the launcher's rule these take 4 wavefronts x 2 columns, 8 x 4, 8 x 2 (K tail: 25
# groups in chunks of 8), 4 x 4, and conv-shaped results with 4 and 8 wavefronts.
KSPLIT_SHAPES = [(70, 1, 1, 100, 16), (256, 1, 1, 256, 64), (90, 1, 1, 70, 100), (64, 1, 1, 2048, 20), (2, 7, 9, 50, 24),
                 (3, 5, 5, 40, 36), (1, 1, 1, 64, 16), (64, 1, 1, 3, 44)]


def _ksplit_case(hip, oracle, typ, shape, alpha=0.5):
    import torch
    n, oh, ow, kn, kw = shape
    m = n * oh * ow
    rng = np.random.default_rng(1000 * typ + m + kn + kw)
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    a = rng.integers(-2 ** 63, 2 ** 63, size=m * kw * (2 if at else 1), dtype=np.int64)
    b = rng.integers(-2 ** 63, 2 ** 63, size=kn * kw * (2 if wt else 1), dtype=np.int64)
    ku = 64 * kw - 7
    want = oracle.mm(typ, a, b, n, oh, ow, kn, kw, alpha, ku)
    y = torch.full((n, kn, oh, ow), float("nan"), dtype=torch.float32, device="cuda")
    hip.mm_engine(hip.ENGINE_VALU, typ, _dev(a), _dev(b), n, oh, ow, kn, kw, alpha, ku, out=y)
    assert y.cpu().numpy().tobytes() == want.tobytes(), (typ, shape, alpha)


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
@pytest.mark.parametrize("shape", KSPLIT_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_vector_alu_gemm_splits_k_for_small_problems(hip, oracle, typ, shape):
    """small GEMMs (the reference's CPU-sized case among them) run with the wavefronts of a workgroup sharing K and
    their partial counts summed through LDS: every type, row-major and NCHW results, ragged rows and columns, K tails
    that leave wavefronts without a group, both slopes"""
    print("case", TYPE_NAMES[typ], shape, flush=True)
    for alpha in (0.5, -0.25):
        _ksplit_case(hip, oracle, typ, shape, alpha)


_KSPLIT_CHILD = r"""
import sys
import torch    # before the library, as in every other test process: both then share torch's HIP runtime
sys.path.insert(0, sys.argv[1])
import fastertnn_amd.lib as hip
from oracle.ftnn_oracle import Oracle
from tests.test_gpu_engines import KSPLIT_SHAPES, _ksplit_case
oracle = Oracle()
for typ in range(4):
    for shape in KSPLIT_SHAPES:
        print("case", typ, shape, flush=True)
        _ksplit_case(hip, oracle, typ, shape)
print("child ok")
"""


@pytest.mark.parametrize("variant", ["4,2", "4,4", "8,2", "8,4", "0"])
def test_every_k_split_variant_forced(variant):
    """FTNN_MM_KSPLIT forces each split variant (wavefronts, columns) onto every shape above, whatever the launcher's
    own rule would pick, and switches the split off; the switch is read once per process, hence child processes"""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    print("case forced K split", variant, flush=True)
    r = subprocess.run([sys.executable, "-c", _KSPLIT_CHILD, root], env=dict(os.environ, FTNN_MM_KSPLIT=variant),
                       capture_output=True, text=True, timeout=280)
    assert r.returncode == 0 and "child ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


def test_lanes_flagged_zero_and_negative_count_as_zero(hip, oracle):
    """a lane with both its sign and its zero bit set is zero in the reference's formula
    (za|zb masks it); the expanded operands must agree"""
    rng = np.random.default_rng(3)
    m, n, kw = 70, 40, 8
    a = rng.integers(-2 ** 63, 2 ** 63, size=m * 2 * kw, dtype=np.int64)
    b = rng.integers(-2 ** 63, 2 ** 63, size=n * 2 * kw, dtype=np.int64)
    want = oracle.mm(TNN, a, b, m, 1, 1, n, kw, 0.5)
    for eng in (hip.ENGINE_VALU, hip.ENGINE_MFMA_I8, hip.ENGINE_MFMA_F4):
        got = hip.mm_engine(eng, TNN, _dev(a), _dev(b), m, 1, 1, n, kw, 0.5).cpu().numpy()
        assert got.tobytes() == want.tobytes(), "engine %d" % eng


def test_fp4_gemm_is_exact_on_its_longest_rows(hip):
    """The fp4 GEMM sums lanes coded (a + 1) / 2 in fp32: quarters up to the lane count, exact up to 65536 words per row.
    Rows of that length, almost all lanes +1 on both sides (sums just below 2^22, where fp32 resolves 1/4 and no
    less), against the vector-ALU engine and against numpy on the bit planes."""
    import torch
    rng = np.random.default_rng(11)
    m, n, kw = 40, 33, 1 << 16

    def sparse(shape):
        r = rng.integers(-2 ** 63, 2 ** 63, size=(5,) + shape, dtype=np.int64)
        return r[0] & r[1] & r[2] & r[3] & r[4]

    def operand(rows):
        v = np.empty((rows, kw // 4, 2, 4), dtype=np.int64)
        v[:, :, 0, :] = sparse((rows, kw // 4, 4))     # sign bits: 1 lane in 32 negative
        v[:, :, 1, :] = sparse((rows, kw // 4, 4))     # zero bits: 1 lane in 32 zero
        return v
    a, b = operand(m), operand(n)
    print("case longest fp4 rows", m, n, kw, flush=True)
    a_d, b_d = _dev(a.reshape(-1)), _dev(b.reshape(-1))
    want = hip.mm_engine(hip.ENGINE_VALU, TNN, a_d, b_d, m, 1, 1, n, kw, 0.5).cpu().numpy()
    got = hip.mm_engine(hip.ENGINE_MFMA_F4, TNN, a_d, b_d, m, 1, 1, n, kw, 0.5).cpu().numpy()
    assert got.tobytes() == want.tobytes()
    # numpy on the planes for a few (row, column) pairs: sum over lanes of a * b
    pop = lambda x: int(np.unpackbits(x.view(np.uint8)).sum())
    for i, j in ((0, 0), (39, 32), (17, 5)):
        sa, za, sb, zb = a[i, :, 0, :], a[i, :, 1, :], b[j, :, 0, :], b[j, :, 1, :]
        nz = ~(za | zb)
        dot = pop(nz) - 2 * pop((sa ^ sb) & nz)
        assert dot > 3_000_000                       # the case is near the top of the range
        assert got.reshape(m, n)[i, j] == np.float32(dot)
    # one group of words more is refused, and AUTO does not pick the engine there
    L, s = hip._L, hip._stream()
    y = torch.empty(16, device="cuda")
    assert L.ftnn_mm_engine(hip.ENGINE_MFMA_F4, 0, a_d.data_ptr(), b_d.data_ptr(), 1, 1, 1, 1, kw + 4, 0, 0.5, y.data_ptr(),
                            a_d.data_ptr(), 1 << 20, s) == -1
    assert b"too long" in L.ftnn_last_error()
    assert hip.select_engine(0, 4096, 1, 1, 4096, kw + 4) == hip.ENGINE_VALU


def test_engine_argument_checks(hip):
    import torch
    a = torch.zeros(64 * 8, dtype=torch.int64, device="cuda")
    y = torch.empty((8, 8, 1, 1), device="cuda")
    L = hip._L
    s = hip._stream()
    assert L.ftnn_mm_engine(9, 0, a.data_ptr(), a.data_ptr(), 8, 1, 1, 8, 4, 0, 0.5, y.data_ptr(), None, 0, s) == -1
    # an explicit matrix-core engine without scratch is an error ...
    assert L.ftnn_mm_engine(hip.ENGINE_MFMA_F4, 0, a.data_ptr(), a.data_ptr(), 8, 1, 1, 8, 4, 0, 0.5, y.data_ptr(),
                            None, 0, s) == -1
    assert b"scratch" in L.ftnn_last_error()
    # ... AUTO without scratch falls back to the engine that needs none
    assert L.ftnn_mm_engine(hip.ENGINE_AUTO, 0, a.data_ptr(), a.data_ptr(), 8, 1, 1, 8, 4, 0, 0.5, y.data_ptr(),
                            None, 0, s) == 0
    torch.cuda.synchronize()
    assert hip.mm_scratch_bytes(hip.ENGINE_VALU, 0, 8192, 1, 1, 8192, 512) == 0
    assert hip.mm_scratch_bytes(hip.ENGINE_MFMA_F4, 0, 8192, 1, 1, 8192, 512) == 2 * (256 * 256 * 1024 + 8192 * 4)   # two bits per lane + a sum per row
    assert hip.mm_scratch_bytes(hip.ENGINE_MFMA_I8, 0, 33, 1, 1, 1, 4) == (2 + 1) * 8 * 1024
    assert hip.select_engine(0, 8192, 1, 1, 8192, 512) == hip.ENGINE_MFMA_F4
    assert hip.select_engine(0, 1, 56, 56, 256, 36) == hip.ENGINE_VALU


def test_layer_engine_argument_checks(hip):
    import torch
    x = torch.zeros((2, 64, 8, 8), device="cuda")
    thr = torch.zeros(2, device="cuda")
    qw = torch.zeros(16 * 2 * 12, dtype=torch.int64, device="cuda")
    scratch = torch.empty(hip.conv_scratch_bytes(0, 2, 64, 8, 8, 16, 3, 3, 1, 1), dtype=torch.uint8, device="cuda")
    y = torch.empty((2, 16, 8, 8), device="cuda")
    L, s = hip._L, hip._stream()
    args = (0, x.data_ptr(), thr.data_ptr(), qw.data_ptr(), 2, 64, 8, 8, 16, 3, 3, 1, 1, 1, 1, 0.5, scratch.data_ptr(),
            y.data_ptr(), s)
    assert L.ftnn_conv_engine(hip.ENGINE_MFMA_I8, *args) == -1          # layers run on the vector ALU or on fp4
    assert b"engine" in L.ftnn_last_error()
    assert L.ftnn_conv_engine(7, *args) == -1
    for eng in (hip.ENGINE_AUTO, hip.ENGINE_VALU, hip.ENGINE_MFMA_F4):
        assert L.ftnn_conv_engine(eng, *args) == 0
    bad = list(args)
    bad[16] = scratch.data_ptr() + 4                                     # misaligned scratch
    assert L.ftnn_conv_engine(hip.ENGINE_MFMA_F4, *bad) == -1
    assert L.ftnn_conv_prepared(0, x.data_ptr(), thr.data_ptr(), None, 2, 64, 8, 8, 16, 3, 3, 1, 1, 1, 1, 0.5,
                                scratch.data_ptr(), y.data_ptr(), s) == -1
    assert L.ftnn_conv_weights_bytes(0, 64, 16, 3, 3) == 1 * 12 * 1024    # one block of 32 kernels x 12 words
    assert L.ftnn_conv_weights_bytes(5, 64, 16, 3, 3) == 0
    torch.cuda.synchronize()
