"""The reference's host-memory entry points (t2r_p2_opt, b2r, mm_*, tnns_conv) through the
C ABI: results bit-exact against the oracle, returned buffers are caller-owned heap memory,
repeated calls with changing shapes reuse the library's device workspace correctly."""
import numpy as np
import pytest

from fastertnn_amd import TNN, TBN, BTN, BNN, TYPE_NAMES, act_is_ternary, weight_is_ternary
from tests.cases import ALL_TYPES, EXTRA_SHAPES, REF_TEST_SHAPES, make_layer

pytestmark = pytest.mark.gpu

# shapes in an order that grows, shrinks and grows the workspace again
ORDER = [6, 0, 11, 2, 10, 9, 5]


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
def test_host_entry_points(hip, oracle, typ):
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    for si in ORDER:
        shape = REF_TEST_SHAPES[si]
        print("case", TYPE_NAMES[typ], shape, flush=True)
        L = make_layer(typ, shape, 4, seed=2000 + si)
        qw = oracle.pack_weights(L["w"], L["wthr"], wt)
        rows_o = oracle.quantize_im2row(L["x"], L["thr"], L["kh"], L["kw"], L["pad"], L["stride"], at)
        rows_h = hip.host_quantize_im2row(L["x"], L["thr"], L["kh"], L["kw"], L["pad"], L["stride"], at)
        assert np.array_equal(rows_h, rows_o)
        oh = hip.out_dim(L["ih"], L["pad"], L["kh"], L["stride"])
        ow = hip.out_dim(L["iw"], L["pad"], L["kw"], L["stride"])
        k, ku = ((L["c"] + 63) // 64) * L["kh"] * L["kw"], L["c"] * L["kh"] * L["kw"]
        y_o = oracle.mm(typ, rows_o, qw, 4, oh, ow, L["kn"], k, L["alpha"], ku)
        y_h = hip.host_mm(typ, rows_o, qw, 4, oh, ow, L["kn"], k, L["alpha"], ku)
        assert y_h.tobytes() == y_o.tobytes()
        y_c = hip.host_conv(typ, L["x"], L["thr"], qw, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"])
        assert y_c.tobytes() == y_o.tobytes()


def test_e2e_chaining_like_the_reference_driver(hip, oracle):
    """src/timing_layers.c:189-201: the output of one tnns_conv is the next layer's input"""
    shapes = [(64, 16, 16, 64, 3, 3, 1, 1), (64, 16, 16, 128, 1, 1, 0, 2), (128, 8, 8, 128, 3, 3, 1, 1),
              (128, 8, 8, 10, 1, 1, 0, 1)]
    L0 = make_layer(TNN, shapes[0], 8, seed=31)
    thr = np.full(8, 0.5, np.float32)
    xh, xo = L0["x"], L0["x"]
    for i, shape in enumerate(shapes):
        c, ih, iw, kn, kw, kh, pad, stride = shape
        Lw = make_layer(TNN, shape, 1, seed=40 + i)
        qw = oracle.pack_weights(Lw["w"], Lw["wthr"], True)
        xh = hip.host_conv(TNN, xh, thr, qw, kn, kh, kw, pad, stride, 0.5)
        xo = oracle.conv(TNN, xo, thr, qw, kn, kh, kw, pad, stride, 0.5)
        assert xh.tobytes() == xo.tobytes(), "layer %d" % i


def test_negative_alpha_and_alpha_one(hip, oracle):
    """the two PReLU forms (f<=0 -> f*=alpha for TNN, r>=0 ? r : alpha*r otherwise) differ only
    in the sign of zero for alpha < 0; both must follow the reference's form"""
    for typ in ALL_TYPES:
        at, wt = act_is_ternary(typ), weight_is_ternary(typ)
        L = make_layer(typ, REF_TEST_SHAPES[1], 2, seed=77)
        qw = oracle.pack_weights(L["w"], L["wthr"], wt)
        for alpha in (1.0, -0.25, 0.0):
            want = oracle.conv(typ, L["x"], L["thr"], qw, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], alpha)
            got = hip.host_conv(typ, L["x"], L["thr"], qw, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], alpha)
            assert got.tobytes() == want.tobytes(), (TYPE_NAMES[typ], alpha)


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
def test_hip_layer_equals_the_reference_baseline_build(hip, oracle, reference_baseline, typ):
    """second reference: the Packing-0 "baseline" build (src/tnns/tnns_cpu_naive.c:255-292), which shares
    no kernel code with the Packing-2 path the library replaces"""
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    shapes = REF_TEST_SHAPES + EXTRA_SHAPES
    for si in (1, 2, 5, 6, 9, 10, 12, 13, 18, 22):
        L = make_layer(typ, shapes[si], 4, seed=2500 + si)
        print("case", TYPE_NAMES[typ], shapes[si], flush=True)
        qw0 = reference_baseline.pack_weights(L["w"], L["wthr"], wt)
        try:
            want = reference_baseline.conv(typ, L["x"], L["thr"], qw0, L["kn"], L["kh"], L["kw"], L["pad"],
                                           L["stride"], L["alpha"])
        finally:
            reference_baseline.free_weights(qw0)
        qw2 = oracle.pack_weights(L["w"], L["wthr"], wt)
        got = hip.host_conv(typ, L["x"], L["thr"], qw2, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"])
        assert got.tobytes() == want.tobytes()


def test_large_buffers_through_the_host_entry_points(hip, oracle):
    """inputs and results of 20 MB: the host entry points move them through their ring of pinned chunks (several
    trips round the ring, a partial last chunk) with the copy threads; twice, so that the ring is reused"""
    shape = (64, 100, 101, 64, 3, 3, 1, 1)
    L = make_layer(TNN, shape, 8, seed=4242)
    assert L["x"].nbytes > 16 << 20
    qw = oracle.pack_weights(L["w"], L["wthr"], True)
    want = oracle.conv(TNN, L["x"], L["thr"], qw, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"])
    for rep in range(2):
        got = hip.host_conv(TNN, L["x"], L["thr"], qw, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"])
        assert got.nbytes > 16 << 20 and got.tobytes() == want.tobytes(), rep
    rows_o = oracle.quantize_im2row(L["x"], L["thr"], 3, 3, 1, 1, True)
    rows_h = hip.host_quantize_im2row(L["x"], L["thr"], 3, 3, 1, 1, True)
    assert rows_h.nbytes > 12 << 20 and np.array_equal(rows_h, rows_o)
    y_h = hip.host_mm(TNN, rows_o, qw, 8, 100, 101, 64, 9, L["alpha"], 0)
    assert y_h.tobytes() == want.tobytes()


def test_results_prepared_ahead_of_time(hip, oracle):
    """From the second request for a size on, large results come from buffers a helper thread allocated and touched
    beforehand: a run of calls with two alternating result sizes, some results held while later ones are made, every
    one complete, distinct and the caller's to free."""
    import ctypes
    la = make_layer(TNN, (16, 64, 64, 40, 3, 3, 1, 1), 8, seed=77)     # 5.2 MB result
    lb = make_layer(TNN, (16, 64, 64, 72, 1, 1, 0, 1), 8, seed=78)     # 9.4 MB result
    cases = []
    for L in (la, lb):
        qw = oracle.pack_weights(L["w"], L["wthr"], True)
        want = oracle.conv(TNN, L["x"], L["thr"], qw, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"])
        assert want.nbytes >= 4 << 20
        cases.append((L, qw, want))
    held = []
    for rep in range(10):
        L, qw, want = cases[rep % 2]
        x, thr = np.ascontiguousarray(L["x"]), np.ascontiguousarray(L["thr"])
        t = hip.Testcase(type=TNN, batchcount=8, channelcount=L["c"], inputW=L["iw"], inputH=L["ih"], kernelcount=L["kn"],
                         kernelW=L["kw"], kernelH=L["kh"], paddingW=L["pad"], paddingH=L["pad"], strideW=L["stride"],
                         strideH=L["stride"], preluAlpha=L["alpha"], input_thresholds=thr.ctypes.data, input=x.ctypes.data,
                         quantized_kernel_packing2=qw.ctypes.data)
        print("case prepared results", rep, flush=True)
        hip._L.tnns_conv(ctypes.byref(t))
        got = np.ctypeslib.as_array(ctypes.cast(t.output, ctypes.POINTER(ctypes.c_float)), shape=(want.size,))
        assert got.tobytes() == want.tobytes(), rep
        held.append(t.output)
        if len(held) > 3:                      # the caller frees in its own order, three results later
            hip._libc.free(ctypes.c_void_p(held.pop(0)))
    assert len(set(held)) == len(held)
    for p in held:
        hip._libc.free(ctypes.c_void_p(p))


_CHILD = r"""
import sys
import numpy as np, torch
sys.path.insert(0, sys.argv[1])
import fastertnn_amd.lib as hip
from fastertnn_amd import TNN
from tests.cases import make_layer
L = make_layer(TNN, (64, 100, 101, 64, 3, 3, 1, 1), 8, seed=4242)
qw = hip.pack_weights(torch.from_numpy(L["w"]).cuda(), torch.from_numpy(L["wthr"]).cuda(), True)
want = hip.conv(TNN, torch.from_numpy(L["x"]).cuda(), torch.from_numpy(L["thr"]).cuda(), qw, L["kn"], 3, 3, 1, 1,
                L["alpha"]).cpu().numpy()
for rep in range(2):
    got = hip.host_conv(TNN, L["x"], L["thr"], qw.cpu().numpy(), L["kn"], 3, 3, 1, 1, L["alpha"])
    assert got.tobytes() == want.tobytes(), rep
print("child ok")
"""


@pytest.mark.parametrize("threads", ["1", "3"])
def test_host_copies_with_other_thread_counts(threads):
    """the copy threads of the host entry points are a per-process choice (CPU affinity, or FTNN_HOST_COPY_THREADS):
    one thread takes the runtime's plain copies, three an odd split of every chunk; a child process each, checked
    against the device-resident call"""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, FTNN_HOST_COPY_THREADS=threads)
    print("case host copy threads", threads, flush=True)
    r = subprocess.run([sys.executable, "-c", _CHILD, root], env=env, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and "child ok" in r.stdout, r.stdout[-1500:] + r.stderr[-1500:]


def _conv_at(hip, typ, L, qw_buf, alpha=0.5):
    """tnns_conv with the packed weights at the address of qw_buf (no copy on the way in)"""
    import ctypes as C
    x, thr = np.ascontiguousarray(L["x"]), np.ascontiguousarray(L["thr"])
    t = hip.Testcase(type=typ, batchcount=x.shape[0], channelcount=L["c"], inputW=L["iw"], inputH=L["ih"], kernelcount=L["kn"],
                     kernelW=L["kw"], kernelH=L["kh"], paddingW=L["pad"], paddingH=L["pad"], strideW=L["stride"],
                     strideH=L["stride"], preluAlpha=alpha, input_thresholds=thr.ctypes.data, input=x.ctypes.data,
                     quantized_kernel_packing2=qw_buf.ctypes.data)
    hip._L.tnns_conv(C.byref(t))
    oh, ow = hip.out_dim(L["ih"], L["pad"], L["kh"], L["stride"]), hip.out_dim(L["iw"], L["pad"], L["kw"], L["stride"])
    return hip._take(t.output, x.shape[0] * L["kn"] * oh * ow, np.float32)


@pytest.mark.parametrize("typ", ALL_TYPES, ids=lambda t: TYPE_NAMES[t])
def test_weights_rewritten_in_place_at_the_same_address(hip, oracle, typ):
    """tnns_conv keeps a layer's weights on the device in engine form, found again by address, size and a hash of the
    contents: rewriting the rows in place -- or packing another layer's into the same buffer, as the reference's
    driver does when malloc hands the address out again (src/timing_layers.c:127-137,212-215) -- must be seen"""
    wt = weight_is_ternary(typ)
    shape = (128, 9, 9, 64, 3, 3, 1, 1)
    L = make_layer(typ, shape, 2, seed=5100 + typ)
    q1 = oracle.pack_weights(L["w"], L["wthr"], wt)
    L2 = make_layer(typ, shape, 2, seed=5200 + typ)
    q2 = oracle.pack_weights(L2["w"], L2["wthr"], wt)
    assert q1.tobytes() != q2.tobytes()
    buf = np.empty_like(q1)
    for rep, q in enumerate((q1, q1, q2, q2, q1)):
        buf[:] = q                                  # same address every time
        want = oracle.conv(typ, L["x"], L["thr"], q, L["kn"], 3, 3, 1, 1, 0.5).reshape(-1)
        got = _conv_at(hip, typ, L, buf)
        assert got.tobytes() == want.tobytes(), rep
    # one flipped lane is another layer too
    buf[:] = q1
    buf[3] ^= 1 << 17
    want = oracle.conv(typ, L["x"], L["thr"], buf.copy(), L["kn"], 3, 3, 1, 1, 0.5).reshape(-1)
    assert _conv_at(hip, typ, L, buf).tobytes() == want.tobytes()
    # the same address and bytes under another layer shape (same row length, other kernel count / channel split)
    shape_b = (64, 9, 9, 128, 3, 3, 1, 1)
    Lb = make_layer(typ, shape_b, 2, seed=5300 + typ)
    qb = oracle.pack_weights(Lb["w"], Lb["wthr"], wt)
    if qb.size == buf.size:
        buf[:] = qb
        want = oracle.conv(typ, Lb["x"], Lb["thr"], qb, Lb["kn"], 3, 3, 1, 1, 0.5).reshape(-1)
        assert _conv_at(hip, typ, Lb, buf).tobytes() == want.tobytes()


def test_more_layers_than_the_weight_cache_holds(hip, oracle):
    """600 distinct small layers, then the first ones again: entries are dropped least recently used first and come back"""
    L = make_layer(TNN, (64, 5, 5, 32, 3, 3, 1, 1), 1, seed=6000)
    rng = np.random.default_rng(6)
    packs, wants = [], []
    for i in range(600):
        w = rng.integers(-1, 2, size=(32, 64, 3, 3)).astype(np.float32)
        q = oracle.pack_weights(w, np.full(32, 0.5, np.float32), True)
        packs.append(q)
        if i < 3 or i > 596:
            wants.append((i, oracle.conv(TNN, L["x"], L["thr"], q, 32, 3, 3, 1, 1, 0.5).reshape(-1)))
        got = _conv_at(hip, TNN, L, q)
        if i < 3 or i > 596:
            assert got.tobytes() == wants[-1][1].tobytes(), i
    for i, want in wants:
        assert _conv_at(hip, TNN, L, packs[i]).tobytes() == want.tobytes(), i


@pytest.mark.parametrize("pixels", [127, 512, 1023, 1024, 1025, 4095])
def test_copy_sizes_around_the_staging_chunks(hip, oracle, pixels):
    """tensors from half a KiB to just under 4 MiB go through the small pinned areas in chunks of 1 MiB: sizes below,
    at and above whole chunks, results up to 4 MiB minus a row"""
    c, kn = 64, 250                                    # x: pixels * 256 B, y: pixels * 1000 B
    L = make_layer(TBN, (c, 1, pixels, kn, 1, 1, 0, 1), 1, seed=6400 + pixels)
    qw = oracle.pack_weights(L["w"], L["wthr"], False)
    want = oracle.conv(TBN, L["x"], L["thr"], qw, kn, 1, 1, 0, 1, 0.5)
    for rep in range(2):
        got = hip.host_conv(TBN, L["x"], L["thr"], qw, kn, 1, 1, 0, 1, 0.5)
        assert got.tobytes() == want.tobytes(), rep


def test_same_rows_at_another_address_are_found_again(hip, oracle):
    """the prepared-weight cache knows a layer by the contents of its rows, their size and the layer shape, not by where
    they lie: a caller that packs the same weights again into fresh memory (the reference's e2e driver packs per layer
    and pass) adds no entry; different rows do; ftnn_host_forget_weights() drops them all"""
    L = make_layer(TNN, (128, 9, 9, 96, 3, 3, 1, 1), 2, seed=7100)
    q = oracle.pack_weights(L["w"], L["wthr"], True)
    want = oracle.conv(TNN, L["x"], L["thr"], q, L["kn"], 3, 3, 1, 1, 0.5).reshape(-1)
    hip.host_forget_weights()
    assert hip.host_cached_weight_bytes() == 0
    assert _conv_at(hip, TNN, L, q).tobytes() == want.tobytes()
    held = hip.host_cached_weight_bytes()
    assert held > 0
    for rep in range(3):
        other = np.empty(q.size + 8 * rep + 8, np.int64)[8 * rep + 4:][:q.size]      # another address every time
        other[:] = q
        assert other.ctypes.data != q.ctypes.data
        assert _conv_at(hip, TNN, L, other).tobytes() == want.tobytes()
        assert hip.host_cached_weight_bytes() == held, "identical rows must not add an entry"
    q2 = q.copy()
    q2[5] ^= 1 << 40
    want2 = oracle.conv(TNN, L["x"], L["thr"], q2, L["kn"], 3, 3, 1, 1, 0.5).reshape(-1)
    assert _conv_at(hip, TNN, L, q2).tobytes() == want2.tobytes()
    assert hip.host_cached_weight_bytes() == 2 * held
    hip.host_forget_weights()
    assert hip.host_cached_weight_bytes() == 0
    assert _conv_at(hip, TNN, L, q).tobytes() == want.tobytes()       # and the layer still runs
    assert hip.host_cached_weight_bytes() == held


def test_large_weight_rows_are_hashed_in_slices_and_kept(hip, oracle):
    """rows of 17 MiB: hashed in slices on the copy threads, kept like any other layer's, and a single flipped bit
    anywhere in them is seen"""
    c, kn, n = 16384, 4100, 2
    rng = np.random.default_rng(72)
    q = rng.integers(-2 ** 63, 2 ** 63, size=kn * 2 * (c // 64), dtype=np.int64)
    assert q.nbytes > 16 << 20
    x = rng.standard_normal((n, c, 1, 1)).astype(np.float32)
    thr = np.full(n, 0.5, np.float32)
    L = dict(x=x, thr=thr, c=c, ih=1, iw=1, kn=kn, kh=1, kw=1, pad=0, stride=1)
    want = oracle.conv(TNN, x, thr, q, kn, 1, 1, 0, 1, 0.5).reshape(-1)
    hip.host_forget_weights()
    for rep in range(2):
        assert _conv_at(hip, TNN, L, q).tobytes() == want.tobytes(), rep
    held = hip.host_cached_weight_bytes()
    assert held > 0
    for pos in (11, q.size // 2 + 3, q.size - 2):      # rewritten in place, in the first, a middle and the last slice
        q[pos] ^= 1 << 3
        want = oracle.conv(TNN, x, thr, q, kn, 1, 1, 0, 1, 0.5).reshape(-1)
        assert _conv_at(hip, TNN, L, q).tobytes() == want.tobytes(), pos
    assert hip.host_cached_weight_bytes() == 4 * held
    hip.host_forget_weights()


_NO_CACHE_CHILD = r"""
import sys
import numpy as np, torch
sys.path.insert(0, sys.argv[1])
import fastertnn_amd.lib as hip
from fastertnn_amd import TNN
from oracle.ftnn_oracle import Oracle
from tests.cases import make_layer
oracle = Oracle()
L = make_layer(TNN, (128, 9, 9, 96, 3, 3, 1, 1), 2, seed=7100)
q = oracle.pack_weights(L["w"], L["wthr"], True)
want = oracle.conv(TNN, L["x"], L["thr"], q, L["kn"], 3, 3, 1, 1, 0.5)
for rep in range(3):
    got = hip.host_conv(TNN, L["x"], L["thr"], q, L["kn"], 3, 3, 1, 1, 0.5)
    assert got.tobytes() == want.tobytes(), rep
    assert hip.host_cached_weight_bytes() == int(sys.argv[2]) * (rep >= 0), hip.host_cached_weight_bytes()
print("child ok")
"""


@pytest.mark.parametrize("env", [{"FTNN_HOST_NO_WEIGHT_CACHE": "1"}, {"FTNN_HOST_WEIGHT_CACHE_MB": "0"}])
def test_weight_cache_switched_off(env):
    """with the cache off (or capped below the layer's prepared weights) every call uploads and prepares its weights"""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    print("case weight cache off", env, flush=True)
    r = subprocess.run([sys.executable, "-c", _NO_CACHE_CHILD, root, "0"], env=dict(os.environ, **env), capture_output=True,
                       text=True, timeout=110)
    assert r.returncode == 0 and "child ok" in r.stdout, r.stdout[-1500:] + r.stderr[-1500:]


@pytest.mark.parametrize("ternary", [True, False], ids=["ternarize_opt_avx2", "binarize_opt_avx2"])
def test_host_weight_packers(hip, oracle, ternary):
    """the reference's weight packers on host pointers (src/utils.c:468-521, 634-675) against the oracle's restatement,
    word for word: channel tails, padding words, thresholds of either sign, a tensor beyond the 4 MiB staging chunks"""
    from fastertnn_amd import synth
    for shape in ((5, 3, 7, 7), (64, 64, 3, 3), (33, 65, 1, 1), (130, 127, 3, 3), (300, 1024, 2, 2)):
        kn, c, kh, kw = shape
        print("case host weight packer", ternary, shape, flush=True)
        w = synth.normal(kn * 31 + c, shape)
        for thr_value in (0.5, 0.0, -0.25):
            thr = np.full(kn, thr_value, np.float32)
            thr[::2] *= 0.5
            want = oracle.pack_weights(w, thr, ternary)
            got = hip.host_pack_weights(w, thr, ternary)
            assert got.tobytes() == np.ascontiguousarray(want).tobytes(), (shape, thr_value)


@pytest.mark.parametrize("rows,cols", [(1, 256), (3, 1280), (257, 4096), (600, 8192)])
def test_host_bitpacking2(hip, oracle, rows, cols):
    """bitpacking2 on host pointers (src/utils.c:257-291) against the oracle's, word for word; the last case moves 19 MB
    through the staging ring"""
    from fastertnn_amd import synth
    x = synth.ternary(rows * 7 + cols, (rows, cols))
    want = oracle.pack_gemm_operand(x)
    got = hip.host_pack_gemm_operand(x)
    assert got.tobytes() == np.ascontiguousarray(want).tobytes()
    # values outside {-1, 0} count as +1 (neither bit), as in the reference's if / else if
    x2 = x.copy()
    x2[0, :7] = (2.0, -3.0, 0.5, -0.0, 1e-30, -1.0, 7.0)
    assert hip.host_pack_gemm_operand(x2).tobytes() == np.ascontiguousarray(oracle.pack_gemm_operand(x2)).tobytes()
