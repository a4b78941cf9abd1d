"""ftnn_conv_static, the layer entry point that allocates nothing, through the C ABI: its results against
ftnn_conv's on the same inputs (bit-exact), on consecutive calls that share the library's fixed work space --
a larger layer first, then a smaller one whose scratch layout lies inside what the first call left behind --
and against the oracle.  Also its size limit."""
import numpy as np
import pytest

from fastertnn_amd import TNN, TBN, BTN, BNN, TYPE_NAMES, act_is_ternary, weight_is_ternary
from tests.cases import make_layer

pytestmark = pytest.mark.gpu


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _layer_on_device(hip, typ, shape, batch, seed):
    L = make_layer(typ, shape, batch, seed)
    qw = hip.pack_weights(_dev(L["w"]), _dev(L["wthr"]), weight_is_ternary(typ))
    return L, _dev(L["x"]), _dev(L["thr"]), qw


# (C, IH, IW, KN, KW, KH, pad, stride): a big layer, then smaller ones of other forms (fp4 64 x 64 tiles, 32 x 32
# tiles, a few-channel first layer in one kernel, the vector-ALU dense path with 8 < C <= 32)
SEQUENCE = [
    ((128, 28, 28, 128, 3, 3, 1, 1), 8),
    ((64, 9, 9, 40, 3, 3, 1, 1), 2),
    ((3, 32, 32, 16, 7, 7, 3, 2), 2),
    ((16, 11, 7, 40, 5, 5, 2, 2), 3),
    ((256, 14, 14, 256, 3, 3, 1, 2), 4),
    ((200, 1, 1, 10, 1, 1, 0, 1), 1),
]


@pytest.mark.parametrize("typ", (TNN, TBN, BTN, BNN), ids=lambda t: TYPE_NAMES[t])
def test_static_scratch_layer_matches_ftnn_conv_on_calls_in_a_row(hip, oracle, typ):
    import torch
    for i, (shape, batch) in enumerate(SEQUENCE):
        print("case", TYPE_NAMES[typ], shape, "batch", batch, flush=True)
        L, x, thr, qw = _layer_on_device(hip, typ, shape, batch, seed=4000 + 31 * i + typ)
        assert hip.conv_scratch_bytes(typ, batch, L["c"], L["ih"], L["iw"], L["kn"], L["kh"], L["kw"], L["pad"],
                                      L["stride"]) <= hip.STATIC_SCRATCH_BYTES
        want = hip.conv(typ, x, thr, qw, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"])
        got = torch.full_like(want, float("nan"))
        hip.conv_static(typ, x, thr, qw, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"], out=got)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), (TYPE_NAMES[typ], shape)
        if i < 2:   # and against the oracle itself
            qw_o = oracle.pack_weights(L["w"], L["wthr"], weight_is_ternary(typ))
            y_o = oracle.conv(typ, L["x"], L["thr"], qw_o, L["kn"], L["kh"], L["kw"], L["pad"], L["stride"], L["alpha"])
            assert got.cpu().numpy().tobytes() == np.ascontiguousarray(y_o).tobytes()


def test_static_scratch_layer_allocates_nothing(hip):
    """device memory in use does not move across calls once the entry point has run on this device"""
    import torch
    L, x, thr, qw = _layer_on_device(hip, TNN, (64, 9, 9, 40, 3, 3, 1, 1), 2, seed=77)
    out = torch.empty((2, 40, 9, 9), device="cuda")
    hip.conv_static(TNN, x, thr, qw, 40, 3, 3, 1, 1, 0.5, out=out)   # first call: looks the array's address up
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(20):
        hip.conv_static(TNN, x, thr, qw, 40, 3, 3, 1, 1, 0.5, out=out)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0


def test_static_scratch_layer_refuses_what_does_not_fit(hip):
    import ctypes as C
    n, c, h, w, kn = 64, 512, 56, 56, 512
    need = hip.conv_scratch_bytes(TNN, n, c, h, w, kn, 3, 3, 1, 1)
    assert need > hip.STATIC_SCRATCH_BYTES
    p = C.c_void_p(256)   # never read: the size check comes first
    rc = hip._L.ftnn_conv_static(TNN, p, p, p, n, c, h, w, kn, 3, 3, 1, 1, 1, 1, 0.5, p, None)
    assert rc == -1 and b"ftnn_conv_static holds" in hip._L.ftnn_last_error()
