"""ctypes binding of libftnn_hip.so (the C ABI declared in include/ftnn.h).

Device-memory entry points take torch CUDA tensors (used only as device buffers)
and run on torch's current stream.  Host-memory entry points are the reference's
own (`tnns_conv`, `tnns_gemm`, `t2r_p2_opt`, `b2r`, `mm_*`): they take numpy
arrays, and the heap buffer each one returns is copied into numpy and freed, as a
C caller would free it.
"""
import ctypes as C
import os

import numpy as np

from . import TNN, TBN, BTN, BNN, act_is_ternary, weight_is_ternary

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libftnn_hip.so")

if not os.path.exists(LIB_PATH):
    raise ImportError("%s is missing: build it with `python -m fastertnn_amd.build` "
                      "(there is no CPU fallback)" % LIB_PATH)

_L = C.CDLL(LIB_PATH)
_libc = C.CDLL(None)
_libc.free.argtypes = [C.c_void_p]

_vp = C.c_void_p
_L.ftnn_last_error.restype = C.c_char_p
_L.ftnn_version.restype = C.c_char_p
_L.ftnn_row_words.restype = C.c_int64
_L.ftnn_pack_scratch_bytes.restype = C.c_int64
_L.ftnn_quantize_im2row.argtypes = [C.c_int, _vp, _vp] + [C.c_int] * 10 + [_vp, _vp, _vp]
_L.ftnn_mm.argtypes = [C.c_int, _vp, _vp] + [C.c_int] * 6 + [C.c_float, _vp, _vp]
_L.ftnn_mm_scratch_bytes.restype = C.c_int64
_L.ftnn_mm_scratch_bytes.argtypes = [C.c_int] * 7
_L.ftnn_select_engine.argtypes = [C.c_int] * 6
_L.ftnn_mm_engine.argtypes = [C.c_int, C.c_int, _vp, _vp] + [C.c_int] * 6 + [C.c_float, _vp, _vp, C.c_int64, _vp]
_L.ftnn_expand_bytes.restype = C.c_int64
_L.ftnn_expand_bytes.argtypes = [C.c_int] * 3
_L.ftnn_expand_rows.argtypes = [C.c_int, C.c_int, _vp, C.c_int, C.c_int, _vp, _vp]
_L.ftnn_mm_expanded.argtypes = [C.c_int, C.c_int, _vp, _vp] + [C.c_int] * 6 + [C.c_float, _vp, _vp]
_L.ftnn_conv_scratch_bytes.restype = C.c_int64
_L.ftnn_conv_scratch_bytes.argtypes = [C.c_int] * 12
_L.ftnn_conv.argtypes = [C.c_int, _vp, _vp, _vp] + [C.c_int] * 11 + [C.c_float, _vp, _vp, _vp]
_L.ftnn_conv_static.argtypes = [C.c_int, _vp, _vp, _vp] + [C.c_int] * 11 + [C.c_float, _vp, _vp]
_L.ftnn_conv_engine.argtypes = [C.c_int, C.c_int, _vp, _vp, _vp] + [C.c_int] * 11 + [C.c_float, _vp, _vp, _vp]
_L.ftnn_select_conv_engine.argtypes = [C.c_int] * 12
_L.ftnn_conv_weights_bytes.restype = C.c_int64
_L.ftnn_conv_weights_bytes.argtypes = [C.c_int] * 5
_L.ftnn_conv_prepare_weights.argtypes = [C.c_int, _vp] + [C.c_int] * 4 + [_vp, _vp]
_L.ftnn_conv_prepared.argtypes = [C.c_int, _vp, _vp, _vp] + [C.c_int] * 11 + [C.c_float, _vp, _vp, _vp]
_L.ftnn_pack_weights.argtypes = [C.c_int, _vp, _vp] + [C.c_int] * 4 + [_vp, _vp]
_L.ftnn_pack_gemm_operand.argtypes = [_vp, C.c_int, C.c_int, _vp, _vp]
for _n in ("t2r_p2_opt", "b2r"):
    getattr(_L, _n).restype = _vp
    getattr(_L, _n).argtypes = [_vp, _vp] + [C.c_int] * 10
for _n in ("mm_tnn", "mm_tbn", "mm_btn"):
    getattr(_L, _n).restype = _vp
    getattr(_L, _n).argtypes = [_vp, _vp] + [C.c_int] * 5 + [C.c_float]
_L.mm_bnn.restype = _vp
_L.mm_bnn.argtypes = [_vp, _vp] + [C.c_int] * 6 + [C.c_float]
_L.tnns_conv.restype = None
_L.tnns_gemm.restype = None
_L.bitpacking2.restype = _vp
_L.bitpacking2.argtypes = [_vp, C.c_int, C.c_int]
for _n in ("ternarize_opt_avx2", "binarize_opt_avx2"):
    getattr(_L, _n).restype = _vp
    getattr(_L, _n).argtypes = [_vp, _vp] + [C.c_int] * 4
_L.ftnn_host_forget_weights.restype = None
_L.ftnn_host_release_spares.restype = None
_L.ftnn_host_cached_weight_bytes.restype = C.c_int64
_L.ftnn_host_hash128.restype = None
_L.ftnn_host_hash128.argtypes = [_vp, C.c_int64, C.c_int, C.POINTER(C.c_uint64)]
_L.ftnn_static_scratch_bytes.restype = C.c_int64

EXPORTS = ("tnns_conv", "tnns_gemm", "t2r_p2_opt", "b2r", "mm_tnn", "mm_tbn", "mm_btn", "mm_bnn",
           "bitpacking2", "ternarize_opt_avx2", "binarize_opt_avx2", "ftnn_host_forget_weights",
           "ftnn_host_release_spares", "ftnn_host_cached_weight_bytes", "ftnn_host_hash128", "ftnn_host_hash_uses_aes",
           "ftnn_static_scratch_bytes",
           "ftnn_last_error", "ftnn_version", "ftnn_out_dim", "ftnn_row_words",
           "ftnn_pack_scratch_bytes", "ftnn_quantize_im2row", "ftnn_mm", "ftnn_conv",
           "ftnn_pack_weights", "ftnn_pack_gemm_operand", "ftnn_select_engine", "ftnn_mm_scratch_bytes",
           "ftnn_mm_engine", "ftnn_expand_bytes", "ftnn_expand_rows", "ftnn_mm_expanded",
           "ftnn_conv_scratch_bytes", "ftnn_conv_engine", "ftnn_select_conv_engine",
           "ftnn_conv_static",
           "ftnn_conv_weights_bytes", "ftnn_conv_prepare_weights", "ftnn_conv_prepared", "ftnn_net_create", "ftnn_net_create_ex", "ftnn_net_destroy", "ftnn_net_output_elems", "ftnn_net_run")

ENGINE_AUTO, ENGINE_VALU, ENGINE_MFMA_I8, ENGINE_MFMA_F4 = 0, 1, 2, 3
ENGINE_NAMES = {ENGINE_VALU: "valu", ENGINE_MFMA_I8: "mfma_i8", ENGINE_MFMA_F4: "mfma_f4"}


class FtnnError(RuntimeError):
    pass


def _check(rc):
    if rc != 0:
        raise FtnnError("ftnn error %d: %s" % (rc, _L.ftnn_last_error().decode()))


def version():
    return _L.ftnn_version().decode()


def out_dim(n, pad, k, stride):
    return int(_L.ftnn_out_dim(n, pad, k, stride))


def row_words(c, kh, kw, ternary):
    return int(_L.ftnn_row_words(c, kh, kw, int(ternary)))


def pack_scratch_bytes(n, c, h, w, ternary):
    return int(_L.ftnn_pack_scratch_bytes(n, c, h, w, int(ternary)))


# ------------------------------------------------------------ device entry points

def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def _dev(t, dtype=None):
    import torch
    assert t.is_cuda and t.is_contiguous(), "expected a contiguous CUDA tensor"
    if dtype is not None:
        assert t.dtype == dtype, "expected %s, got %s" % (dtype, t.dtype)
    return t.data_ptr()


def quantize_im2row(x, thr, kh, kw, pad, stride, ternary, out=None, scratch=None):
    """t2r_p2_opt (ternary) / b2r (binary) on device tensors; returns int64 rows."""
    import torch
    n, c, h, w = x.shape
    oh, ow = out_dim(h, pad, kh, stride), out_dim(w, pad, kw, stride)
    if oh <= 0 or ow <= 0:
        raise FtnnError("kernel larger than padded input")
    words = row_words(c, kh, kw, ternary)
    if out is None:
        out = torch.empty(n * oh * ow * words, dtype=torch.int64, device=x.device)
    if scratch is None:
        scratch = torch.empty(pack_scratch_bytes(n, c, h, w, ternary), dtype=torch.uint8, device=x.device)
    _check(_L.ftnn_quantize_im2row(int(ternary), _dev(x, torch.float32), _dev(thr, torch.float32),
                                   n, c, h, w, pad, pad, kh, kw, stride, stride, _dev(out), _dev(scratch),
                                   _stream()))
    return out


def mm(typ, a, b, n, oh, ow, kn, k, alpha, k_unpack=0, out=None):
    """mm_tnn / mm_tbn / mm_btn / mm_bnn on device tensors; returns fp32 (n, kn, oh, ow)."""
    import torch
    if out is None:
        out = torch.empty((n, kn, oh, ow), dtype=torch.float32, device=a.device)
    _check(_L.ftnn_mm(typ, _dev(a), _dev(b), n, oh, ow, kn, k, k_unpack, alpha, _dev(out, torch.float32),
                      _stream()))
    return out


def conv_scratch_bytes(typ, n, c, h, w, kn, kh, kw, pad, stride):
    return int(_L.ftnn_conv_scratch_bytes(typ, n, c, h, w, kn, kh, kw, pad, pad, stride, stride))


def select_engine(typ, n, oh, ow, kn, k):
    return int(_L.ftnn_select_engine(typ, n, oh, ow, kn, k))


def mm_scratch_bytes(engine, typ, n, oh, ow, kn, k):
    return int(_L.ftnn_mm_scratch_bytes(engine, typ, n, oh, ow, kn, k))


def mm_engine(engine, typ, a, b, n, oh, ow, kn, k, alpha, k_unpack=0, out=None, scratch=None):
    """ftnn_mm_engine: the GEMM on an explicit engine (or AUTO); scratch is allocated if not given."""
    import torch
    if out is None:
        out = torch.empty((n, kn, oh, ow), dtype=torch.float32, device=a.device)
    need = mm_scratch_bytes(engine, typ, n, oh, ow, kn, k)
    if scratch is None and need > 0:
        scratch = torch.empty(need, dtype=torch.uint8, device=a.device)
    sp = _dev(scratch) if scratch is not None else None
    sb = scratch.numel() * scratch.element_size() if scratch is not None else 0
    _check(_L.ftnn_mm_engine(engine, typ, _dev(a), _dev(b), n, oh, ow, kn, k, k_unpack, alpha,
                             _dev(out, torch.float32), sp, sb, _stream()))
    return out


def expand_rows(engine, rows_t, n_rows, k, ternary, out=None):
    """ftnn_expand_rows: packed rows -> the operand format of a matrix-core engine."""
    import torch
    if out is None:
        out = torch.empty(int(_L.ftnn_expand_bytes(engine, n_rows, k)), dtype=torch.uint8, device=rows_t.device)
    _check(_L.ftnn_expand_rows(engine, int(ternary), _dev(rows_t), n_rows, k, _dev(out), _stream()))
    return out


def mm_expanded(engine, typ, a_exp, b_exp, n, oh, ow, kn, k, alpha, k_unpack=0, out=None):
    """ftnn_mm_expanded: the matrix-core GEMM on two expanded operands."""
    import torch
    if out is None:
        out = torch.empty((n, kn, oh, ow), dtype=torch.float32, device=a_exp.device)
    _check(_L.ftnn_mm_expanded(engine, typ, _dev(a_exp), _dev(b_exp), n, oh, ow, kn, k, k_unpack, alpha,
                               _dev(out, torch.float32), _stream()))
    return out


def select_conv_engine(typ, n, c, h, w, kn, kh, kw, pad, stride):
    return int(_L.ftnn_select_conv_engine(typ, n, c, h, w, kn, kh, kw, pad, pad, stride, stride))


def conv(typ, x, thr, qw, kn, kh, kw, pad, stride, alpha, scratch=None, out=None, engine=ENGINE_AUTO):
    """One conv layer (tnn_conv_p2 & co.) on device tensors; engine: AUTO, VALU or MFMA_F4."""
    import torch
    n, c, h, w = x.shape
    oh, ow = out_dim(h, pad, kh, stride), out_dim(w, pad, kw, stride)
    if oh <= 0 or ow <= 0:
        raise FtnnError("kernel larger than padded input")
    tern = act_is_ternary(typ)
    if scratch is None:
        scratch = torch.empty(conv_scratch_bytes(typ, n, c, h, w, kn, kh, kw, pad, stride), dtype=torch.uint8,
                              device=x.device)
    if out is None:
        out = torch.empty((n, kn, oh, ow), dtype=torch.float32, device=x.device)
    args = (typ, _dev(x, torch.float32), _dev(thr, torch.float32), _dev(qw), n, c, h, w, kn, kh, kw, pad, pad,
            stride, stride, alpha, _dev(scratch), _dev(out, torch.float32), _stream())
    _check(_L.ftnn_conv(*args) if engine == ENGINE_AUTO else _L.ftnn_conv_engine(engine, *args))
    return out


STATIC_SCRATCH_BYTES = int(_L.ftnn_static_scratch_bytes())   # FTNN_STATIC_SCRATCH_BYTES of the build


def conv_static(typ, x, thr, qw, kn, kh, kw, pad, stride, alpha, out):
    """ftnn_conv_static: the layer on the library's own fixed work space; allocates nothing (out is required)."""
    import torch
    n, c, h, w = x.shape
    _check(_L.ftnn_conv_static(typ, _dev(x, torch.float32), _dev(thr, torch.float32), _dev(qw), n, c, h, w, kn, kh,
                               kw, pad, pad, stride, stride, alpha, _dev(out, torch.float32), _stream()))
    return out


def prepare_conv_weights(typ, qw, c, kn, kh, kw):
    """ftnn_conv_prepare_weights: the packed rows in the form the layer's engine reads (once per layer)."""
    import torch
    out = torch.empty(int(_L.ftnn_conv_weights_bytes(typ, c, kn, kh, kw)), dtype=torch.uint8, device=qw.device)
    _check(_L.ftnn_conv_prepare_weights(typ, _dev(qw), c, kn, kh, kw, _dev(out), _stream()))
    return out


def conv_prepared(typ, x, thr, prepared, kn, kh, kw, pad, stride, alpha, scratch=None, out=None):
    """ftnn_conv_prepared: one conv layer with weights from prepare_conv_weights."""
    import torch
    n, c, h, w = x.shape
    oh, ow = out_dim(h, pad, kh, stride), out_dim(w, pad, kw, stride)
    if oh <= 0 or ow <= 0:
        raise FtnnError("kernel larger than padded input")
    if scratch is None:
        scratch = torch.empty(conv_scratch_bytes(typ, n, c, h, w, kn, kh, kw, pad, stride), dtype=torch.uint8,
                              device=x.device)
    if out is None:
        out = torch.empty((n, kn, oh, ow), dtype=torch.float32, device=x.device)
    _check(_L.ftnn_conv_prepared(typ, _dev(x, torch.float32), _dev(thr, torch.float32), _dev(prepared), n, c, h, w,
                                 kn, kh, kw, pad, pad, stride, stride, alpha, _dev(scratch),
                                 _dev(out, torch.float32), _stream()))
    return out


def pack_weights(w, thr, ternary):
    """ternarize_opt_avx2 / binarize_opt_avx2 on device tensors."""
    import torch
    kn, c, kh, kw = w.shape
    out = torch.empty(kn * row_words(c, kh, kw, ternary), dtype=torch.int64, device=w.device)
    _check(_L.ftnn_pack_weights(int(ternary), _dev(w, torch.float32), _dev(thr, torch.float32), kn, c, kh, kw,
                                _dev(out), _stream()))
    return out


def pack_gemm_operand(x):
    """bitpacking2 on a device tensor [I][J] of {-1,0,+1} floats."""
    import torch
    i, j = x.shape
    out = torch.empty(max(i * j // 32, 1), dtype=torch.int64, device=x.device)
    _check(_L.ftnn_pack_gemm_operand(_dev(x, torch.float32), i, j, _dev(out), _stream()))
    return out


class LayerDesc(C.Structure):
    """ftnn_layer_t"""
    _fields_ = [("type", C.c_int), ("C", C.c_int), ("H", C.c_int), ("W", C.c_int), ("KN", C.c_int),
                ("KH", C.c_int), ("KW", C.c_int), ("pad", C.c_int), ("stride", C.c_int),
                ("threshold", C.c_float), ("prelu_alpha", C.c_float), ("d_qw", _vp)]


_L.ftnn_net_create.restype = _vp
_L.ftnn_net_create.argtypes = [C.c_int, C.c_int, C.POINTER(LayerDesc)]
_L.ftnn_net_create_ex.restype = _vp
_L.ftnn_net_create_ex.argtypes = [C.c_int, C.c_int, C.POINTER(LayerDesc), C.c_int]
NET_REREAD_PREFIX = 1
_L.ftnn_net_destroy.restype = None
_L.ftnn_net_destroy.argtypes = [_vp]
_L.ftnn_net_output_elems.restype = C.c_int64
_L.ftnn_net_output_elems.argtypes = [_vp]
_L.ftnn_net_run.argtypes = [_vp, _vp, _vp, C.c_int, _vp]


class Net:
    """ftnn_net_*: a chain of conv layers with device-resident activations.
    `layers` is a list of dicts with keys type, shape (C, IH, IW, KN, KW, KH, pad, stride),
    threshold, alpha, qw (packed weights, int64 CUDA tensor, kept alive here)."""

    def __init__(self, batch, layers, flags=0):
        self.batch = batch
        self._weights = [l["qw"] for l in layers]
        arr = (LayerDesc * len(layers))()
        for d, l in zip(arr, layers):
            c, ih, iw, kn, kw, kh, pad, stride = l["shape"]
            d.type, d.C, d.H, d.W, d.KN, d.KH, d.KW, d.pad, d.stride = l["type"], c, ih, iw, kn, kh, kw, pad, stride
            d.threshold, d.prelu_alpha, d.d_qw = l["threshold"], l["alpha"], _dev(l["qw"])
        self._h = _L.ftnn_net_create_ex(batch, len(layers), arr, flags) if flags else _L.ftnn_net_create(batch, len(layers), arr)
        if not self._h:
            raise FtnnError(_L.ftnn_last_error().decode())
        c, ih, iw, kn, kw, kh, pad, stride = layers[-1]["shape"]
        self.out_shape = (batch, kn, out_dim(ih, pad, kh, stride), out_dim(iw, pad, kw, stride))
        assert int(_L.ftnn_net_output_elems(self._h)) == int(np.prod(self.out_shape))

    def run(self, x, out=None, graph=False):
        import torch
        if out is None:
            out = torch.empty(self.out_shape, dtype=torch.float32, device=x.device)
        _check(_L.ftnn_net_run(self._h, _dev(x, torch.float32), _dev(out, torch.float32), int(graph), _stream()))
        return out

    def close(self):
        if self._h and _L is not None:   # at interpreter shutdown the module's globals may be gone already
            _L.ftnn_net_destroy(self._h)
        self._h = None

    def __del__(self):
        self.close()


# -------------------------------------------------- reference (host) entry points

class Testcase(C.Structure):
    """testcase_t, include/tnns/data.h:4-25."""
    _fields_ = [("type", C.c_int), ("batchcount", C.c_int), ("channelcount", C.c_int),
                ("inputW", C.c_int), ("inputH", C.c_int), ("kernelcount", C.c_int),
                ("kernelW", C.c_int), ("kernelH", C.c_int), ("paddingW", C.c_int),
                ("paddingH", C.c_int), ("strideW", C.c_int), ("strideH", C.c_int),
                ("preluAlpha", C.c_float), ("input_thresholds", _vp), ("input", _vp),
                ("kernel", _vp), ("quantized_kernel_packing0", _vp),
                ("quantized_kernel_packing1", _vp), ("quantized_kernel_packing2", _vp),
                ("output", _vp)]


class TestcaseGemm(C.Structure):
    """testcase_tnns_gemm_t, include/tnns/data.h:27-41."""
    _fields_ = [("m", C.c_int), ("p", C.c_int), ("p_packed", C.c_int), ("n", C.c_int),
                ("x", _vp), ("w", _vp), ("x_packing0", _vp), ("x_packing1", _vp), ("x_packing2", _vp),
                ("w_packing0", _vp), ("w_packing1", _vp), ("w_packing2", _vp), ("output", _vp)]


def _take(ptr, n, dtype):
    buf = (C.c_char * (n * np.dtype(dtype).itemsize)).from_address(ptr)
    out = np.frombuffer(buf, dtype=dtype).copy()
    _libc.free(ptr)
    return out


def _np(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def host_quantize_im2row(x, thr, kh, kw, pad, stride, ternary):
    x, thr = _np(x, np.float32), _np(thr, np.float32)
    n, c, h, w = x.shape
    oh, ow = out_dim(h, pad, kh, stride), out_dim(w, pad, kw, stride)
    fn = _L.t2r_p2_opt if ternary else _L.b2r
    ptr = fn(x.ctypes.data, thr.ctypes.data, n, c, h, w, pad, pad, kh, kw, stride, stride)
    return _take(ptr, n * oh * ow * row_words(c, kh, kw, ternary), np.int64)


def host_mm(typ, a, b, n, oh, ow, kn, k, alpha, k_unpack=0):
    a, b = _np(a, np.int64), _np(b, np.int64)
    if typ == BNN:
        ptr = _L.mm_bnn(a.ctypes.data, b.ctypes.data, n, oh, ow, kn, k, k_unpack, alpha)
    else:
        fn = (_L.mm_tnn, _L.mm_tbn, _L.mm_btn)[typ]
        ptr = fn(a.ctypes.data, b.ctypes.data, n, oh, ow, kn, k, alpha)
    return _take(ptr, n * kn * oh * ow, np.float32).reshape(n, kn, oh, ow)


def host_conv(typ, x, thr, qw, kn, kh, kw, pad, stride, alpha):
    """tnns_conv on a testcase_t built from numpy arrays."""
    x, thr, qw = _np(x, np.float32), _np(thr, np.float32), _np(qw, np.int64)
    n, c, h, w = x.shape
    t = Testcase(type=typ, batchcount=n, channelcount=c, inputW=w, inputH=h, kernelcount=kn, kernelW=kw,
                 kernelH=kh, paddingW=pad, paddingH=pad, strideW=stride, strideH=stride, preluAlpha=alpha,
                 input_thresholds=thr.ctypes.data, input=x.ctypes.data,
                 quantized_kernel_packing2=qw.ctypes.data)
    _L.tnns_conv(C.byref(t))
    oh, ow = out_dim(h, pad, kh, stride), out_dim(w, pad, kw, stride)
    return _take(t.output, n * kn * oh * ow, np.float32).reshape(n, kn, oh, ow)


def host_pack_weights(w, thr, ternary):
    """ternarize_opt_avx2 / binarize_opt_avx2 on host pointers: fp32 (KN, C, KH, KW) -> Packing-2 rows"""
    w, thr = _np(w, np.float32), _np(thr, np.float32)
    kn, c, kh, kw = w.shape
    fn = _L.ternarize_opt_avx2 if ternary else _L.binarize_opt_avx2
    return _take(fn(w.ctypes.data, thr.ctypes.data, kn, c, kh, kw), kn * row_words(c, kh, kw, ternary), np.int64)


def host_pack_gemm_operand(x):
    """bitpacking2 on host pointers: fp32 [I][J] of {-1, 0, +1} -> Packing 2"""
    x = _np(x, np.float32)
    i, j = x.shape
    return _take(_L.bitpacking2(x.ctypes.data, i, j), i * j // 32, np.int64)


def host_hash128(a, portable=False):
    """the prepared-weight cache's content hash of a numpy array's bytes, as (low, high)"""
    a = np.ascontiguousarray(a)
    out = (C.c_uint64 * 2)()
    _L.ftnn_host_hash128(a.ctypes.data, a.nbytes, int(portable), out)
    return int(out[0]), int(out[1])


def host_forget_weights():
    _L.ftnn_host_forget_weights()


def host_cached_weight_bytes():
    return int(_L.ftnn_host_cached_weight_bytes())


def host_gemm(xp, wp, m, n, p_packed, into=None):
    """tnns_gemm; `into` (m x n float32) exercises the copy-into-output branch."""
    xp, wp = _np(xp, np.int64), _np(wp, np.int64)
    t = TestcaseGemm(m=m, p=p_packed * 64, p_packed=p_packed, n=n, x_packing2=xp.ctypes.data,
                     w_packing2=wp.ctypes.data)
    if into is not None:
        assert into.dtype == np.float32 and into.size == m * n and into.flags.c_contiguous
        t.output = into.ctypes.data
        _L.tnns_gemm(C.byref(t))
        return into
    _L.tnns_gemm(C.byref(t))
    return _take(t.output, m * n, np.float32).reshape(m, n)
