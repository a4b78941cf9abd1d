"""ctypes bindings of the checker: TEST INFRASTRUCTURE ONLY.

Three libraries are bound here:

* ``Oracle``     -- ``libftnn_oracle.so``, the plain-C restatement in this directory.
* ``OracleAvx2`` -- ``libftnn_oracle_avx2.so``, the TNN GEMM restated with AVX2 intrinsics
  (the reference's blocking and popcount scheme): the benchmark's CPU baseline where the
  compiled reference is absent.
* ``Reference``  -- ``_ref/libref_final.so``, the reference's own AVX2 "final" path
  compiled from its sources (present only where ``make ref`` ran or its output
  was carried along).  It validates the restatement, writes the golden vectors
  and serves as the CPU baseline of the benchmark.
* ``ReferenceBaseline`` -- ``_ref/libref_baseline.so``, the reference's Packing-0
  "baseline" build (src/tnns/tnns_cpu_naive.c), an independent second reference.

Only the test-suite, the smoke check and the benchmark's CPU-baseline leg may
import this module; the shipped library never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "libftnn_oracle.so")
ORACLE_AVX2_SO = os.path.join(HERE, "libftnn_oracle_avx2.so")
REF_SO = os.path.join(HERE, "_ref", "libref_final.so")
REF_BASELINE_SO = os.path.join(HERE, "_ref", "libref_baseline.so")

TNN, TBN, BTN, BNN = 0, 1, 2, 3
TYPE_NAMES = {TNN: "tnn", TBN: "tbn", BTN: "btn", BNN: "bnn"}

_i64p = C.POINTER(C.c_int64)
_f32p = C.POINTER(C.c_float)
_i32p = C.POINTER(C.c_int32)


def build(with_reference=True):
    """Compile the checker (and the reference where its tree is present)."""
    subprocess.run(["make", "-C", HERE, "oracle"] + (["ref"] if with_reference else []),
                   check=True, stdout=subprocess.DEVNULL)


def aligned_empty(n, dtype, align=64):
    """1-D array whose data pointer is `align`-byte aligned (the reference's GEMM
    uses aligned 256-bit loads, mm_p2_final_tnn_avx2.c:130-133)."""
    dtype = np.dtype(dtype)
    raw = np.empty(n * dtype.itemsize + align, dtype=np.uint8)
    off = (-raw.ctypes.data) % align
    return raw[off:off + n * dtype.itemsize].view(dtype)


def aligned_copy(a, align=64):
    out = aligned_empty(a.size, a.dtype, align)
    out[:] = a.reshape(-1)
    return out.reshape(a.shape)


def _p(a, typ):
    return a.ctypes.data_as(typ)


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def cpack(c):
    return (c + 63) // 64


def round4(k):
    return 4 * ((k + 3) // 4)


def out_dim(n, pad, k, stride):
    return (n + 2 * pad - k) // stride + 1


class Oracle:
    def __init__(self, path=ORACLE_SO):
        if not os.path.exists(path):
            build(with_reference=False)
        L = self.lib = C.CDLL(path)
        L.orc_row_words.restype = C.c_int64
        L.orc_pack_gemm_operand.restype = C.c_int
        for name in ("orc_pack_weights_ternary", "orc_pack_weights_binary", "orc_t2r_p2", "orc_b2r",
                     "orc_mm_tnn", "orc_mm_tbn", "orc_mm_btn", "orc_mm_bnn", "orc_tnns_conv",
                     "orc_tnns_gemm"):
            getattr(L, name).restype = None

    def row_words(self, c, kh, kw, ternary):
        return int(self.lib.orc_row_words(c, kh, kw, int(ternary)))

    def pack_weights(self, w, thr, ternary):
        w = _f32(w)
        thr = _f32(thr)
        kn, c, kh, kw = w.shape
        out = aligned_empty(kn * self.row_words(c, kh, kw, ternary), np.int64)
        fn = self.lib.orc_pack_weights_ternary if ternary else self.lib.orc_pack_weights_binary
        fn(_p(w, _f32p), _p(thr, _f32p), kn, c, kh, kw, _p(out, _i64p))
        return out

    def pack_gemm_operand(self, x):
        x = _f32(x)
        i, j = x.shape
        out = aligned_empty(i * j // 32, np.int64)
        if self.lib.orc_pack_gemm_operand(_p(x, _f32p), i, j, _p(out, _i64p)) != 0:
            raise ValueError("J must be a multiple of 256")
        return out

    def quantize_im2row(self, x, thr, kh, kw, pad, stride, ternary):
        x = _f32(x)
        thr = _f32(thr)
        n, c, h, w = x.shape
        oh, ow = out_dim(h, pad, kh, stride), out_dim(w, pad, kw, stride)
        out = aligned_empty(n * oh * ow * self.row_words(c, kh, kw, ternary), np.int64)
        fn = self.lib.orc_t2r_p2 if ternary else self.lib.orc_b2r
        fn(_p(x, _f32p), _p(thr, _f32p), n, c, h, w, pad, pad, kh, kw, stride, stride, _p(out, _i64p))
        return out

    def mm(self, typ, a, b, n, oh, ow, kn, k, alpha, k_unpack=0, want_acc=False):
        y = np.empty(n * kn * oh * ow, dtype=np.float32)
        acc = np.empty(n * kn * oh * ow, dtype=np.int32) if want_acc else None
        accp = _p(acc, _i32p) if want_acc else None
        args = [_p(a, _i64p), _p(b, _i64p), n, oh, ow, kn, k]
        if typ == BNN:
            self.lib.orc_mm_bnn(*args, k_unpack, C.c_float(alpha), _p(y, _f32p), accp)
        else:
            fn = (self.lib.orc_mm_tnn, self.lib.orc_mm_tbn, self.lib.orc_mm_btn)[typ]
            fn(*args, C.c_float(alpha), _p(y, _f32p), accp)
        return (y, acc) if want_acc else y

    def conv(self, typ, x, thr, qw, kn, kh, kw, pad, stride, alpha):
        x = _f32(x)
        thr = _f32(thr)
        n, c, h, w = x.shape
        oh, ow = out_dim(h, pad, kh, stride), out_dim(w, pad, kw, stride)
        scratch = aligned_empty(n * oh * ow * self.row_words(c, kh, kw, typ in (TNN, TBN)), np.int64)
        y = np.empty((n, kn, oh, ow), dtype=np.float32)
        self.lib.orc_tnns_conv(typ, _p(x, _f32p), _p(thr, _f32p), _p(qw, _i64p), n, c, h, w, kn, kh, kw,
                               pad, pad, stride, stride, C.c_float(alpha), _p(scratch, _i64p), _p(y, _f32p))
        return y

    def gemm(self, xp, wp, m, n, p_packed):
        y = np.empty((m, n), dtype=np.float32)
        self.lib.orc_tnns_gemm(_p(xp, _i64p), _p(wp, _i64p), m, n, p_packed, _p(y, _f32p))
        return y


class OracleAvx2:
    """orc_avx2_mm_tnn: needs a CPU with AVX2 and 32-byte aligned operands (aligned_copy)"""

    @staticmethod
    def available():
        try:
            flags = next(l for l in open("/proc/cpuinfo") if l.startswith("flags"))
        except (OSError, StopIteration):
            return False
        return " avx2" in flags and os.path.exists(ORACLE_AVX2_SO)

    def __init__(self, path=ORACLE_AVX2_SO):
        self.lib = C.CDLL(path)
        self.lib.orc_avx2_mm_tnn.restype = None

    def mm(self, typ, a, b, n, oh, ow, kn, k, alpha, k_unpack=0):
        assert typ == TNN, "the AVX2 restatement covers the TNN GEMM"
        assert a.ctypes.data % 32 == 0 and b.ctypes.data % 32 == 0
        y = np.empty(n * kn * oh * ow, dtype=np.float32)
        self.lib.orc_avx2_mm_tnn(_p(a, _i64p), _p(b, _i64p), n, oh, ow, kn, k, C.c_float(alpha), _p(y, _f32p))
        return y


class _Testcase(C.Structure):
    # include/tnns/data.h:4-25
    _fields_ = [("type", C.c_int), ("batchcount", C.c_int), ("channelcount", C.c_int),
                ("inputW", C.c_int), ("inputH", C.c_int), ("kernelcount", C.c_int),
                ("kernelW", C.c_int), ("kernelH", C.c_int), ("paddingW", C.c_int),
                ("paddingH", C.c_int), ("strideW", C.c_int), ("strideH", C.c_int),
                ("preluAlpha", C.c_float), ("input_thresholds", C.c_void_p), ("input", C.c_void_p),
                ("kernel", C.c_void_p), ("quantized_kernel_packing0", C.c_void_p),
                ("quantized_kernel_packing1", C.c_void_p), ("quantized_kernel_packing2", C.c_void_p),
                ("output", C.c_void_p)]


class Reference:
    """The compiled reference.  Every routine returns heap memory that the caller
    frees (src/timing_layers.c:160,176); results are copied into numpy and freed."""

    def __init__(self, path=REF_SO):
        if not os.path.exists(path):
            raise FileNotFoundError(path)
        L = self.lib = C.CDLL(path)
        self.libc = C.CDLL(None)
        self.libc.free.argtypes = [C.c_void_p]
        for name in ("t2r_p2_opt", "b2r", "mm_tnn", "mm_tbn", "mm_btn", "mm_bnn", "ternarize_opt_avx2",
                     "binarize_opt_avx2", "bitpacking2", "direct_pad", "direct_conv2d", "direct_mmm"):
            getattr(L, name).restype = C.c_void_p
        L.tnns_conv.restype = None

    @staticmethod
    def available():
        return os.path.exists(REF_SO)

    def _take(self, ptr, n, dtype):
        if not ptr:
            raise MemoryError("reference returned NULL")
        buf = (C.c_char * (n * np.dtype(dtype).itemsize)).from_address(ptr)
        out = aligned_copy(np.frombuffer(buf, dtype=dtype))
        self.libc.free(ptr)
        return out

    def pack_weights(self, w, thr, ternary):
        w = _f32(w)
        thr = _f32(thr)
        kn, c, kh, kw = w.shape
        words = round4(cpack(c) * kh * kw) * (2 if ternary else 1)
        fn = self.lib.ternarize_opt_avx2 if ternary else self.lib.binarize_opt_avx2
        return self._take(fn(_p(w, _f32p), _p(thr, _f32p), kn, c, kh, kw), kn * words, np.int64)

    def pack_gemm_operand(self, x):
        x = _f32(x)
        i, j = x.shape
        return self._take(self.lib.bitpacking2(_p(x, _f32p), i, j), i * j // 32, np.int64)

    def quantize_im2row(self, x, thr, kh, kw, pad, stride, ternary):
        x = aligned_copy(_f32(x))
        thr = _f32(thr)
        n, c, h, w = x.shape
        oh, ow = out_dim(h, pad, kh, stride), out_dim(w, pad, kw, stride)
        words = round4(cpack(c) * kh * kw) * (2 if ternary else 1)
        fn = self.lib.t2r_p2_opt if ternary else self.lib.b2r
        ptr = fn(_p(x, _f32p), _p(thr, _f32p), n, c, h, w, pad, pad, kh, kw, stride, stride)
        return self._take(ptr, n * oh * ow * words, np.int64)

    def mm(self, typ, a, b, n, oh, ow, kn, k, alpha, k_unpack=0):
        args = [_p(a, _i64p), _p(b, _i64p), n, oh, ow, kn, k]
        if typ == BNN:
            ptr = self.lib.mm_bnn(*args, k_unpack, C.c_float(alpha))
        else:
            ptr = (self.lib.mm_tnn, self.lib.mm_tbn, self.lib.mm_btn)[typ](*args, C.c_float(alpha))
        return self._take(ptr, n * kn * oh * ow, np.float32)

    def conv(self, typ, x, thr, qw, kn, kh, kw, pad, stride, alpha):
        x = aligned_copy(_f32(x))
        thr = _f32(thr)
        n, c, h, w = x.shape
        t = _Testcase(type=typ, batchcount=n, channelcount=c, inputW=w, inputH=h, kernelcount=kn,
                      kernelW=kw, kernelH=kh, paddingW=pad, paddingH=pad, strideW=stride, strideH=stride,
                      preluAlpha=alpha, input_thresholds=thr.ctypes.data, input=x.ctypes.data,
                      quantized_kernel_packing2=qw.ctypes.data)
        self.lib.tnns_conv(C.byref(t))
        oh, ow = out_dim(h, pad, kh, stride), out_dim(w, pad, kw, stride)
        return self._take(t.output, n * kn * oh * ow, np.float32).reshape(n, kn, oh, ow)

    def direct_conv(self, x, w, pad, stride, alpha, pad_val):
        """The reference's own fp32 self-test path (src/timing_layers.c:150-152)."""
        x = _f32(x)
        w = _f32(w)
        n, c, h, wd = x.shape
        kn, _, kh, kw = w.shape
        px = self.lib.direct_pad(_p(x, _f32p), pad, pad, n, c, h, wd, pad_val)
        y = self.lib.direct_conv2d(C.c_void_p(px), _p(w, _f32p), stride, stride, n, c, h + 2 * pad,
                                   wd + 2 * pad, kn, kh, kw, C.c_float(alpha))
        self.libc.free(px)
        oh, ow = out_dim(h, pad, kh, stride), out_dim(wd, pad, kw, stride)
        return self._take(y, n * kn * oh * ow, np.float32).reshape(n, kn, oh, ow)


class ReferenceBaseline:
    """The reference's "baseline" build (Packing 0, separate ternarise / img2row / popcount GEMM /
    PReLU passes, src/tnns/tnns_cpu_naive.c:255-292): an implementation independent of the Packing-2
    path, used as a second reference and for the reference's own "baseline vs final" comparison
    (Makefile:50)."""

    def __init__(self, path=REF_BASELINE_SO):
        if not os.path.exists(path):
            raise FileNotFoundError(path)
        L = self.lib = C.CDLL(path)
        self.libc = C.CDLL(None)
        self.libc.free.argtypes = [C.c_void_p]
        L.ternarize_naive.restype = C.c_void_p
        L.binarize_naive.restype = C.c_void_p
        L.tnns_conv.restype = None

    @staticmethod
    def available():
        return os.path.exists(REF_BASELINE_SO)

    def pack_weights(self, w, wthr, ternary):
        """ternarize_naive / binarize_naive on the weights, as src/timing_layers.c:129-133 does;
        returns the raw pointer (freed by free_weights)"""
        w = _f32(w)
        wthr = _f32(wthr)
        kn, c, kh, kw = w.shape
        fn = self.lib.ternarize_naive if ternary else self.lib.binarize_naive
        ptr = fn(_p(w, _f32p), _p(wthr, _f32p), kn, c, kh, kw, 0, 0)
        if not ptr:
            raise MemoryError("reference returned NULL")
        return ptr

    def free_weights(self, ptr):
        self.libc.free(ptr)

    def conv(self, typ, x, thr, qw0_ptr, kn, kh, kw, pad, stride, alpha):
        x = aligned_copy(_f32(x))
        thr = _f32(thr)
        n, c, h, w = x.shape
        t = _Testcase(type=typ, batchcount=n, channelcount=c, inputW=w, inputH=h, kernelcount=kn,
                      kernelW=kw, kernelH=kh, paddingW=pad, paddingH=pad, strideW=stride, strideH=stride,
                      preluAlpha=alpha, input_thresholds=thr.ctypes.data, input=x.ctypes.data,
                      quantized_kernel_packing0=qw0_ptr)
        self.lib.tnns_conv(C.byref(t))
        oh, ow = out_dim(h, pad, kh, stride), out_dim(w, pad, kw, stride)
        buf = (C.c_char * (n * kn * oh * ow * 4)).from_address(t.output)
        out = np.frombuffer(buf, dtype=np.float32).copy().reshape(n, kn, oh, ow)
        self.libc.free(t.output)
        return out
