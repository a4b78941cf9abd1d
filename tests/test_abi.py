"""The C-ABI library without a GPU: it loads, exports every symbol that include/ftnn.h
declares, keeps the reference's struct layouts, and rejects bad arguments before any
device work.  Also pins the seeded input generators.  CPU only."""
import ctypes as C
import os
import re
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ftnn.h")


def declared_symbols():
    text = open(HEADER).read()
    return sorted(set(re.findall(r"^FTNN_API [^;(]*?\**\s*\*?(\w+)\(", text, flags=re.M)))


def test_header_declares_the_reference_entry_points():
    names = declared_symbols()
    for want in ("tnns_conv", "tnns_gemm", "t2r_p2_opt", "b2r", "mm_tnn", "mm_tbn", "mm_btn", "mm_bnn"):
        assert want in names
    assert len(names) >= 18


def test_library_exports_every_declared_symbol():
    import fastertnn_amd.lib as lib
    dll = C.CDLL(lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(dll, name), "libftnn_hip.so does not export " + name
    assert sorted(lib.EXPORTS) == declared_symbols()


def test_struct_layout_matches_the_reference(tmp_path):
    """testcase_t is 112 bytes with `output` at 104, testcase_tnns_gemm_t 88 bytes with
    `output` at 80 (include/tnns/data.h:4-41 on LP64)"""
    src = tmp_path / "layout.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "ftnn.h"\n'
                   "int main(void){printf(\"%zu %zu %zu %zu %zu %zu %d\\n\", sizeof(testcase_t),"
                   "offsetof(testcase_t, preluAlpha), offsetof(testcase_t, input_thresholds),"
                   "offsetof(testcase_t, output), sizeof(testcase_tnns_gemm_t),"
                   "offsetof(testcase_tnns_gemm_t, output), (int)BNN);return 0;}\n")
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)],
                   check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    assert out == ["112", "48", "56", "104", "88", "80", "3"]
    import fastertnn_amd.lib as lib
    assert C.sizeof(lib.Testcase) == 112 and C.sizeof(lib.TestcaseGemm) == 88
    assert lib.Testcase.output.offset == 104 and lib.TestcaseGemm.output.offset == 80


def test_shape_helpers_match_the_oracle(oracle):
    import fastertnn_amd.lib as lib
    for c in (1, 3, 63, 64, 65, 127, 128, 257, 1024):
        for (kh, kw) in ((1, 1), (3, 3), (5, 3), (7, 7)):
            for tern in (0, 1):
                assert lib.row_words(c, kh, kw, tern) == oracle.row_words(c, kh, kw, tern)
    assert lib.out_dim(224, 3, 7, 2) == 112 and lib.out_dim(14, 1, 5, 2) == 6 and lib.out_dim(1, 0, 1, 1) == 1
    assert lib.pack_scratch_bytes(2, 65, 3, 5, 1) == 2 * 15 * 2 * 16
    assert lib.pack_scratch_bytes(2, 65, 3, 5, 0) == 2 * 15 * 2 * 8


def test_bad_arguments_are_rejected_without_touching_the_device():
    import fastertnn_amd.lib as lib
    L = lib._L
    buf = (C.c_char * 4096)()
    p = C.addressof(buf) & ~15
    assert L.ftnn_pack_gemm_operand(p, 4, 100, p, None) == -1          # J % 256 != 0 (src/utils.c:258)
    assert b"256" in L.ftnn_last_error()
    assert L.ftnn_pack_gemm_operand(None, 4, 256, p, None) == -1
    assert L.ftnn_mm(7, p, p, 1, 1, 1, 1, 4, 0, 0.5, p, None) == -1         # unknown type
    assert L.ftnn_mm(0, p, p, 0, 1, 1, 1, 4, 0, 0.5, p, None) == -1         # empty batch
    assert L.ftnn_mm(0, p + 8, p, 1, 1, 1, 1, 4, 0, 0.5, p, None) == -1     # misaligned operand
    assert L.ftnn_mm(0, None, p, 1, 1, 1, 1, 4, 0, 0.5, p, None) == -1
    # kernel larger than the padded input
    assert L.ftnn_quantize_im2row(1, p, p, 1, 8, 2, 2, 0, 0, 3, 3, 1, 1, p, p, None) == -1
    assert L.ftnn_quantize_im2row(1, p, p, 1, 8, 4, 4, 0, 0, 3, 3, 0, 1, p, p, None) == -1  # stride 0
    assert L.ftnn_conv(9, p, p, p, 1, 8, 4, 4, 4, 3, 3, 1, 1, 1, 1, 0.5, p, p, None) == -1
    assert L.ftnn_pack_weights(1, p, p, 0, 8, 3, 3, p, None) == -1


def test_engine_selection_and_scratch_sizes_need_no_device():
    import fastertnn_amd.lib as lib
    # the large GEMM goes to the fp4 matrix-core engine, layer-sized problems stay on the vector ALU
    assert lib.select_engine(0, 8192, 1, 1, 8192, 512) == lib.ENGINE_MFMA_F4
    assert lib.select_engine(0, 2048, 1, 1, 2048, 256) == lib.ENGINE_MFMA_F4
    assert lib.select_engine(0, 1, 56, 56, 256, 36) == lib.ENGINE_VALU
    assert lib.select_engine(0, 32, 56, 56, 64, 9) == lib.ENGINE_VALU
    assert lib.select_engine(0, 1024, 1, 1, 1024, 128) == lib.ENGINE_MFMA_F4      # the mid sizes of the reference's sweep too
    assert lib.select_engine(0, 512, 1, 1, 512, 64) == lib.ENGINE_VALU            # too little work for three launches
    # fp32 accumulation of the fp4 GEMM's products (multiples of 1/4) is exact up to 2^22 lanes: never chosen beyond
    assert lib.select_engine(0, 4096, 1, 1, 4096, 1 << 16) == lib.ENGINE_MFMA_F4
    assert lib.select_engine(0, 4096, 1, 1, 4096, (1 << 16) + 4) == lib.ENGINE_VALU
    assert lib.select_engine(0, 4096, 1, 1, 4096, 1 << 18) == lib.ENGINE_VALU
    assert lib.mm_scratch_bytes(lib.ENGINE_VALU, 0, 8192, 1, 1, 8192, 512) == 0
    assert lib.mm_scratch_bytes(lib.ENGINE_MFMA_F4, 0, 8192, 1, 1, 8192, 512) == 2 * (256 * 256 * 1024 + 8192 * 4)   # two bits per lane + a sum per row
    assert lib.mm_scratch_bytes(lib.ENGINE_MFMA_I8, 0, 33, 1, 1, 1, 4) == (2 + 1) * 8 * 1024
    assert lib.mm_scratch_bytes(lib.ENGINE_AUTO, 0, 8192, 1, 1, 8192, 512) == 2 * (256 * 256 * 1024 + 8192 * 4)
    assert lib._L.ftnn_expand_bytes(lib.ENGINE_MFMA_F4, 100, 6) == 4 * 4 * 1024 + 128 * 4   # 4 row blocks x 4 pairs of K words, 128 row sums
    assert lib._L.ftnn_expand_bytes(lib.ENGINE_MFMA_I8, 100, 6) == 4 * 16 * 1024
    assert lib._L.ftnn_expand_bytes(lib.ENGINE_VALU, 100, 6) == 0
    # conv scratch covers either layer engine.  Vector ALU: the quantised input (16 bytes per pixel and 64
    # channels), plus dense rows and weights when C <= 32 packs several taps per word.  fp4 matrix cores: 32 bytes
    # per pixel and 64 channels, plus 1 KiB per 32 kernels and word of the rounded-up row.
    assert lib.pack_scratch_bytes(2, 64, 8, 8, 1) == 2 * 8 * 8 * 16
    assert lib.conv_scratch_bytes(0, 2, 64, 8, 8, 16, 3, 3, 1, 1) == 2 * 8 * 8 * 32 + 1 * 12 * 1024
    valu_dense = 2 * 32 * 32 * 16 + 2 * 16 * 16 * 4 * 16 + 16 * 4 * 16
    # fp4 with C <= 8: a nibble dword per input pixel, 32 bytes per output pixel and dense word, fragments and
    # re-packed rows of the weights
    fp4_dense = 2 * 32 * 32 * 4 + 2 * 16 * 16 * 3 * 32 + 1 * 4 * 1024 + 16 * 4 * 16
    assert lib.conv_scratch_bytes(0, 2, 3, 32, 32, 16, 7, 7, 3, 2) == max(valu_dense, fp4_dense)
    # layer engine: fp4 wherever the dense re-packing does not apply and fp32 accumulation stays exact
    assert lib.select_conv_engine(0, 1, 256, 56, 56, 256, 3, 3, 1, 1) == lib.ENGINE_MFMA_F4
    assert lib.select_conv_engine(0, 32, 3, 224, 224, 64, 7, 7, 3, 2) == lib.ENGINE_MFMA_F4   # dense re-packing, C <= 8
    assert lib.select_conv_engine(0, 4, 16, 20, 20, 64, 3, 3, 1, 1) == lib.ENGINE_VALU         # dense re-packing, C > 8


def test_missing_library_is_an_import_error(tmp_path):
    """no silent CPU fallback: the binding refuses to import without the built library"""
    pkg = tmp_path / "fastertnn_amd"
    pkg.mkdir()
    for f in ("__init__.py", "lib.py"):
        (pkg / f).write_text(open(os.path.join(ROOT, "fastertnn_amd", f)).read())
    r = subprocess.run(["python3", "-c", "import fastertnn_amd.lib"], cwd=str(tmp_path), capture_output=True,
                       text=True, env={**os.environ, "PYTHONPATH": str(tmp_path)})
    assert r.returncode != 0 and "no CPU fallback" in r.stderr


def test_seeded_generators_are_pinned():
    from fastertnn_amd import synth
    z = synth.splitmix64(0, 3)
    # SplitMix64 reference outputs for seed 0 (first three of the published test vector)
    assert [int(v) for v in z] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    t = synth.ternary(1, (4096,))
    assert set(np.unique(t)) == {-1.0, 0.0, 1.0} and abs(float(t.mean())) < 0.05
    b = synth.binary(1, (4096,))
    assert set(np.unique(b)) == {-1.0, 1.0}
    g = synth.normal(1, (1 << 16,))
    assert abs(float(g.mean())) < 0.02 and abs(float(g.std()) - 1.0) < 0.02
    assert np.array_equal(synth.normal(9, (1000,))[100:200], synth.normal(9, (200,))[100:200])


def test_build_refuses_scratch_in_hand_counted_kernels():
    """the build's guard for kernels whose loads are counted by hand: scratch use there is an error"""
    from fastertnn_amd import build
    ok = ("x.hip:1:1: remark: Function Name: _ZN4ftnn9k_conv_f4ILb0EEEvv [-Rpass-analysis=kernel-resource-usage]\n"
          "x.hip:1:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]\n"
          "x.hip:1:1: remark: Function Name: _ZN4ftnn6k_mfmaEvv [-Rpass-analysis=kernel-resource-usage]\n"
          "x.hip:1:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]\n"
          "x.hip:1:1: remark: Function Name: _ZN4ftnn8k_expandEvv [-Rpass-analysis=kernel-resource-usage]\n"
          "x.hip:1:1: remark:     ScratchSize [bytes/lane]: 64 [-Rpass-analysis=kernel-resource-usage]\n")
    build.check_no_scratch("mfma_kernels.hip", ok)   # scratch in a kernel that counts nothing by hand is no error
    for kernel in ("k_conv_f4", "k_mfma"):           # in either guarded kernel it is
        lines = ok.splitlines(True)
        at = next(i for i, l in enumerate(lines) if kernel in l)
        lines[at + 1] = lines[at + 1].replace("lane]: 0", "lane]: 60")
        with pytest.raises(RuntimeError, match="scratch"):
            build.check_no_scratch("mfma_kernels.hip", "".join(lines))
    with pytest.raises(RuntimeError, match="no resource remarks"):
        build.check_no_scratch("mfma_kernels.hip", "")
    with pytest.raises(RuntimeError, match="k_mfma"):   # remarks for one of the two only
        build.check_no_scratch("mfma_kernels.hip", "".join(ok.splitlines(True)[:2]))


def test_benchmark_probe_is_built_outside_the_library():
    """bench.py loads them for the measured vector-ALU issue rate and for the cost of a grid-wide synchronisation; they
    are no part of the shipped package"""
    import ctypes
    import os
    from bench_probe import build as probe_build
    from fastertnn_amd import build
    assert os.path.exists(build.LIB) and os.path.exists(probe_build.LIB) and os.path.exists(probe_build.LIB_GRIDSYNC)
    dll = ctypes.CDLL(probe_build.LIB)
    for name in ("probe_valu_init", "probe_valu_run", "probe_clock_run", "probe_copy_run", "probe_mfma_run", "probe_lds_run"):
        assert hasattr(dll, name)
    assert hasattr(ctypes.CDLL(probe_build.LIB_GRIDSYNC), "probe_gridsync_run")
    assert not os.path.exists(os.path.join(os.path.dirname(build.LIB), "probe_valu"))


def test_size_limits_need_no_device():
    """shapes beyond the documented limits are refused (a scratch size of 0 is how the size query says so)"""
    import fastertnn_amd.lib as lib
    assert lib.conv_scratch_bytes(0, 1, 1, 8192, 8191, 1, 1, 1, 0, 1) > 0         # just below 2^26 pixels per plane
    assert lib.conv_scratch_bytes(0, 1, 1, 8192, 8192, 1, 1, 1, 0, 1) == 0        # 2^26: refused
    assert lib.conv_scratch_bytes(0, 65536, 1, 4, 4, 1, 1, 1, 0, 1) == 0          # batch above 65535
    # a very large layer sizes its scratch for the im2row + GEMM form: planes + rows + fragments
    big = lib.conv_scratch_bytes(0, 8, 1024, 56, 56, 1024, 3, 3, 1, 2)
    small = lib.conv_scratch_bytes(0, 8, 1024, 56, 56, 128, 3, 3, 1, 2)
    assert big > small > 0
    # shape arithmetic that would overflow 32 bits is refused, not wrapped
    assert lib.conv_scratch_bytes(0, 1, 1, 8, 8, 1, 3, 3, 2 ** 30, 1) == 0          # padding of 2^30
    assert lib.conv_scratch_bytes(0, 1, 2 ** 31 - 1, 8, 8, 1, 3, 3, 1, 1) == 0      # channels near 2^31
    assert lib.row_words(2 ** 31 - 1, 3, 3, True) == 0
    assert lib.row_words(64 * (2 ** 24 - 4), 1, 1, False) == 2 ** 24 - 4            # the longest row
    assert lib.row_words(64 * (2 ** 24 - 4) + 1, 1, 1, False) == 0
    assert lib.mm_scratch_bytes(lib.ENGINE_MFMA_I8, 0, 256, 1, 1, 256, 2 ** 24) == 0


def test_layer_chain_refuses_bad_descriptions_before_touching_the_device():
    """ftnn_net_create validates every layer with the rules of a single layer call; nothing is allocated before"""
    import ctypes
    import fastertnn_amd.lib as lib

    def create(batch, *shapes):
        arr = (lib.LayerDesc * len(shapes))()
        for d, (c, h, w, kn, kh, kw, pad, stride) in zip(arr, shapes):
            d.type, d.C, d.H, d.W, d.KN, d.KH, d.KW, d.pad, d.stride = 0, c, h, w, kn, kh, kw, pad, stride
            d.threshold, d.prelu_alpha, d.d_qw = 0.5, 0.5, ctypes.c_void_p(256)   # never read: validation fails first
        return lib._L.ftnn_net_create(batch, len(shapes), arr), lib._L.ftnn_last_error().decode()

    for batch, shapes, text in (
            (1, [(64, 8, 8, 64, 3, 3, 2 ** 30, 1)], "2^26"),                       # padding that overflows 32 bits
            (1, [(2 ** 31 - 1, 8, 8, 64, 3, 3, 1, 1)], "words per"),              # rows longer than 32-bit sums hold
            (1, [(64, 8, 8, 64, 9, 9, 0, 1)], "larger than padded input"),
            (70000, [(64, 8, 8, 64, 3, 3, 1, 1)], "batch"),
            (1, [(64, 8, 8, 64, 3, 3, 1, 1), (32, 8, 8, 64, 3, 3, 1, 1)], "is not the output"),
    ):
        handle, err = create(batch, *shapes)
        assert not handle and text in err, (shapes, err)


def test_layer_chain_refuses_unknown_flags():
    import ctypes
    import fastertnn_amd.lib as lib
    arr = (lib.LayerDesc * 1)()
    d = arr[0]
    d.type, d.C, d.H, d.W, d.KN, d.KH, d.KW, d.pad, d.stride = 0, 64, 8, 8, 64, 3, 3, 1, 1
    d.threshold, d.prelu_alpha, d.d_qw = 0.5, 0.5, ctypes.c_void_p(256)
    assert not lib._L.ftnn_net_create_ex(1, 1, arr, 6)
    assert "flags" in lib._L.ftnn_last_error().decode()
