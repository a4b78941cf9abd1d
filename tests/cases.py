"""Shapes and input recipes shared by the tests.

A shape is (C, IH, IW, KN, KW, KH, pad, stride) in the order of the reference's
shape tables (include/timing/shapes_test.h:2, src/timing_layers.c:29-40: the
fifth entry is the kernel WIDTH, the sixth its height).
"""
import numpy as np

from fastertnn_amd import synth, TNN, TBN, BTN, BNN, act_is_ternary, weight_is_ternary

# the reference's 12 self-test shapes (include/timing/shapes_test.h:6-17)
REF_TEST_SHAPES = [
    (32, 7, 7, 32, 3, 3, 0, 1),
    (32, 7, 7, 32, 3, 3, 1, 2),
    (127, 7, 7, 32, 3, 3, 1, 1),
    (127, 7, 7, 32, 3, 3, 1, 1),
    (128, 7, 7, 32, 3, 3, 1, 2),
    (193, 7, 7, 32, 3, 3, 1, 2),
    (256, 14, 14, 256, 3, 5, 1, 2),
    (256, 14, 14, 256, 3, 3, 1, 2),
    (257, 14, 14, 257, 3, 3, 1, 2),
    (320, 15, 23, 320, 3, 3, 1, 2),
    (512, 1, 1, 512, 1, 1, 0, 1),
    (1024, 14, 14, 1024, 5, 5, 1, 2),
]

# extra edge shapes: 7x7 stem with C=3 (include/timing/shapes_e2e.h:10, shrunk input),
# 1x1 stride-2 projection (shapes_e2e.h:17), one-pixel output, KN not a multiple of any tile,
# FC with C not a multiple of 256, kernel covering the whole padded input
EXTRA_SHAPES = [
    (3, 32, 32, 16, 7, 7, 3, 2),
    (64, 12, 12, 128, 1, 1, 0, 2),
    (65, 3, 3, 5, 3, 3, 0, 1),
    (70, 9, 5, 33, 2, 4, 2, 3),
    (200, 1, 1, 10, 1, 1, 0, 1),
    (64, 4, 4, 7, 6, 6, 1, 1),
    # few channels: several kernel taps share a 64-lane word in the device's dense re-packing
    (8, 9, 9, 12, 3, 3, 1, 1),
    (16, 11, 7, 40, 5, 5, 2, 2),
    (1, 6, 6, 3, 3, 3, 1, 1),
    (21, 8, 8, 9, 3, 3, 0, 1),
    (20, 16, 16, 33, 7, 7, 3, 2),
]

ALL_TYPES = (TNN, TBN, BTN, BNN)


def make_layer(typ, shape, batch, seed, alpha=0.5):
    """Seeded inputs for one layer: N(0,1) activations, uniform ternary/binary weights,
    thresholds as the reference's driver sets them (src/timing_layers.c:100-107) but with a
    different activation threshold per batch item so that the per-item indexing is exercised."""
    c, ih, iw, kn, kw, kh, pad, stride = shape
    x = synth.normal(seed, (batch, c, ih, iw))
    if act_is_ternary(typ):
        thr = (0.5 + 0.125 * (np.arange(batch) % 3)).astype(np.float32)
    else:
        thr = (0.25 * ((np.arange(batch) % 3) - 1)).astype(np.float32)
    if weight_is_ternary(typ):
        w = synth.ternary(seed + 1, (kn, c, kh, kw))
        wthr = np.full(kn, 0.5, np.float32)
    else:
        w = synth.binary(seed + 1, (kn, c, kh, kw))
        wthr = np.zeros(kn, np.float32)
    return dict(type=typ, shape=shape, batch=batch, x=x, thr=thr, w=w, wthr=wthr, alpha=alpha,
                c=c, ih=ih, iw=iw, kn=kn, kw=kw, kh=kh, pad=pad, stride=stride)


def decode_ternary_rows(rows, n_rows, kw_words):
    """Packing-2 rows -> int8 matrix [n_rows][64*kw_words] of {-1,0,+1}."""
    r = np.asarray(rows, dtype=np.int64).view(np.uint64).reshape(n_rows, kw_words // 4, 2, 4)
    sign = r[:, :, 0, :].reshape(n_rows, kw_words)
    zero = r[:, :, 1, :].reshape(n_rows, kw_words)
    sb = np.unpackbits(sign.view(np.uint8), axis=1, bitorder="little").astype(np.int8)
    zb = np.unpackbits(zero.view(np.uint8), axis=1, bitorder="little").astype(np.int8)
    assert not np.any(sb & zb), "a lane is both negative and zero"
    return (1 - 2 * sb) * (1 - zb)


def decode_binary_rows(rows, n_rows, kw_words):
    """single-plane rows -> int8 matrix of {-1,+1} (bit set = -1)."""
    r = np.asarray(rows, dtype=np.int64).view(np.uint64).reshape(n_rows, kw_words)
    sb = np.unpackbits(r.view(np.uint8), axis=1, bitorder="little").astype(np.int8)
    return 1 - 2 * sb
