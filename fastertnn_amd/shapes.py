"""Layer tables as data: the reference's own (data/reference_shape_tables.txt, written by
data/make_shape_tables.py from include/timing/shapes_{e2e,layers,test}.h) and the ResNet-18-like stack of the
end-to-end configuration.  A row is (C, IH, IW, KN, KW, KH, pad, stride): the fifth entry is the kernel WIDTH, the
sixth its height (src/timing_layers.c:29-40)."""
import os

TABLES_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "data", "reference_shape_tables.txt")

# stem, four stages of 3x3 layers with stride-2 transitions, fully connected layer as 1x1: the 19 layers of the
# batch-32 end-to-end configuration (3 x 224 x 224 input)
RESNET18_LIKE = [
    (3, 224, 224, 64, 7, 7, 3, 2), (64, 112, 112, 64, 3, 3, 1, 2),
    (64, 56, 56, 64, 3, 3, 1, 1), (64, 56, 56, 64, 3, 3, 1, 1), (64, 56, 56, 64, 3, 3, 1, 1), (64, 56, 56, 64, 3, 3, 1, 1),
    (64, 56, 56, 128, 3, 3, 1, 2), (128, 28, 28, 128, 3, 3, 1, 1), (128, 28, 28, 128, 3, 3, 1, 1), (128, 28, 28, 128, 3, 3, 1, 1),
    (128, 28, 28, 256, 3, 3, 1, 2), (256, 14, 14, 256, 3, 3, 1, 1), (256, 14, 14, 256, 3, 3, 1, 1), (256, 14, 14, 256, 3, 3, 1, 1),
    (256, 14, 14, 512, 3, 3, 1, 2), (512, 7, 7, 512, 3, 3, 1, 1), (512, 7, 7, 512, 3, 3, 1, 1), (512, 7, 7, 512, 3, 3, 1, 1),
    (512, 7, 7, 1000, 1, 1, 0, 1),
]


def reference_tables(path=TABLES_PATH):
    """{"e2e": [{"name", "layers"}...] in the reference's order, "layers": [row...], "test": [row...]}"""
    out = {"e2e": [], "layers": [], "test": []}
    rows = None
    for line in open(path):
        line = line.strip()
        if not line or line.startswith("#"):
            continue
        if line.startswith("["):
            mode, name = line.strip("[]").split()
            if mode == "e2e":
                rows = []
                out["e2e"].append({"name": name, "layers": rows})
            else:
                rows = out["layers" if mode == "layer" else "test"]
            continue
        row = tuple(int(v) for v in line.split())
        assert len(row) == 8, line
        rows.append(row)
    return out


def layer_macs(batch, row):
    c, ih, iw, kn, kw, kh, pad, stride = row
    oh, ow = (ih + 2 * pad - kh) // stride + 1, (iw + 2 * pad - kw) // stride + 1
    return batch * oh * ow * kn * c * kh * kw
