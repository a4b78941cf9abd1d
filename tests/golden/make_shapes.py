"""Writes tests/golden/reference_shape_tables.json: the layer tables of the reference's timing drivers as data --
include/timing/shapes_e2e.h (seven networks, the e2e mode of src/timing_layers.c:182-207) and
include/timing/shapes_layers.h (the 17 single layers of its layer mode).  Each row is
(C, IH, IW, KN, KW, KH, pad, stride), the reference's own order (shapes_e2e.h:2).

Run here, where the reference tree is mounted:  python tests/golden/make_shapes.py [/root/reference]
"""
import json
import os
import re
import sys

ROW = re.compile(r"\{\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*\}")


def tables(path, prefix):
    """name -> rows for every 'static int <prefix><name>[...][PARAMCOUNT] = {...};' in the header"""
    text = open(path).read()
    text = re.sub(r"//[^\n]*", "", text)
    out = {}
    for m in re.finditer(r"static\s+int\s+" + prefix + r"(\w+)\s*\[[^\]]*\]\s*\[PARAMCOUNT\]\s*=\s*\{(.*?)\};", text, re.S):
        rows = [[int(v) for v in r] for r in ROW.findall(m.group(2))]
        if rows:
            out[m.group(1)] = rows
    return out


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    inc = os.path.join(ref, "include", "timing")
    e2e = tables(os.path.join(inc, "shapes_e2e.h"), "shapes_")
    # the order of the reference's table of tables (shapes_e2e.h:408-410)
    order = ["resnet18", "resnet34", "vgg16", "vgg19", "darknet19", "darknet53", "resnet152"]
    assert sorted(e2e) == sorted(order), sorted(e2e)
    layers = tables(os.path.join(inc, "shapes_layers.h"), "shape_")
    single = [layers[str(i)][0] for i in range(len(layers))]
    doc = {"row": ["C", "IH", "IW", "KN", "KW", "KH", "pad", "stride"],
           "source": {"e2e": "include/timing/shapes_e2e.h", "layers": "include/timing/shapes_layers.h:5-21"},
           "e2e": [{"name": n, "layers": e2e[n]} for n in order], "layers": single}
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "reference_shape_tables.json"), "w") as f:
        json.dump(doc, f, indent=0, separators=(",", ":"))
        f.write("\n")
    print({n: len(e2e[n]) for n in order}, len(single))


if __name__ == "__main__":
    main()
