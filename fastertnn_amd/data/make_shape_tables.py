"""Writes reference_shape_tables.txt beside this script: the layer tables of the reference's timing drivers as
plain data -- include/timing/shapes_e2e.h (seven networks, the e2e mode of src/timing_layers.c:182-207),
include/timing/shapes_layers.h (the 17 single layers of its layer mode) and include/timing/shapes_test.h (the 12
shapes of its self-test mode).  One row per line, eight integers `C IH IW KN KW KH pad stride` in the reference's
own order (shapes_e2e.h:2); a line `[mode name]` opens a table.  The Python side (fastertnn_amd/shapes.py) and
the C++ timing driver (harness/) read the same file.

Run where the reference tree is mounted:  python fastertnn_amd/data/make_shape_tables.py [/root/reference]
"""
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
    tests = tables(os.path.join(inc, "shapes_test.h"), "test_shape_")
    selftest = [tests[str(i)][0] for i in range(len(tests))]
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "reference_shape_tables.txt"), "w") as f:
        f.write("# C IH IW KN KW KH pad stride; from include/timing/shapes_{e2e,layers,test}.h of the reference\n")
        for n in order:
            f.write("[e2e %s]\n" % n)
            for r in e2e[n]:
                f.write(" ".join(str(v) for v in r) + "\n")
        for i, r in enumerate(single):
            f.write("[layer %d]\n%s\n" % (i, " ".join(str(v) for v in r)))
        for i, r in enumerate(selftest):
            f.write("[test %d]\n%s\n" % (i, " ".join(str(v) for v in r)))
    print({n: len(e2e[n]) for n in order}, len(single), len(selftest))


if __name__ == "__main__":
    main()
