"""Builds the two timing drivers beside this file (ftnn_timing_layers, ftnn_timing_gemm) with hipcc for gfx950 and
links them against fastertnn_amd/libftnn_hip.so (found at run time through an $ORIGIN-relative rpath)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIBDIR = os.path.join(os.path.dirname(HERE), "fastertnn_amd")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
TARGETS = {"ftnn_timing_layers": "timing_layers.hip", "ftnn_timing_gemm": "timing_gemm.hip"}


def build_harness():
    out = []
    for exe, src in TARGETS.items():
        cmd = [HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-Wall", "-Xclang", "-target-feature", "-Xclang",
               "-packed-fp32-ops", os.path.join(HERE, src), "-L" + LIBDIR, "-lftnn_hip", "-Wl,-rpath,$ORIGIN/../fastertnn_amd",
               "-o", os.path.join(HERE, exe)]
        p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, p.stdout))
        out.append(os.path.join(HERE, exe))
    return out


if __name__ == "__main__":
    print(build_harness())
