"""Builds the benchmark's measurement aids beside this file (not part of the shipped library): libprobe_valu.so, the
vector-ALU issue-rate, matrix-core chain and shader-clock probe, and libprobe_gridsync.so, the cost of a grid-wide
synchronisation inside a cooperative launch against that of a launch boundary."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libprobe_valu.so")
LIB_GRIDSYNC = os.path.join(HERE, "libprobe_gridsync.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _build(src, lib):
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", os.path.join(HERE, src), "-o", lib]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, p.stdout))
    return lib


def build_probe():
    _build("probe_gridsync.hip", LIB_GRIDSYNC)
    return _build("probe_valu.hip", LIB)


if __name__ == "__main__":
    print(build_probe())
