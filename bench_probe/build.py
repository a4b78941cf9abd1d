"""Builds libprobe_valu.so beside this file: the vector-ALU issue-rate and shader-clock probe that bench.py loads
(a measurement aid of the benchmark, not part of the shipped library)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libprobe_valu.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def build_probe():
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", os.path.join(HERE, "probe_valu.hip"), "-o", LIB]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("hipcc failed on probe_valu.hip:\n%s" % p.stdout)
    return LIB


if __name__ == "__main__":
    print(build_probe())
