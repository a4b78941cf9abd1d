"""AddressSanitizer + UndefinedBehaviorSanitizer legs (host code only; CPU): `make -C oracle sanitize` builds the checker
(ftnn_oracle.c, ftnn_oracle_avx2.c) and the host side of the shipped library (ftnn_api.hip, ftnn_net.hip) with both
sanitizers and runs their drivers: every routine of the checker on exact-size buffers, and the library's size
arithmetic and argument checks on shapes up to INT_MAX."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("make") is None or not os.path.exists("/opt/rocm/bin/hipcc"), reason="needs make and hipcc")
def test_checker_and_library_host_code_under_asan_and_ubsan():
    objs = [os.path.join(ROOT, "fastertnn_amd", "csrc", n + ".o") for n in ("pack_kernels", "mm_kernels", "mfma_kernels", "stem_kernels")]
    assert all(os.path.exists(o) for o in objs), "build the library first (python -m fastertnn_amd.build)"
    r = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "sanitize"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "sanitize ok" in r.stdout and "sanitize abi ok" in r.stdout
