"""Writes profiles/traffic_tnn_gemm_<M>x<N>x<K>.json: HBM-side bytes per launch of the GEMM kernels, from two
rocprofv3 counter runs of bench.py (one counter per run) and the plain device copy of known size that bench.py runs
with --copy-calibration.  bench.py reads that file for `roofline.traffic`; it holds no literal of its own.

    cd /tmp && export TMPDIR=/tmp
    rocprofv3 --pmc FETCH_SIZE -d <out>/pmc_fetch -o r -- python3 <repo>/bench.py --cpu-rows 0 --no-extra --steps 3 --warmup 1 --copy-calibration
    rocprofv3 --pmc WRITE_SIZE -d <out>/pmc_write -o r -- python3 <repo>/bench.py --cpu-rows 0 --no-extra --steps 3 --warmup 1 --copy-calibration
    python3 bench_probe/traffic_from_pmc.py <out>/pmc_fetch <out>/pmc_write 8192 8192 32768

Both counters report KiB per dispatch.  The calibration copy moves 256 MiB each way; the factor between that and what
a counter reads for it scales every other dispatch of the same run.
"""
import collections
import datetime
import glob
import json
import os
import sqlite3
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
COPY_BYTES = 256 << 20

# kernel-name fragment and grid (workgroups) -> key in the JSON; grids are those of the 8192 x 8192 x 32768 launch
KERNELS = {"k_mfma_p4": "k_mfma_p4<", "k_mfma_i8": "k_mfma<false", "k_mm": "k_mm<0"}


def per_dispatch(dirname, counter):
    """[(kernel name, workgroups, value)] in dispatch order from the rocprofv3 database under dirname"""
    dbs = sorted(glob.glob(os.path.join(dirname, "**", "*.db"), recursive=True))
    if not dbs:
        raise SystemExit("no rocprofv3 database under %s" % dirname)
    c = sqlite3.connect(dbs[-1])
    acc = collections.OrderedDict()
    for did, name, gx, gy, gz, wx, wy, wz, cn, v in c.execute(
            "select dispatch_id, kernel_name, grid_size_x, grid_size_y, grid_size_z, workgroup_size_x, workgroup_size_y, "
            "workgroup_size_z, counter_name, value from counters_collection order by dispatch_id"):
        if cn != counter:
            continue
        wgs = (gx // max(wx, 1)) * (gy // max(wy, 1)) * (gz // max(wz, 1))
        key = (did, name, wgs)
        acc[key] = acc.get(key, 0.0) + v      # one row per XCD / instance: a dispatch is their sum
    return [(k[1], k[2], v) for k, v in acc.items()]


def summarise(rows, m, n):
    copy = [v for name, wgs, v in rows if "k_probe_copy" in name]
    big = sum(copy) / len(copy) if copy else None
    out = {}
    for key, frag in KERNELS.items():
        # the launch on the full operands: the grid with the most workgroups for this kernel
        mine = [(wgs, v) for name, wgs, v in rows if frag in name]
        if not mine:
            continue
        top = max(w for w, _ in mine)
        vals = [v for w, v in mine if w == top]
        out[key] = {"kib_reported_mean": sum(vals) / len(vals), "dispatches": len(vals), "workgroups": top}
    return big, out


def main():
    fetch_dir, write_dir = sys.argv[1], sys.argv[2]
    m, n, k = (int(v) for v in sys.argv[3:6])
    f_copy, f = summarise(per_dispatch(fetch_dir, "FETCH_SIZE"), m, n)
    w_copy, w = summarise(per_dispatch(write_dir, "WRITE_SIZE"), m, n)
    if not f_copy or not w_copy:
        raise SystemExit("no calibration copy in the runs: pass --copy-calibration to bench.py")
    fs, ws = COPY_BYTES / 1024.0 / f_copy, COPY_BYTES / 1024.0 / w_copy
    kernels = {}
    for key in f:
        if key not in w:
            continue
        fb, wb = f[key]["kib_reported_mean"] * fs * 1024, w[key]["kib_reported_mean"] * ws * 1024
        kernels[key] = {"fetch_kib_reported": round(f[key]["kib_reported_mean"], 1),
                        "write_kib_reported": round(w[key]["kib_reported_mean"], 1),
                        "dispatches": [f[key]["dispatches"], w[key]["dispatches"]],
                        "fetch_bytes": int(fb), "write_bytes": int(wb), "bytes_per_launch": int(fb + wb)}
    try:
        commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip()
    except OSError:
        commit = None
    doc = {"workload": "TNN GEMM M=%d N=%d K=%d" % (m, n, k), "date": datetime.date.today().isoformat(),
           "commit": commit or os.environ.get("FTNN_COMMIT"),
           "command": "rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE -- python3 bench.py --cpu-rows 0 --no-extra --steps 3 --warmup 1 --copy-calibration",
           "calibration_copy_kib_reported": {"FETCH_SIZE": round(f_copy, 1), "WRITE_SIZE": round(w_copy, 1)},
           "fetch_scale": round(fs, 3), "write_scale": round(ws, 3), "kernels": kernels}
    path = os.path.join(ROOT, "profiles", "traffic_tnn_gemm_%dx%dx%d.json" % (m, n, k))
    with open(path, "w") as fjson:
        json.dump(doc, fjson, indent=1)
        fjson.write("\n")
    print(json.dumps(doc))


if __name__ == "__main__":
    main()
