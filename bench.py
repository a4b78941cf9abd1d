#!/usr/bin/env python3
"""Benchmark of the TNN hot path on one MI355X.

Headline workload: the large compute-bound TNN GEMM (M = N = 8192, K = 32768,
uniform ternary operands in Packing 2, PReLU(0.5) fused).  One "step" is one call
of the GEMM entry point of the C ABI (`ftnn_mm`) with both packed operands and
the output resident in HBM.  Prints ONE JSON line:

  value        ternary GMAC/s = M*N*K / time
  roofline     vector-ALU roofline of the GEMM kernel: algorithmic lane-ops per
               launch (4 VALU ops per pair of 32-lane dwords for TNN) over the
               HIP-event duration of the launches, against 256 CU x 4 SIMD x 16
               lanes x 2.4 GHz
  cpu_baseline the reference's own AVX2 GEMM (compiled from its sources into
               oracle/_ref) on one host core over a bounded row sample of the same
               operands; the GPU rows of that sample are compared bit-for-bit
  extra        conv-layer latencies (kernel-only and host-pointer ABI inclusive)
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

VALU_PEAK_TOPS = 256 * 4 * 16 * 2.4e9 / 1e12  # 39.32 T lane-ops/s (int32 VALU, one op per lane per clock)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # a step is under a millisecond: the defaults are long enough for the clocks to settle under load (with 3 + 10
    # steps the timed region still ran 13 % slower per step than with these) and still take 0.1 s in all
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--m", type=int, default=8192)
    ap.add_argument("--n", type=int, default=8192)
    ap.add_argument("--k", type=int, default=32768)
    ap.add_argument("--cpu-rows", type=int, default=8192, help="rows of A in the CPU-baseline sample (0 = skip)")
    ap.add_argument("--no-extra", action="store_true", help="skip the conv-layer latency section")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 256 MiB device copy, the known-size dispatch that "
                         "FETCH_SIZE / WRITE_SIZE counter runs are scaled by")
    return ap.parse_args()


def ternary_operand(torch, lib, rows, k, seed):
    """uniform {-1,0,+1} fp32 [rows][k] generated on the device, packed by the library"""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    out = torch.empty(rows * k // 32, dtype=torch.int64, device="cuda")
    step = max(1, (1 << 28) // k)  # <= 1 GiB of fp32 at a time
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        x = torch.randint(-1, 2, (r1 - r0, k), generator=g, device="cuda", dtype=torch.int8).float()
        out[r0 * k // 32:r1 * k // 32] = lib.pack_gemm_operand(x)
    return out


def event_times(torch, fn, reps):
    """per-launch duration in ms from HIP events recorded on the launch stream"""
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for a, b in ev:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return [a.elapsed_time(b) for a, b in ev]


def host_cpu():
    """the host the CPU baseline ran on: model name and the cores present (the baseline itself uses one)"""
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return {"model": model, "cores_present": os.cpu_count()}


def cpu_gemm_baseline(a_host, b_host, rows, n, kw, alpha):
    """reference mm_tnn on one core (its protocol pins the process to core 0, Makefile:21);
    falls back to the plain-C port when the compiled reference is absent"""
    from oracle import ftnn_oracle as O
    try:
        os.sched_setaffinity(0, {sorted(os.sched_getaffinity(0))[0]})
    except (AttributeError, OSError):
        pass
    if O.Reference.available():
        ref, kind = O.Reference(), "reference"
        t0 = time.perf_counter()
        y = ref.mm(O.TNN, a_host, b_host, rows, 1, 1, n, kw, alpha)
        dt = time.perf_counter() - t0
    else:
        orc, kind = O.Oracle(), "port"
        t0 = time.perf_counter()
        y = orc.mm(O.TNN, a_host, b_host, rows, 1, 1, n, kw, alpha)
        dt = time.perf_counter() - t0
    return y, dt, kind


def small_gemm(torch, lib, m, n, k, reps=30):
    """the reference's own CPU-runnable GEMM case on every engine (whole call, HIP events), the
    host entry point mm_tnn (host pointers in and out) and the CPU reference on one core"""
    import numpy as np
    from fastertnn_amd import TNN
    from oracle import ftnn_oracle as O
    kw, alpha = k // 64, 0.5
    a = ternary_operand(torch, lib, m, k, seed=1)
    b = ternary_operand(torch, lib, n, k, seed=7)
    y = torch.empty((m, n, 1, 1), dtype=torch.float32, device="cuda")
    scratch = torch.empty(max(lib.mm_scratch_bytes(e, TNN, m, 1, 1, n, kw) for e in lib.ENGINE_NAMES) or 16,
                          dtype=torch.uint8, device="cuda")
    a_h, b_h = O.aligned_copy(a.cpu().numpy()), O.aligned_copy(b.cpu().numpy())
    cpu = O.Reference() if O.Reference.available() else O.Oracle()
    t_cpu = []
    for _ in range(5):
        t0 = time.perf_counter()
        want = cpu.mm(TNN, a_h, b_h, m, 1, 1, n, kw, alpha)
        t_cpu.append(time.perf_counter() - t0)
    out = {"cpu_ms": round(min(t_cpu) * 1e3, 3), "cpu_gmacs": round(float(m) * n * k / min(t_cpu) / 1e9, 1),
           "auto_engine": lib.ENGINE_NAMES[lib.select_engine(TNN, m, 1, 1, n, kw)]}
    for eng, name in lib.ENGINE_NAMES.items():
        def run(eng=eng):
            lib.mm_engine(eng, TNN, a, b, m, 1, 1, n, kw, alpha, out=y, scratch=scratch)
        run()
        t = event_times(torch, run, reps)
        t = sum(t) / len(t)
        out[name] = {"call_ms": round(t, 4), "gmacs": round(float(m) * n * k / t / 1e6, 1),
                     "bit_exact_vs_cpu": bool(y.cpu().numpy().tobytes() == np.ascontiguousarray(want).tobytes())}
    t_abi = []
    for _ in range(10):
        t0 = time.perf_counter()
        got = lib.host_mm(TNN, a_h, b_h, m, 1, 1, n, kw, alpha)
        t_abi.append(time.perf_counter() - t0)
    out["abi_ms"] = round(min(t_abi) * 1e3, 3)
    out["abi_bit_exact_vs_cpu"] = bool(got.tobytes() == np.ascontiguousarray(want).tobytes())
    return out


def other_types(torch, lib, a_tern, b_tern, m, n, k, reps=5):
    """TBN / BTN / BNN on the headline shape: every engine's whole call and the vector-ALU kernel's
    fraction of its roofline (2 lane-ops per dword pair for these types); binary operands are
    uniform random words"""
    from fastertnn_amd import TBN, BTN, BNN, act_is_ternary, weight_is_ternary
    kw = k // 64
    g = torch.Generator(device="cuda")
    g.manual_seed(9)
    a_bin = torch.randint(-2 ** 62, 2 ** 62, (m * kw,), generator=g, device="cuda", dtype=torch.int64)
    b_bin = torch.randint(-2 ** 62, 2 ** 62, (n * kw,), generator=g, device="cuda", dtype=torch.int64)
    y = torch.empty((m, n, 1, 1), dtype=torch.float32, device="cuda")
    out = {}
    for typ, name in ((TBN, "tbn"), (BTN, "btn"), (BNN, "bnn")):
        a = a_tern if act_is_ternary(typ) else a_bin
        b = b_tern if weight_is_ternary(typ) else b_bin
        scratch = torch.empty(max(lib.mm_scratch_bytes(e, typ, m, 1, 1, n, kw) for e in lib.ENGINE_NAMES) or 16,
                              dtype=torch.uint8, device="cuda")
        row, first = {}, None
        for eng, en in lib.ENGINE_NAMES.items():
            def run(eng=eng):
                lib.mm_engine(eng, typ, a, b, m, 1, 1, n, kw, 0.5, k if typ == BNN else 0, out=y, scratch=scratch)
            run()
            torch.cuda.synchronize()
            if first is None:
                first = y.clone()
            same = bool(torch.equal(first, y))
            t = event_times(torch, run, reps)
            t = sum(t) / len(t)
            row[en] = {"call_ms": round(t, 4), "gmacs": round(float(m) * n * k / t / 1e6, 1), "same_bits_as_valu": same}
        row["valu_roofline_frac"] = round(2.0 * m * n * 2 * kw / (row["valu"]["call_ms"] * 1e-3) / 1e12 / VALU_PEAK_TOPS, 4)
        out[name] = row
        del scratch, first
    return out


def pack_rates(torch, lib, reps=10):
    """the quantise + im2row + bit-pack stage alone (t2r_p2_opt / b2r on device memory): algorithmic bytes (fp32
    input once, packed rows once) over the time of its two launches, against the 8 TB/s of HBM"""
    out = {}
    g = torch.Generator(device="cuda")
    g.manual_seed(11)
    for name, tern, (n, c, h, w, k, pad, stride) in (("t2r_b1_c256_56x56_k3", True, (1, 256, 56, 56, 3, 1, 1)),
                                                      ("t2r_b32_c256_56x56_k3", True, (32, 256, 56, 56, 3, 1, 1)),
                                                      ("b2r_b32_c256_56x56_k3", False, (32, 256, 56, 56, 3, 1, 1))):
        x = torch.randn((n, c, h, w), generator=g, device="cuda")
        thr = torch.full((n,), 0.5 if tern else 0.0, device="cuda")
        oh, ow = lib.out_dim(h, pad, k, stride), lib.out_dim(w, pad, k, stride)
        rows = torch.empty(n * oh * ow * lib.row_words(c, k, k, tern), dtype=torch.int64, device="cuda")
        scratch = torch.empty(lib.pack_scratch_bytes(n, c, h, w, tern), dtype=torch.uint8, device="cuda")

        def step():
            lib.quantize_im2row(x, thr, k, k, pad, stride, tern, out=rows, scratch=scratch)
        for _ in range(3):
            step()
        t = sorted(event_times(torch, step, reps))[reps // 2]
        nbytes = 4.0 * x.numel() + 8.0 * rows.numel()
        out[name] = {"ms": round(t, 4), "algorithmic_mb": round(nbytes / 1e6, 1), "gbps": round(nbytes / t / 1e6, 1),
                     "frac_of_8tbps": round(nbytes / t / 1e6 / 8000.0, 3)}
        del x, rows, scratch
    return out


def conv_latency(torch, lib, typ, shape, batch, seed, reps=20):
    """kernel-only (device buffers, HIP events) and ABI-inclusive (host pointers) latency"""
    import numpy as np
    from fastertnn_amd import act_is_ternary, weight_is_ternary
    c, ih, iw, kn, kw, kh, pad, stride = shape
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    x = torch.randn((batch, c, ih, iw), generator=g, device="cuda")
    thr = torch.full((batch,), 0.5 if at else 0.0, device="cuda")
    if wt:
        w = torch.randint(-1, 2, (kn, c, kh, kw), generator=g, device="cuda", dtype=torch.int8).float()
    else:
        w = torch.randint(0, 2, (kn, c, kh, kw), generator=g, device="cuda", dtype=torch.int8).float() * 2 - 1
    wthr = torch.full((kn,), 0.5 if wt else 0.0, device="cuda")
    qw = lib.pack_weights(w, wthr, wt)
    oh, ow = lib.out_dim(ih, pad, kh, stride), lib.out_dim(iw, pad, kw, stride)
    scratch = torch.empty(lib.conv_scratch_bytes(typ, batch, c, ih, iw, kn, kh, kw, pad, stride), dtype=torch.uint8,
                          device="cuda")
    y = torch.empty((batch, kn, oh, ow), device="cuda")

    # weights are prepared once per layer (matrix-core fragments), as a layer of a network holds them;
    # the packed-rows call ftnn_conv repeats that step on every call and is timed beside it
    prepared = lib.prepare_conv_weights(typ, qw, c, kn, kh, kw)

    def step():
        lib.conv_prepared(typ, x, thr, prepared, kn, kh, kw, pad, stride, 0.5, scratch=scratch, out=y)

    def step_rows():
        lib.conv(typ, x, thr, qw, kn, kh, kw, pad, stride, 0.5, scratch=scratch, out=y)

    for _ in range(3):
        step()
        step_rows()
    kernel_ms = sorted(event_times(torch, step, reps))[reps // 2]
    rows_ms = sorted(event_times(torch, step_rows, reps))[reps // 2]
    xh, thrh, qwh = x.cpu().numpy(), thr.cpu().numpy(), qw.cpu().numpy()
    lib.host_conv(typ, xh, thrh, qwh, kn, kh, kw, pad, stride, 0.5)
    t = []
    for _ in range(5):
        t0 = time.perf_counter()
        yh = lib.host_conv(typ, xh, thrh, qwh, kn, kh, kw, pad, stride, 0.5)
        t.append((time.perf_counter() - t0) * 1e3)
    out = {"kernel_ms": round(kernel_ms, 4), "kernel_ms_from_packed_rows": round(rows_ms, 4),
           "engine": lib.ENGINE_NAMES[lib.select_conv_engine(typ, batch, c, ih, iw, kn, kh, kw, pad, stride)],
           "abi_ms": round(sorted(t)[2], 3),
           "gmacs_kernel": round(batch * oh * ow * kn * c * kh * kw / kernel_ms / 1e6, 1)}
    # the reference's layer on one host core, same inputs
    from oracle import ftnn_oracle as O
    if O.Reference.available():
        ref = O.Reference()
        ref.conv(typ, xh, thrh, qwh, kn, kh, kw, pad, stride, 0.5)
        t0 = time.perf_counter()
        yr = ref.conv(typ, xh, thrh, qwh, kn, kh, kw, pad, stride, 0.5)
        out["cpu_ms"] = round((time.perf_counter() - t0) * 1e3, 2)
        out["bit_exact_vs_reference"] = bool(np.ascontiguousarray(yh).tobytes() == yr.tobytes())
    # the reference's "baseline" (Packing 0) build beside its "final" one, as its Makefile pairs them
    if O.ReferenceBaseline.available():
        base = O.ReferenceBaseline()
        qw0 = base.pack_weights(w.cpu().numpy(), wthr.cpu().numpy(), wt)
        try:
            t0 = time.perf_counter()
            yb = base.conv(typ, xh, thrh, qw0, kn, kh, kw, pad, stride, 0.5)
            out["cpu_reference_baseline_build_ms"] = round((time.perf_counter() - t0) * 1e3, 1)
            out["bit_exact_vs_reference_baseline_build"] = bool(np.ascontiguousarray(yh).tobytes() == yb.tobytes())
        finally:
            base.free_weights(qw0)
    return out




def e2e_latency(torch, lib, batch, reps=50, cpu=True, typ=None):
    """the ResNet-18-like TNN stack chained on the device (eager launches and HIP-graph replay), and
    (cpu=True) the same chain through the reference's tnns_conv on one host core"""
    import numpy as np
    from fastertnn_amd import TNN, act_is_ternary, weight_is_ternary
    from fastertnn_amd.shapes import RESNET18_LIKE
    typ = TNN if typ is None else typ
    at, wt = act_is_ternary(typ), weight_is_ternary(typ)
    g = torch.Generator(device="cuda")
    g.manual_seed(6)
    x = torch.randn((batch, 3, 224, 224), generator=g, device="cuda")
    layers = []
    for (c, ih, iw, kn, kw, kh, pad, stride) in RESNET18_LIKE:
        if wt:
            w = torch.randint(-1, 2, (kn, c, kh, kw), generator=g, device="cuda", dtype=torch.int8).float()
        else:
            w = torch.randint(0, 2, (kn, c, kh, kw), generator=g, device="cuda", dtype=torch.int8).float() * 2 - 1
        qw = lib.pack_weights(w, torch.full((kn,), 0.5 if wt else 0.0, device="cuda"), wt)
        layers.append(dict(type=typ, shape=(c, ih, iw, kn, kw, kh, pad, stride), threshold=0.5 if at else 0.0,
                           alpha=0.5, qw=qw))
    net = lib.Net(batch, layers)
    y = torch.empty(net.out_shape, device="cuda")
    macs = sum(batch * lib.out_dim(ih, p, kh, s) * lib.out_dim(iw, p, kw, s) * kn * c * kh * kw
               for (c, ih, iw, kn, kw, kh, p, s) in RESNET18_LIKE)
    out = {"layers": len(layers), "batch": batch, "gmac": round(macs / 1e9, 2)}
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        for graph, key in ((False, "eager_ms"), (True, "graph_ms")):
            for _ in range(3):
                net.run(x, out=y, graph=graph)
            t = sorted(event_times(torch, lambda: net.run(x, out=y, graph=graph), reps))[reps // 2]
            out[key] = round(t, 4)
    st.synchronize()
    from oracle import ftnn_oracle as O
    if cpu and O.Reference.available():
        ref = O.Reference()
        xh = x.cpu().numpy()
        thr = np.full(batch, 0.5 if at else 0.0, np.float32)
        t0 = time.perf_counter()
        for l in layers:
            c, ih, iw, kn, kw, kh, pad, stride = l["shape"]
            xh = ref.conv(typ, xh, thr, O.aligned_copy(l["qw"].cpu().numpy()), kn, kh, kw, pad, stride, 0.5)
        out["cpu_ms"] = round((time.perf_counter() - t0) * 1e3, 1)
        out["bit_exact_vs_reference"] = bool(y.cpu().numpy().tobytes() == np.ascontiguousarray(xh).tobytes())
    net.close()
    return out


def valu_probe():
    """the measured issue rate of v_bcnt_u32_b32 over the whole chip (fastertnn_amd/csrc/probe_valu.hip, a child
    process): what the nominal 39.3 T lane-op/s of the vector-ALU roofline comes to at the clock the chip holds"""
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fastertnn_amd", "probe_valu")
    if not os.path.exists(exe):
        return {"skipped": "fastertnn_amd/probe_valu is not built"}
    p = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    for line in p.stdout.splitlines():
        if line.startswith("{"):
            return json.loads(line)
    return {"failed": p.stdout[-200:]}


def reference_gemm_sweep(torch, lib, reps=10):
    """the sweep of the reference's GEMM driver, m = n in {32 .. 4096}, p = 8 m (src/timing_gemm.c:90-97), alpha = 1 as
    tnns_gemm (src/tnns/tnns_cpu_mm_p2.c:123): device-resident operands, the engine the library picks, against the
    reference on one host core"""
    import numpy as np
    from fastertnn_amd import TNN
    from oracle import ftnn_oracle as O
    out = {}
    for m in (32, 64, 128, 256, 512, 1024, 2048, 4096):
        p = 8 * m
        kw = p // 64
        a = ternary_operand(torch, lib, m, p, seed=20 + m)
        b = ternary_operand(torch, lib, m, p, seed=21 + m)
        y = torch.empty((m, m, 1, 1), dtype=torch.float32, device="cuda")
        need = lib.mm_scratch_bytes(lib.ENGINE_AUTO, TNN, m, 1, 1, m, kw)
        scratch = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")

        def run():
            lib.mm_engine(lib.ENGINE_AUTO, TNN, a, b, m, 1, 1, m, kw, 1.0, out=y, scratch=scratch)
        for _ in range(3):
            run()
        t = sorted(event_times(torch, run, reps))[reps // 2]
        row = {"engine": lib.ENGINE_NAMES[lib.select_engine(TNN, m, 1, 1, m, kw)], "device_ms": round(t, 4),
               "gmacs": round(float(m) * m * p / t / 1e6, 1)}
        if O.Reference.available():
            ref = O.Reference()
            ah, bh = O.aligned_copy(a.cpu().numpy()), O.aligned_copy(b.cpu().numpy())
            t0 = time.perf_counter()
            want = ref.mm(TNN, ah, bh, m, 1, 1, m, kw, 1.0)
            row["cpu_ms"] = round((time.perf_counter() - t0) * 1e3, 3)
            row["bit_exact_vs_reference"] = bool(y.cpu().numpy().tobytes() == np.ascontiguousarray(want).tobytes())
        out["m%d" % m] = row
        del a, b, y, scratch
    return out


def reference_single_layers(torch, lib, batch=8, reps=10):
    """the 17 layers of the reference's `layer` mode (include/timing/shapes_layers.h, kept as data in
    fastertnn_amd/data/reference_shape_tables.txt), TNN, batch 8 (src/timing_layers.c:46): device-resident call with
    prepared weights against the reference's tnns_conv on one host core"""
    import numpy as np
    from fastertnn_amd import TNN
    from oracle import ftnn_oracle as O
    from fastertnn_amd import shapes
    tables = shapes.reference_tables()
    out = {}
    g = torch.Generator(device="cuda")
    g.manual_seed(9)
    for shape in tables["layers"]:
        c, ih, iw, kn, kw, kh, p, s = shape
        x = torch.randn((batch, c, ih, iw), generator=g, device="cuda")
        thr = torch.full((batch,), 0.5, device="cuda")
        w = torch.randint(-1, 2, (kn, c, kh, kw), generator=g, device="cuda", dtype=torch.int8).float()
        qw = lib.pack_weights(w, torch.full((kn,), 0.5, device="cuda"), True)
        del w
        prepared = lib.prepare_conv_weights(TNN, qw, c, kn, kh, kw)
        oh, ow = lib.out_dim(ih, p, kh, s), lib.out_dim(iw, p, kw, s)
        scratch = torch.empty(lib.conv_scratch_bytes(TNN, batch, c, ih, iw, kn, kh, kw, p, s), dtype=torch.uint8,
                              device="cuda")
        y = torch.empty((batch, kn, oh, ow), device="cuda")

        def step():
            lib.conv_prepared(TNN, x, thr, prepared, kn, kh, kw, p, s, 0.5, scratch=scratch, out=y)
        for _ in range(3):
            step()
        t = sorted(event_times(torch, step, reps))[reps // 2]
        row = {"engine": lib.ENGINE_NAMES[lib.select_conv_engine(TNN, batch, c, ih, iw, kn, kh, kw, p, s)],
               "device_ms": round(t, 4), "gmac": round(batch * oh * ow * kn * c * kh * kw / 1e9, 2)}
        if O.Reference.available():
            ref = O.Reference()
            xh, qwh = x.cpu().numpy(), O.aligned_copy(qw.cpu().numpy())
            t0 = time.perf_counter()
            want = ref.conv(TNN, xh, np.full(batch, 0.5, np.float32), qwh, kn, kh, kw, p, s, 0.5)
            row["cpu_ms"] = round((time.perf_counter() - t0) * 1e3, 2)
            row["bit_exact_vs_reference"] = bool(y.cpu().numpy().tobytes() == np.ascontiguousarray(want).tobytes())
        out["c%d_%dx%d_k%d_s%d" % (c, ih, iw, kh, s)] = row
        del x, qw, prepared, scratch, y
    return out


def reference_networks(torch, lib, batch=8, reps=5):
    """the seven networks of the reference's e2e mode (include/timing/shapes_e2e.h, kept as data in
    fastertnn_amd/data/reference_shape_tables.txt), at the reference's batch of 8 (src/timing_layers.c:46): device-resident
    layer chain against the same tnns_conv chain on one host core.  Three tables leave out their pooling layers; there
    the reference's driver hands the previous output buffer on under the next row's shape
    (src/timing_layers.c:187-200), and so do the chain (FTNN_NET_REREAD_PREFIX) and the CPU side here."""
    import numpy as np
    from fastertnn_amd import TNN
    from oracle import ftnn_oracle as O
    from fastertnn_amd import shapes
    tables = shapes.reference_tables()
    out = {}
    g = torch.Generator(device="cuda")
    g.manual_seed(8)
    for net_t in tables["e2e"]:
        shapes = [tuple(r) for r in net_t["layers"]]
        c, h, w = shapes[0][:3]
        ok = True
        for (cc, ih, iw, kn, kw, kh, p, s) in shapes:
            ok = ok and (cc, ih, iw) == (c, h, w)
            c, h, w = kn, lib.out_dim(ih, p, kh, s), lib.out_dim(iw, p, kw, s)
        layers = []
        for (c, ih, iw, kn, kw, kh, p, s) in shapes:
            wgt = torch.randint(-1, 2, (kn, c, kh, kw), generator=g, device="cuda", dtype=torch.int8).float()
            qw = lib.pack_weights(wgt, torch.full((kn,), 0.5, device="cuda"), True)
            layers.append(dict(type=TNN, shape=(c, ih, iw, kn, kw, kh, p, s), threshold=0.5, alpha=0.5, qw=qw))
        x = torch.randn((batch,) + shapes[0][:3], generator=g, device="cuda")
        net = lib.Net(batch, layers, flags=0 if ok else lib.NET_REREAD_PREFIX)
        y = torch.empty(net.out_shape, device="cuda")
        for _ in range(2):
            net.run(x, out=y)
        t = sorted(event_times(torch, lambda: net.run(x, out=y), reps))[reps // 2]
        macs = sum(batch * lib.out_dim(ih, p, kh, s) * lib.out_dim(iw, p, kw, s) * kn * c * kh * kw
                   for (c, ih, iw, kn, kw, kh, p, s) in shapes)
        row = {"layers": len(shapes), "gmac": round(macs / 1e9, 1), "device_ms": round(t, 4), "chains_shape_to_shape": ok}
        if O.Reference.available():
            ref = O.Reference()
            xh = x.cpu().numpy()
            thr = np.full(batch, 0.5, np.float32)
            t0 = time.perf_counter()
            for l in layers:
                c, ih, iw, kn, kw, kh, p, s = l["shape"]
                if xh.shape[1:] != (c, ih, iw):
                    xh = np.ascontiguousarray(xh).reshape(-1)[:batch * c * ih * iw].reshape(batch, c, ih, iw)
                xh = ref.conv(TNN, xh, thr, O.aligned_copy(l["qw"].cpu().numpy()), kn, kh, kw, p, s, 0.5)
            row["cpu_ms"] = round((time.perf_counter() - t0) * 1e3, 1)
            row["bit_exact_vs_reference"] = bool(y.cpu().numpy().tobytes() == np.ascontiguousarray(xh).tobytes())
        net.close()
        out[net_t["name"]] = row
        del layers, x, y
    return out


def main():
    args = parse()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus %d is not supported "
                 "(the path would shard over output rows with no exchange)" % args.gpus)
    import numpy as np
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    import fastertnn_amd.lib as lib
    from fastertnn_amd import TNN, TBN, BTN

    m, n, k = args.m, args.n, args.k
    assert k % 256 == 0
    kw = k // 64
    alpha = 0.5
    a = ternary_operand(torch, lib, m, k, seed=5)
    b = ternary_operand(torch, lib, n, k, seed=6)
    y = torch.empty((m, n, 1, 1), dtype=torch.float32, device="cuda")
    auto = lib.select_engine(TNN, m, 1, 1, n, kw)
    scratch = torch.empty(max(lib.mm_scratch_bytes(e, TNN, m, 1, 1, n, kw) for e in lib.ENGINE_NAMES) or 16,
                          dtype=torch.uint8, device="cuda")

    def step():   # the timed hot path: packed operands in, fp32 result out, engine chosen by the library
        lib.mm_engine(lib.ENGINE_AUTO, TNN, a, b, m, 1, 1, n, kw, alpha, out=y, scratch=scratch)

    if args.copy_calibration:
        src = torch.empty(1 << 26, dtype=torch.float32, device="cuda").fill_(1.0)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    macs = float(m) * n * k
    reps = min(max(args.steps, 5), 50)   # launches per event-timed mean below

    def mean(v):
        return sum(v) / len(v)

    # every engine on the same operands, per-launch HIP events; the whole call (expansion included)
    engines = {}
    y_ref = None
    for eng, name in lib.ENGINE_NAMES.items():
        def run(eng=eng):
            lib.mm_engine(eng, TNN, a, b, m, 1, 1, n, kw, alpha, out=y, scratch=scratch)
        run()
        torch.cuda.synchronize()
        if y_ref is None:
            y_ref = y.clone()
        same = bool(torch.equal(y, y_ref))
        t = mean(event_times(torch, run, reps))
        engines[name] = {"call_ms": round(t, 4), "gmacs": round(macs / t / 1e6, 1), "same_bits_as_valu": same}
    del y_ref

    # rooflines of the dominant kernels, each timed alone with HIP events on the launch stream
    valu_ms = engines["valu"]["call_ms"]   # the VALU engine is one kernel
    valu_ops = 4.0 * m * n * (2 * kw)      # 4 vector ops per pair of 32-lane dwords, 2*kw dwords per plane
    valu_ach = valu_ops / (valu_ms * 1e-3) / 1e12
    roofline_valu = {"bound": "valu", "achieved": round(valu_ach, 3), "peak": round(VALU_PEAK_TOPS, 3),
                     "unit": "Tlaneop/s", "frac": round(valu_ach / VALU_PEAK_TOPS, 4), "traffic": None,
                     "kernel": "k_mm<TNN,2,8,1>", "avg_launch_ms": valu_ms,
                     "popcount_frac": round(valu_ach / 2 / VALU_PEAK_TOPS, 4),
                     "note": "peak = 256 CU x 4 SIMD x 16 lanes x 2.4 GHz int32 VALU lane-ops; "
                             "algorithmic ops = 4 per dword pair (v_or, v_bitop3, 2 x v_bcnt)"}
    mfma = {}
    for eng, kernel, peak in ((lib.ENGINE_MFMA_I8, "k_mfma<int8>", 5000.0), (lib.ENGINE_MFMA_F4, "k_mfma<fp4>", 10100.0)):
        a_exp = lib.expand_rows(eng, a, m, kw, True)
        b_exp = lib.expand_rows(eng, b, n, kw, True)

        def gemm(eng=eng, a_exp=a_exp, b_exp=b_exp):
            lib.mm_expanded(eng, TNN, a_exp, b_exp, m, 1, 1, n, kw, alpha, out=y)

        def expand(eng=eng, a_exp=a_exp):
            lib.expand_rows(eng, a, m, kw, True, out=a_exp)
        gemm()
        t = mean(event_times(torch, gemm, reps))
        te = mean(event_times(torch, expand, reps))
        ach = 2.0 * macs / (t * 1e-3) / 1e12
        mfma[eng] = {"bound": "mfma", "achieved": round(ach, 1), "peak": peak, "unit": "TOP/s" if eng == lib.ENGINE_MFMA_I8 else "TFLOP/s",
                     "frac": round(ach / peak, 4), "traffic": None, "kernel": kernel, "avg_launch_ms": round(t, 4),
                     "expand_one_operand_ms": round(te, 4)}
        del a_exp, b_exp
    if (m, n, k) == (8192, 8192, 32768):
        # HBM bytes per launch from rocprofv3 FETCH_SIZE / WRITE_SIZE (KiB per dispatch, scaled by a plain 256 MiB
        # copy: x2.0 / x1.0), measured with this script under the profiler: profiles/tnn_gemm_8192x8192x32768_all_engines.md
        roofline_valu["traffic"] = int((2049521.1 * 2.0 + 262183.5) * 1024)
        mfma[lib.ENGINE_MFMA_I8]["traffic"] = int((1574007.8 * 2.0 + 262144.0) * 1024)
        mfma[lib.ENGINE_MFMA_F4]["traffic"] = int((790714.8 * 2.0 + 262144.0) * 1024)
    roofline = {lib.ENGINE_VALU: roofline_valu, lib.ENGINE_MFMA_I8: mfma[lib.ENGINE_MFMA_I8],
                lib.ENGINE_MFMA_F4: mfma[lib.ENGINE_MFMA_F4]}[auto]

    cpu = None
    if args.cpu_rows > 0:
        rows = min(args.cpu_rows, m)
        a_host = a[:rows * 2 * kw].cpu().numpy()
        b_host = b.cpu().numpy()
        from oracle.ftnn_oracle import aligned_copy
        y_cpu, dt, kind = cpu_gemm_baseline(aligned_copy(a_host), aligned_copy(b_host), rows, n, kw, alpha)
        y_gpu = y.view(m, n)[:rows].cpu().numpy()
        cpu = {"value": round(float(rows) * n * k / dt / 1e9, 2), "unit": "GMAC/s", "cores": 1, "kind": kind,
               "sample": "first %d of %d rows of A against all %d columns, K=%d (%.1f s on one core)"
                         % (rows, m, n, k, dt),
               "gpu_rows_bit_exact": bool(y_gpu.tobytes() == np.ascontiguousarray(y_cpu).tobytes()),
               "host": host_cpu()}

    extra = None
    if not args.no_extra:
        extra = {
            "other_types_same_gemm_shape": other_types(torch, lib, a, b, m, n, k),
            "tnn_gemm_256x256x4096": small_gemm(torch, lib, 256, 256, 4096),
            "quantize_im2row_pack": pack_rates(torch, lib),
            "tnn_conv_b1_c256_56x56_k3": conv_latency(torch, lib, TNN, (256, 56, 56, 256, 3, 3, 1, 1), 1, 2),
            "tbn_conv_b8_c128_28x28_k3": conv_latency(torch, lib, TBN, (128, 28, 28, 128, 3, 3, 1, 1), 8, 3),
            "btn_conv_b8_c128_28x28_k3": conv_latency(torch, lib, BTN, (128, 28, 28, 128, 3, 3, 1, 1), 8, 4),
            "tnn_resnet18_like_b32_e2e": e2e_latency(torch, lib, 32),
            "valu_popcount_probe": valu_probe(),
            "reference_gemm_sweep": reference_gemm_sweep(torch, lib),
            "reference_single_layers_b8": reference_single_layers(torch, lib),
            "reference_e2e_networks_b8": reference_networks(torch, lib),
            "tnn_resnet18_like_other_batches": {"b%d" % b: e2e_latency(torch, lib, b, cpu=False) for b in (1, 8, 128)},
            "other_types_resnet18_like_b32": {n: e2e_latency(torch, lib, 32, cpu=False, typ=t)
                                              for n, t in (("tbn", 1), ("btn", 2), ("bnn", 3))},
        }

    line = {
        "metric": "TNN GEMM ternary GMAC/s", "value": round(macs / (ms_per_step * 1e-3) / 1e9, 1),
        "unit": "GMAC/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": {1: "u32", 2: "int8", 3: "fp4 (E2M1, exact for -1/0/+1) with fp32 accumulate"}[auto], "data": "synthetic",
        "config": {"workload": "TNN GEMM M=%d N=%d K=%d, uniform ternary, Packing 2, PReLU 0.5 fused" % (m, n, k),
                   "m": m, "n": n, "k": k},
        "roofline": roofline, "cpu_baseline": cpu,
        "engine": lib.ENGINE_NAMES[auto], "engines": engines,
        "roofline_valu_kernel": roofline_valu, "roofline_mfma_i8_kernel": mfma[lib.ENGINE_MFMA_I8],
        "roofline_mfma_f4_kernel": mfma[lib.ENGINE_MFMA_F4], "extra": extra,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
