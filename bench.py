#!/usr/bin/env python3
"""Benchmark of the TNN hot path on one MI355X.

Headline workload: the large compute-bound TNN GEMM (M = N = 8192, K = 32768,
uniform ternary operands in Packing 2, PReLU(0.5) fused).  One "step" is one pass of
the GEMM from two PACKED operands resident in HBM, as the reference's mm_tnn takes
them: both are brought into the engine's operand form (ftnn_expand_rows) and
multiplied (ftnn_mm_expanded) -- what one ftnn_mm_engine call does, as three calls so that
the GEMM launch can be timed by itself (the one call is timed beside it).  Where the
library's engine choice for the shape is the vector ALU the step is that one call.
The step of a layer that keeps its weights in engine form is reported beside it
(step_with_weights_kept_in_engine_form).  Prints ONE JSON line:

  value        ternary GMAC/s = M*N*K / time of a step
  roofline     the dominant kernel of the step (the fp4 matrix-core GEMM): its launches
               inside the timed region are bracketed by HIP events on the launch
               stream; algorithmic FLOP per launch over their mean duration against
               the published dense fp4 peak.  `traffic` comes from the tracked counter
               summary under profiles/ (never a literal here).  Nested in it,
               `valu_popcount`: the vector-ALU popcount kernel on the same operands
               against 256 CU x 4 SIMD x 16 lanes x 2.4 GHz (the figure the metric
               names), with the measured v_bcnt issue rate and the shader clocks of
               probe and kernel, taken back to back in this process
  cpu_baseline the reference's own AVX2 GEMM (compiled from its sources into
               oracle/_ref) on one host core over a bounded row sample of the same
               operands, or the AVX2 restatement under oracle/ where that build is
               absent; the GPU rows of the sample are compared bit-for-bit
  extra        conv-layer and layer-chain latencies (kernel-only and host-pointer ABI
               inclusive), the other types on the headline shape, the reference's GEMM
               sweep, its 17 single layers and two of its networks, each with a roofline
               object and a bit-for-bit comparison with the reference's CPU path; --full
               adds the other networks, batch sizes and types
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


MFMA_F4_PEAK_TFLOPS = 10100.0   # dense fp4 matrix rate of MI355X


def roofline_mfma_f4(macs, ms):
    """roofline object of a kernel (or chain of kernels) on the fp4 matrix cores: 2 FLOP per lane-MAC"""
    ach = 2.0 * macs / (ms * 1e-3) / 1e12
    return {"bound": "mfma", "achieved": round(ach, 1), "peak": MFMA_F4_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(ach / MFMA_F4_PEAK_TFLOPS, 4)}


def roofline_valu(m, n, kw, ms, ops_per_pair=4):
    """roofline object of the vector-ALU popcount GEMM: ops_per_pair lane-ops per pair of 32-lane dwords (4 for TNN, 2
    for the types with a binary operand) against 256 CU x 4 SIMD x 16 lanes x 2.4 GHz"""
    ach = float(ops_per_pair) * m * n * (2 * kw) / (ms * 1e-3) / 1e12
    return {"bound": "valu", "achieved": round(ach, 3), "peak": round(VALU_PEAK_TOPS, 3), "unit": "Tlaneop/s",
            "frac": round(ach / VALU_PEAK_TOPS, 4)}


def roofline_for(engine_name, m, n, kw, ms, ops_per_pair=4):
    return roofline_mfma_f4(float(m) * n * kw * 64, ms) if engine_name == "mfma_f4" else roofline_valu(m, n, kw, ms, ops_per_pair)


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
    ap.add_argument("--full", action="store_true",
                    help="also run the long sections (the reference's GEMM sweep, its 17 single layers and seven "
                         "networks, other batch sizes and types); they go into the same JSON line under extra")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 256 MiB device copy, the known-size dispatch that "
                         "FETCH_SIZE / WRITE_SIZE counter runs are scaled by")
    ap.add_argument("--chain-codes", action="store_true",
                    help="run the registers-only MFMA chain on every code table of the probe (lane content against "
                         "clock), not only the two the GEMM's history needs")
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
    """mm_tnn on ONE host core (the reference's protocol pins its drivers to core 0, Makefile:21): the reference's
    own AVX2 path where its compiled form is present (kind "reference"), else the AVX2 restatement under oracle/
    (kind "port"), else nothing -- the scalar oracle is a checker, not a baseline.  The affinity of the process is
    restored afterwards.  Returns (y, seconds, kind) or (None, reason, None)."""
    from oracle import ftnn_oracle as O
    if O.Reference.available():
        impl, kind = O.Reference(), "reference"
    elif O.OracleAvx2.available():
        impl, kind = O.OracleAvx2(), "port"
    else:
        return None, "neither oracle/_ref/libref_final.so nor an AVX2 host: no CPU path of reference grade to time", None
    saved = None
    try:
        saved = os.sched_getaffinity(0)
        os.sched_setaffinity(0, {sorted(saved)[0]})
    except (AttributeError, OSError):
        saved = None
    try:
        t0 = time.perf_counter()
        y = impl.mm(O.TNN, a_host, b_host, rows, 1, 1, n, kw, alpha)
        dt = time.perf_counter() - t0
    finally:
        if saved is not None:
            os.sched_setaffinity(0, saved)
    return y, dt, kind


def graph_times(torch, fn, y, reps, n_graph=10):
    """device time of `fn` with no host in the loop: n_graph calls recorded into one graph, HIP events around its
    replay, per call; every replay must leave in y what the eager call left there (returns ms, same_bits)"""
    fn()
    torch.cuda.synchronize()
    y_eager = y.clone()
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(n_graph):
                fn()
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        same = bool(torch.equal(y, y_eager))
        ms = sorted(event_times(torch, graph.replay, reps))[reps // 2] / n_graph
        same = same and bool(torch.equal(y, y_eager))
        del graph
        return ms, same
    except RuntimeError as e:      # no graph on this runtime: eager calls back to back instead, and say so
        sys.stderr.write("bench.py: graph capture failed (%s); timing %d eager calls back to back\n" % (e, n_graph))
        torch.cuda.synchronize()

        def many():
            for _ in range(n_graph):
                fn()
        return sorted(event_times(torch, many, reps))[reps // 2] / n_graph, None


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
        exact = bool(y.cpu().numpy().tobytes() == np.ascontiguousarray(want).tobytes())
        tg, same = graph_times(torch, run, y, reps)
        out[name] = {"call_ms": round(t, 4), "gmacs": round(float(m) * n * k / t / 1e6, 1), "bit_exact_vs_cpu": exact,
                     "device_ms_in_a_graph_of_10_calls": round(tg, 4), "graph_replays_same_bits_as_eager": same}
        if name != "mfma_i8":   # whole call (expansions included for fp4) over the device time of a call in the graph
            out[name]["roofline"] = roofline_for(name, m, n, kw, tg)
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
            for _ in range(4):   # the clocks settle over the first calls after the idle time of the allocations
                run()
            t = event_times(torch, run, reps)
            t = sum(t) / len(t)
            row[en] = {"call_ms": round(t, 4), "gmacs": round(float(m) * n * k / t / 1e6, 1), "same_bits_as_valu": same}
        row["valu_roofline_frac"] = round(2.0 * m * n * 2 * kw / (row["valu"]["call_ms"] * 1e-3) / 1e12 / VALU_PEAK_TOPS, 4)
        row["valu"]["roofline"] = roofline_valu(m, n, kw, row["valu"]["call_ms"], 2)
        row["mfma_f4"]["roofline"] = roofline_mfma_f4(float(m) * n * k, row["mfma_f4"]["call_ms"])
        row["all_engines_same_bits"] = all(r["same_bits_as_valu"] for r in (row["valu"], row["mfma_i8"], row["mfma_f4"]))
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
    call_ms = sorted(event_times(torch, step, reps))[reps // 2]
    rows_ms = sorted(event_times(torch, step_rows, reps))[reps // 2]
    # device time of the layer with no host in the loop (a single call issued from Python leaves the device idle
    # between its two launches)
    n_graph = 10
    kernel_ms, graph_same = graph_times(torch, step, y, reps, n_graph)
    xh, thrh, qwh = x.cpu().numpy(), thr.cpu().numpy(), qw.cpu().numpy()
    yh = lib.host_conv(typ, xh, thrh, qwh, kn, kh, kw, pad, stride, 0.5)
    # ABI-inclusive: the C call tnns_conv alone, host pointers in, malloc'd host pointer out (freed as a C caller would)
    import ctypes
    tc = lib.Testcase(type=typ, batchcount=batch, channelcount=c, inputW=iw, inputH=ih, kernelcount=kn, kernelW=kw,
                      kernelH=kh, paddingW=pad, paddingH=pad, strideW=stride, strideH=stride, preluAlpha=0.5,
                      input_thresholds=thrh.ctypes.data, input=xh.ctypes.data, quantized_kernel_packing2=qwh.ctypes.data)
    t = []
    for _ in range(15):
        t0 = time.perf_counter()
        lib._L.tnns_conv(ctypes.byref(tc))
        t.append((time.perf_counter() - t0) * 1e3)
        lib._libc.free(tc.output)
    out = {"kernel_ms": round(kernel_ms, 4),
           "kernel_ms_is": "HIP events around a graph replay of %d calls (weights prepared), per call" % n_graph,
           "graph_replays_same_bits_as_eager": graph_same,
           "single_call_ms_from_python": round(call_ms, 4), "single_call_ms_from_packed_rows": round(rows_ms, 4),
           "engine": lib.ENGINE_NAMES[lib.select_conv_engine(typ, batch, c, ih, iw, kn, kh, kw, pad, stride)],
           "abi_ms": round(sorted(t)[7], 3),
           "gmacs_kernel": round(batch * oh * ow * kn * c * kh * kw / kernel_ms / 1e6, 1)}
    out["roofline"] = roofline_for(out["engine"], batch * oh * ow, kn, ((c + 63) // 64) * kh * kw, kernel_ms,
                                   4 if typ == 0 else 2)
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

            # ten passes queued behind each other: the device's time per pass without the host's part in a single call
            def ten(graph=graph):
                for _ in range(10):
                    net.run(x, out=y, graph=graph)
            t10 = sorted(event_times(torch, ten, max(5, reps // 2)))[max(5, reps // 2) // 2] / 10
            out[key.replace("_ms", "_ms_per_pass_of_ten_queued")] = round(t10, 4)
    st.synchronize()
    # the chain's layers run on the fp4 matrix cores: logical MACs of the whole pass over its device time
    out["roofline"] = roofline_mfma_f4(macs, out["eager_ms_per_pass_of_ten_queued"])
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


class Probe:
    """bench_probe/libprobe_valu.so: the v_bcnt issue-rate chain and the shader-clock sampler, run in this process on
    torch's current stream"""

    def __init__(self):
        import ctypes as C
        path = os.path.join(ROOT, "bench_probe", "libprobe_valu.so")
        self.lib = C.CDLL(path) if os.path.exists(path) else None
        self.C = C
        if self.lib is not None and self.lib.probe_valu_init() != 0:
            self.lib = None

    def _call(self, fn, trips, torch, n):
        out = (self.C.c_double * n)()
        if fn(int(trips), self.C.c_void_p(torch.cuda.current_stream().cuda_stream), out) != 0:
            return None
        return list(out)

    def copy(self, torch, src, dst):
        out = (self.C.c_double * 1)()
        rc = self.lib.probe_copy_run(self.C.c_void_p(src.data_ptr()), self.C.c_void_p(dst.data_ptr()),
                                     self.C.c_size_t(src.numel() * src.element_size()),
                                     self.C.c_void_p(torch.cuda.current_stream().cuda_stream), out)
        return None if rc != 0 else out[0]

    def issue_rate(self, torch, trips=2500):
        r = self._call(self.lib.probe_valu_run, trips, torch, 5)
        if r is None:
            return None
        return {"ms": round(r[0], 4), "lane_ops_per_s": float("%.4e" % r[1]), "frac_of_nominal": round(r[1] / (VALU_PEAK_TOPS * 1e12), 4),
                "shader_mhz": round(r[2], 1), "lane_ops_per_lane_cycle": round(r[3], 4), "result_ok": bool(r[4])}

    MFMA_CHAIN_FORMS = ("lanes_as_minus1_0_plus1", "lanes_as_0_half_1", "all_zero", "lanes_as_0_0_1", "lanes_as_0_1_2",
                        "lanes_as_minus1.5_0_plus1.5", "lanes_as_minus6_0_plus6")

    def mfma_rate(self, torch, form, trips=10000):
        """the fp4 matrix-core chain with operands from registers (k_mfma_chain) on uniformly random ternary lanes
        coded by table `form` (index into MFMA_CHAIN_FORMS; 0 = -1 / 0 / +1, 1 = the GEMM's offset codes 0 / 0.5 / 1):
        what the chip sustains with no operand traffic, and the clock it holds meanwhile"""
        out = (self.C.c_double * 4)()
        if self.lib.probe_mfma_run(int(trips), int(form), self.C.c_void_p(torch.cuda.current_stream().cuda_stream), out) != 0:
            return None
        r = list(out)
        return {"ms": round(r[0], 4), "tflops": round(r[1] / 1e12, 1), "frac_of_10100": round(r[1] / 10100e12, 4),
                "shader_mhz": round(r[2], 1), "matrix_pipe_busy": round(r[3], 4)}

    def lds_read_rate(self, torch, trips=20000):
        """bytes per shader cycle and compute unit that wavefronts reading LDS with 16-byte reads reach (k_lds_read: four
        wavefronts per workgroup, fragment layout), with one workgroup per compute unit -- how the 256 x 256 matrix-core
        tiles run -- and with two"""
        if self.lib is None or not hasattr(self.lib, "probe_lds_run"):
            return None
        res = {}
        for wgs, key in ((1, "one_workgroup_per_cu"), (2, "two_workgroups_per_cu")):
            out = (self.C.c_double * 2)()
            if self.lib.probe_lds_run(wgs, int(trips), self.C.c_void_p(torch.cuda.current_stream().cuda_stream), out) != 0:
                return None
            res[key] = {"ms": round(out[0], 4), "bytes_per_cycle_and_cu": round(out[1], 1)}
        return res

    def clock_after(self, torch, trips=16):
        """shader clock seen by a short, nearly idle kernel queued directly behind whatever ran last on the stream"""
        r = self._call(self.lib.probe_clock_run, trips, torch, 2)
        return None if r is None else {"ms": round(r[0], 4), "shader_mhz": round(r[1], 1)}


_GRID_SYNC_CHILD = r"""
import ctypes as C, json, sys
import torch
lib = C.CDLL(sys.argv[1])
lib.probe_gridsync_run.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.POINTER(C.c_double)]
out = {}
buf = (C.c_double * 4)()
st = torch.cuda.current_stream().cuda_stream
for mode, key in ((2, "launch_boundary"), (0, "cooperative_groups_grid_sync"), (1, "counter_barrier_bounded_wait")):
    best = None
    for _ in range(5):
        if lib.probe_gridsync_run(mode, 1, 18, st, buf) != 0:
            out = {"failed": key}
            break
        if buf[3] != 1.0:
            out = {"failed": key + ": data passed through the synchronisations is wrong"}
            break
        best = buf[1] if best is None else min(best, buf[1])
    if "failed" in out:
        break
    out[key + "_us"] = round(best, 2)
    out["workgroups"] = int(buf[2])
print("GRIDSYNC " + json.dumps(out), flush=True)
"""


def grid_sync_cost(torch):
    """bench_probe/libprobe_gridsync.so: microseconds per grid-wide synchronisation inside one cooperative launch (the
    library's cooperative_groups grid sync, and a counter barrier with a bounded wait) against microseconds per launch
    boundary of plain launches, 18 synchronisations each (a 19-layer chain), one workgroup of 256 threads per compute
    unit.  What decides whether a chain of small layers should be one resident kernel.  Runs in a child process: a
    process that has made a cooperative launch ends in a segmentation fault inside rocprofv3's exit handler when it is
    traced, which must not be this one's end (the child has printed its figures by then)."""
    import subprocess
    path = os.path.join(ROOT, "bench_probe", "libprobe_gridsync.so")
    if not os.path.exists(path):
        return {"skipped": "bench_probe/libprobe_gridsync.so is not built"}
    try:
        p = subprocess.run([sys.executable, "-c", _GRID_SYNC_CHILD, path], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                           text=True, timeout=120)
    except subprocess.TimeoutExpired:
        return {"failed": "timeout"}
    for line in p.stdout.splitlines():
        if line.startswith("GRIDSYNC "):
            return json.loads(line[len("GRIDSYNC "):])
    return {"failed": "child exit %d: %s" % (p.returncode, p.stderr[-300:])}


def valu_reconciliation(torch, probe, run_valu, valu_ops, reps=12):
    """The v_bcnt chain and the vector-ALU GEMM kernel back to back on one stream, with the shader clock each one
    left behind (sampled by a 30 us kernel queued directly after it): the kernel's fraction of the NOMINAL roofline
    (2.4 GHz) can exceed the probe's only when it ran at a higher clock, and its lane-ops per lane and cycle -- the
    schedule-only figure -- is what compares like with like."""
    if probe.lib is None:
        return {"skipped": "bench_probe/libprobe_valu.so is not built"}
    lanes = 256 * 4 * 16
    out = {}
    for _ in range(3):          # the same thermal / clock state for both: alternate them
        probe.issue_rate(torch, 500)
        run_valu()
    p = probe.issue_rate(torch)
    p["clock_after_mhz"] = (probe.clock_after(torch) or {}).get("shader_mhz")
    out["probe"] = p
    t = event_times(torch, run_valu, reps)
    k_ms = sum(t) / len(t)
    clk = probe.clock_after(torch)
    out["kernel"] = {"avg_launch_ms": round(k_ms, 4), "frac_of_nominal": round(valu_ops / (k_ms * 1e-3) / 1e12 / VALU_PEAK_TOPS, 4),
                     "clock_after_mhz": clk["shader_mhz"] if clk else None}
    if clk and clk["shader_mhz"] > 0:
        out["kernel"]["lane_ops_per_lane_cycle_at_that_clock"] = round(valu_ops / (k_ms * 1e-3) / (lanes * clk["shader_mhz"] * 1e6), 4)
    p2 = probe.issue_rate(torch)
    out["probe_again"] = {"frac_of_nominal": p2["frac_of_nominal"], "shader_mhz": p2["shader_mhz"],
                          "lane_ops_per_lane_cycle": p2["lane_ops_per_lane_cycle"]}
    return out


def traffic_record(kernel_key, shape):
    """HBM-side bytes per launch of `kernel_key` from the tracked counter summary profiles/traffic_*.json (written
    by bench_probe/traffic_from_pmc.py from two rocprofv3 --pmc runs of this script); None when there is no record for
    this shape"""
    path = os.path.join(ROOT, "profiles", "traffic_tnn_gemm_%dx%dx%d.json" % shape)
    try:
        doc = json.load(open(path))
        k = doc["kernels"][kernel_key]
        return int(k["bytes_per_launch"]), {"file": os.path.relpath(path, ROOT), "commit": doc.get("commit"),
                                            "date": doc.get("date"), "fetch_scale": doc.get("fetch_scale"),
                                            "write_scale": doc.get("write_scale")}
    except (OSError, KeyError, ValueError):
        return None, None


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
        tg, same = graph_times(torch, run, y, reps)
        row["device_ms_in_a_graph_of_10_calls"], row["graph_replays_same_bits_as_eager"] = round(tg, 4), same
        row["roofline"] = roofline_for(row["engine"], m, m, kw, min(t, tg))
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
        tg, same = graph_times(torch, step, y, reps)
        row["device_ms_in_a_graph_of_10_calls"], row["graph_replays_same_bits_as_eager"] = round(tg, 4), same
        row["roofline"] = roofline_for(row["engine"], batch * oh * ow, kn, ((c + 63) // 64) * kh * kw, min(t, tg))
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


def reference_networks(torch, lib, batch=8, reps=5, only=None):
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
        if only is not None and net_t["name"] not in only:
            continue
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
        row = {"layers": len(shapes), "gmac": round(macs / 1e9, 1), "device_ms": round(t, 4), "chains_shape_to_shape": ok,
               "roofline": roofline_mfma_f4(macs, t)}
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


def host_gemm_cfg4(torch, lib, a, b, m, n, kw, alpha=0.5):
    """mm_tnn with host pointers on the headline shape (128 MiB in, 256 MiB out through PCIe): with the copy threads
    the caller's CPU affinity allows, and pinned to one core as the reference's Makefile runs its drivers (then the
    runtime's plain copies).  The library reads the affinity once, so each case runs in a child process."""
    import subprocess
    code = ("import sys, time, os, numpy as np\n"
            "sys.path.insert(0, %r)\n"
            "if sys.argv[1] == 'one': os.sched_setaffinity(0, {sorted(os.sched_getaffinity(0))[0]})\n"
            "import fastertnn_amd.lib as lib\n"
            "m, n, kw = %d, %d, %d\n"
            "rng = np.random.default_rng(1)\n"
            "def op(rows):\n"
            "    r = rng.integers(0, 2 ** 63, size=(rows, kw // 4, 2, 4), dtype=np.int64)\n"
            "    r[:, :, 0, :] &= ~r[:, :, 1, :]\n"
            "    return r.reshape(-1)\n"
            "a, b = op(m), op(n)\n"
            "lib.host_mm(0, a, b, m, 1, 1, n, kw, 0.5)\n"
            "t = []\n"
            "for _ in range(3):\n"
            "    t0 = time.perf_counter(); y = lib._L.mm_tnn(a.ctypes.data, b.ctypes.data, m, 1, 1, n, kw, 0.5); t.append(time.perf_counter() - t0); lib._libc.free(y)\n"
            "print(min(t) * 1e3)\n" % (ROOT, m, n, kw))
    out = {}
    for mode in ("all", "one"):
        try:
            p = subprocess.run([sys.executable, "-c", code, mode], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
            ms = float(p.stdout.strip().splitlines()[-1])
            out["caller_on_%s_core%s" % (mode, "s" if mode == "all" else "")] = {
                "abi_ms": round(ms, 2), "gmacs_pcie_inclusive": round(float(m) * n * kw * 64 / ms / 1e6, 1)}
        except Exception as e:   # noqa: BLE001 -- a failed side measurement must not lose the benchmark line
            out["caller_on_%s_core%s" % (mode, "s" if mode == "all" else "")] = {"failed": str(e)[:200]}
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
    macs = float(m) * n * k

    # The timed hot path: what the reference's mm_tnn does per call -- both operands arrive as packed rows.  On a
    # matrix-core engine a step therefore brings BOTH operands into engine form (ftnn_expand_rows on A and on B) and
    # multiplies (ftnn_mm_expanded); these are the launches of the one C call ftnn_mm_engine, issued as three calls so
    # that the GEMM kernel of every timed step sits between two HIP events on the launch stream.  The cheaper step of a
    # layer that keeps its weights in engine form (B expanded once) is timed beside it, outside the timed region.
    gemm_events = []
    if auto == lib.ENGINE_VALU:
        def step(timed=False):
            if timed:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                gemm_events.append((e0, e1))
                e0.record()
            lib.mm_engine(lib.ENGINE_VALU, TNN, a, b, m, 1, 1, n, kw, alpha, out=y)
            if timed:
                e1.record()
        step_desc = "ftnn_mm_engine (vector ALU) on the packed operands"
        step_kept = None
    else:
        b_exp = torch.empty(int(lib._L.ftnn_expand_bytes(auto, n, kw)), dtype=torch.uint8, device="cuda")
        a_exp = torch.empty(int(lib._L.ftnn_expand_bytes(auto, m, kw)), dtype=torch.uint8, device="cuda")

        def step(timed=False):
            lib.expand_rows(auto, a, m, kw, True, out=a_exp)
            lib.expand_rows(auto, b, n, kw, True, out=b_exp)
            if timed:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                gemm_events.append((e0, e1))
                e0.record()
            lib.mm_expanded(auto, TNN, a_exp, b_exp, m, 1, 1, n, kw, alpha, out=y)
            if timed:
                e1.record()

        def step_kept():
            lib.expand_rows(auto, a, m, kw, True, out=a_exp)
            lib.mm_expanded(auto, TNN, a_exp, b_exp, m, 1, 1, n, kw, alpha, out=y)
        step_desc = ("ftnn_expand_rows(A) + ftnn_expand_rows(B) + ftnn_mm_expanded: both operands from packed rows in "
                     "every step, as mm_tnn takes them (what one ftnn_mm_engine call does, as three calls so that the GEMM "
                     "launch is timed by itself)")

    if args.copy_calibration:
        src = torch.empty(1 << 26, dtype=torch.float32, device="cuda").fill_(1.0)
        dst = torch.empty_like(src)
        Probe().copy(torch, src, dst)    # k_probe_copy, 256 MiB each way
        torch.cuda.synchronize()
        del src, dst

    def mean(v):
        return sum(v) / len(v)

    REPS = 30   # launches per event-timed mean in the untimed sections, whatever --steps says

    # every engine on the same packed operands, per-launch HIP events: the whole call ftnn_mm_engine, both
    # expansions included for the matrix-core engines
    # (run before the timed region: auxiliary measurements, and the chip reaches the clocks it holds under load)
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
        t = mean(event_times(torch, run, REPS if name != "valu" else 12))
        engines[name] = {"call_ms": round(t, 4), "gmacs": round(macs / t / 1e6, 1), "same_bits_as_valu": same}


    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(timed=True)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    gemm_ms = [e0.elapsed_time(e1) for e0, e1 in gemm_events]
    gemm_avg = sum(gemm_ms) / len(gemm_ms)
    step_same = bool(torch.equal(y, y_ref))
    del y_ref
    kept = None
    if step_kept is not None:
        # a layer's step: the weights stay in engine form, only the activation rows are expanded per step
        for _ in range(args.warmup):
            step_kept()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step_kept()
        torch.cuda.synchronize()
        ms_kept = (time.perf_counter() - t0) / args.steps * 1e3
        kept = {"ms_per_step": round(ms_kept, 4), "gmacs": round(macs / (ms_kept * 1e-3) / 1e9, 1),
                "step": "ftnn_expand_rows(A) + ftnn_mm_expanded with B expanded once (weights kept in engine form)"}

    # the vector-ALU kernel against the roofline the metric names, with the issue-rate probe beside it
    valu_ops = 4.0 * m * n * (2 * kw)      # 4 vector ops per pair of 32-lane dwords, 2*kw dwords per plane
    probe = Probe()

    def run_valu():
        lib.mm_engine(lib.ENGINE_VALU, TNN, a, b, m, 1, 1, n, kw, alpha, out=y)
    recon = valu_reconciliation(torch, probe, run_valu, valu_ops)
    valu_ms = recon["kernel"]["avg_launch_ms"] if "kernel" in recon else engines["valu"]["call_ms"]
    valu_ach = valu_ops / (valu_ms * 1e-3) / 1e12
    traffic, traffic_src = traffic_record("k_mm", (m, n, k))
    roofline_valu = {"bound": "valu", "achieved": round(valu_ach, 3), "peak": round(VALU_PEAK_TOPS, 3),
                     "unit": "Tlaneop/s", "frac": round(valu_ach / VALU_PEAK_TOPS, 4), "traffic": traffic,
                     "kernel": "k_mm<TNN,2,8,1>", "avg_launch_ms": round(valu_ms, 4),
                     "popcount_frac": round(valu_ach / 2 / VALU_PEAK_TOPS, 4),
                     "gmacs": round(macs / valu_ms / 1e6, 1),
                     "probe_and_clocks": recon,
                     "note": "peak = 256 CU x 4 SIMD x 16 lanes x 2.4 GHz int32 VALU lane-ops; "
                             "algorithmic ops = 4 per dword pair (v_or, v_bitop3, 2 x v_bcnt)"}
    mfma = {}
    for eng, key, kernel, peak in ((lib.ENGINE_MFMA_I8, "k_mfma_i8", "k_mfma<int8>", 5000.0),
                                   (lib.ENGINE_MFMA_F4, "k_mfma_p4", "k_mfma_p4<fp4, operands at 2 bits per lane>", 10100.0)):
        ae = lib.expand_rows(eng, a, m, kw, True)
        be = lib.expand_rows(eng, b, n, kw, True)

        def gemm(eng=eng, ae=ae, be=be):
            lib.mm_expanded(eng, TNN, ae, be, m, 1, 1, n, kw, alpha, out=y)

        def expand(eng=eng, ae=ae):
            lib.expand_rows(eng, a, m, kw, True, out=ae)
        gemm()
        t = mean(event_times(torch, gemm, REPS))
        te = mean(event_times(torch, expand, REPS))
        if eng == auto:
            t = gemm_avg          # the headline kernel: its launches inside the timed region
        ach = 2.0 * macs / (t * 1e-3) / 1e12
        traffic, src = traffic_record(key, (m, n, k))
        mfma[eng] = {"bound": "mfma", "achieved": round(ach, 1), "peak": peak, "unit": "TOP/s" if eng == lib.ENGINE_MFMA_I8 else "TFLOP/s",
                     "frac": round(ach / peak, 4), "traffic": traffic, "kernel": kernel, "avg_launch_ms": round(t, 4),
                     "expand_one_operand_ms": round(te, 4)}
        if eng == lib.ENGINE_MFMA_F4:
            # the same launch on operand buffers of all-zero codes: the same instruction stream without the switching
            # activity of real data, i.e. what the schedule alone allows when power does not bound it
            az, bz = torch.zeros_like(ae), torch.zeros_like(be)

            def gemm_zero(eng=eng, az=az, bz=bz):
                lib.mm_expanded(eng, TNN, az, bz, m, 1, 1, n, kw, alpha, out=y)
            gemm_zero()
            tz = mean(event_times(torch, gemm_zero, REPS))
            mfma[eng]["same_kernel_on_all_zero_operands"] = {"avg_launch_ms": round(tz, 4),
                                                             "frac": round(2.0 * macs / (tz * 1e-3) / 1e12 / peak, 4)}
            del az, bz
        if eng == lib.ENGINE_MFMA_F4 and probe.lib is not None:
            # registers-only chain of the same instruction, directly behind a run of the kernel
            for _ in range(REPS):
                gemm()
            mfma[eng]["mfma_chain_from_registers"] = {}
            for form in ((1, 0) if not args.chain_codes else range(len(Probe.MFMA_CHAIN_FORMS))):
                probe.mfma_rate(torch, form, 2000)
                mfma[eng]["mfma_chain_from_registers"][Probe.MFMA_CHAIN_FORMS[form]] = probe.mfma_rate(torch, form)
        if eng == auto:
            mfma[eng]["launches_timed"] = len(gemm_ms)
            mfma[eng]["timed"] = "HIP events around each GEMM launch of the timed region"
            mfma[eng]["traffic_source"] = src
        del ae, be
    if auto == lib.ENGINE_VALU:
        roofline = dict(roofline_valu)
    else:
        roofline = dict(mfma[auto])
        roofline["valu_popcount"] = {"frac": roofline_valu["frac"], "popcount_frac": roofline_valu["popcount_frac"],
                                     "achieved": roofline_valu["achieved"], "peak": roofline_valu["peak"], "unit": "Tlaneop/s",
                                     "avg_launch_ms": roofline_valu["avg_launch_ms"], "kernel": roofline_valu["kernel"],
                                     "gmacs": roofline_valu["gmacs"], "traffic": roofline_valu["traffic"],
                                     "probe_and_clocks": recon}

    cpu = None
    if args.cpu_rows > 0:
        rows = min(args.cpu_rows, m)
        a_host = a[:rows * 2 * kw].cpu().numpy()
        b_host = b.cpu().numpy()
        from oracle.ftnn_oracle import aligned_copy
        y_cpu, dt, kind = cpu_gemm_baseline(aligned_copy(a_host), aligned_copy(b_host), rows, n, kw, alpha)
        if y_cpu is None:
            cpu = {"value": None, "reason": dt}
        else:
            step()
            torch.cuda.synchronize()
            y_gpu = y.view(m, n)[:rows].cpu().numpy()
            cpu = {"value": round(float(rows) * n * k / dt / 1e9, 2), "unit": "GMAC/s", "cores": 1, "kind": kind,
                   "sample": "first %d of %d rows of A against all %d columns, K=%d (%.1f s on one core)"
                             % (rows, m, n, k, dt),
                   "gpu_rows_bit_exact": bool(y_gpu.tobytes() == np.ascontiguousarray(y_cpu).tobytes()),
                   "host": host_cpu()}

    extra = None
    if not args.no_extra:
        extra = {
            "tnn_gemm_256x256x4096": small_gemm(torch, lib, 256, 256, 4096),
            "tnn_conv_b1_c256_56x56_k3": conv_latency(torch, lib, TNN, (256, 56, 56, 256, 3, 3, 1, 1), 1, 2),
            "tbn_conv_b8_c128_28x28_k3": conv_latency(torch, lib, TBN, (128, 28, 28, 128, 3, 3, 1, 1), 8, 3),
            "btn_conv_b8_c128_28x28_k3": conv_latency(torch, lib, BTN, (128, 28, 28, 128, 3, 3, 1, 1), 8, 4),
            "tnn_resnet18_like_b32_e2e": e2e_latency(torch, lib, 32),
            "quantize_im2row_pack": pack_rates(torch, lib),
            "host_mm_8192x8192x32768": host_gemm_cfg4(torch, lib, a, b, m, n, kw) if (m, n, k) == (8192, 8192, 32768) else None,
            "other_types_same_gemm_shape": other_types(torch, lib, a, b, m, n, k),
            "reference_gemm_sweep": reference_gemm_sweep(torch, lib),
            "reference_single_layers_b8": reference_single_layers(torch, lib),
            "reference_e2e_networks_b8": reference_networks(torch, lib, only=None if args.full else ("resnet18", "resnet152")),
            "grid_sync_against_launch_boundary": grid_sync_cost(torch),
            "lds_read_rate_16_byte_reads": probe.lds_read_rate(torch) if probe.lib is not None else None,
        }
        if args.full:
            extra.update({
                "tnn_resnet18_like_other_batches": {"b%d" % bb: e2e_latency(torch, lib, bb, cpu=False) for bb in (1, 8, 128)},
                "other_types_resnet18_like_b32": {nm: e2e_latency(torch, lib, 32, cpu=False, typ=t)
                                                  for nm, t in (("tbn", 1), ("btn", 2), ("bnn", 3))},
            })

    line = {
        "metric": "TNN GEMM ternary GMAC/s", "value": round(macs / (ms_per_step * 1e-3) / 1e9, 1),
        "unit": "GMAC/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": {1: "u32", 2: "int8", 3: "fp4 (E2M1, exact for -1/0/+1) with fp32 accumulate"}[auto], "data": "synthetic",
        "config": {"workload": "TNN GEMM M=%d N=%d K=%d, uniform ternary, Packing 2, PReLU 0.5 fused" % (m, n, k),
                   "m": m, "n": n, "k": k, "step": step_desc},
        "roofline": roofline, "cpu_baseline": cpu,
        "engine": lib.ENGINE_NAMES[auto], "step_same_bits_as_valu": step_same,
        "step_with_weights_kept_in_engine_form": kept,
        "engines_whole_call_from_packed_operands": engines,
        "roofline_mfma_i8_kernel": mfma[lib.ENGINE_MFMA_I8] if auto != lib.ENGINE_MFMA_I8 else None,
        "extra": extra,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
