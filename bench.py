#!/usr/bin/env python3
"""Benchmark of the SMaLL layer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--model mobilenet_v1] [--batch 64]

A step is one forward pass of the model over one batch of synthetic images that are already
resident in HBM.  The headline workload is MobileNetV1 1.0 (224x224x3, float32) at batch 64; the
line also carries ResNet-8 uint8 at batch 64 and 256, the per-layer roofline table, the roofline
of the dominant kernel and the reference's CPU build timed on this host.

Prints ONE compact JSON line on stdout (headline, roofline, cpu_baseline, a per-configuration summary);
the per-layer tables go to bench_<workload>_full.json in the output folder (OUT_DIR), progress and readable tables to stderr.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
OUT_DIR = "gpurun_out"      # results that are too long for the one JSON line on stdout
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_HBM = 8.0e12          # B/s, MI355X HBM3E
PEAK_MFMA_F32 = 157.3e12   # FLOP/s, dense fp32 MFMA
PEAK_MFMA_I8 = 5.0e15      # OP/s, dense int8 MFMA

# HBM bytes per launch of the dominant kernel come from the committed counter summary (rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE over this same benchmark, two runs, scaled by what the counters read for an in-place ReLU of 822 MB): the
# figure is read from that file, together with the number of launches it was measured over, and is reported only while
# the forward pass still issues that many launches of the kernel family (another kernel mix: null, measure again).
TRAFFIC_PROFILES = {("mobilenet_v1", 64, "conv_mfma_f32_*"): "profiles/mobilenet_v1_b64_traffic_and_mfma.md"}


def measured_traffic_bytes(model_name, batch, family, launches):
    """-> HBM bytes per launch of `family` from the committed profile, or None (no profile, or measured on another mix)."""
    rel = TRAFFIC_PROFILES.get((model_name, batch, family))
    if rel is None:
        return None
    try:
        text = open(os.path.join(ROOT, rel)).read()
    except OSError:
        return None
    import re
    row = re.search(r"^\| %s \| (\d+) \|" % re.escape(family), text, re.M)
    per = re.search(r"HBM traffic ([0-9.]+) MB", text)
    if not row or not per or int(row.group(1)) != launches:
        return None
    return round(float(per.group(1)) * 1e6)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def cpu_model_name():
    """The host CPU's model string (first "model name" of /proc/cpuinfo)."""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def table_summary(entry, batch):
    """images/s + min / median per-layer roofline fraction of one configuration's per-layer table."""
    fr = sorted(r["roofline_frac"] for r in entry["layers"] if r.get("roofline_frac"))
    out = {"images_per_s": entry["images_per_s"], "ms_per_step": entry["ms_per_step"]}
    if fr:
        out["layer_frac_min"] = round(fr[0], 3)
        out["layer_frac_median"] = round(statistics.median(fr), 3)
    fl = [r["frac_of_stream_floor"] for r in entry["layers"] if r.get("frac_of_stream_floor")]
    if len(entry["layers"]) == 1 and fl:
        out["of_bytes_only_kernel"] = fl[0]         # single bandwidth-bound layer: against a kernel that only moves its bytes
    for k in ("hip_graph_ms_per_step", "one_launch_ms_per_step", "one_launch_images_per_s", "roofline"):
        if k in entry:
            out[k] = entry[k]
    return out


def emit(out, tag):
    """The full result (per-layer tables, extras) goes to bench_<tag>_full.json in OUT_DIR and to stderr; stdout gets
    ONE compact JSON line: the headline fields, roofline, cpu_baseline and a short per-configuration summary."""
    full = json.dumps(out)
    path = os.path.join(ROOT, OUT_DIR, "bench_%s_full.json" % tag)
    try:
        os.makedirs(os.path.dirname(path), exist_ok=True)
        with open(path, "w") as f:
            f.write(full + "\n")
        log("full per-layer tables and extras: %s" % path)
    except OSError as e:
        log("could not write %s: %r" % (path, e))
    extras = out.get("extras") or {}
    summary = {}
    for key, e in extras.items():
        # the batch-1 single layers are launch-latency-bound: in the full file, not in the compact line
        single_b1 = key.endswith("_b1") and len(e.get("layers", ())) == 1 if isinstance(e, dict) else False
        if isinstance(e, dict) and "layers" in e and "images_per_s" in e and not single_b1:
            summary[key] = table_summary(e, None)
    head_fr = sorted(r["roofline_frac"] for r in out.get("layers", []) if r.get("roofline_frac"))
    if head_fr:
        summary["headline_layers"] = {"n": len(head_fr), "frac_min": round(head_fr[0], 3),
                                      "frac_median": round(statistics.median(head_fr), 3)}
        fl = sorted(r["frac_of_stream_floor"] for r in out.get("layers", []) if r.get("frac_of_stream_floor"))
        if fl:
            # bandwidth-bound layers against a kernel that only moves their bytes (same place in the model)
            summary["headline_layers"].update({"bandwidth_layers": len(fl), "of_bytes_only_kernel_min": fl[0],
                                               "of_bytes_only_kernel_median": round(statistics.median(fl), 3)})
    for k in ("fresh_process_ms_per_step", "mfma_f32_sustained_TFLOPs", "hbm_copy_sustained_GBs", "mfma_and_vector_alu_same_simd", "hip_graph_ms_per_step",
              "host_buffers_ms_per_step", "host_buffers_images_per_s", "host_buffers_serial_ms_per_step",
              "host_buffers_result_unchanged"):
        if k in extras:
            summary[k] = extras[k]
    for k in ("resnet8_u8_cpu", "dscnn_cpu", "tiny_yolo_v2_cpu"):
        if extras.get(k):
            summary[k] = {f: extras[k][f] for f in ("value", "unit", "cores", "kind")}
    compact = {k: v for k, v in out.items() if k not in ("layers", "extras")}
    compact["summary"] = summary
    compact["full_result"] = os.path.relpath(path, ROOT)
    print(json.dumps(compact), flush=True)


def op_bytes(model, op, batch):
    """Algorithmic HBM bytes of one op for `batch` images: every tensor once; in-place
    activations count a read and a write; Accum reads both operands and writes one."""
    es = model.esize()
    n_in, n_out = op.act_elems()
    w = op.weight_elems() * es
    if op.kind == "accum":
        return batch * 3 * n_out * es
    return batch * (n_in + n_out) * es + w


def op_bound(model, op, batch):
    """-> (seconds at the roofline, 'hbm' | 'mfma')."""
    t_hbm = op_bytes(model, op, batch) / PEAK_HBM
    peak = PEAK_MFMA_F32 if model.dtype == "f32" else PEAK_MFMA_I8
    on_mfma = op.kind in ("conv", "dense") and op.C % 16 == 0
    t_mfma = batch * op.flops() / peak if on_mfma else 0.0
    return (t_mfma, "mfma") if t_mfma > t_hbm else (t_hbm, "hbm")


# (timed steps, warm-up steps) per headline model when the command line gives none: ~200 ms timed after ~100 ms of load
DEFAULT_COUNTS = {"mobilenet_v1": (200, 100), "tiny_yolo_v2": (200, 100), "layer_sweep": (200, 100),
                  "resnet8_u8": (6000, 3000), "dscnn": (6000, 3000)}


def counts_for(step_fn, args, at_least=0):
    """(timed steps, warm-up steps) for a side measurement, from the duration of `step_fn` (3 + 10 probe calls): the
    warm-up is about 100 ms of load and the timed region about 200 ms whatever the model's size, and never fewer than
    the counts on the command line.  (The command line's counts are the headline's; a side configuration is built after
    host work during which the GPU idles, and 5 + 20 passes of a small model would time the machine's way back from
    idle, not the kernels.)"""
    import torch
    for _ in range(3):
        step_fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(10):
        step_fn()
    torch.cuda.synchronize()
    est = max((time.perf_counter() - t0) / 10, 1e-6)
    k, w = min(8000, max(200, int(0.2 / est) + 1)), min(4000, max(100, int(0.1 / est) + 1))
    if not args.auto_counts:
        k, w = max(k, args.steps), max(w, args.warmup)
    return max(k, at_least), w


def time_forward(ex, steps, warmup):
    import torch
    for _ in range(warmup):
        ex.forward()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        ex.forward()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def time_forward_one_launch(ex, steps, warmup):
    """Seconds per small_hip_qmodel_forward launch, HIP events on the launch stream."""
    import torch
    for _ in range(warmup):
        ex.forward_one_launch()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(steps):
        ex.forward_one_launch()
    ev1.record()
    torch.cuda.synchronize()
    return ev0.elapsed_time(ev1) * 1e-3 / steps


def time_ops(ex, steps):
    """Per-op device time (ms) from HIP events on the launch stream, the median over `steps` passes.  Float32 models are
    timed launch by launch as the forward pass issues them: a convolution that carries its 2x2 max-pool has the
    time of the fused launch, and the pool's own row reads 0.  (uint8 models are timed op by op, unfused.)"""
    import torch
    ops = ex.model.ops
    st = ex.stream()
    # Events for all passes are made first and the passes are issued back to back with one synchronisation at the end:
    # the GPU stays loaded (a pause between passes lets its clock drop), and the host never waits inside a pass.
    if ex.model.dtype == "f32" and ex.fused:
        entries = ex.plan
        index = {op.name: i for i, op in enumerate(ops)}
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(len(entries) + 1)] for _ in range(steps)]
        for ev in evs:
            ev[0].record()
            for i, e in enumerate(entries):
                ex.run_entry(e, st)
                ev[i + 1].record()
        torch.cuda.synchronize()
        seen = [[] for _ in ops]
        for ev in evs:
            for i, e in enumerate(entries):
                seen[index[e[0].name]].append(ev[i].elapsed_time(ev[i + 1]))
        return [statistics.median(t) if t else 0.0 for t in seen]
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(len(ops) + 1)] for _ in range(steps)]
    for ev in evs:
        ev[0].record()
        for i, op in enumerate(ops):
            ex.run_op(op, st)
            ev[i + 1].record()
    torch.cuda.synchronize()
    seen = [[] for _ in ops]
    for ev in evs:
        for i in range(len(ops)):
            seen[i].append(ev[i].elapsed_time(ev[i + 1]))
    return [statistics.median(t) for t in seen]


def layer_table(model, batch, ms):
    """Per-op rows.  A convolution that carried the following 2x2 max-pool (or, a first layer, the following depthwise
    layer) in its launch is priced on the fused launch's own algorithmic bytes (its input + the second layer's output +
    the filters); the second layer's row is empty."""
    rows = []
    ops = model.ops
    es = model.esize()
    for i, (op, t) in enumerate(zip(ops, ms)):
        tb, kind = op_bound(model, op, batch)
        nbytes = op_bytes(model, op, batch)
        if t == 0.0 and op.kind in ("maxpool", "dw"):
            rows.append({"layer": op.name, "ms": 0.0, "bound": kind, "roofline_frac": None, "GB/s": None,
                         "TFLOP/s": None, "fused_into": "previous convolution"})
            continue
        if op.kind == "conv" and i + 1 < len(ops) and ops[i + 1].kind in ("maxpool", "dw") and ms[i + 1] == 0.0:
            nbytes = batch * (op.act_elems()[0] + ops[i + 1].act_elems()[1]) * es + \
                (op.weight_elems() + ops[i + 1].weight_elems()) * es
            # the fused launch's own roofline: its bytes at the HBM peak, or the convolution's flops at the MFMA peak
            t_mfma = batch * op.flops() / (PEAK_MFMA_F32 if model.dtype == "f32" else PEAK_MFMA_I8) if op.C % 16 == 0 else 0.0
            tb, kind = (t_mfma, "mfma") if t_mfma > nbytes / PEAK_HBM else (nbytes / PEAK_HBM, "hbm")
        rows.append({"layer": op.name, "ms": round(t, 5), "bound": kind,
                     "roofline_frac": round(tb / (t * 1e-3), 4) if t > 0 else None,
                     "GB/s": round(nbytes / (t * 1e-3) / 1e9, 1) if t > 0 else None,
                     "TFLOP/s": round(batch * op.flops() / (t * 1e-3) / 1e12, 2) if t > 0 and op.flops() else None})
    return rows


def stream_floors(ex, steps):
    """For every bandwidth-bound layer of a float32 model (depthwise convolution, pooling, activation): the time of a
    kernel that only moves the layer's bytes (reads the input tensor, writes the output tensor: shp_probe_stream of
    libsmall_hip_probe.so, a measurement aid outside the product library), launched where the layer is launched, i.e.
    right after the layer that produces its input, so that the caches are in the state the layer finds.
    -> {layer name: ms}, median over `steps`."""
    import ctypes as C
    import torch
    from smallframework_amd import capi
    path = os.path.join(os.path.dirname(capi.LIB_PATH), "libsmall_hip_probe.so")
    if not os.path.exists(path) or ex.model.dtype != "f32":
        return {}
    probe = C.CDLL(path).shp_probe_stream
    probe.restype, probe.argtypes = C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p]
    st = ex.stream()
    out = {}
    for j, entry in enumerate(ex.plan):
        op = entry[0]
        if op.kind not in ("dw", "maxpool", "avgpool", "relu", "leaky") or entry[1] is not None:
            continue
        n_in, n_out = (ex.batch * e for e in op.act_elems())
        n_in16, n_out16 = n_in // 4, min(n_out, n_in) // 4
        src, dst = ex.buf[op.src], ex.buf[op.dst]
        if src.data_ptr() == dst.data_ptr():
            continue
        ts = []
        for _ in range(steps):
            if j > 0:
                ex.run_entry(ex.plan[j - 1], st)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            rc = probe(C.c_void_p(src.data_ptr()), n_in16, C.c_void_p(dst.data_ptr()), n_out16, st)
            e1.record()
            if rc:
                raise RuntimeError("shp_probe_stream: status %d" % rc)
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1))
        out[op.name] = statistics.median(ts)
    return out


def add_floor_column(table, floors):
    for r in table:
        f = floors.get(r["layer"])
        if f and r.get("ms"):
            r["stream_floor_ms"] = round(f, 5)
            r["frac_of_stream_floor"] = round(f / r["ms"], 3)


def mfma_probe_tflops(steps=5):
    """Calibration: float32 MFMA instructions on registers only (libsmall_hip_probe.so, a measurement aid that is
    not part of the product library), 4 workgroups per CU (one wave per SIMD and workgroup).  With 8 workgroups per CU
    this four-accumulator loop reads 138 instead of 155 TFLOP/s; a one-accumulator loop sustains 155 with eight waves per
    SIMD as well, so that figure says something about the probe at that occupancy, not about the machine.
    -> sustained TFLOP/s of the matrix pipes on this machine (to set beside the published 157.3), or None when the probe
    library is not built."""
    import ctypes as C
    import torch
    from smallframework_amd import capi
    path = os.path.join(os.path.dirname(capi.LIB_PATH), "libsmall_hip_probe.so")
    if not os.path.exists(path):
        return None
    probe = C.CDLL(path).shp_probe_mfma_f32
    probe.restype, probe.argtypes = C.c_int, [C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    sink = torch.zeros(4, device="cuda")
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    wgs, iters = 256 * 4, 20000

    def call():
        rc = probe(wgs, iters, C.c_void_p(sink.data_ptr()), st)
        if rc:
            raise RuntimeError("shp_probe_mfma_f32: status %d" % rc)
    call()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        call()
    e1.record()
    torch.cuda.synchronize()
    flops = steps * float(wgs) * 4 * iters * 4 * 4096
    return flops / (e0.elapsed_time(e1) * 1e-3) / 1e12


def hbm_copy_gbs(nbytes=822083584, steps=10):
    """Calibration: a device-to-device copy of `nbytes` through the runtime (read + write counted), GB/s."""
    import torch
    x = torch.empty(nbytes // 4, dtype=torch.float32, device="cuda").normal_()
    y = torch.empty_like(x)
    y.copy_(x)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        y.copy_(x)
    e1.record()
    torch.cuda.synchronize()
    return 2.0 * nbytes * steps / (e0.elapsed_time(e1) * 1e-3) / 1e9


def issue_overlap_us(iters=500):
    """Calibration: matrix instructions of one wave and vector-ALU instructions of another wave on the same SIMD, timed
    apart and together (libsmall_hip_probe.so, one workgroup of eight waves per CU; each side is 1024 issue cycles per
    iteration).  -> {"matrix_us", "vector_us", "both_us"} or None when the probe library is not built.  both = matrix +
    vector means the two do not overlap: a kernel's vector instructions are time its matrix pipe stands still."""
    import ctypes as C
    import torch
    from smallframework_amd import capi
    path = os.path.join(os.path.dirname(capi.LIB_PATH), "libsmall_hip_probe.so")
    if not os.path.exists(path) or not hasattr(C.CDLL(path), "shp_probe_issue_overlap"):
        return None
    probe = C.CDLL(path).shp_probe_issue_overlap
    probe.restype, probe.argtypes = C.c_int, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    sink = torch.zeros(4, device="cuda")
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {}
    for name, mode in (("matrix_us", 1), ("vector_us", 2), ("both_us", 3)):
        for timed in (False, True):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(3):
                rc = probe(256, mode, iters, C.c_void_p(sink.data_ptr()), st)
                if rc:
                    raise RuntimeError("shp_probe_issue_overlap: status %d" % rc)
            e1.record()
            torch.cuda.synchronize()
            if timed:
                out[name] = round(e0.elapsed_time(e1) / 3 * 1e3, 1)
    return out


def library_gemm_ms(model, batch, steps, warmup):
    """Calibration, not part of the product path: the contraction of every MFMA-sized convolution as a plain
    float32 GEMM [Co x K] . [K x pixels] through torch.mm (the vendor BLAS; no im2col cost counted, TF32 off).
    -> {layer name: milliseconds}.  It shows what a tuned library reaches on this machine for the same shapes."""
    import torch
    torch.backends.cuda.matmul.allow_tf32 = False
    out = {}
    for op in model.ops:
        if op.kind not in ("conv", "dense") or op.C % 16 != 0:
            continue
        M, K = op.Co, op.C * op.kh * op.kw
        N = batch * op.Ho * op.Wo
        a = torch.randn(M, K, device="cuda")
        b = torch.randn(K, N, device="cuda")
        c = torch.empty(M, N, device="cuda")
        for _ in range(warmup):
            torch.mm(a, b, out=c)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            torch.mm(a, b, out=c)
        e1.record()
        torch.cuda.synchronize()
        out[op.name] = e0.elapsed_time(e1) / steps
    return out


def cpu_threads():
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    threads = min(threads, os.cpu_count() or threads)
    os.environ["OMP_NUM_THREADS"] = str(threads)
    return threads


def cpu_reference_model(model, weights, x_one, budget_s=10.0, max_passes=4096):
    """The reference's own ZEN2 build (AVX2 + OpenMP) on this host, batch-1 calls.
    -> (cpu_baseline object, per-layer mean milliseconds per image)."""
    from oracle.binding import have_ref
    if not have_ref("ZEN2"):
        return None, None
    from oracle.model_exec import RefExecutor
    threads = cpu_threads()
    ex = RefExecutor(model, weights, x_one, "ZEN2")
    ex.forward()                     # warm-up (the reference's protocol: 1 warm-up call)
    per_op = [0.0] * len(model.ops)
    t0 = time.perf_counter()
    n = 0
    ts = []
    while n < max_passes and (time.perf_counter() - t0) < budget_s:
        t1 = time.perf_counter()
        ex.forward(per_op)
        ts.append(time.perf_counter() - t1)
        n += 1
    mean = sum(ts) / len(ts)
    base = {"value": round(1.0 / mean, 2), "unit": "images/s", "cores": threads, "cpu": cpu_model_name(),
            "kind": "reference", "sample": "%d batch-1 forward passes of %s (all layers, unfused Conv2D+ReLU as the reference's "
                      "Layer classes issue them) on the reference's ZEN2 build, 1 warm-up; min %.2f ms mean %.2f ms"
                      % (n, model.name, 1e3 * min(ts), 1e3 * mean)}
    return base, [1e3 * t / n for t in per_op]


def add_cpu_column(table, cpu_ms, batch):
    """Per layer: the reference CPU build's milliseconds per image and the GPU/CPU throughput ratio."""
    if cpu_ms is None:
        return
    for row, c in zip(table, cpu_ms):
        row["cpu_ref_ms_per_image"] = round(c, 4)
        if row.get("ms"):
            row["gpu_over_cpu"] = round(c / (row["ms"] / batch), 1)


def cpu_port_u8(model, batch=8):
    """A model on the scalar C port (1 core).  ResNet-8 uint8: the reference has no uint8 Accum/AveragePool;
    DS-CNN: its AVX2 build cannot run the 10x4 first layer."""
    from smallframework_amd import models
    from oracle.model_exec import OracleExecutor
    w = models.make_weights(model)
    x = models.make_input(model, batch)
    ex = OracleExecutor(model, batch, w, x)
    ex.forward()
    t0 = time.perf_counter()
    reps = 3
    for _ in range(reps):
        OracleExecutor(model, batch, w, x).forward()
    dt = (time.perf_counter() - t0) / reps
    return {"value": round(batch / dt, 1), "unit": "images/s", "cores": 1, "cpu": cpu_model_name(), "kind": "port",
            "sample": "%d images x %d passes of %s on this build's scalar C restatement, 1 core (not the reference's "
                      "build)" % (batch, reps, model.name)}


def layout_rows(lib, torch, steps, warmup):
    """On-device pack_buffer / unpack_buffer (NCHW <-> packed), HIP-event timed; pure data movement,
    bound = HBM with one read and one write per element."""
    import ctypes as C
    cases = [("pack_input_3x224x224_b64", "pack", 64, 3, 224, 224),
             ("pack_256x56x56_b64", "pack", 64, 256, 56, 56),
             ("unpack_256x56x56_b64", "unpack", 64, 256, 56, 56),
             ("unpack_logits_1008_b64", "unpack", 64, 1008, 1, 1)]
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rows = []
    for name, way, b, c, h, w in cases:
        n = b * c * h * w
        src = torch.randn(n, device="cuda")
        dst = torch.empty_like(src)
        fn = lib.small_hip_pack if way == "pack" else lib.small_hip_unpack
        call = lambda: fn(0, b, 1, c, h, w, 16, 16, C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), 4, st)
        for _ in range(warmup):
            assert call() == 0
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            call()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        nbytes = 2 * n * 4
        rows.append({"layer": name, "ms": round(ms, 5), "bound": "hbm", "GB/s": round(nbytes / ms / 1e6, 1),
                     "roofline_frac": round(nbytes / PEAK_HBM / (ms * 1e-3), 4)})
        log("%-26s %.4f ms  %.0f GB/s  %.1f%% of HBM peak" % (name, ms, nbytes / ms / 1e6, 100 * rows[-1]["roofline_frac"]))
        del src, dst
    torch.cuda.empty_cache()
    return rows


def sweep_only(args, torch, models):
    """--model layer_sweep: the four single layers at C = 256, 56x56 (Conv2D 3x3, DepthwiseConv2D 3x3,
    MaxPool2D 3x3 stride 2, ReLU), each run `steps` times at --batch (default 64).  The JSON line is
    about the Conv2D layer; the others are in "layers"."""
    batch = args.batch or 64
    rows, head = [], None
    for m in models.layer_sweep():
        ex = models.HipExecutor(m, batch)
        k, w = counts_for(ex.forward, args)
        sec = time_forward(ex, k, w)
        ms = time_ops(ex, min(k, 200))
        r = layer_table(m, batch, ms)[0]
        r["layer"] = m.name
        r["images_per_s"] = round(batch / (r["ms"] * 1e-3), 1)
        rows.append(r)
        log("%-20s batch %d: %.4f ms  %.0f images/s  %s %.1f%% of roofline" % (
            m.name, batch, r["ms"], r["images_per_s"], r["bound"], 100 * (r["roofline_frac"] or 0)))
        if head is None:
            head = (m, sec, r)
        del ex
        torch.cuda.empty_cache()
    from smallframework_amd import capi
    rows += layout_rows(capi.load(), torch, args.steps, args.warmup)
    m, sec, r = head
    op = m.ops[0]
    out = {"metric": "images/s @batch%d %s fp32" % (batch, m.name), "value": round(batch / sec, 2),
           "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "f32", "data": "synthetic",
           "config": {"workload": "single layers at C=256, 56x56, batch %d: Conv2D 3x3 s1 same, DepthwiseConv2D "
                                  "3x3 s1, MaxPool2D 3x3 s2 valid, ReLU" % batch, "batch": batch},
           "roofline": {"bound": "mfma", "achieved": r["TFLOP/s"], "peak": round(PEAK_MFMA_F32 / 1e12, 1),
                        "unit": "TFLOP/s", "frac": r["roofline_frac"], "traffic": None,
                        "kernel": "conv_mfma_f32_*", "launches_per_step": 1, "avg_launch_ms": r["ms"],
                        "algorithmic_per_launch": {"GFLOP": round(batch * op.flops() / 1e9, 3),
                                                   "MB": round(op_bytes(m, op, batch) / 1e6, 3)}},
           "cpu_baseline": None, "layers": rows}
    emit(out, "layer_sweep_b%d" % batch)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # defaults (DEFAULT_COUNTS): a GPU that has idled needs some tens of milliseconds of convolution load to reach its
    # sustained state (see the order of the measurements in main), so the default warm-up is about 100 ms of forward
    # passes and the timed region about 200 ms
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--model", default="mobilenet_v1",
                    choices=["mobilenet_v1", "resnet8_u8", "tiny_yolo_v2", "dscnn", "layer_sweep"])
    ap.add_argument("--batch", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="headline model only")
    ap.add_argument("--unfused", action="store_true", help="issue Conv2D and the activation as separate calls")
    ap.add_argument("--library-gemm", action="store_true",
                    help="calibration: also time every MFMA-sized convolution's contraction as a torch.mm float32 GEMM")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this build measures one GPU; the path shards by image with no collective, "
            "so --gpus N > 1 is not run here.")
        sys.exit(2)

    import torch
    from smallframework_amd import capi, models
    if not torch.cuda.is_available():
        log("bench.py: no GPU visible")
        sys.exit(1)
    capi.load()
    args.auto_counts = args.steps is None and args.warmup is None
    if args.steps is None:
        args.steps = DEFAULT_COUNTS[args.model][0]
    if args.warmup is None:
        args.warmup = DEFAULT_COUNTS[args.model][1]
    if args.model == "layer_sweep":
        return sweep_only(args, torch, models)
    default_batch = {"mobilenet_v1": 64, "resnet8_u8": 64, "tiny_yolo_v2": 16, "dscnn": 64}
    batch = args.batch or default_batch[args.model]
    model = getattr(models, args.model)()
    log("building %s batch %d ..." % (model.name, batch))
    weights = models.make_weights(model)
    x = models.make_input(model, batch)
    ex = models.HipExecutor(model, batch, weights, x, fused=not args.unfused)

    # Order of the measurements.  A GPU that has been idle runs its first 30-odd forward passes up to 12% slower, whatever
    # ran before that was not convolution-like: half a second of MFMA instructions on registers or of device copies
    # leaves the ramp in place, 100 passes of any convolution model (this one on other buffers, another model) remove
    # it, and the core clock the driver reports stays at 2.36-2.38 GHz throughout.  So the state is the machine's, not
    # this process's or these buffers', and every figure that is read against a roofline has to be taken in it:
    #   1. the first `warmup` + `steps` passes of the process, reported beside the headline as the fresh-process figure;
    #   2. machine calibration (float32 MFMA on registers only, a device-to-device copy, the issue probe);
    #   3. the per-layer pass (HIP events around every launch, at least 60 passes; medians);
    #   4. `warmup` untimed and `steps` timed passes: the headline.
    calib = {}
    fresh = None
    if model.dtype == "f32" and not args.no_extras:
        fresh = time_forward(ex, args.steps, args.warmup)
        log("%s: %.3f ms/step over the first %d + %d passes of the process" % (model.name, fresh * 1e3, args.warmup, args.steps))
        sustained = mfma_probe_tflops()
        if sustained is not None:
            calib["mfma_f32_sustained_TFLOPs"] = round(sustained, 1)
        calib["hbm_copy_sustained_GBs"] = round(hbm_copy_gbs(), 1)
        ov = issue_overlap_us()
        if ov is not None:
            calib["mfma_and_vector_alu_same_simd"] = ov
    # per-op device times (HIP events on the launch stream); the headline-only runs the profile commands make keep to
    # the command line's count
    layer_passes = min(args.steps, 200) if args.no_extras else max(60, min(args.steps, 200))
    ms = time_ops(ex, layer_passes)
    sec = time_forward(ex, args.steps, args.warmup)
    one_launch = None
    if model.dtype == "u8" or model.name == "dscnn":
        # quantised models and the DS-CNN run as ONE launch (small_hip_qmodel_forward / small_hip_fmodel_forward: a
        # workgroup per image, tensors in LDS); that is the step that is reported, the layer-by-layer time stays beside it
        ex.build_one_launch()
        sec_layers, sec = sec, time_forward_one_launch(ex, args.steps, args.warmup)
        one_launch = {"layer_by_layer_ms_per_step": round(sec_layers * 1e3, 4), "ms_per_step": round(sec * 1e3, 4),
                      "TOPs": round(batch * model.flops_per_image() / sec / 1e12, 3)}
        log("%s: layer by layer %.4f ms/step, one launch %.4f ms/step" % (model.name, sec_layers * 1e3, sec * 1e3))
    ips = batch / sec
    log("%s: %.3f ms/step, %.1f images/s" % (model.name, sec * 1e3, ips))

    table = layer_table(model, batch, ms)
    if not args.no_extras:
        # what a kernel that only moves each bandwidth-bound layer's bytes takes in the same place of the model
        add_floor_column(table, stream_floors(ex, max(5, min(args.steps, 200) // 2)))
    if args.library_gemm:
        log("float32 MFMA on registers only: %s TFLOP/s sustained (published peak 157.3)" % mfma_probe_tflops())
        log("device-to-device copy of 822 MB: %.0f GB/s read + write (published peak 8000)" % hbm_copy_gbs())
        lib_ms = library_gemm_ms(model, batch, args.steps, args.warmup)
        for r in table:
            if r["layer"] in lib_ms:
                r["library_gemm_ms"] = round(lib_ms[r["layer"]], 5)
    for r in table:
        log("  %-28s %9.4f ms  %-4s %6.1f%%%s%s" % (r["layer"], r["ms"], r["bound"], 100 * (r["roofline_frac"] or 0),
                                                    "   library GEMM %.4f ms" % r["library_gemm_ms"]
                                                    if "library_gemm_ms" in r else "",
                                                    "   bytes-only kernel %.4f ms (%.0f%% of it)" % (
                                                        r["stream_floor_ms"], 100 * r["frac_of_stream_floor"])
                                                    if "stream_floor_ms" in r else ""))

    # dominant kernel = the one with the largest summed time
    # convolutions that carry the depthwise layer after them run in kernels of their own (first layer: conv_stem3x3_dw3x3,
    # pointwise: conv_pw_dw3x3); the depthwise layer's row has no launch
    with_dw = {e[0].name for e in getattr(ex, "plan", []) if e[1] is not None and e[1].kind == "dw"} \
        if model.dtype == "f32" and getattr(ex, "fused", False) else set()

    def kernel_of(op):
        if op.kind in ("conv", "dense"):
            if op.name in with_dw:
                return "conv_stem3x3_dw3x3_f32_kernel" if op.C % 16 != 0 else "conv_pw_dw3x3_f32_kernel"
            if op.C % 16 != 0:
                return "conv_smallci_%s_kernel" % model.dtype
            return "conv_mfma_%s_*" % model.dtype
        return {"dw": "dw_%s_kernel" % model.dtype, "maxpool": "pool_%s_kernel" % model.dtype,
                "avgpool": "pool_%s_kernel" % model.dtype}.get(op.kind, "ew_%s_kernel" % model.dtype)

    per_kernel = {}
    for i, (op, t) in enumerate(zip(model.ops, ms)):
        if t == 0.0 and op.kind in ("maxpool", "dw") and i > 0 and model.ops[i - 1].kind == "conv":
            continue                                   # ran inside the previous convolution's launch
        k = kernel_of(op)
        d = per_kernel.setdefault(k, {"ms": 0.0, "launches": 0, "flops": 0.0, "bytes": 0.0})
        d["ms"] += t
        d["launches"] += 1
        d["flops"] += batch * op.flops()
        d["bytes"] += op_bytes(model, op, batch)
    dom = max(per_kernel, key=lambda k: per_kernel[k]["ms"])
    d = per_kernel[dom]
    if "mfma" in dom:
        peak = (PEAK_MFMA_F32 if model.dtype == "f32" else PEAK_MFMA_I8) / 1e12
        ach = d["flops"] / (d["ms"] * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": round(ach, 2), "peak": round(peak, 1), "unit": "TFLOP/s",
                "frac": round(ach / peak, 4), "traffic": None}
    else:
        ach = d["bytes"] / (d["ms"] * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": round(ach, 1), "peak": 8000.0, "unit": "GB/s",
                "frac": round(ach / 8000.0, 4), "traffic": None}
    if not args.unfused:
        roof["traffic"] = measured_traffic_bytes(model.name, batch, dom, d["launches"])   # bytes per launch, or None
    roof.update({"kernel": dom, "launches_per_step": d["launches"],
                 "avg_launch_ms": round(d["ms"] / d["launches"], 5),
                 "algorithmic_per_launch": {"GFLOP": round(d["flops"] / d["launches"] / 1e9, 3),
                                            "MB": round(d["bytes"] / d["launches"] / 1e6, 3)}})

    extras = {"per_kernel_ms": {k: round(v["ms"], 4) for k, v in per_kernel.items()},
              "sum_of_layer_ms": round(sum(ms), 4)}
    if one_launch:
        # the step IS one kernel: its roofline is the whole model's arithmetic over the launch time (int8 MFMA peak);
        # algorithmic bytes = the images in, the logits out, every filter once
        extras["one_launch"] = one_launch
        extras["layer_by_layer_roofline"] = roof
        algo = batch * (model.in_shape[0] * model.in_shape[1] * model.in_shape[2] + model.ops[-1].Co) + \
            sum(o.weight_elems() for o in model.ops)
        ach = batch * model.flops_per_image() / sec / 1e12
        pk = PEAK_MFMA_I8 if model.dtype == "u8" else PEAK_MFMA_F32
        roof = {"bound": "mfma", "achieved": round(ach, 3), "peak": round(pk / 1e12, 1),
                "unit": "TOP/s" if model.dtype == "u8" else "TFLOP/s",
                "frac": round(ach / (pk / 1e12), 4), "traffic": None,
                "kernel": "qmodel_u8_kernel" if model.dtype == "u8" else "fmodel_f32_kernel",
                "launches_per_step": 1, "avg_launch_ms": round(sec * 1e3, 5),
                "algorithmic_per_launch": {"GOP": round(batch * model.flops_per_image() / 1e9, 3),
                                           "MB": round(algo / 1e6, 3)},
                "note": "instruction-, LDS- and latency-bound: one workgroup per image, 16 waves per compute unit, only "
                        "`batch` of the 256 compute units busy"}
    if model.dtype == "f32" and not args.no_extras:
        # what the float32 matrix pipes sustain on registers alone, beside the published peak used in `roofline`
        extras.update(calib)
        extras["fresh_process_ms_per_step"] = round(fresh * 1e3, 4)
        # the same forward pass replayed from a HIP graph (no host work between the launches)
        ex.capture()
        for _ in range(args.warmup):
            ex.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            ex.replay()
        torch.cuda.synchronize()
        sg = (time.perf_counter() - t0) / args.steps
        extras["hip_graph_ms_per_step"] = round(sg * 1e3, 4)
        log("%s: HIP graph replay %.3f ms/step (eager %.3f)" % (model.name, sg * 1e3, sec * 1e3))
        # the same step when the caller holds host buffers: pinned input uploaded, forward pass, output downloaded
        # (a note beside the headline, which is measured with the input resident in device memory)
        op = model.ops[-1]
        c, h, w = op.out_shape()
        n_out = ex.batch * c * h * w
        hx = torch.empty(ex.buf["in"].numel(), dtype=ex.tdtype, pin_memory=True)
        hx.copy_(ex.buf["in"])
        hy = torch.empty(n_out, dtype=ex.tdtype, pin_memory=True)

        def host_step():
            ex.buf["in"].copy_(hx, non_blocking=True)
            ex.forward()
            hy.copy_(ex.buf[ex.out_name][:n_out], non_blocking=True)
        # a side measurement whose pipeline needs some steps to fill: at least 100 timed steps after 30
        h_steps, h_warm = max(args.steps, 100), max(args.warmup, 30)
        for _ in range(h_warm):
            host_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(h_steps):
            host_step()
        torch.cuda.synchronize()
        sh = (time.perf_counter() - t0) / h_steps
        extras["host_buffers_serial_ms_per_step"] = round(sh * 1e3, 4)
        extras["host_buffers_MB_per_step"] = round((hx.numel() * hx.element_size() + hy.numel() * hy.element_size()) / 1e6, 2)
        log("%s: with host buffers, serial (upload + forward + download on one stream) %.3f ms/step" % (model.name, sh * 1e3))
        # the same with the upload of batch i + 1 under the layers of batch i (small_hip_upload_begin / _wait: the library's
        # copy stream and an event; what Tensor::prefetch() does in the C++ classes): two device inputs in turn
        import ctypes as C
        lib = capi.load()
        ref_out = ex.output().copy()
        din = [ex.buf["in"], torch.empty_like(ex.buf["in"])]
        hxs = [hx, torch.empty(hx.numel(), dtype=ex.tdtype, pin_memory=True)]
        hxs[1].copy_(hx)
        nbytes = hx.numel() * hx.element_size()
        pending = [None, None]

        def begin(i):
            e = C.c_void_p()
            capi.check(lib.small_hip_upload_begin(C.c_void_p(din[i].data_ptr()), C.c_void_p(hxs[i].data_ptr()), nbytes,
                                                  ex.stream(), C.byref(e)))
            pending[i] = e

        step_no = [0]

        def host_step_overlapped():
            b = step_no[0] & 1
            step_no[0] += 1
            begin(b ^ 1)                                   # batch i + 1 starts going up ...
            capi.check(lib.small_hip_upload_wait(pending[b], ex.stream()))
            ex.buf["in"] = din[b]
            ex.forward()                                   # ... while batch i runs
            hy.copy_(ex.buf[ex.out_name][:n_out], non_blocking=True)
        begin(0)
        for _ in range(h_warm):
            host_step_overlapped()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(h_steps):
            host_step_overlapped()
        torch.cuda.synchronize()
        so = (time.perf_counter() - t0) / h_steps
        capi.check(lib.small_hip_upload_finish(pending[step_no[0] & 1]))
        same = bool((hy.numpy() == ref_out).all())
        ex.buf["in"] = din[0]
        extras["host_buffers_ms_per_step"] = round(so * 1e3, 4)
        extras["host_buffers_images_per_s"] = round(ex.batch / so, 1)
        extras["host_buffers_result_unchanged"] = same
        log("%s: with host buffers, next upload under the current pass %.3f ms/step (logits %s the resident run's)"
            % (model.name, so * 1e3, "equal" if same else "DIFFER FROM"))
    if not args.no_extras and args.model == "mobilenet_v1":
        for name, b in (("resnet8_u8", 64), ("resnet8_u8", 256)):
            m2 = getattr(models, name)()
            e2 = models.HipExecutor(m2, b)
            k2, w2 = counts_for(e2.forward, args, 50)
            s2 = time_forward(e2, k2, w2)
            ms2 = time_ops(e2, 10)
            # the same forward pass replayed from a HIP graph (21 launches, no host work in between)
            e2.capture()
            for _ in range(w2):
                e2.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(k2):
                e2.replay()
            torch.cuda.synchronize()
            s3 = (time.perf_counter() - t0) / k2
            # the whole model in one launch (one workgroup per image, tensors and filters in LDS), HIP-event timed
            e2.build_one_launch()
            k4, w4 = counts_for(e2.forward_one_launch, args, 50)
            s4 = time_forward_one_launch(e2, k4, w4)
            algo = b * (m2.in_shape[0] * m2.in_shape[1] * m2.in_shape[2] + m2.ops[-1].Co) + \
                sum(o.weight_elems() for o in m2.ops)
            extras["%s_b%d" % (name, b)] = {"images_per_s": round(b / s2, 1), "ms_per_step": round(s2 * 1e3, 4),
                                            "hip_graph_images_per_s": round(b / s3, 1),
                                            "hip_graph_ms_per_step": round(s3 * 1e3, 4),
                                            "one_launch_ms_per_step": round(s4 * 1e3, 4),
                                            "one_launch_images_per_s": round(b / s4, 1),
                                            "one_launch_TOPs": round(b * m2.flops_per_image() / s4 / 1e12, 2),
                                            "one_launch_algorithmic_MB": round(algo / 1e6, 3),
                                            # the step is one kernel: the model's arithmetic over its launch time, HIP events
                                            # on the launch stream, against the int8 MFMA peak (neither roofline binds a
                                            # 25 MOP model of 16..64-channel layers: the figure says how far away they are)
                                            "roofline": {"bound": "mfma", "kernel": "qmodel_u8_kernel",
                                                         "achieved": round(b * m2.flops_per_image() / s4 / 1e12, 2),
                                                         "peak": round(PEAK_MFMA_I8 / 1e12, 1), "unit": "TOP/s",
                                                         "frac": round(b * m2.flops_per_image() / s4 / PEAK_MFMA_I8, 4),
                                                         "traffic": None, "launches_per_step": 1,
                                                         "avg_launch_ms": round(s4 * 1e3, 5),
                                                         "algorithmic_per_launch": {"GOP": round(b * m2.flops_per_image() / 1e9, 3),
                                                                                    "MB": round(algo / 1e6, 3)}},
                                            "layers": layer_table(m2, b, ms2)}
            log("%s batch %d: layer by layer %.4f ms/step %.0f images/s | HIP graph %.4f ms/step | ONE LAUNCH %.4f ms/step "
                "%.0f images/s" % (name, b, s2 * 1e3, b / s2, s3 * 1e3, s4 * 1e3, b / s4))
            e2.close()
            del e2
        torch.cuda.empty_cache()
        # the other float32 configurations: whole models and the single-layer sweep at C = 256, 56x56
        others = [(models.tiny_yolo_v2(), 16), (models.dscnn(), 1), (models.dscnn(), 64)]
        others += [(m, b) for b in (1, 64) for m in models.layer_sweep()]
        for m2, b in others:
            e2 = models.HipExecutor(m2, b)
            k2, w2 = counts_for(e2.forward, args)
            s2 = time_forward(e2, k2, w2)
            ms2 = time_ops(e2, 10)
            tab = layer_table(m2, b, ms2)
            if b > 1:
                add_floor_column(tab, stream_floors(e2, 5))
            extras["%s_b%d" % (m2.name, b)] = {"images_per_s": round(b / s2, 1), "ms_per_step": round(s2 * 1e3, 4),
                                               "layers": tab}
            if m2.name == "dscnn":
                # the whole model in one launch (small_hip_fmodel_forward: a workgroup per image, activations in LDS)
                e2.build_one_launch()
                k4, w4 = counts_for(e2.forward_one_launch, args, 50)
                s4 = time_forward_one_launch(e2, k4, w4)
                extras["%s_b%d" % (m2.name, b)].update({"one_launch_ms_per_step": round(s4 * 1e3, 4),
                                                        "one_launch_images_per_s": round(b / s4, 1),
                                                        "one_launch_TFLOPs": round(b * m2.flops_per_image() / s4 / 1e12, 3)})
                log("%s batch %d: ONE LAUNCH %.4f ms/step %.0f images/s" % (m2.name, b, s4 * 1e3, b / s4))
                e2.close()
            if len(m2.ops) == 1:
                log("%-20s batch %2d: %.4f ms  %.0f images/s  %s %.1f%% of roofline%s" % (
                    m2.name, b, tab[0]["ms"], b / (tab[0]["ms"] * 1e-3), tab[0]["bound"],
                    100 * (tab[0]["roofline_frac"] or 0),
                    "   bytes-only kernel %.4f ms" % tab[0]["stream_floor_ms"] if "stream_floor_ms" in tab[0] else ""))
            else:
                log("%s batch %d: %.4f ms/step %.0f images/s" % (m2.name, b, s2 * 1e3, b / s2))
                for r in tab:
                    log("  %-28s %9.4f ms  %-4s %6.1f%%%s" % (r["layer"], r["ms"], r["bound"], 100 * (r["roofline_frac"] or 0),
                                                             "   bytes-only kernel %.4f ms" % r["stream_floor_ms"]
                                                             if "stream_floor_ms" in r else ""))
            del e2
            torch.cuda.empty_cache()

        extras["layout"] = {"layers": layout_rows(capi.load(), torch, args.steps, args.warmup)}

    cpu = None
    if not args.no_cpu:
        try:
            if model.dtype == "f32" and model.name != "dscnn":   # the reference cannot run the 10x4 stem
                x1 = models.make_input(model, 1)
                cpu, cpu_ms = cpu_reference_model(model, weights, x1)
                add_cpu_column(table, cpu_ms, batch)
            if cpu is None:
                cpu = cpu_port_u8(model) if model.dtype == "u8" else None
            if not args.no_extras and args.model == "mobilenet_v1":
                extras["resnet8_u8_cpu"] = cpu_port_u8(models.resnet8_u8())
                extras["dscnn_cpu"] = cpu_port_u8(models.dscnn())
                # reference CPU build beside the other float32 configurations (bounded samples)
                for m2 in [models.tiny_yolo_v2()] + models.layer_sweep():
                    w2 = models.make_weights(m2)
                    c2, ms2 = cpu_reference_model(m2, w2, models.make_input(m2, 1), budget_s=3.0, max_passes=8)
                    if c2 is None:
                        continue
                    extras["%s_cpu" % m2.name] = c2
                    for key, e in extras.items():
                        if key.startswith(m2.name + "_b") and "layers" in e:
                            add_cpu_column(e["layers"], ms2, int(key.rsplit("_b", 1)[1]))
                    log("%s on the reference ZEN2 build, %d threads: %.2f images/s" % (m2.name, c2["cores"], c2["value"]))
        except Exception as e:            # the baseline leg must not take the GPU numbers down
            log("cpu baseline failed: %r" % (e,))

    out = {
        "metric": "images/s @batch%d %s %s" % (batch, model.name, "fp32" if model.dtype == "f32" else "u8"),
        "value": round(ips, 2), "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if model.dtype == "f32" else "u8", "data": "synthetic",
        "config": {"workload": "%s forward, batch %d, %dx%dx%d input, %s" % (
            model.name, batch, model.in_shape[1], model.in_shape[2], model.in_shape[0],
            "whole model in one launch" if one_launch else
            "Conv2D+bias+activation fused" if not args.unfused else "unfused layer calls"),
            "batch": batch, "GFLOP_per_image": round(model.flops_per_image() / 1e9, 4),
            "before_warmup": (("the process's first `warmup` + `steps` passes (summary.fresh_process_ms_per_step), machine "
                               "calibration (MFMA probe, device copy), " if calib else "") +
                              "the per-layer pass (%d passes with an event after every launch); then `warmup` untimed and "
                              "`steps` timed forward passes" % layer_passes)},
        "roofline": roof,
        "cpu_baseline": cpu,
        "layers": table,
        "extras": extras,
    }
    emit(out, "%s_b%d" % (model.name, batch))


if __name__ == "__main__":
    main()
