#!/usr/bin/env python3
"""Benchmark of the darknet convolution forward path on one MI355X.

A step is one forward pass of the whole network over one batch of synthetic input that is
already resident in device memory (the layer loop the reference runs inside
forward_network_gpu, src/network.c:773-785, without the host<->device copies around it).
Default workload: yolov3 at 416x416, batch 64, fp32 - the configuration the headline metric is
quoted on.  Prints ONE JSON line on stdout; progress goes to stderr.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload yolov3-416|yolov3-608|yolov3-tiny-416|
                    yolov3-tiny-xnor-416|resnext50-224|yolov1-448|yolov1-tiny-448|sweep] [--batch B]
                    [--precision fp32|bf16x3|bf16] [--per-layer FILE] [--no-cpu]
Without --batch the default workload is measured at batch 64 (the line's `value`) and then at
batch 1 in the same process (the line's `batch1` object): the metric is quoted at both.
    python bench.py --post      (letterbox and detection decode + NMS latency instead of the forward pass)

The line carries, besides the driver's fields:
  roofline      the dominant kernel's algorithmic FLOP/s against the fp32 MFMA peak, from HIP
                events attached to each of its dispatches (the kernel's own start and end on
                the launch stream, what a profiler's kernel trace reports), over K more steps
                right after the timed ones; the same pass records an event after every layer
                for the per-layer table (the timed steps themselves carry no events: those
                cost a few microseconds each, 20% of a batch-1 pass)
  roofline      also carries, per network, the conv layer furthest below its own ceiling
                min(MFMA peak, arithmetic intensity x 8 TB/s); XNOR networks are priced against HBM
  cpu_baseline  the reference CPU path (compiled reference when oracle/_ref is present, else
                this repository's restatement, both -Ofast -fopenmp) timed on the host cores
                on a bounded sample of the same network
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_BF16_MFMA_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0
XNOR_CUS = 256
XNOR_CLOCK_HZ = 2.4e9

WORKLOADS = {
    "yolov3-416": ("yolov3", 416),
    "yolov3-608": ("yolov3", 608),
    "yolov3-tiny-416": ("yolov3_tiny", 416),
    "resnext50-224": ("resnext50", 224),
    "yolov3-tiny-xnor-416": ("yolov3_tiny_xnor", 416),
    "yolov1-448": ("yolov1", 448),
    "yolov1-tiny-448": ("yolov1_tiny", 448),
}


def cfg_generator(cfg_name):
    from darknet_amd import cfgs
    if cfg_name == "yolov3_tiny_xnor":       # binary=1 xnor=1 on every conv but the first and the last
        return lambda batch, size: cfgs.yolov3_tiny(batch, size, xnor=True)
    return getattr(cfgs, cfg_name)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def fill_params(setter, layers, seed=1000):
    """uniform(-1,1)*sqrt(2/(k*k*c/groups)) weights, biases 0, BN mean 0 / variance 1 / scale 1."""
    import numpy as np
    from darknet_amd import synth
    for i, L in enumerate(layers):
        if L["type"] == "local":         # one weight matrix per output location, one bias per output
            setter(i, synth.conv_weights(seed + i, L["out_h"] * L["out_w"] * L["n"], L["c"], L["size"]),
                   np.zeros(L["outputs"], np.float32), None, None, None)
            continue
        if L["type"] == "connected":
            setter(i, synth.conv_weights(seed + i, L["outputs"], L["inputs"], 1), np.zeros(L["outputs"], np.float32),
                   None, None, None)
            continue
        if L["type"] != "convolutional":
            continue
        w = synth.conv_weights(seed + i, L["n"], L["c"] // L["groups"], L["size"])
        b, s, m, v = synth.bn_identity(L["n"])
        if L["batch_normalize"]:
            setter(i, w, b, s, m, v)
        else:
            setter(i, w, b, None, None, None)


def layer_bytes(L):
    """Algorithmic HBM bytes of one layer for the whole batch (read operands once, write once)."""
    b = L["batch"]
    t = L["type"]
    if t == "convolutional":
        wbytes = 4 * L["nweights"] + (16 * L["n"] if L["batch_normalize"] else 4 * L["n"])
        return 4 * b * (L["inputs"] + L["outputs"]) + wbytes
    if t == "local":
        return 4 * b * (L["inputs"] + L["outputs"]) + 4 * (L["nweights"] + L["outputs"])
    if t == "connected":
        return 4 * b * (L["inputs"] + L["outputs"]) + 4 * (L["inputs"] * L["outputs"] + L["outputs"])
    if t == "maxpool":
        return 4 * b * (L["inputs"] + L["outputs"])  # inference leaves the argmax indexes out
    if t == "shortcut":
        add = min(L["c"], L["out_c"]) * min(L["h"], L["out_h"]) * min(L["w"], L["out_w"])
        return 4 * b * (2 * L["outputs"] + add)
    if t in ("route", "yolo", "softmax"):
        return 8 * b * L["outputs"]
    return 4 * b * (L["inputs"] + L["outputs"])


def profiled_traffic(workload, batch, kernel):
    """HBM bytes per launch of `kernel`, as measured by the committed rocprofv3 --pmc runs of this
    very command (profiles/bench_<workload>_b<batch>.md carries the figure and how it was scaled).
    Counters cannot be read from inside the process, so this is a constant read from that file, not
    a measurement of the present run: returns (bytes, "profiles/<file>"), or (None, None) when no
    such profile exists."""
    import re
    name = f"bench_{workload.replace('-', '_')}_b{batch}.md"
    try:
        text = open(os.path.join(ROOT, "profiles", name)).read()
    except OSError:
        return None, None
    m = re.search(r"traffic_bytes_per_launch\(" + re.escape(kernel) + r"\):\s*([0-9.]+)", text)
    return (float(m.group(1)), "profiles/" + name) if m else (None, None)


DATA_DEPENDENCE = ("fp32 MFMA on this part is power-limited: the clock it holds, and with it the fraction, depends "
                   "on how many operand bits toggle. Inside the network (activations decayed by the benchmark's "
                   "initialisation) the 3x3 256->512 @26x26 layer runs 0.71 ms at batch 64; alone on uniform(-1,1) "
                   "data (`--workload sweep`) the same layer takes 0.82 ms (79% against 89% of peak). The sweep "
                   "figure is the conservative one.")


def host_description():
    """nproc, physical cores and model string of the host the CPU baseline runs on."""
    info = {"nproc": os.cpu_count(), "physical_cores": None, "cpu_model": None}
    try:
        cores, phys, core = set(), None, None
        for line in open("/proc/cpuinfo"):
            key, _, val = line.partition(":")
            key, val = key.strip(), val.strip()
            if key == "model name" and not info["cpu_model"]:
                info["cpu_model"] = val
            elif key == "physical id":
                phys = val
            elif key == "core id":
                core = val
            elif not key and phys is not None:
                cores.add((phys, core))
                phys = core = None
        if phys is not None:
            cores.add((phys, core))
        info["physical_cores"] = len(cores) or None
    except OSError:
        pass
    try:
        info["cpus_allowed"] = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        pass
    return info


def cpu_baseline(kind_pref, cfg_name, size, budget_s=20.0):
    """Time the reference CPU path on a bounded sample: the same network at a small batch."""
    from darknet_amd import cfgs, synth
    from oracle import ref
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    gen = cfg_generator(cfg_name)
    if kind_pref == "reference" and ref.available("fast"):
        kind = "reference"

        def make(batch):
            text = gen(batch, size)
            with tempfile.NamedTemporaryFile("w", suffix=".cfg", delete=False) as f:
                f.write(text)
            # the reference prints its layer table to stderr; keep the bench's stderr readable
            devnull = os.open(os.devnull, os.O_WRONLY)
            saved = os.dup(2)
            os.dup2(devnull, 2)
            try:
                net = ref.RefNet(f.name, "fast")
            finally:
                os.dup2(saved, 2)
                os.close(devnull)
                os.close(saved)
                os.unlink(f.name)
            fill_params(net.set_conv, net.layers)
            return net, (lambda x: net.predict(x)), net.inputs
    else:
        kind = "port"
        from oracle.net import OracleNet

        def make(batch):
            net = OracleNet(gen(batch, size), fast=True)
            fill_params(net.set_conv, net.layers)
            return net, (lambda x: net.forward(x)), net.net["inputs"]

    # one image first to size the sample
    net, run, inputs = make(1)
    x = synth.uniform01(7, inputs)
    run(x)  # warm-up
    t0 = time.perf_counter()
    run(x)
    t1 = time.perf_counter() - t0
    batch = int(max(1, min(8, budget_s / 2 / max(t1, 1e-3))))
    reps = 2
    if batch > 1:
        net, run, inputs = make(batch)
        x = synth.uniform01(7, inputs * batch)
        run(x)
    t0 = time.perf_counter()
    for _ in range(reps):
        run(x)
    dt = (time.perf_counter() - t0) / reps
    return {"value": batch / dt, "unit": "images/s", "cores": threads, "kind": kind,
            "sample": f"{cfg_name}-{size} forward at batch {batch}, 1 warm-up + {reps} timed passes, "
                      f"-Ofast -fopenmp, OMP_NUM_THREADS={threads}, {dt:.3f} s/pass",
            **host_description()}


def cpu_baseline_sweep(kind_pref, budget_s=20.0):
    """The three single-layer shapes of the sweep on the reference CPU path (im2col + gemm_nn +
    batch-norm + leaky, src/convolutional_layer.c:445-485), one image each: GFLOP/s per layer."""
    from darknet_amd import cfgs, synth
    from oracle import ref
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    use_ref = kind_pref == "reference" and ref.available("fast")
    rows, spent = [], 0.0
    for name, (c, h, w, n, size, stride) in cfgs.SWEEP.items():
        text = cfgs.single_conv(1, c, h, w, n, size, stride, pad=1)
        if use_ref:
            with tempfile.NamedTemporaryFile("w", suffix=".cfg", delete=False) as f:
                f.write(text)
            devnull = os.open(os.devnull, os.O_WRONLY)
            saved = os.dup(2)
            os.dup2(devnull, 2)
            try:
                net = ref.RefNet(f.name, "fast")
            finally:
                os.dup2(saved, 2)
                os.close(devnull)
                os.close(saved)
                os.unlink(f.name)
            run, inputs = (lambda x, net=net: net.predict(x)), net.inputs
        else:
            from oracle.net import OracleNet
            net = OracleNet(text, fast=True)
            run, inputs = (lambda x, net=net: net.forward(x)), net.net["inputs"]
        fill_params(net.set_conv, net.layers)
        x = synth.uniform(7, inputs, -1, 1)
        run(x)
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or (time.perf_counter() - t0 < budget_s / 6 and reps < 50):
            run(x)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        spent += dt * reps
        out_hw = (h + 2 * (size // 2) - size) // stride + 1
        fl = 2.0 * n * size * size * c * out_hw * out_hw
        rows.append({"name": name, "ms": round(dt * 1e3, 3), "gflops": round(fl / dt / 1e9, 2), "passes": reps})
    mean = sum(r["gflops"] for r in rows) / len(rows)
    return {"value": round(mean / 1e3, 5), "unit": "TFLOP/s", "cores": threads,
            "kind": "reference" if use_ref else "port",
            "sample": f"the three sweep layers at batch 1, 1 warm-up + 3..50 timed passes each ({spent:.1f} s in all), "
                      f"-Ofast -fopenmp, OMP_NUM_THREADS={threads}; mean of the three layers' GFLOP/s",
            "layers": rows, **host_description()}


def post_bench(args):
    """--post: latency of the steps either side of the forward pass for one 416x416 yolov3 image -
    letterbox of a 1920x1080 frame into the network input and get_network_boxes + do_nms_sort on the
    three yolo heads - on the device, and the compiled reference's CPU functions on the same data
    (resize/letterbox_image, get_network_boxes, do_nms_sort).  Prints one JSON line of its own."""
    import ctypes as C
    import numpy as np
    from darknet_amd import api, cfgs, synth
    api.set_gpu(0)
    L = api._lib.load()
    text = cfgs.yolov3(1, 416)
    net = api.Network(cfg_text=text)
    fill_params(net.set_conv, net.layers)
    frame = synth.uniform01(3, 3 * 1080 * 1920).reshape(3, 1080, 1920)
    x = synth.uniform01(7, net.inputs)
    net.predict(x)
    heads = {i: net.layer_output(i) for i, Ly in enumerate(net.layers) if Ly["type"] == "yolo"}

    def timed(fn, reps):
        fn()
        L.hip_synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        L.hip_synchronize()
        return (time.perf_counter() - t0) * 1e3 / reps

    out = {"metric": "post-processing latency", "unit": "ms", "workload": "yolov3-416, one 1920x1080 frame", "gpu": {},
           "cpu_reference": {}}
    out["gpu"]["letterbox_1080p_into_input_ms"] = round(timed(lambda: net.letterbox_input(0, frame), 20), 4)
    obj = np.concatenate([h.reshape(3, 85, -1)[:, 4, :].ravel() for h in heads.values()])
    num = C.c_int(0)
    for want in (50, 500, 5000):
        thresh = float(np.sort(obj)[-want])
        def boxes():
            d = L.get_network_boxes_image(net.net, 0, 1920, 1080, thresh, 1, 0.45, C.byref(num))
            L.free_detections(d, num.value)
        ms = timed(boxes, 20)
        out["gpu"][f"boxes_nms_{want}_candidates_ms"] = round(ms, 4)
        out["gpu"][f"boxes_nms_{want}_candidates_kept"] = int(num.value)
    net.free()
    try:
        from oracle import ref
        if ref.available("fast"):
            with tempfile.NamedTemporaryFile("w", suffix=".cfg", delete=False) as f:
                f.write(text)
            devnull = os.open(os.devnull, os.O_WRONLY)
            saved = os.dup(2)
            os.dup2(devnull, 2)
            try:
                rnet = ref.RefNet(f.name, "fast")
            finally:
                os.dup2(saved, 2)
                os.close(devnull)
                os.close(saved)
                os.unlink(f.name)
            for i, h in heads.items():
                rnet.set_output(i, h)
            t0 = time.perf_counter()
            ref.letterbox_image(frame, 416, 416, "fast")
            out["cpu_reference"]["letterbox_1080p_ms"] = round((time.perf_counter() - t0) * 1e3, 3)
            for want in (50, 500, 5000):
                thresh = float(np.sort(obj)[-want])
                t0 = time.perf_counter()
                rows = rnet.get_boxes(1920, 1080, thresh, 1, 0.45)
                out["cpu_reference"][f"boxes_nms_{want}_candidates_ms"] = round((time.perf_counter() - t0) * 1e3, 3)
            out["cpu_reference"]["kind"] = "compiled reference, -Ofast -fopenmp"
    except Exception as e:  # the CPU leg is a comparison only
        log("cpu reference leg failed:", repr(e))
    print(json.dumps(out), flush=True)


def measure(L, api, synth, workload, batch, precision, steps, warmup, per_layer=""):
    """One workload at one batch size: the timed steps, then the same steps with events for the
    roofline and the per-layer table, then the PCIe-inclusive figure.  Returns the JSON fields."""
    import numpy as np
    cfg_name, size = WORKLOADS[workload]
    text = cfg_generator(cfg_name)(batch, size)
    dev = L.hip_device_name().decode()
    L.conv_set_precision({"fp32": 0, "bf16": 1, "bf16x3": 2}[precision])
    # bf16x3 issues six bf16 MFMAs per fp32-equivalent multiply-add: its algorithmic FLOPs are priced
    # against a sixth of the bf16 peak
    peak = {"fp32": PEAK_FP32_MFMA_TFLOPS, "bf16": PEAK_BF16_MFMA_TFLOPS,
            "bf16x3": PEAK_BF16_MFMA_TFLOPS / 6}[precision]
    net = api.Network(cfg_text=text)
    fill_params(net.set_conv, net.layers)
    x = synth.uniform01(7, net.inputs * net.batch)
    net.push_input(x)
    flops_img = net.conv_flops()

    for _ in range(warmup):
        net.forward_device()
    net.synchronize()

    # ---- timed region: K steps of the device-resident forward (what a caller runs), input already
    # in HBM, bracketed by HIP events on the launch stream and a synchronize on both sides
    ev0, ev1 = L.hip_event_create(), L.hip_event_create()
    net.synchronize()
    t0 = time.perf_counter()
    L.hip_event_record(ev0)
    for _ in range(steps):
        net.forward_device()
    L.hip_event_record(ev1)
    net.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    total_ms = L.hip_event_elapsed_ms(ev0, ev1)
    ms_per_step = max(total_ms, 0.0) / steps
    value = batch / (ms_per_step / 1e3)

    # ---- the same K steps again with a HIP event after every layer (same stream): per-kernel
    # launch durations for the roofline.  The extra events cost a few microseconds per layer, so
    # this pass is a little slower than the timed one; both figures are reported.
    layer_ms = np.zeros(net.n)
    kernel_ms = np.zeros(net.n)
    L.hip_event_record(ev0)
    for _ in range(steps):
        _, ms, kms = net.forward_profiled_kernels()
        layer_ms += np.asarray(ms)
        kernel_ms += np.asarray(kms)
    L.hip_event_record(ev1)
    net.synchronize()
    layer_ms /= steps
    kernel_ms /= steps          # -1 stays -1: a layer takes the same kernel every step
    ms_per_step_events = L.hip_event_elapsed_ms(ev0, ev1) / steps

    # ---- PCIe-inclusive figure (network_predict: H2D input + D2H yolo/last outputs), untimed extra
    t0 = time.perf_counter()
    for _ in range(2):
        net.predict(x)
    pcie_ms = (time.perf_counter() - t0) * 1e3 / 2
    # the same with the batch built in pinned host memory (hip_host_alloc): no staging memcpy
    xp = api.pinned_array(x.size)
    xp[:] = x
    net.predict(xp)
    t0 = time.perf_counter()
    for _ in range(2):
        net.predict(xp)
    pcie_pinned_ms = (time.perf_counter() - t0) * 1e3 / 2
    api.free_pinned_array(xp)
    del xp
    # the same work with the copies overlapped: network_predict_submit / _collect keep two batches in
    # flight, so the upload of batch n+1 and the download of batch n-1 run while batch n computes
    # (pageable input, as network_predict takes it; the outputs are the same bits)
    reps = 6 if batch > 1 else 40
    net.submit(x)
    net.collect(copy=False)
    t0 = time.perf_counter()
    net.submit(x)
    for _ in range(reps - 1):
        net.submit(x)
        net.collect(copy=False)
    net.collect(copy=False)
    pcie_pipelined_ms = (time.perf_counter() - t0) * 1e3 / reps

    # ---- per-layer accounting, grouped by kernel
    kernels = {}
    rows = []
    for i, Ly in enumerate(net.layers):
        ms = float(layer_ms[i])
        row = {"layer": i, "type": Ly["type"], "ms": ms, "bytes": layer_bytes(Ly)}
        if Ly["type"] == "convolutional":
            fl = 2.0 * Ly["n"] * Ly["size"] ** 2 * (Ly["c"] // Ly["groups"]) * Ly["out_h"] * Ly["out_w"] * Ly["batch"]
            name = ("xnor_conv_kernel" if Ly["xnor"] else
                    L.conv_kernel_name_geometry(Ly["batch"], Ly["c"], Ly["h"], Ly["w"], Ly["n"], Ly["groups"],
                                                Ly["size"], Ly["stride"], Ly["pad"]).decode())
            # what bounds the layer: the matrix cores, or HBM at its arithmetic intensity
            ceiling = min(peak, fl / row["bytes"] * PEAK_HBM_GBS / 1e3)
            tfl = fl / ms / 1e9 if ms > 0 else 0.0
            row.update(flops=fl, kernel=name, tflops=tfl, ceiling_tflops=ceiling,
                       frac_of_ceiling=tfl / ceiling if ceiling > 0 else 0.0,
                       shape=f'{Ly["size"]}x{Ly["size"]}/{Ly["stride"]} {Ly["c"]}->{Ly["n"]} @{Ly["w"]}x{Ly["h"]}')
            row["kernel_ms"] = float(kernel_ms[i])   # the main kernel alone; -1 = not stamped
            k = kernels.setdefault(name, {"ms": 0.0, "kernel_ms": 0.0, "stamped": 0, "flops": 0.0,
                                          "launches": 0, "bytes": 0.0})
            k["ms"] += ms
            if kernel_ms[i] > 0:
                k["kernel_ms"] += float(kernel_ms[i])
                k["stamped"] += 1
            k["flops"] += fl
            k["bytes"] += row["bytes"]
            k["launches"] += 1
        # a same-geometry shortcut, a yolo head or a 2x2 stride-2 maxpool right after a convolution can
        # run inside that convolution's kernel (the library says which do at the present fusion level):
        # its event interval is empty and its traffic belongs to the conv kernel
        row["fused"] = bool(L.network_layer_runs_fused(net.net, i))
        # a route of one source is a view of that source's buffer: no launch, no traffic
        view = Ly["type"] == "route" and len(Ly.get("input_layers", [])) == 1
        row["fused"] = row["fused"] or view
        row["gbs"] = row["bytes"] / ms / 1e6 if ms > 0 and not row["fused"] else 0.0
        if row["fused"] and not view:
            # the conv kernel reads the shortcut's second operand and writes the fused layer's output
            # beside its own (both layer outputs stay observable, as in the reference)
            # (a fused maxpool's input is the conv's own output: only its output is added)
            extra = 4 * Ly["batch"] * Ly["outputs"] * (2 if Ly["type"] == "shortcut" else 1)
            kernels[rows[i - 1]["kernel"]]["fused_bytes"] = kernels[rows[i - 1]["kernel"]].get("fused_bytes", 0.0) + extra
        rows.append(row)
    dom_name, dom = max(kernels.items(), key=lambda kv: kv[1]["ms"])
    # the kernel's own duration when every one of its launches was stamped; else (a kernel outside
    # the MFMA path) the interval between the events around its layers
    stamped = dom["stamped"] == dom["launches"]
    dom_ms = dom["kernel_ms"] if stamped else dom["ms"]
    conv_ms = sum(k["ms"] for k in kernels.values())
    conv_tflops = sum(k["flops"] for k in kernels.values()) / conv_ms / 1e9
    traffic, traffic_source = profiled_traffic(workload, batch, dom_name)
    common = {"kernel": dom_name, "launches_per_step": dom["launches"],
              "avg_launch_ms": round(dom_ms / dom["launches"], 4),
              "timing": "events on the kernel's dispatch" if stamped else "events between layers",
              "avg_layer_interval_ms": round(dom["ms"] / dom["launches"], 4),
              "traffic": traffic, "traffic_source": traffic_source,
              "algorithmic_bytes_per_launch": round((dom["bytes"] + dom.get("fused_bytes", 0.0)) / dom["launches"])}
    if dom_name == "xnor_conv_kernel":
        # Two ceilings, reported against whichever binds.  HBM: the activations stay fp32 in memory.
        # Bit-ops: one 32-bit word of XNOR + popcount stands for 32 multiply-adds (64 FLOPs of the
        # fp32 formulation) and costs two vector-ALU instructions (v_xor_b32, v_bcnt_u32_b32 with
        # accumulate); a CU issues 64 lanes per clock, so 32 words per clock per CU.
        gbs = dom["bytes"] / dom_ms / 1e6
        words_per_s = dom["flops"] / 64.0 / (dom_ms / 1e3)
        word_peak = 32.0 * XNOR_CUS * XNOR_CLOCK_HZ
        hbm_frac, bit_frac = gbs / PEAK_HBM_GBS, words_per_s / word_peak
        if hbm_frac >= bit_frac:
            roofline = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                        "frac": round(hbm_frac, 4)}
        else:
            roofline = {"bound": "valu-bitops", "achieved": round(words_per_s / 1e12, 3),
                        "peak": round(word_peak / 1e12, 3), "unit": "Tword/s (32 XNOR+popcount bits each)",
                        "frac": round(bit_frac, 4)}
        roofline.update(common)
        roofline.update({"hbm_gbs": round(gbs, 1), "hbm_frac": round(hbm_frac, 4),
                         "bitop_twords_per_s": round(words_per_s / 1e12, 3), "bitop_frac": round(bit_frac, 4),
                         "bitop_peak_note": "32 words/clk/CU (64 lanes, 2 instructions per word) x 256 CUs x 2.4 GHz",
                         "bytes_per_launch": dom["bytes"] / dom["launches"],
                         "kernel_family": "every instance of xnor_conv_kernel<ACT,SIZE,BITS> and "
                                          "xnor_conv_pool_kernel<ACT> (the variant that also writes the 2x2 maxpool "
                                          "and the next layer's sign bits), accounted as one kernel",
                         "equivalent_fp32_tflops": round(dom["flops"] / dom_ms / 1e9, 3)})
    else:
        achieved = dom["flops"] / dom_ms / 1e9  # TFLOP/s
        roofline = {"bound": "mfma", "achieved": round(achieved, 3), "peak": peak, "unit": "TFLOP/s",
                    "frac": round(achieved / peak, 4), **common,
                    "flops_per_launch": dom["flops"] / dom["launches"]}
        if precision == "fp32":
            roofline["data_dependence"] = DATA_DEPENDENCE
    if any(Ly["type"] == "convolutional" and Ly["xnor"] for Ly in net.layers):
        # equivalent fp32 FLOPs of bit-op layers over the fp32 MFMA peak is not a fraction of anything
        roofline["all_conv_equivalent_tflops"] = round(conv_tflops, 3)
    else:
        roofline["all_conv_tflops"] = round(conv_tflops, 3)
        roofline["all_conv_frac"] = round(conv_tflops / peak, 4)
    conv_rows = [r for r in rows if r["type"] == "convolutional" and r["ms"] > 0]
    if conv_rows:
        worst = min(conv_rows, key=lambda r: r["frac_of_ceiling"])
        roofline["min_conv_frac_of_ceiling"] = round(worst["frac_of_ceiling"], 4)
        roofline["min_conv_layer"] = f'{worst["layer"]}: {worst["shape"]}'

    if per_layer:
        with open(per_layer, "w") as f:
            json.dump({"device": dev, "workload": workload, "batch": batch,
                       "ms_per_step": ms_per_step, "layers": rows, "kernels": kernels}, f, indent=1)
        log("per-layer table written to", per_layer)
    memk = [r for r in rows if r["type"] != "convolutional" and not r["fused"] and r["ms"] > 0]
    mem = None
    if memk:
        mb = sum(r["bytes"] for r in memk)
        mm = sum(r["ms"] for r in memk)
        mem = {"ms_per_step": round(mm, 4), "gbs": round(mb / mm / 1e6, 1), "frac_of_hbm_peak": round(mb / mm / 1e6 / PEAK_HBM_GBS, 4)}
        log(f"[{workload} b{batch}] memory-bound layers: {mm:.3f} ms/step, {mb / mm / 1e6:.0f} GB/s "
            f"({mb / mm / 1e6 / PEAK_HBM_GBS:.1%} of HBM peak; {sum(r['fused'] for r in rows)} shortcuts "
            f"and yolo heads that run inside the preceding convolution and one-source routes, which are views, are not counted); conv layers {conv_ms:.3f} ms/step, "
            f"{conv_tflops:.1f} TFLOP/s")
    net.free()
    return {"value": round(value, 2), "ms_per_step": round(ms_per_step, 4), "batch": batch,
            "gflop_per_image": round(flops_img / 1e9, 3), "device": dev,
            "wall_ms_per_step": round(wall_ms / steps, 4),
            "ms_per_step_with_layer_events": round(ms_per_step_events, 4),
            "pcie_inclusive_ms_per_step": round(pcie_pipelined_ms, 3),
            "pcie_inclusive_images_per_s": round(batch / (pcie_pipelined_ms / 1e3), 2),
            "pcie_inclusive_note": "network_predict_submit/_collect, two batches in flight, pageable input; "
                                   "the synchronous network_predict is the _sync_ figure",
            "pcie_inclusive_sync_ms_per_step": round(pcie_ms, 3),
            "pcie_inclusive_sync_images_per_s": round(batch / (pcie_ms / 1e3), 2),
            "pcie_inclusive_pinned_input_ms_per_step": round(pcie_pinned_ms, 3),
            "memory_bound_layers": mem, "roofline": roofline}


def sweep_bench(args, L):
    """--workload sweep: the three single-layer shapes of the benchmark configurations (3x3 s1
    256->512 @26, 1x1 512->256 @52, 3x3 s2 128->256 @104, batch-norm + leaky) at batch 1 and 64,
    each timed alone through forward_convolutional_gpu.  One JSON line: `value` is the mean
    TFLOP/s of the three batch-64 layers, `layers` holds all six."""
    from darknet_amd import cfgs, layerbench
    rows = []
    for name, (c, h, w, n, size, stride) in cfgs.SWEEP.items():
        for batch in (1, 64):
            r = layerbench.time_layer(batch, c, h, w, n, size, stride, pad=size // 2 if size > 1 else 0,
                                      iters=max(args.steps, 20), warmup=max(args.warmup, 3))
            fl = 2.0 * n * size * size * c * batch * ((h + 2 * (size // 2) - size) // stride + 1) ** 2
            byts = r["algorithmic_gbs"] * r["ms"] * 1e6
            ceiling = min(PEAK_FP32_MFMA_TFLOPS, fl / byts * PEAK_HBM_GBS / 1e3)
            r.update(name=name, ceiling_tflops=round(ceiling, 1), frac_of_ceiling=round(r["tflops"] / ceiling, 4))
            rows.append(r)
            log(json.dumps(r))
    b64 = [r for r in rows if r["batch"] == 64]
    dom = max(b64, key=lambda r: r["ms"])
    mean = sum(r["tflops"] for r in b64) / len(b64)
    out = {"metric": "conv TFLOP/s, single-layer sweep (mean of the three batch-64 layers)", "value": round(mean, 2),
           "unit": "TFLOP/s", "n_gpus": 1, "steps": max(args.steps, 20), "warmup": max(args.warmup, 3),
           "ms_per_step": round(sum(r["ms"] for r in b64), 4), "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "single conv layer sweep, fp32, batch 1 and 64, BN + leaky, activations and weights "
                                  "uniform(-1,1)", "device": L.hip_device_name().decode()},
           "roofline": {"bound": "mfma", "achieved": dom["tflops"], "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                        "frac": round(dom["tflops"] / PEAK_FP32_MFMA_TFLOPS, 4), "traffic": None, "traffic_source": None,
                        "data_dependence": DATA_DEPENDENCE,
                        "kernel": dom["kernel"], "layer": dom["shape"], "avg_launch_ms": dom["ms"],
                        "timing": "events around the layer's launches"},
           "layers": rows}
    if not args.no_cpu:
        try:
            out["cpu_baseline"] = cpu_baseline_sweep(args.cpu_kind)
        except Exception as e:  # the CPU leg must not take the GPU result down with it
            log("cpu_baseline failed:", repr(e))
            out["cpu_baseline"] = None
    print(json.dumps(out), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="yolov3-416", choices=sorted(WORKLOADS) + ["sweep"])
    ap.add_argument("--batch", type=int, default=0,
                    help="default: 64, followed (for the default workload) by a batch-1 leg reported as `batch1`")
    ap.add_argument("--per-layer", default="")
    ap.add_argument("--precision", default="fp32", choices=["fp32", "bf16", "bf16x3"],
                    help="bf16: the tap-blocked MFMA kernels round their operands to bf16 (opt-in, not the "
                         "headline configuration; its error against fp32 is reported by the tests)")
    ap.add_argument("--fusion", type=int, default=1, choices=[0, 1, 2],
                    help="network_set_fusion: 0 layer by layer, 1 layer pairs in one launch with every layer's "
                         "output written (default), 2 lean (maps only a fused maxpool reads are not written)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--post", action="store_true",
                    help="time letterbox and detection decode + NMS around the forward pass instead")
    ap.add_argument("--cpu-kind", default="reference", choices=["reference", "port"])
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on one GPU only (the forward path has no exchange step: it shards "
            "by batch, every GPU running the same forward on its share of the images). Use --gpus 1.")
        sys.exit(2)

    if args.post:
        post_bench(args)
        return

    from darknet_amd import api, synth

    api.set_gpu(0)
    L = api._lib.load()
    log("device:", L.hip_device_name().decode())
    L.network_set_fusion(args.fusion)
    if args.workload == "sweep":
        sweep_bench(args, L)
        return

    # One plain copy of known size (256 MiB read + 256 MiB written): the yardstick that turns a
    # profiler's FETCH_SIZE / WRITE_SIZE readings for the conv kernel into bytes.
    cal = api.DeviceArray(n=64 << 20), api.DeviceArray(n=64 << 20)
    L.copy_gpu(64 << 20, cal[0].ptr, 1, cal[1].ptr, 1)
    L.hip_synchronize()
    del cal

    batch = args.batch or 64
    m = measure(L, api, synth, args.workload, batch, args.precision, args.steps, args.warmup, args.per_layer)
    # The metric is quoted at batch 64 and batch 1 (the reference's own `speed` loop runs at batch 1,
    # examples/darknet.c:116-134): the default run measures both in one process, batch 64 first.
    m1 = None
    if not args.batch and args.workload == "yolov3-416":
        m1 = measure(L, api, synth, args.workload, 1, args.precision, max(args.steps, 50), max(args.warmup, 10))

    cfg_name, size = WORKLOADS[args.workload]
    config = {"workload": f"{args.workload} forward, batch {batch}, {args.precision}, input uniform[0,1), "
                          f"weights uniform(-1,1)*sqrt(2/(k*k*c)), BN mean 0 var 1 scale 1",
              "fusion": args.fusion}
    config.update({k: m[k] for k in ("gflop_per_image", "device", "wall_ms_per_step", "ms_per_step_with_layer_events",
                                     "pcie_inclusive_ms_per_step", "pcie_inclusive_images_per_s",
                                     "pcie_inclusive_note", "pcie_inclusive_sync_ms_per_step",
                                     "pcie_inclusive_sync_images_per_s",
                                     "pcie_inclusive_pinned_input_ms_per_step", "memory_bound_layers")})
    out = {
        "metric": "images/sec", "value": m["value"], "unit": "images/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": m["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"fp32": "f32", "bf16": "bf16 operands, f32 accumulate and storage",
                  "bf16x3": "f32 emulated with three bf16 pieces per operand, f32 accumulate and storage"}[args.precision],
        "data": "synthetic", "config": config, "roofline": m["roofline"],
    }
    if m1:
        out["batch1"] = {"metric": "images/sec", "value": m1["value"], "unit": "images/s", "ms_per_step": m1["ms_per_step"],
                         "steps": max(args.steps, 50), "warmup": max(args.warmup, 10),
                         "workload": f"{args.workload} forward, batch 1, {args.precision}, same process, after the batch-64 leg",
                         "pcie_inclusive_ms_per_step": m1["pcie_inclusive_ms_per_step"],
                         "memory_bound_layers": m1["memory_bound_layers"], "roofline": m1["roofline"]}
    if not args.no_cpu:
        try:
            cb = cpu_baseline(args.cpu_kind, cfg_name, size)
            cb["gflops"] = round(cb["value"] * m["gflop_per_image"], 2)
            out["cpu_baseline"] = cb
        except Exception as e:  # the CPU leg must not take the GPU result down with it
            log("cpu_baseline failed:", repr(e))
            out["cpu_baseline"] = None
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
