#!/usr/bin/env python3
"""Benchmark of the deepRacin CNN layer path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload vgg16|squeezenet|vgg_conv3|fire|conv3x3]
    python bench.py --summarise DIR [DIR ...]       # tables from rocprofv3 output directories (see below)

A step is one dR_apply (one batch-1 forward pass) over a synthetic input that is already resident in
the feed node's HBM buffer.  W untimed warm-up passes, then BLOCKS blocks of exactly K passes, each block
enqueued back to back and closed by one synchronisation; `ms_per_step` is the MEDIAN block / K (one block
of 20 passes is a few milliseconds long and a single sample of it says little), `ms_per_step_min` /
`_max` are the fastest and slowest block.  Prints ONE JSON line:

  metric/value   batch-1 images/s through dR_apply = 1000 / ms_per_step
  roofline       the dominant kernel of the workload (the fused Winograd MFMA convolution for the VGG
                 workloads).  `achieved` = direct-equivalent FLOPs (2*9*H*W*I*O per layer, the
                 algorithmic work) of its launches in one pass / their summed device time; `frac` =
                 achieved / 157.3 TFLOP/s.  Winograd F(2x2,3x3) issues 2.25x fewer multiplications than
                 that, so `frac` is credit for the algorithm, NOT matrix-pipe utilisation: that is
                 `issued_tflops` (the FLOPs the kernel really issues, 2*16*tiles*I*O with tiles, I and O
                 padded to its blocks -- the counter SQ_INSTS_VALU_MFMA_MOPS_F32 reads exactly this, see
                 profiles/) and `mfma_busy_frac` = issued_tflops / 157.3, the share of the data-sheet
                 matrix peak the pipe was issuing at; the >= 50 % target is judged on `mfma_busy_frac`.
                 `mfma_busy_frac_counters` is the same share from SQ_VALU_MFMA_BUSY_CYCLES of the
                 committed rocprofv3 run (profiles/counters.json: busy cycles per SIMD / (this run's device
                 time x 2.4 GHz)), `mfma_busy_frac_profiled` the share over the profiler's own, longer,
                 kernel durations; null when there is no such run (or when profiles/counters.json was written for
                 other kernel sources).  `mfma_stream_clock_mhz` = the shader clock under a stream of fp32 MFMAs,
                 measured in this run (drhip_mfma_clock_probe): the data-sheet peak assumes 2400 MHz, so
                 `mfma_busy_frac_at_stream_clock` = mfma_busy_frac x 2400 / that clock is the share of the matrix
                 cycles the part really offers under such load.  Device
                 times come from HIP events on the graph's own stream in a separate instrumented region:
                 with profilingGPU set the library attaches a start and a stop event to every kernel
                 launch, so a launch's span is the kernel alone, as in a rocprofv3 kernel trace.
                 `traffic` = HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE runs recorded in
                 profiles/counters.json (null when that file has no entry for the workload)
  roofline_fc    the same for the FC GEMVs against the 8 TB/s HBM peak, with one row per layer
  layers         per layer: device time, direct-equivalent TFLOP/s, for Winograd layers issued TFLOP/s
  cpu_baseline   the CPU oracle (a scalar C restatement of the reference kernels, OpenMP over the host
                 cores) on the same network and input; reported, not a target.  `pocl` says whether the
                 reference's own OpenCL kernels could run on the host cores through a CPU OpenCL runtime
                 (they cannot on these boxes: the probe's finding is reported)
  secondary      the other network of the headline metric (SqueezeNet v1.1 when the workload is VGG16
                 and vice versa), measured the same way, with its own layers and roofline
  configs        the three small configurations of the benchmark list (single 3x3 layer as Winograd and
                 as direct convolution, fire module, VGG16 conv3 block): time, layers, CPU oracle time

This script drives exactly one GPU.

--summarise turns rocprofv3 output into the tables kept under profiles/: a directory with a
*_results.db (from --kernel-trace --stats) gives the per-kernel duration table; directories with
*_counter_collection.csv (from --pmc) give per-dispatch counter tables of the last forward pass --
FETCH_SIZE and WRITE_SIZE scaled by what the same run read for the plain 256 MiB copies of
--calibrate-copy, the matrix-core counters as issued FLOPs and busy share per Winograd launch -- and
`--counters-json FILE` stores the figures bench.py reports (`traffic`, `mfma_busy_frac_counters`).
"""
import argparse
import collections
import csv
import ctypes
import glob
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_MFMA_F32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
PEAK_CLOCK_GHZ = 2.4            # the clock the data-sheet peak is quoted at
COUNTERS_JSON = os.path.join(ROOT, "profiles", "counters.json")
BLOCKS = 25


class _QuietStdout:
    """Silences the library's printf output (profiling lines) at the file-descriptor level."""

    def __enter__(self):
        sys.stdout.flush()
        self._saved = os.dup(1)
        self._null = os.open(os.devnull, os.O_WRONLY)
        os.dup2(self._null, 1)

    def __exit__(self, *exc):
        os.dup2(self._saved, 1)
        os.close(self._null)
        os.close(self._saved)


def kind_of(node):
    if node["op"] == "conv":
        _, _, kh, kw = node["w"].shape
        s = tuple(node.get("stride", (1, 1)))
        if kh == 3 and kw == 3 and s == (1, 1) and os.environ.get("DR_CONV3X3") != "direct":
            return "winograd"
        return "conv1x1" if (kh == 1 and kw == 1 and s == (1, 1)) else "direct"
    return node["op"]


KERNEL_NAMES = {"winograd": "winograd_f23_mfma_kernel", "conv1x1": "conv1x1_mfma_kernel", "direct": "conv3x3_direct_mfma_kernel"}


def winograd_issued_flops(lib, W, H, I, O):
    """FLOPs the Winograd kernel issues for a layer: 16 GEMMs over tiles x I x O, each padded to the blocks of
    the variant the scheduler picks (tile blocks of 32 or 16, 8 input channels per stage, 32/64/128 or 16/32/64
    output channels per workgroup); drhip_conv3x3_winograd_f32 decides the same way."""
    v = lib.drhip_conv3x3_winograd_pick_variant(W, H, I, O)
    tb = 16 if v & 0x100 else 32
    ob = tb * {1: 1, 2: 2, 3: 4}[v & 0xf]
    tiles = ((W + 1) // 2) * ((H + 1) // 2)
    pad = lambda n, m: -(-n // m) * m
    # (an image layer -- at most 4 input channels, 32-tile blocks, unsplit, four waves -- runs its one stage without
    # the two k-steps that would multiply zeros)
    few = I <= 4 and tb == 32 and (v & 0xf) <= 2 and not (v & 0x400) and not (v >> 4) & 0xf
    return 2 * 16 * pad(tiles, tb) * (4 if few else pad(I, 8)) * pad(O, ob)


def measure(workload, seed, steps, warmup, blocks=BLOCKS, instrument=True, env_vars=None):
    """Build the graph, time `blocks` blocks of `steps` passes, optionally run the instrumented region."""
    import numpy as np
    import deepracin_amd as dr
    from deepracin_amd import configs

    old = {k: os.environ.get(k) for k in (env_vars or {})}
    os.environ.update(env_vars or {})
    try:
        lib = dr.load_library()
        spec, feeds, outs = configs.CONFIGS[workload](seed=seed)
        flops, shapes = configs.flops(spec)

        env = dr.Environment()
        g = env.create_graph()
        nodes = configs.build_graph(g, spec, outs)
        dr.prepare(g)
        for i, a in feeds.items():
            configs.feed_chw(nodes[i], a)

        def sync():
            # dR_downloadArray is the API's synchronisation point; 4 bytes are enough
            buf = np.empty(1, np.float32)
            mem = (dr.c_void_p * max(g.num_outputs, 1))()
            lib.dR_getOutputBuffers(g.ptr, mem)
            lib.dR_downloadArray(g.ptr, b"", mem[0], 0, 4, buf.ctypes.data_as(dr.c_void_p))

        for _ in range(warmup):
            assert lib.dR_apply(g.ptr)
        sync()
        block_ms = []
        for _ in range(blocks):
            t0 = time.perf_counter()
            for _ in range(steps):
                lib.dR_apply(g.ptr)
            sync()
            block_ms.append((time.perf_counter() - t0) * 1e3 / steps)
        res = {"spec": spec, "feeds": feeds, "flops": flops, "shapes": shapes, "outs": outs,
               "ms_per_step": statistics.median(block_ms), "ms_min": min(block_ms), "ms_max": max(block_ms),
               "launch_graph": bool(dr.graph_struct(g).drGraphExec)}

        # wall-clock rate of the loop the reference's users run: feed (H2D over PCIe), pass, download of the output
        # (the three C calls with buffers set up once, as a C caller has them: no array is created inside the loop)
        feed_idx, feed_arr = next(iter(feeds.items()))
        feed_arr = np.ascontiguousarray(feed_arr, np.float32)
        feed_ptr, feed_node = feed_arr.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), nodes[feed_idx].ptr
        mem = (dr.c_void_p * max(g.num_outputs, 1))()
        n_out = lib.dR_getOutputBuffers(g.ptr, mem)
        host = [np.empty(int(np.prod(g.outnodes[i].out_shape)), np.float32) for i in range(n_out)]
        host_ptr = [h.ctypes.data_as(dr.c_void_p) for h in host]

        def one_round():
            lib.dR_feedData(g.ptr, feed_node, feed_ptr, 0, feed_arr.size)
            lib.dR_apply(g.ptr)
            for i in range(n_out):
                lib.dR_downloadArray(g.ptr, b"output", mem[i], 0, host[i].nbytes, host_ptr[i])

        n_e2e = max(steps, 100)
        for _ in range(3):
            one_round()
        t0 = time.perf_counter()
        for _ in range(n_e2e):
            one_round()
        res["e2e_ms"] = (time.perf_counter() - t0) * 1e3 / n_e2e

        if instrument:
            cfg = dr.graph_config(g)
            cfg.profilingGPU = 1
            per_node = np.zeros(len(spec))
            n_inst = max(steps, 20)
            with _QuietStdout():
                for _ in range(3):
                    lib.dR_apply(g.ptr)
                for _ in range(n_inst):
                    lib.dR_apply(g.ptr)
                    for i, n in enumerate(nodes):
                        per_node[i] += dr.node_struct(n).drLastKernelMs
            cfg.profilingGPU = 0
            res["per_node"] = per_node / n_inst
        env.close()
        return res
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v


def analyse(lib, m, workload, counters):
    """Per-layer rows, kernel groups and the roofline blocks of one measured workload."""
    spec, flops, shapes, per_node = m["spec"], m["flops"], m["shapes"], m["per_node"]
    ms = [float(v) for v in per_node]
    # an expand 1x1 that rides in its 3x3 sibling's Winograd launch has no kernel of its own: its work is
    # credited to the launch that does it
    merged, joint_o = dict(flops), {}
    for i, n in enumerate(spec):
        if n["op"] == "conv" and kind_of(n) == "conv1x1" and ms[i] == 0.0:
            for j, o in enumerate(spec):
                if j != i and o["op"] == "conv" and kind_of(o) == "winograd" and o["in"] == n["in"] and ms[j] > 0.0:
                    merged[j] = merged.get(j, 0) + merged.pop(i, 0)
                    joint_o[j] = o["w"].shape[1] + n["w"].shape[1]      # the 1x1 channels travel as centre-tap 3x3 filters
                    break
    groups, layers = {}, []
    for i, n in enumerate(spec):
        if n["op"] == "feed":
            continue
        k = kind_of(n)
        gk = groups.setdefault(k, {"ms": 0.0, "flops": 0, "issued": 0, "bytes": 0, "launches": 0})
        gk["ms"] += ms[i]
        gk["flops"] += merged.get(i, 0)
        gk["launches"] += 1 if ms[i] > 0 else 0
        gk["kernels"] = gk.get("kernels", 0) + (1 if ms[i] > 0 else 0)
        row = None
        if i in merged and ms[i] > 0:
            row = {"node": i, "kind": k, "out": list(shapes[i]), "us": round(ms[i] * 1e3, 2),
                   "tflops": round(merged[i] / (ms[i] * 1e-3) / 1e12, 2)}
        if k == "winograd" and ms[i] > 0:
            W, H, _ = shapes[n["in"]]
            I, O = n["w"].shape[0], joint_o.get(i, n["w"].shape[1])
            issued = winograd_issued_flops(lib, W, H, I, O)
            gk["issued"] += issued
            v = lib.drhip_conv3x3_winograd_pick_variant(W, H, I, O)
            if (v >> 4) & 0xf and not v & 0x800:       # split layers whose partial tiles are summed by a second kernel
                gk["kernels"] += 1
            row["issued_tflops"] = round(issued / (ms[i] * 1e-3) / 1e12, 2)
            row["mfma_busy_frac"] = round(issued / (ms[i] * 1e-3) / 1e12 / PEAK_MFMA_F32_TFLOPS, 4)
        if k == "fc" and ms[i] > 0:
            K, N = n["w"].shape
            b = 4 * (K * N + K + 2 * N)
            gk["bytes"] += b
            row["gbs"] = round(b / (ms[i] * 1e-3) / 1e9, 1)
            row["hbm_frac"] = round(b / (ms[i] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)
        if row:
            layers.append(row)

    conv_kinds = [k for k in ("winograd", "conv1x1", "direct") if k in groups and groups[k]["ms"] > 0]
    dominant = max(conv_kinds, key=lambda k: groups[k]["ms"]) if conv_kinds else None
    roofline = None
    if dominant:
        gk = groups[dominant]
        ach = gk["flops"] / (gk["ms"] * 1e-3) / 1e12
        rec = (counters.get(workload) or {}).get(dominant) or {}
        roofline = {"kernel": KERNEL_NAMES[dominant], "bound": "mfma", "achieved": round(ach, 3), "peak": PEAK_MFMA_F32_TFLOPS,
                    "unit": "TFLOP/s", "frac": round(ach / PEAK_MFMA_F32_TFLOPS, 4),
                    "frac_is": "direct-equivalent FLOPs / peak (algorithmic credit)",
                    "traffic": rec.get("traffic_bytes_per_launch"),
                    "launches_per_step": gk["launches"], "avg_launch_ms": round(gk["ms"] / max(gk["launches"], 1), 5),
                    "flops_per_launch": gk["flops"] / max(gk["launches"], 1)}
        if dominant == "winograd":
            issued = gk["issued"] / (gk["ms"] * 1e-3) / 1e12
            # counters of the committed rocprofv3 run: busy cycles per SIMD over THIS run's device time (the profiler's own
            # timestamps run ~10 % long), and the share under the profiler itself
            cyc = rec.get("mfma_busy_cycles_per_simd")
            roofline.update({"issued_tflops": round(issued, 3), "frac_issued": round(issued / PEAK_MFMA_F32_TFLOPS, 4),
                             "mfma_busy_frac": round(issued / PEAK_MFMA_F32_TFLOPS, 4),
                             "mfma_busy_frac_counters": round(cyc / (gk["ms"] * 1e3 * PEAK_CLOCK_GHZ * 1e3), 4) if cyc else None,
                             "mfma_busy_frac_profiled": rec.get("mfma_busy_frac"),
                             "target": "mfma_busy_frac >= 0.50"})
        if rec.get("measured"):
            roofline["counters_measured"] = rec["measured"]
    roofline_fc = None
    if "fc" in groups and groups["fc"]["ms"] > 0:
        gk = groups["fc"]
        ach = gk["bytes"] / (gk["ms"] * 1e-3) / 1e9
        rec = (counters.get(workload) or {}).get("fc") or {}
        roofline_fc = {"kernel": "fc_gemv_kernel", "bound": "hbm", "achieved": round(ach, 1), "peak": PEAK_HBM_GBS,
                       "unit": "GB/s", "frac": round(ach / PEAK_HBM_GBS, 4), "traffic": rec.get("traffic_bytes_per_launch"),
                       "launches_per_step": gk["launches"], "avg_launch_ms": round(gk["ms"] / gk["launches"], 5),
                       "bytes_per_launch": gk["bytes"] / gk["launches"],
                       "layers": [{"node": l["node"], "us": l["us"], "gbs": l["gbs"], "frac": l["hbm_frac"]} for l in layers if l["kind"] == "fc"]}
    out_groups = {k: {"ms": round(v["ms"], 4), "launches": v["launches"], "kernels": v.get("kernels", 0),
                      "tflops": round(v["flops"] / (v["ms"] * 1e-3) / 1e12, 2) if v["ms"] > 0 and v["flops"] else None}
                  for k, v in groups.items()}
    return layers, out_groups, roofline, roofline_fc


def kernel_sources_sha1():
    """Hash over the device sources (csrc/device): identifies the kernels a profile was taken on."""
    import hashlib
    h = hashlib.sha1()
    d = os.path.join(ROOT, "deepracin_amd", "csrc", "device")
    for f in sorted(os.listdir(d)):
        if f.endswith((".hip", ".hpp")):
            h.update(f.encode())
            h.update(open(os.path.join(d, f), "rb").read())
    return h.hexdigest()


def compact_roofline(r):
    """The roofline block without its explanatory strings (for the one-line summary)."""
    if not r:
        return r
    keep = ("kernel", "bound", "achieved", "peak", "unit", "frac", "frac_issued", "traffic", "mfma_busy_frac_counters",
            "mfma_busy_frac_profiled", "mfma_stream_clock_mhz", "mfma_busy_frac_at_stream_clock", "launches_per_step", "avg_launch_ms")
    return {k: r[k] for k in keep if k in r}


def probe_pocl():
    """Could the reference's own OpenCL kernels run on the host cores?  Needs an OpenCL device of type CPU (PoCL)
    and a checkout of the reference (DR_REFERENCE_DIR).  Nothing is installed or downloaded; this only looks."""
    ref = os.environ.get("DR_REFERENCE_DIR")
    have_ref = bool(ref) and os.path.isdir(os.path.join(ref, "Kernels"))
    try:
        cl = ctypes.CDLL("libOpenCL.so.1")
    except OSError:
        return "unavailable (no OpenCL loader: libOpenCL.so.1 not found%s)" % ("" if have_ref else "; no reference checkout at DR_REFERENCE_DIR")
    n = ctypes.c_uint(0)
    if cl.clGetPlatformIDs(0, None, ctypes.byref(n)) != 0 or n.value == 0:
        return "unavailable (OpenCL loader present, 0 platforms%s)" % ("" if have_ref else "; no reference checkout at DR_REFERENCE_DIR")
    plats = (ctypes.c_void_p * n.value)()
    cl.clGetPlatformIDs(n.value, plats, None)
    cpu_devices = 0
    for p in plats:
        k = ctypes.c_uint(0)
        if cl.clGetDeviceIDs(ctypes.c_void_p(p), ctypes.c_ulong(2), 0, None, ctypes.byref(k)) == 0:   # CL_DEVICE_TYPE_CPU
            cpu_devices += k.value
    if cpu_devices == 0:
        return "unavailable (%d OpenCL platform(s), 0 devices of type CPU: no PoCL on this machine%s)" % (
            n.value, "" if have_ref else "; no reference checkout at DR_REFERENCE_DIR")
    if not have_ref:
        return "unavailable (a CPU OpenCL device exists, but no reference checkout at DR_REFERENCE_DIR: only this repository travels to the GPU box)"
    return "unavailable (CPU OpenCL device and reference checkout found, but building the reference needs glib and cmake, which this harness does not drive)"


def time_oracle(spec, feeds, budget_s, min_reps=3, max_reps=200):
    from oracle import oracle
    oracle.load()
    oracle.run_spec(spec, feeds)                     # warm-up (page-in, thread pool)
    reps, t0 = 0, time.perf_counter()
    while reps < min_reps or (time.perf_counter() - t0 < budget_s and reps < max_reps):
        oracle.run_spec(spec, feeds)
        reps += 1
    return (time.perf_counter() - t0) / reps, reps, oracle.num_threads()


def calibrate_copy(lib, dr):
    """4 device-to-device copies of 64 Mi floats: 256 MiB read and 256 MiB written per launch."""
    n = 64 << 20
    info = dr.DeviceInfo()
    assert lib.drhip_init(0, info) == 0
    src, dst = ctypes.c_void_p(), ctypes.c_void_p()
    assert lib.drhip_malloc(ctypes.byref(src), 4 * n) == 0 and lib.drhip_malloc(ctypes.byref(dst), 4 * n) == 0
    assert lib.drhip_fill_f32(src, 1.0, n, None) == 0
    for _ in range(4):
        assert lib.drhip_copy3d_f32(src, 8192, 8192, 0, 0, 0, dst, 8192, 8192, 0, 0, 0, 8192, 8192, 1, None) == 0
    assert lib.drhip_stream_sync(None) == 0
    lib.drhip_free(src)
    lib.drhip_free(dst)


# ---------------------------------------------------------------------------------------------------------
# --summarise: rocprofv3 output -> the tables of profiles/
# ---------------------------------------------------------------------------------------------------------

def _short(name):
    return name.split("(")[0].replace("void ", "").replace("drhip::", "")


def _last_pass(rows, last=0):
    """Dispatches of the last complete forward pass: those after the second-to-last softmax launch up to the last
    one; for workloads without a softmax the trailing `last` dispatches (all of them when `last` is 0), the
    runtime's own copy kernels (a synchronous read-back at the end of the run) not counted."""
    rows = [r for r in rows if not r["kernel"].startswith("__amd_rocclr")]
    ends = [i for i, r in enumerate(rows) if "softmax" in r["kernel"]]
    if len(ends) >= 2 and not last:
        return rows[ends[-2] + 1: ends[-1] + 1]
    return rows[-last:] if last else rows


def _load_counters(path):
    """{counter: [ {dispatch, kernel, grid, value, start, end} in dispatch order ]} of one counter_collection.csv."""
    per = collections.OrderedDict()
    for r in csv.DictReader(open(path)):
        d = per.setdefault(r["Counter_Name"], collections.OrderedDict())
        k = int(r["Dispatch_Id"])
        if k in d:
            d[k]["value"] += float(r["Counter_Value"])      # one row per XCD / shader engine on some builds
        else:
            d[k] = {"dispatch": k, "kernel": _short(r["Kernel_Name"]), "grid": int(r["Grid_Size"]), "value": float(r["Counter_Value"]),
                    "start": int(r["Start_Timestamp"]), "end": int(r["End_Timestamp"])}
    return {c: list(d.values()) for c, d in per.items()}


def summarise(dirs, workload, counters_json, last=0):
    import sqlite3
    fetch = write = mfma = None
    record = {}
    for d in dirs:
        for db in sorted(glob.glob(os.path.join(d, "**", "*_results.db"), recursive=True)):
            c = sqlite3.connect(db)
            rows = list(c.execute("select name,total_calls,total_duration,average,percentage from top_kernels"))
            print("rocprofv3 kernel-trace statistics of %s (durations in microseconds):\n" % os.path.relpath(db, ROOT))
            print("| kernel | calls | avg us | total us | % |")
            print("|---|---:|---:|---:|---:|")
            for n, calls, tot, avg, pct in rows:
                print("| `%s` | %d | %.3f | %.1f | %.2f |" % (_short(n), calls, avg, tot, pct))
            print()
        for f in sorted(glob.glob(os.path.join(d, "**", "*_counter_collection.csv"), recursive=True)):
            per = _load_counters(f)
            if "FETCH_SIZE" in per:
                fetch = per["FETCH_SIZE"]
            if "WRITE_SIZE" in per:
                write = per["WRITE_SIZE"]
            if "SQ_INSTS_VALU_MFMA_MOPS_F32" in per:
                mfma = per
    if fetch and write:
        cf = [r["value"] for r in fetch if "copy3d" in r["kernel"]][1:]
        cw = [r["value"] for r in write if "copy3d" in r["kernel"]][1:]
        assert cf and cw, "no copy3d_kernel dispatches: run bench.py with --calibrate-copy under the profiler"
        kib = 256 * 1024
        sf, sw = kib / (sum(cf) / len(cf)), kib / (sum(cw) / len(cw))
        print("HBM traffic per dispatch of the last forward pass.  Calibration: the 256 MiB copies read FETCH_SIZE = %.0f and "
              "WRITE_SIZE = %.0f per launch, so one FETCH_SIZE unit is %.3f KiB and one WRITE_SIZE unit %.3f KiB.\n" % (
                  sum(cf) / len(cf), sum(cw) / len(cw), sf, sw))
        pf, pw = _last_pass(fetch, last), _last_pass(write, last)
        assert [r["kernel"] for r in pf] == [r["kernel"] for r in pw], "the two counter runs saw different passes"
        print("| kernel | grid (lanes) | fetch KiB | write KiB |")
        print("|---|---:|---:|---:|")
        tot = collections.OrderedDict()
        for a, b in zip(pf, pw):
            print("| `%s` | %d | %.1f | %.1f |" % (a["kernel"], a["grid"], a["value"] * sf, b["value"] * sw))
            t = tot.setdefault(a["kernel"], [0, 0.0, 0.0])
            t[0] += 1; t[1] += a["value"] * sf; t[2] += b["value"] * sw
        print("\n| kernel | launches | fetch KiB | write KiB | KiB per launch |")
        print("|---|---:|---:|---:|---:|")
        for k, (n, a, b) in tot.items():
            print("| `%s` | %d | %.1f | %.1f | %.1f |" % (k, n, a, b, (a + b) / n))
        print()
        for group, match in (("winograd", "winograd_f23"), ("fc", "fc_gemv"), ("conv1x1", "conv1x1_mfma"), ("direct", "direct_mfma")):
            sel = [(n, a, b) for k, (n, a, b) in tot.items() if match in k]
            if sel:
                n = sum(s[0] for s in sel)
                record.setdefault(group, {})["traffic_bytes_per_launch"] = round(sum(s[1] + s[2] for s in sel) * 1024 / n, 1)
    if mfma:
        mops = _last_pass(mfma["SQ_INSTS_VALU_MFMA_MOPS_F32"], last)
        busy = {r["dispatch"]: r["value"] for r in mfma.get("SQ_VALU_MFMA_BUSY_CYCLES", [])}
        print("Matrix-core counters of the launches of the last forward pass that issue MFMAs.  SQ_INSTS_VALU_MFMA_MOPS_F32 counts "
              "512 FLOP per unit; SQ_VALU_MFMA_BUSY_CYCLES is summed over the chip's 1024 SIMDs; `kernel us` is the dispatch's own "
              "End - Start timestamp under the profiler (longer than in a plain run); busy = busy cycles per SIMD / (kernel us x 2.4 GHz).\n")
        print("| # | kernel | grid (lanes) | MOPS | issued GFLOP | MFMA busy cycles/SIMD | kernel us | busy |")
        print("|---:|---|---:|---:|---:|---:|---:|---:|")
        families = (("winograd", "winograd_f23"), ("direct", "direct_mfma"), ("conv1x1", "conv1x1_mfma"), ("first_layer", "fewc"))
        tot = collections.OrderedDict()
        k = 0
        reduce_us = 0.0
        for r in mops:
            if r["value"] <= 0:
                if "winograd_split_reduce" in r["kernel"]:      # second kernel of a split layer: no MFMAs, but part of the node's time
                    reduce_us += (r["end"] - r["start"]) / 1e3
                continue
            k += 1
            us = (r["end"] - r["start"]) / 1e3
            b = busy.get(r["dispatch"], 0.0) / 1024.0
            fam = next((f for f, m in families if m in r["kernel"]), "other")
            t = tot.setdefault(fam, [0, 0.0, 0.0, 0.0])
            t[0] += 1; t[1] += b; t[2] += r["value"] * 512; t[3] += us
            print("| %d | `%s` | %d | %d | %.3f | %.0f | %.1f | %.1f %% |" % (k, r["kernel"], r["grid"], r["value"], r["value"] * 512 / 1e9, b, us,
                                                                         100.0 * b / (us * 1e3 * PEAK_CLOCK_GHZ)))
        print()
        if reduce_us and "winograd" in tot:
            print("The split layers' second kernels (winograd_split_reduce_kernel) add %.1f us to the Winograd nodes; the figure below includes them.\n" % reduce_us)
            tot["winograd"][3] += reduce_us
        for fam, (n, tb, tc, tt) in tot.items():
            print("%s: %d launches, %.3f GFLOP issued, %.0f busy cycles per SIMD in %.1f us under the profiler = %.1f %% of the cycles at 2.4 GHz." % (
                fam, n, tc / 1e9, tb, tt, 100.0 * tb / (tt * 1e3 * PEAK_CLOCK_GHZ)))
            rec = record.setdefault(fam, {})
            rec["mfma_busy_cycles_per_simd"] = round(tb, 1)
            rec["issued_gflop"] = round(tc / 1e9, 4)
            rec["profiled_us"] = round(tt, 2)
            rec["mfma_busy_frac"] = round(tb / (tt * 1e3 * PEAK_CLOCK_GHZ), 4)
        print()
    if counters_json and record:
        data = json.load(open(counters_json)) if os.path.exists(counters_json) else {}
        sha = kernel_sources_sha1()
        if data.get("kernel_sources_sha1") != sha:      # figures of other kernel sources do not mix with these
            data = {"kernel_sources_sha1": sha}
        entry = data.setdefault(workload, {})
        for g, rec in record.items():
            rec["measured"] = time.strftime("%Y-%m-%d")
            entry.setdefault(g, {}).update(rec)
        json.dump(data, open(counters_json, "w"), indent=1, sort_keys=True)
        print("figures stored in %s under \"%s\"" % (os.path.relpath(counters_json, ROOT), workload))


# ---------------------------------------------------------------------------------------------------------

def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--blocks", type=int, default=BLOCKS, help="timed blocks of --steps passes; the median block is reported")
    ap.add_argument("--workload", default="vgg16", choices=["vgg16", "squeezenet", "vgg_conv3", "fire", "conv3x3"])
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true", help="skip the second network of the headline metric")
    ap.add_argument("--no-configs", action="store_true", help="skip the three small configurations")
    ap.add_argument("--layers", action="store_true", help="also print a per-layer table to stderr")
    ap.add_argument("--no-clock-probe", action="store_true", help="skip the measurement of the shader clock under a stream of MFMAs (profile runs)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="before the workload, run 4 plain copies of 256 MiB (copy3d_kernel): under rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE their known traffic gives the scale of the counters")
    ap.add_argument("--summarise", nargs="+", metavar="DIR", help="print the profile tables of rocprofv3 output directories and exit")
    ap.add_argument("--counters-json", default=None, help="with --summarise: store traffic / MFMA busy figures in this file")
    ap.add_argument("--last", type=int, default=0, help="with --summarise: table the trailing N dispatches (workloads without a softmax)")
    args = ap.parse_args()
    if args.summarise:
        summarise(args.summarise, args.workload, args.counters_json, args.last)
        return
    if args.gpus != 1:
        print("bench.py drives exactly one GPU (batch-1 inference has no multi-GPU path); got --gpus %d" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import deepracin_amd as dr

    lib = dr.load_library()
    if lib.drhip_device_count() <= 0:
        print("bench.py: no HIP device visible; the hot path has no CPU fallback", file=sys.stderr)
        sys.exit(1)
    counters = json.load(open(COUNTERS_JSON)) if os.path.exists(COUNTERS_JSON) else {}
    # Counter figures belong to the kernels they were measured on: a file written for other kernel sources is not replayed.
    counters_stale = bool(counters) and counters.get("kernel_sources_sha1") != kernel_sources_sha1()
    if counters_stale:
        counters = {}

    if args.calibrate_copy:
        calibrate_copy(lib, dr)
    m = measure(args.workload, args.seed, args.steps, args.warmup, args.blocks)
    spec, feeds, flops = m["spec"], m["feeds"], m["flops"]
    layers, groups, roofline, roofline_fc = analyse(lib, m, args.workload, counters)

    # The data-sheet matrix peak is quoted at 2.4 GHz; under a stream of fp32 MFMAs the part runs slower (power).  The
    # clock of such a stream, measured now on this GPU, caps every utilisation figure against the data-sheet peak.
    mhz, probe_us = ctypes.c_float(0.0), ctypes.c_float(0.0)
    lib.drhip_mfma_clock_probe.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float), ctypes.c_void_p]
    if not args.no_clock_probe and lib.drhip_mfma_clock_probe(200, 500, ctypes.byref(mhz), ctypes.byref(probe_us), None) == 0 and mhz.value > 0 and roofline and "mfma_busy_frac" in roofline:
        roofline["mfma_stream_clock_mhz"] = round(mhz.value, 1)
        roofline["mfma_stream_probe_us"] = round(probe_us.value, 1)
        roofline["mfma_busy_frac_at_stream_clock"] = round(roofline["mfma_busy_frac"] * PEAK_CLOCK_GHZ * 1e3 / mhz.value, 4)

    secondary = None
    other = {"vgg16": "squeezenet", "squeezenet": "vgg16"}.get(args.workload)
    if other and not args.no_secondary:
        m2 = measure(other, args.seed, args.steps, args.warmup, args.blocks)
        l2, g2, r2, rfc2 = analyse(lib, m2, other, counters)
        secondary = {"workload": other, "value": round(1e3 / m2["ms_per_step"], 2), "unit": "images/s",
                     "ms_per_step": round(m2["ms_per_step"], 4), "ms_per_step_min": round(m2["ms_min"], 4), "ms_per_step_max": round(m2["ms_max"], 4),
                     "kernel_ms_per_step": round(float(m2["per_node"].sum()), 4),
                     "kernels_per_step": sum(v["kernels"] for v in g2.values()),
                     "e2e_ms_per_step_with_feed_and_download": round(m2["e2e_ms"], 4),
                     "conv_gflop": round(sum(v for i, v in m2["flops"].items() if m2["spec"][i]["op"] == "conv") / 1e9, 3),
                     "roofline": r2, "roofline_fc": rfc2, "groups": g2, "layers": l2}

    pocl = probe_pocl()
    configs_out = None
    if not args.no_configs and args.workload in ("vgg16", "squeezenet"):
        configs_out = {}
        for name, env_vars, label in (("conv3x3", None, "conv3x3.winograd"), ("conv3x3", {"DR_CONV3X3": "direct"}, "conv3x3.direct"),
                                      ("fire", None, "fire"), ("vgg_conv3", None, "vgg_conv3"), ("vgg_conv3", {"DR_CONV3X3": "direct"}, "vgg_conv3.direct")):
            old = os.environ.get("DR_CONV3X3")
            if env_vars:
                os.environ.update(env_vars)
            try:
                mc = measure(name, args.seed, args.steps, args.warmup, max(5, args.blocks // 5))
                lc, gc, rc, _ = analyse(lib, mc, name, counters)
            finally:
                if env_vars:
                    if old is None:
                        os.environ.pop("DR_CONV3X3", None)
                    else:
                        os.environ["DR_CONV3X3"] = old
            conv_flops = sum(v for i, v in mc["flops"].items() if mc["spec"][i]["op"] == "conv")
            kms = float(mc["per_node"].sum())
            blk = {"ms_per_step": round(mc["ms_per_step"], 4), "images_per_s": round(1e3 / mc["ms_per_step"], 1),
                   "gpu_kernels_ms": round(kms, 4), "gpu_ms_with_feed_and_download": round(mc["e2e_ms"], 4),
                   "conv_gflop": round(conv_flops / 1e9, 4),
                   "conv_tflops": round(conv_flops / (kms * 1e-3) / 1e12, 2), "frac_of_mfma_peak": round(conv_flops / (kms * 1e-3) / 1e12 / PEAK_MFMA_F32_TFLOPS, 4),
                   "roofline": rc, "layers": lc, "pocl_reference_ms": pocl}
            if not args.no_cpu_baseline and not env_vars:
                cpu_s, reps, cores = time_oracle(mc["spec"], mc["feeds"], 1.0)
                blk["cpu_oracle_ms"] = round(cpu_s * 1e3, 3)
                blk["cpu_cores"] = cores
            configs_out[label] = blk

    cpu_baseline = None
    if not args.no_cpu_baseline:
        cpu_s, reps, cores = time_oracle(spec, feeds, 10.0)
        cpu_baseline = {"value": round(1.0 / cpu_s, 4), "unit": "images/s", "cores": cores, "kind": "port",
                        "sample": "%d full %s forward passes of the scalar-C oracle (same weights and input), OpenMP" % (reps, args.workload),
                        "pocl": pocl}

    if args.layers:
        for l in layers:
            print("node %3d %-8s out %-18s %8.2f us %7.2f TFLOP/s%s" % (l["node"], l["kind"], l["out"], l["us"], l["tflops"],
                  "  issued %6.2f (busy %.3f)" % (l["issued_tflops"], l["mfma_busy_frac"]) if "issued_tflops" in l else ""), file=sys.stderr)
        for k, gk in groups.items():
            print("%-9s %2d launches %8.4f ms" % (k, gk["launches"], gk["ms"]), file=sys.stderr)

    e2e_ips = round(1e3 / m["e2e_ms"], 1)
    detail = {
        "workload": args.workload, "ms_per_step": round(m["ms_per_step"], 4), "timed_blocks": args.blocks,
        "kernel_ms_per_step": round(float(m["per_node"].sum()), 4),
        "kernels_per_step": sum(v["kernels"] for v in groups.values()),
        "roofline": roofline, "roofline_fc": roofline_fc, "groups": groups, "layers": layers,
        "secondary": secondary, "configs": configs_out, "pocl": pocl, "counters_stale": counters_stale,
    }
    # The tables go to stderr (one JSON document); stdout carries ONE short line with both networks of the metric.
    print("bench.py detail: " + json.dumps(detail), file=sys.stderr)
    sec_line = None
    if secondary:
        sec_line = {k: secondary[k] for k in ("workload", "value", "unit", "ms_per_step", "kernel_ms_per_step", "kernels_per_step")}
        sec_line["e2e_images_per_s"] = round(1e3 / secondary["e2e_ms_per_step_with_feed_and_download"], 1)
        sec_line["roofline"] = compact_roofline(secondary["roofline"])
    cfg_line = None
    if configs_out:
        cfg_line = {name: {"ms_per_step": c["ms_per_step"], "kernel_ms": c["gpu_kernels_ms"], "frac": c["frac_of_mfma_peak"],
                           "mfma_busy_frac": (c["roofline"] or {}).get("mfma_busy_frac")} for name, c in configs_out.items()}
    line = {
        "metric": "batch-1 images/s %s fp32 through dR_apply" % args.workload,
        "value": round(1e3 / m["ms_per_step"], 2),
        "unit": "images/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(m["ms_per_step"], 4),
        "ms_per_step_min": round(m["ms_min"], 4),
        "ms_per_step_max": round(m["ms_max"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": args.workload, "batch": 1, "input": list(spec[0]["shape"]), "seed": args.seed,
                   "nodes": len(spec), "conv_gflop": round(sum(v for i, v in flops.items() if spec[i]["op"] == "conv") / 1e9, 3),
                   "launch_graph": m["launch_graph"], "kernels_per_step": detail["kernels_per_step"],
                   "kernel_ms_per_step": detail["kernel_ms_per_step"],
                   "e2e_images_per_s": e2e_ips, "e2e_ms_per_step_with_feed_and_download": round(m["e2e_ms"], 4)},
        "roofline": compact_roofline(roofline),
        "roofline_fc": {k: v for k, v in roofline_fc.items() if k != "bytes_per_launch"} if roofline_fc else None,
        "cpu_baseline": cpu_baseline,
        "secondary": sec_line,
        "configs": cfg_line,
        "counters_stale": counters_stale,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
