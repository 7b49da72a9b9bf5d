#!/usr/bin/env python3
"""Benchmark of the deepRacin CNN layer path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload vgg16|squeezenet|vgg_conv3|fire|conv3x3]

A step is one dR_apply (one batch-1 forward pass) over a synthetic input that is already resident in
the feed node's HBM buffer.  Prints ONE JSON line:

  metric/value  batch-1 images/s through dR_apply (K passes enqueued back to back, one final sync)
  roofline      dominant kernel of the workload (the fused Winograd MFMA conv for the VGG workloads):
                achieved = direct-equivalent FLOPs of its launches in one pass / their summed device
                time, measured with HIP events on the graph's own stream in a separate instrumented
                region of the same length: with profilingGPU set, the library attaches a start and a
                stop event to every kernel launch (hipExtLaunchKernelGGL), so a launch's span is the
                kernel alone, as in a rocprofv3 kernel trace.  (Events in the timed region itself
                would cost a few percent.)  peak = 157.3 TFLOP/s dense fp32 MFMA.  traffic = HBM bytes
                per launch from rocprofv3 FETCH_SIZE / WRITE_SIZE counter runs (a constant copied
                from the committed profile summary, null where none was taken)
  roofline_fc   the same for the FC GEMVs against the 8 TB/s HBM peak
  cpu_baseline  the CPU oracle (a scalar C restatement of the reference kernels, OpenMP over the host
                cores) on the same network and input; reported, not a target
  secondary     the other network of the headline metric (SqueezeNet v1.1 when the workload is VGG16
                and vice versa): images/s through dR_apply, same protocol

The other workloads of the configuration list are parity-test cases; they can be timed with
--workload.  This script drives exactly one GPU.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_MFMA_F32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch of the dominant kernel from `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE`
# runs of this script, scaled by what the same counters read for a copy of known size; the
# commands and the per-layer figures are in profiles/.  Keyed by (workload, kernel group).
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = {
    ("vgg16", "winograd"): 24935.9 * 1024,      # profiles/vgg16_hbm_traffic.md: fetch 263 376 + write 60 784 KiB over 13 launches
    ("vgg16", "fc"): 167699.2 * 1024,         # fetch 501 560 + write 1 533 KiB over 3 launches
}


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


KERNEL_NAMES = {"winograd": "winograd_f23_mfma_kernel", "conv1x1": "conv1x1_mfma_kernel", "direct": "conv_direct_kernel"}


def measure(workload, seed, steps, warmup, instrument=True):
    """Build the graph, time `steps` passes, optionally run the instrumented region.  Returns a dict."""
    import numpy as np
    import deepracin_amd as dr
    from deepracin_amd import configs

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
    t0 = time.perf_counter()
    for _ in range(steps):
        lib.dR_apply(g.ptr)
    sync()
    elapsed = time.perf_counter() - t0
    res = {"spec": spec, "feeds": feeds, "flops": flops, "shapes": shapes,
           "ms_per_step": elapsed * 1e3 / steps, "images_per_s": steps / elapsed,
           "launch_graph": bool(dr.graph_struct(g).drGraphExec)}

    # wall-clock rate including the blocking feed (H2D over PCIe) and logits download each step
    feed_idx, feed_arr = next(iter(feeds.items()))
    n_e2e = max(steps // 4, 5)
    t0 = time.perf_counter()
    for _ in range(n_e2e):
        configs.feed_chw(nodes[feed_idx], feed_arr)
        lib.dR_apply(g.ptr)
        configs.fetch_chw(g)
    res["e2e_ms"] = (time.perf_counter() - t0) * 1e3 / n_e2e

    if instrument:
        # instrumented region: hipEvents between nodes on the graph's stream
        cfg = dr.graph_config(g)
        cfg.profilingGPU = 1
        per_node = np.zeros(len(spec))
        with _QuietStdout():
            for _ in range(3):
                lib.dR_apply(g.ptr)
            for _ in range(steps):
                lib.dR_apply(g.ptr)
                for i, n in enumerate(nodes):
                    per_node[i] += dr.node_struct(n).drLastKernelMs
        cfg.profilingGPU = 0
        res["per_node"] = per_node / steps
    env.close()
    return res


def calibrate_copy(lib, dr):
    """4 device-to-device copies of 64 Mi floats: 256 MiB read and 256 MiB written per launch."""
    import ctypes
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="vgg16", choices=["vgg16", "squeezenet", "vgg_conv3", "fire", "conv3x3"])
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true", help="skip the second network of the headline metric")
    ap.add_argument("--layers", action="store_true", help="also print a per-layer table to stderr")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="before the workload, run 4 plain copies of 256 MiB (copy3d_kernel): under rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE their known traffic gives the scale of the counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py drives exactly one GPU (batch-1 inference has no multi-GPU path); got --gpus %d" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import deepracin_amd as dr

    lib = dr.load_library()
    if lib.drhip_device_count() <= 0:
        print("bench.py: no HIP device visible; the hot path has no CPU fallback", file=sys.stderr)
        sys.exit(1)

    if args.calibrate_copy:
        calibrate_copy(lib, dr)
    m = measure(args.workload, args.seed, args.steps, args.warmup)
    spec, feeds, flops, shapes = m["spec"], m["feeds"], m["flops"], m["shapes"]
    per_node = m["per_node"]

    groups = {}
    for i in range(len(spec)):
        if spec[i]["op"] == "feed":
            continue
        k = kind_of(spec[i])
        gk = groups.setdefault(k, {"ms": 0.0, "flops": 0, "bytes": 0, "launches": 0})
        gk["ms"] += per_node[i]
        gk["flops"] += flops.get(i, 0)
        gk["launches"] += 1
        if k == "fc":
            K, N = spec[i]["w"].shape
            gk["bytes"] += 4 * (K * N + K + 2 * N)
    layers = []
    for i in range(len(spec)):
        if i in flops and per_node[i] > 0:
            layers.append({"node": i, "kind": kind_of(spec[i]), "out": list(shapes[i]), "ms": round(float(per_node[i]), 4),
                           "tflops": round(flops[i] / (per_node[i] * 1e-3) / 1e12, 2)})

    conv_kinds = [k for k in ("winograd", "conv1x1", "direct") if k in groups]
    dominant = max(conv_kinds, key=lambda k: groups[k]["ms"]) if conv_kinds else None
    roofline = None
    if dominant:
        gk = groups[dominant]
        ach = gk["flops"] / (gk["ms"] * 1e-3) / 1e12
        roofline = {"kernel": KERNEL_NAMES[dominant], "bound": "mfma", "achieved": round(ach, 3), "peak": PEAK_MFMA_F32_TFLOPS,
                    "unit": "TFLOP/s", "frac": round(ach / PEAK_MFMA_F32_TFLOPS, 4),
                    "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH.get((args.workload, dominant)),
                    "launches_per_step": gk["launches"], "avg_launch_ms": round(gk["ms"] / gk["launches"], 5),
                    "flops_per_launch": gk["flops"] / gk["launches"]}
    roofline_fc = None
    if "fc" in groups and groups["fc"]["ms"] > 0:
        gk = groups["fc"]
        ach = gk["bytes"] / (gk["ms"] * 1e-3) / 1e9
        roofline_fc = {"kernel": "fc_gemv_kernel", "bound": "hbm", "achieved": round(ach, 1), "peak": PEAK_HBM_GBS,
                       "unit": "GB/s", "frac": round(ach / PEAK_HBM_GBS, 4),
                       "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH.get((args.workload, "fc")),
                       "launches_per_step": gk["launches"], "avg_launch_ms": round(gk["ms"] / gk["launches"], 5),
                          "bytes_per_launch": gk["bytes"] / gk["launches"]}

    secondary = None
    other = {"vgg16": "squeezenet", "squeezenet": "vgg16"}.get(args.workload)
    if other and not args.no_secondary:
        m2 = measure(other, args.seed, args.steps, args.warmup, instrument=False)
        secondary = {"workload": other, "value": round(m2["images_per_s"], 2), "unit": "images/s",
                     "ms_per_step": round(m2["ms_per_step"], 4),
                     "e2e_ms_per_step_with_feed_and_download": round(m2["e2e_ms"], 4)}

    cpu_baseline = None
    if not args.no_cpu_baseline:
        from oracle import oracle
        oracle.load()
        oracle.run_spec(spec, feeds)                     # warm-up (page-in, thread pool)
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or (time.perf_counter() - t0 < 10.0 and reps < 200):
            oracle.run_spec(spec, feeds)
            reps += 1
        cpu_s = (time.perf_counter() - t0) / reps
        cpu_baseline = {"value": round(1.0 / cpu_s, 4), "unit": "images/s", "cores": oracle.num_threads(), "kind": "port",
                        "sample": "%d full %s forward passes of the scalar-C oracle (same weights and input), OpenMP" % (reps, args.workload)}

    if args.layers:
        for l in layers:
            print("node %3d %-8s out %-18s %8.4f ms %7.2f TFLOP/s" % (l["node"], l["kind"], l["out"], l["ms"], l["tflops"]), file=sys.stderr)
        for k, gk in groups.items():
            print("%-9s %2d launches %8.4f ms" % (k, gk["launches"], gk["ms"]), file=sys.stderr)

    line = {
        "metric": "batch-1 images/s %s fp32 through dR_apply" % args.workload,
        "value": round(m["images_per_s"], 2),
        "unit": "images/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(m["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": args.workload, "batch": 1, "input": list(spec[0]["shape"]), "seed": args.seed,
                   "nodes": len(spec), "conv_gflop": round(sum(v for i, v in flops.items() if spec[i]["op"] == "conv") / 1e9, 3),
                   "launch_graph": m["launch_graph"]},
        "roofline": roofline,
        "roofline_fc": roofline_fc,
        "cpu_baseline": cpu_baseline,
        "secondary": secondary,
        "kernel_ms_per_step": round(float(per_node.sum()), 4),
        "e2e_ms_per_step_with_feed_and_download": round(m["e2e_ms"], 4),
        "groups": {k: {"ms": round(v["ms"], 4), "launches": v["launches"],
                       "tflops": round(v["flops"] / (v["ms"] * 1e-3) / 1e12, 2) if v["ms"] > 0 and v["flops"] else None}
                   for k, v in groups.items()},
        "layers": layers,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
