#!/usr/bin/env python3
"""Benchmark of the sparse-convolution hot path on one MI355X.

A step is one pass of the 120k-voxel fp16 VoxelNet sparse backbone (BASELINE
config 3): 8 rulebooks + 13 convolutions through the C ABI, inputs resident in
HBM.  Prints ONE JSON line: latency per step (the whole backbone captured in a
HIP graph and replayed), effective TFLOP/s, the roofline of the dominant
kernel (timed with HIP events on the launch stream in an eager pass) and the
CPU baseline (the oracle on the host cores, one bounded pass).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "sparse backbone latency ms + effective TFLOP/s, 120k voxels fp16, 1×MI355X"
PEAK_FP16_TFLOPS = 2500.0   # MI355X dense fp16 MFMA
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch of the roofline kernel at the default 120 000 voxels, from two `rocprofv3 --pmc` runs of this
# script (FETCH_SIZE 33873, WRITE_SIZE 32768 per dispatch), each scaled by what the same counter read for the
# 256 MiB copy of --pmc-copy-mib (FETCH_SIZE reads half the copied KiB: factor 2.0; WRITE_SIZE factor 1.0).
MEASURED_TRAFFIC_BYTES = {("conv3", 120000): int((33911 * 2.0 + 32768 * 1.0) * 1024)}


def cpu_baseline(cfg, threads):
    """One pass of the same workload through the CPU oracle (fp32 accumulation on fp16-rounded operands)."""
    import numpy as np
    from oracle import oracle

    def r16(a):
        return np.asarray(a, dtype=np.float32).astype(np.float16).astype(np.float32)

    feats, coords, grid = r16(cfg["feats"]), cfg["coords"], list(cfg["grid"])
    rulebooks = {}
    t_rb = t_conv = 0.0
    for spec, (w, b) in zip(cfg["layers"], cfg["weights"]):
        n = len(coords)
        rb = rulebooks.get(spec["key"])
        if rb is None:
            t0 = time.perf_counter()
            if spec["subm"]:
                rb = oracle.rulebook(coords, n, [1] + grid, spec["ksize"], spec["stride"], spec["padding"],
                                     spec["dilation"], n, True)
                rb.update(out_coors=coords, num_act_out=n, out_grid=grid)
            else:
                og = oracle.out_shape(grid, spec["ksize"], spec["stride"], spec["padding"], spec["dilation"])
                rb = oracle.rulebook(coords, n, [1] + og, spec["ksize"], spec["stride"], spec["padding"],
                                     spec["dilation"], 8 * n, False)
                rb["out_coors"] = rb["out_coors"][:rb["num_act_out"]].copy()
                rb["out_grid"] = og
            t_rb += time.perf_counter() - t0
            rulebooks[spec["key"]] = rb
        t0 = time.perf_counter()
        y = oracle.conv(feats, r16(w), r16(b), rb["index"], rb["num_index"], rb["num_act_out"], acc="f32",
                        threads=threads)
        if spec.get("relu"):
            y = np.maximum(y, 0)
        feats = r16(y)
        t_conv += time.perf_counter() - t0
        coords, grid = rb["out_coors"], rb["out_grid"]
    return t_rb, t_conv


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--voxels", type=int, default=120000)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="time eager enqueues instead of HIP-graph replays")
    ap.add_argument("--no-overlap", action="store_true",
                    help="enqueue rulebooks and convolutions on one stream instead of two")
    ap.add_argument("--pmc-copy-mib", type=int, default=0,
                    help="end with ONE device-to-device copy of this many MiB: the dispatch of known size that scales "
                         "the FETCH_SIZE / WRITE_SIZE counters of a `rocprofv3 --pmc` run of this script")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the sparse backbone is a single-GPU inference path); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import deploy3d_amd
    from deploy3d_amd import layers, synth

    deploy3d_amd.load_library()  # raises if the HIP library is missing: no fallback
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    cfg = synth.config3(args.voxels)
    specs, weights = cfg["layers"], cfg["weights"]
    n = len(cfg["coords"])
    counts = layers.measure_output_counts(specs, cfg["coords"], cfg["grid"])
    caps = layers.plan_capacities(specs, n, counts)
    net = layers.SparseBackbone(specs, weights, caps, overlap=not args.no_overlap)
    x = layers.make_input(cfg["coords"], cfg["feats"], cfg["grid"])

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(max(1, args.warmup)):
            y = net.forward(x)
        stream.synchronize()
        ref_out = y.feats.clone()

        # pairs per rulebook -> algorithmic FLOPs
        pairs = {}
        for key, rb in net.rulebooks.items():
            ni = int(rb.num_index.item())
            pairs[key] = int((rb.index[2, :ni] >= 0).sum().item())
        layer_flops = [2.0 * pairs[s["key"]] * s["cin"] * s["cout"] for s in specs]
        total_flops = float(sum(layer_flops))

        # ---- eager pass with HIP events on the launch stream: per-layer times ----
        k_eager = max(3, min(args.steps, 20))
        ev = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in specs]
              for _ in range(k_eager)]
        stream.synchronize()
        t0 = time.perf_counter()
        for it in range(k_eager):
            rulebooks = {}
            cur = x
            for li, (spec, lyr) in enumerate(zip(specs, net.layers)):
                if spec["key"] not in rulebooks:
                    rulebooks[spec["key"]] = lyr.build_rulebook(cur)
                ev[it][li][0].record(stream)
                cur = lyr.forward(cur, rulebooks)
                ev[it][li][1].record(stream)
        stream.synchronize()
        eager_ms = (time.perf_counter() - t0) * 1e3 / k_eager
        layer_ms = [float(np.mean([ev[it][li][0].elapsed_time(ev[it][li][1]) for it in range(k_eager)]))
                    for li in range(len(specs))]

        # ---- timed region: K steps ----
        if args.no_graph:
            stream.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                y = net.forward(x)
            stream.synchronize()
            ms = (time.perf_counter() - t0) * 1e3 / args.steps
            mode = "eager" + ("" if args.no_overlap else ", rulebooks beside convolutions on two side streams")
        else:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                y = net.forward(x)
            for _ in range(2):
                graph.replay()
            stream.synchronize()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                graph.replay()
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) * 1e3 / args.steps
            mode = "hip-graph replay" + ("" if args.no_overlap else ", rulebooks beside convolutions on two side streams")
        same = bool(torch.equal(y.feats, ref_out))
        if args.pmc_copy_mib:
            src = torch.ones(args.pmc_copy_mib << 20, dtype=torch.uint8, device="cuda")
            dst = torch.empty_like(src)
            stream.synchronize()
            dst.copy_(src)
            stream.synchronize()

    # dominant kernel: the convolution with the largest event time among layers that reuse a cached
    # neighbour table (their enqueue launches exactly one kernel)
    first_of_key = {}
    for li, s in enumerate(specs):
        first_of_key.setdefault(s["key"], li)
    single = [li for li, s in enumerate(specs) if first_of_key[s["key"]] != li]
    dom = max(single, key=lambda li: layer_ms[li])
    dspec = specs[dom]
    achieved = layer_flops[dom] / (layer_ms[dom] * 1e-3) / 1e12
    roofline = {
        "kernel": "convStaged<fp16,%d,%d> (layer %s)" % (dspec["cin"], dspec["cout"], dspec["name"]),
        "bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
        "frac": round(achieved / PEAK_FP16_TFLOPS, 4),
        "traffic": MEASURED_TRAFFIC_BYTES.get((dspec["name"][:5], args.voxels)),
        "flops_per_launch": layer_flops[dom], "avg_launch_ms": round(layer_ms[dom], 4),
    }

    out = {
        "metric": METRIC, "value": round(ms, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "fp16", "data": "synthetic",
        "config": {"workload": "config 3: VoxelNet sparse backbone, %d voxels, grid [41,1440,1440], "
                               "8 rulebooks + 13 convs, fp16 storage / fp32 accumulate" % n,
                   "mode": mode, "stage_voxels": counts, "capacities": caps},
        "effective_tflops": round(total_flops / (ms * 1e-3) / 1e12, 2),
        "total_gflop": round(total_flops / 1e9, 2),
        "eager_ms_per_step": round(eager_ms, 4),
        "outputs_match_warmup": same,
        "layer_ms": {s["name"]: round(t, 4) for s, t in zip(specs, layer_ms)},
        "roofline": roofline,
    }

    if not args.no_cpu_baseline:
        threads = min(16, os.cpu_count() or 1)
        t_rb, t_conv = cpu_baseline(cfg, threads)
        out["cpu_baseline"] = {
            "value": round((t_rb + t_conv) * 1e3, 1), "unit": "ms", "cores": threads, "kind": "port",
            "sample": "one full pass of the same workload through the CPU oracle: 8 rulebooks (serial, %.0f ms) + "
                      "13 convolutions (OpenMP, %d threads, %.0f ms)" % (t_rb * 1e3, threads, t_conv * 1e3),
        }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
