#!/usr/bin/env python3
"""Benchmark of the sparse-convolution hot path on one MI355X.

A step is one pass of a BASELINE configuration through the C ABI with inputs resident in HBM; the default is
config 3, the 120k-voxel fp16 VoxelNet sparse backbone (8 rulebooks + 13 convolutions).  Prints ONE JSON line:
latency per step (the whole pass captured in a HIP graph and replayed) and effective TFLOP/s; per operator, the
device time measured with HIP events around graph replays of that operator alone, and from it the roofline of the
dominant kernel (`roofline`) and of every operator (`rooflines`: MFMA for the convolutions with 32 or more input
channels, HBM for the rulebook builds and the narrow convolutions); the peaks this GPU reaches on a dense MFMA loop
and a streaming copy (`measured_peak`); and the CPU baseline (the oracle on the host cores, with the final output
of the GPU pass checked against it).
"""
import argparse
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "sparse backbone latency ms + effective TFLOP/s, 120k voxels fp16, 1×MI355X"
PEAK_TFLOPS = {"float16": 2500.0, "bfloat16": 2500.0, "int8": 5000.0, "float32": 157.3}   # MI355X dense MFMA
PEAK_HBM_GBS = 8000.0
ELEM = {"float16": 2, "bfloat16": 2, "int8": 1, "float32": 4}
# HBM bytes per launch of the roofline kernel, from two `rocprofv3 --pmc` runs of this script at the default
# workload (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what the same counter read for the
# 256 MiB copy of --pmc-copy-mib (FETCH_SIZE reads half the copied KiB: factor 2.0; WRITE_SIZE factor 1.0).
# A cached reading: it belongs to the kernel and workload named here and is null for any other.
TRAFFIC_SOURCE = "profiles/config3_backbone_hbm_traffic_pmc.txt"
# conv3_0 / conv3_1 run the same kernel on the same rulebook: FETCH_SIZE 34792 and WRITE_SIZE 34050 per dispatch.
MEASURED_TRAFFIC = {(3, 120000, "conv3_0"): int((34792 * 2.0 + 34050 * 1.0) * 1024),
                    (3, 120000, "conv3_1"): int((34792 * 2.0 + 34050 * 1.0) * 1024)}
DEFAULT_VOXELS = {1: 20000, 2: 60000, 3: 120000, 4: 120000, 5: 250000}
WORKLOAD = {
    1: "config 1: one SubM 3x3x3 16->16, fp32, %d voxels uniform in grid [41,1600,1408]",
    2: "config 2: one strided SpConv 3x3x3 s2 32->64, fp16 storage / fp32 accumulate, %d voxels, grid [41,1440,1440]",
    3: "config 3: VoxelNet sparse backbone, %d voxels, grid [41,1440,1440], 8 rulebooks + 13 convs, "
       "fp16 storage / fp32 accumulate",
    4: "config 4: config 3 in int8 (per-channel weights, per-tensor activations calibrated on the fp16 pass), "
       "%d voxels, int32 accumulate",
    5: "config 5: Cylinder3D residual block + downsample, fp16, %d voxels, grid [480,360,32]",
}


def r_to(a, dtype):
    import numpy as np
    import torch
    t = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}[dtype]
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(t).float().numpy()


def cpu_pass(cfg, threads, rulebooks_out=None):
    """One pass of the workload through the CPU oracle (fp32 accumulation on storage-rounded operands; int32
    accumulation + the requantize rule for int8).  Returns (rulebook s, conv s, final coords, final features);
    ``rulebooks_out`` (a dict) receives the oracle's rulebook per indice key, with the coordinates it was built on."""
    import numpy as np
    from oracle import oracle
    dtype = cfg["dtype"]
    int8 = dtype == "int8"
    first = dict(feats=cfg["feats_q"] if int8 else r_to(cfg["feats"], dtype), coords=cfg["coords"],
                 grid=list(cfg["grid"]))
    outs = {"input": first}
    rulebooks = {}
    t_rb = t_conv = 0.0
    cur = first
    for spec, (w, b) in zip(cfg["layers"], cfg["weights"]):
        src = spec.get("src")
        if src is None:
            x = cur
        elif "+" in src:
            p, q = (outs[s] for s in src.split("+"))
            x = dict(feats=r_to(p["feats"] + q["feats"], dtype), coords=p["coords"], grid=p["grid"])
        else:
            x = outs[src]
        n = len(x["coords"])
        rb = rulebooks.get(spec["key"])
        if rb is None:
            t0 = time.perf_counter()
            if spec["subm"]:
                rb = oracle.rulebook(x["coords"], n, [1] + x["grid"], spec["ksize"], spec["stride"], spec["padding"],
                                     spec["dilation"], n, True)
                rb.update(out_coors=x["coords"], num_act_out=n, out_grid=x["grid"])
            else:
                og = oracle.out_shape(x["grid"], spec["ksize"], spec["stride"], spec["padding"], spec["dilation"])
                rb = oracle.rulebook(x["coords"], n, [1] + og, spec["ksize"], spec["stride"], spec["padding"],
                                     spec["dilation"], 8 * n, False)
                rb["out_coors"] = rb["out_coors"][:rb["num_act_out"]].copy()
                rb["out_grid"] = og
            t_rb += time.perf_counter() - t0
            rb["in_coors"] = x["coords"]
            rulebooks[spec["key"]] = rb
        t0 = time.perf_counter()
        if int8:
            w_q, s_w = oracle.quantize_weights(w)
            m, bq = oracle.requant_params(spec["s_in"], s_w, spec["s_out"], b)
            acc = oracle.conv_i8(x["feats"], w_q, rb["index"], rb["num_index"], rb["num_act_out"], threads=threads)
            y = oracle.requantize(acc, m, bq, bool(spec.get("relu")))
        else:
            y = oracle.conv(x["feats"], r_to(w, dtype), r_to(b, dtype), rb["index"], rb["num_index"],
                            rb["num_act_out"], acc="f32", threads=threads)
            if spec.get("relu"):
                y = np.maximum(y, 0)
            y = r_to(y, dtype)
        t_conv += time.perf_counter() - t0
        cur = dict(feats=y, coords=rb["out_coors"], grid=rb["out_grid"])
        outs[spec["name"]] = cur
    if rulebooks_out is not None:
        rulebooks_out.update(rulebooks)
    return t_rb, t_conv, cur["coords"], cur["feats"]


def cpu_baseline(cfg, gpu_coords, gpu_feats):
    """All host cores (median of 3 passes) and one thread (1 pass; 3 when a pass takes under 15 s), plus the check of
    the GPU pass's final output against the oracle's: same coordinates, features within the tolerance of the type."""
    import numpy as np
    cores = os.cpu_count() or 1
    runs = []
    for _ in range(3):
        t_rb, t_conv, coords, feats = cpu_pass(cfg, cores)
        runs.append((t_rb + t_conv, t_rb, t_conv))
    runs.sort()
    total, t_rb, t_conv = runs[1]
    single = [cpu_pass(cfg, 1)[:2]]
    if sum(single[0]) < 15.0:
        single += [cpu_pass(cfg, 1)[:2] for _ in range(2)]
    single_s = sorted(sum(s) for s in single)[len(single) // 2]
    # parity of the final output: rows matched by coordinate
    def by_coord(c, f):
        order = np.lexsort(np.asarray(c).T[::-1])
        return np.asarray(c)[order], np.asarray(f)[order]
    c_ref, f_ref = by_coord(coords, feats)
    c_gpu, f_gpu = by_coord(gpu_coords, gpu_feats)
    same_coords = c_ref.shape == c_gpu.shape and bool((c_ref == c_gpu).all())
    parity = {"coords_equal": same_coords}
    if same_coords:
        ref64 = f_ref.astype(np.float64)
        err = np.abs(f_gpu.astype(np.float64) - ref64)
        rms = float(np.sqrt(np.mean(ref64 ** 2))) if ref64.size else 0.0
        dtype = cfg["dtype"]
        # the oracle here accumulates in fp32 like the GPU, in another order: fp32 within 1e-4 relative (+ rms
        # floor) per element, 2-byte types within 2e-2 * rms, int8 exact
        if dtype == "float32":
            ok = bool((err <= 1e-4 * (np.abs(ref64) + rms)).all())
            tol = "1e-4 * (|ref| + rms) per element"
        else:
            bound = 0.0 if dtype == "int8" else 2e-2 * rms
            ok = bool(err.size == 0 or err.max() <= bound)
            tol = bound
        parity.update(max_abs_err=float(err.max()) if err.size else 0.0, rms=rms, tolerance=tol, within_tolerance=ok)
    return {
        "value": round(total * 1e3, 1), "unit": "ms", "cores": cores, "kind": "port",
        "one_thread_ms": round(single_s * 1e3, 1),
        "sample": "the full pass of the same workload through the CPU oracle: %d rulebooks (serial, %.0f ms) + %d "
                  "convolutions (OpenMP over output rows, %.0f ms); %d threads: median of 3 passes; 1 thread: "
                  "median of %d" % (len({s["key"] for s in cfg["layers"]}), t_rb * 1e3, len(cfg["layers"]),
                                    t_conv * 1e3, cores, len(single)),
        "gpu_output_vs_oracle": parity,
    }


def measured_peaks():
    """Runs the peaks program (dense MFMA loop, streaming copy) as a child process; None if it is not built."""
    exe = os.path.join(ROOT, "deploy3d_amd", "libs", "d3d_peaks")
    if not os.path.exists(exe):
        return None
    try:
        out = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, timeout=120, text=True)
        return json.loads(out.stdout.strip().splitlines()[-1]) if out.returncode == 0 else None
    except Exception:
        return None


def build_workload(config, voxels, layers_mod, synth, torch):
    """cfg, torch dtype, and the SparseBackbone + input of the configuration (capacities from a sizing pre-pass)."""
    np_dtype = {"float32": torch.float32, "float16": torch.float16, "int8": torch.int8}
    if config == 4:
        cfg3 = synth.config3(voxels)
        counts = layers_mod.measure_output_counts(cfg3["layers"], cfg3["coords"], cfg3["grid"])
        caps = layers_mod.plan_capacities(cfg3["layers"], len(cfg3["coords"]), counts)
        net3 = layers_mod.SparseBackbone(cfg3["layers"], cfg3["weights"], caps, overlap=False)
        net3.forward(layers_mod.make_input(cfg3["coords"], cfg3["feats"], cfg3["grid"]))
        torch.cuda.synchronize()
        acts = {"input": cfg3["feats"]}
        for s in cfg3["layers"]:
            o = net3.outputs[s["name"]]
            acts[s["name"]] = o.feats[:int(o.num_act.item())].float().cpu().numpy()
        del net3
        cfg = synth.config4(voxels, acts)
        feats = cfg["feats_q"]
    else:
        cfg = {1: synth.config1, 2: synth.config2, 3: synth.config3, 5: synth.config5}[config](voxels)
        feats = cfg["feats"]
        counts = layers_mod.measure_output_counts(cfg["layers"], cfg["coords"], cfg["grid"])
        caps = layers_mod.plan_capacities(cfg["layers"], len(cfg["coords"]), counts)
    dtype = np_dtype[cfg["dtype"]]
    return cfg, dtype, feats, counts, caps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=3, choices=[1, 2, 3, 4, 5],
                    help="BASELINE configuration; 3 (the default) is the one the metric is quoted on")
    ap.add_argument("--voxels", type=int, default=0, help="0 = the configuration's own size")
    ap.add_argument("--capacity-scale", type=float, default=1.0,
                    help="row capacities as a multiple of the live counts (1.0 = the counts rounded up to 1024)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-peaks", action="store_true", help="do not run the measured-peaks program")
    ap.add_argument("--no-graph", action="store_true", help="time eager enqueues instead of HIP-graph replays")
    ap.add_argument("--no-overlap", action="store_true",
                    help="enqueue rulebooks and convolutions on one stream instead of three")
    ap.add_argument("--no-fused", action="store_true", help="skip the second figure (index tensors unwritten)")
    ap.add_argument("--no-op-timing", action="store_true",
                    help="skip the per-operator graphs and the rooflines built on them (counter runs, where every "
                         "extra dispatch is profiled)")
    ap.add_argument("--pmc-copy-mib", type=int, default=0,
                    help="end with ONE device-to-device copy of this many MiB: the dispatch of known size that scales "
                         "the FETCH_SIZE / WRITE_SIZE counters of a `rocprofv3 --pmc` run of this script")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the sparse backbone is a single-GPU inference path); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    peaks = None if args.no_peaks else measured_peaks()

    import numpy as np
    import torch
    import deploy3d_amd
    from deploy3d_amd import layers, synth

    deploy3d_amd.load_library()  # raises if the HIP library is missing: no fallback
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    voxels = args.voxels or DEFAULT_VOXELS[args.config]
    cfg, dtype, feats, counts, caps = build_workload(args.config, voxels, layers, synth, torch)
    specs, weights = cfg["layers"], cfg["weights"]
    n = len(cfg["coords"])
    in_cap = n
    if args.capacity_scale != 1.0:  # head-room over the live counts: every kernel is launched at capacity
        counts_s = {k: int(v * args.capacity_scale) for k, v in counts.items()}
        in_cap = int(n * args.capacity_scale)
        caps = layers.plan_capacities(specs, in_cap, counts_s)
    net = layers.SparseBackbone(specs, weights, caps, dtype=dtype, overlap=not args.no_overlap)
    x = layers.make_input(cfg["coords"], feats, cfg["grid"], dtype=dtype, capacity=in_cap)

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(max(1, args.warmup)):
            y = net.forward(x)
        stream.synchronize()
        ref_out = y.feats.clone()

        # pairs per rulebook -> algorithmic FLOPs and bytes
        pairs, rows_in, rows_out = {}, {}, {}
        for key, rb in net.rulebooks.items():
            ni = int(rb.num_index.item())
            pairs[key] = int((rb.index[2, :ni] >= 0).sum().item())
            rows_in[key] = int(rb.num_act_in.item())
            rows_out[key] = int(rb.num_act_out.item())
        layer_flops = [2.0 * pairs[s["key"]] * s["cin"] * s["cout"] for s in specs]
        total_flops = float(sum(layer_flops))

        # ---- device time per operator: the operator alone, R enqueues captured in a graph, replayed between two
        # HIP events on the launch stream ----
        R, REPLAYS = 8, 3

        def op_ms(enqueue):
            enqueue()
            stream.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                for _ in range(R):
                    enqueue()
            g.replay()
            stream.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(REPLAYS):
                g.replay()
            e1.record(stream)
            stream.synchronize()
            return e0.elapsed_time(e1) / (R * REPLAYS)

        layer_ms, rulebook_ms = [], {}
        first_of_key = {}
        for li, (spec, lyr) in enumerate(zip(specs, net.layers)):
            if args.no_op_timing:
                break
            inp = net.inputs[spec["name"]]
            if spec["key"] not in first_of_key:
                first_of_key[spec["key"]] = li
                rulebook_ms[spec["key"]] = op_ms(lambda: lyr.build_rulebook(inp))
            layer_ms.append(op_ms(lambda: lyr.forward(inp, net.rulebooks)))

        # ---- timed region: K steps ----
        k_eager = max(3, min(args.steps, 20))
        stream.synchronize()
        t0 = time.perf_counter()
        for _ in range(k_eager):
            y = net.forward(x)
        stream.synchronize()
        torch.cuda.synchronize()
        eager_ms = (time.perf_counter() - t0) * 1e3 / k_eager
        streams = "" if args.no_overlap else ", rulebooks beside convolutions on two side streams"
        host_ms = None
        if args.no_graph:
            ms = eager_ms
            mode = "eager" + streams
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
            host_ms = (time.perf_counter() - t0) * 1e3 / args.steps   # host time of one hipGraphLaunch
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) * 1e3 / args.steps
            mode = "hip-graph replay" + streams
        same = bool(torch.equal(y.feats, ref_out))
        # second figure: the same pass by a runner that declares itself the only reader of the index tensors
        # (D3D_OPT_INDEX_UNUSED): rulebook operators write the tables their linked convolutions read and leave the
        # reference-format index tensors unwritten.  Not `value`: the operators' documented outputs are incomplete.
        fused = None
        if not args.no_graph and not args.no_fused:
            net2 = layers.SparseBackbone(specs, weights, caps, dtype=dtype, overlap=not args.no_overlap,
                                         index_tensors=False)
            for _ in range(2):
                y2 = net2.forward(x)
            stream.synchronize()
            graph2 = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph2, stream=stream):
                y2 = net2.forward(x)
            for _ in range(2):
                graph2.replay()
            stream.synchronize()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                graph2.replay()
            torch.cuda.synchronize()
            ms2 = (time.perf_counter() - t0) * 1e3 / args.steps
            n2 = int(y2.num_act.item())
            fused = {"ms_per_step": round(ms2, 4), "effective_tflops": round(total_flops / (ms2 * 1e-3) / 1e12, 2),
                     "what": "same pass with D3D_OPT_INDEX_UNUSED on every rulebook operator: index tensors left "
                             "unwritten, tables and tile masks written by the probe pass, no compaction",
                     "outputs_equal_full_pass": bool(n2 == int(y.num_act.item()) and torch.equal(y2.feats, y.feats)
                                                     and torch.equal(y2.coors[:n2], y.coors[:n2]))}
            del net2, graph2
        # third figure: the same pass recorded once as a native schedule (d3d_schedule_*, three lanes with direct
        # events, no HIP graph) - what a caller without graph capture gets; its host cost per pass is reported
        sched = None
        if not args.no_graph and not args.no_fused and all("+" not in (s.get("src") or "") for s in specs):
            net3 = layers.SparseBackbone(specs, weights, caps, dtype=dtype, overlap=False)
            for _ in range(3):
                y3 = net3.forward_scheduled(x)
            stream.synchronize()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                net3.forward_scheduled(x)
            host3 = (time.perf_counter() - t0) * 1e3 / args.steps
            torch.cuda.synchronize()
            ms3 = (time.perf_counter() - t0) * 1e3 / args.steps
            sched = {"ms_per_step": round(ms3, 4), "host_ms_per_pass": round(host3, 4),
                     "what": "the pass enqueued by one d3d_schedule_run per step: no HIP graph, rulebooks on two "
                             "lanes of their own, events straight between the lanes",
                     "outputs_equal_full_pass": bool(torch.equal(y3.feats, y.feats))}
            del net3
        # further figures beside `value` (same kernels, other conditions): what a caller gets who binds the operators
        # unchanged (`reference_contract`), replays that alternate between two different clouds, and capacities
        # with head-room over the live counts
        def replay_ms(graphs, steps):
            for g in graphs:
                g.replay()
            stream.synchronize()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(steps):
                graphs[i % len(graphs)].replay()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) * 1e3 / steps

        def captured(network, inp):
            for _ in range(2):
                out_t = network.forward(inp)
            stream.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                out_t = network.forward(inp)
            return g, out_t

        extra = {}
        if not args.no_graph and not args.no_fused:
            # (a) no d3d_link_*, no D3D_OPT_PERSISTENT_INDEX: every rulebook operator fills its whole index tensor
            # with -1 (reference: trt/spconv/index.cu:352-354), every convolution derives its table from the tensor
            net_r = layers.SparseBackbone(specs, weights, caps, dtype=dtype, overlap=not args.no_overlap,
                                          extensions=False)
            g_r, y_r = captured(net_r, x)
            ms_r = replay_ms([g_r], args.steps)
            extra["reference_contract"] = {
                "ms_per_step": round(ms_r, 4), "effective_tflops": round(total_flops / (ms_r * 1e-3) / 1e12, 2),
                "what": "the same pass with the operators as the reference's contract alone describes them: no "
                        "d3d_link_rulebook / d3d_link_coords, no D3D_OPT_PERSISTENT_INDEX - index tensors filled with "
                        "-1 at capacity on every enqueue, neighbour tables derived from the index tensor per enqueue",
                "outputs_equal_full_pass": bool(torch.equal(y_r.feats, y.feats))}
            del net_r, g_r
            # (b) two clouds in turn: the full cloud and one with ~8 % fewer voxels (the first rows of a shuffled
            # copy), each in buffers of its own at the same capacities; replays alternate, so the incremental fill of
            # the persistent index tensors and the tile masks see change between passes
            n_b = int(n * 0.92)
            pick = np.sort(np.random.default_rng(5).permutation(n)[:n_b])
            x_b = layers.make_input(cfg["coords"][pick], feats[pick], cfg["grid"], dtype=dtype, capacity=in_cap)
            g_b, y_b = captured(net, x_b)
            g_a, y_a = captured(net, x)
            ms_ab = replay_ms([g_a, g_b], 2 * (args.steps // 2 + 1))
            g_a.replay()
            stream.synchronize()
            extra["alternating_clouds"] = {
                "ms_per_step": round(ms_ab, 4), "voxels": [n, n_b],
                "what": "graph replays alternating between two clouds (the second a random 92 % subset of the "
                        "first) through the same operators and capacities",
                "full_cloud_output_unchanged": bool(torch.equal(y_a.feats, ref_out))}
            del g_b, x_b
            # (c) capacities at 1.5 x the live counts (input rows and every strided layer's maxNumActOut)
            counts15 = {k: int(v * 1.5) for k, v in counts.items()}
            caps15 = layers.plan_capacities(specs, int(n * 1.5), counts15)
            net_c = layers.SparseBackbone(specs, weights, caps15, dtype=dtype, overlap=not args.no_overlap)
            x_c = layers.make_input(cfg["coords"], feats, cfg["grid"], dtype=dtype, capacity=int(n * 1.5))
            g_c, y_c = captured(net_c, x_c)
            ms_c = replay_ms([g_c], args.steps)
            n_c = int(y_c.num_act.item())
            extra["capacity_1p5x"] = {
                "ms_per_step": round(ms_c, 4), "capacities": caps15,
                "what": "the same cloud with every row capacity at 1.5 x the live count (kernels are launched at "
                        "capacity)",
                "outputs_equal_full_pass": bool(n_c == int(y.num_act.item()) and
                                                torch.equal(y_c.feats[:n_c], y.feats[:n_c]))}
            del net_c, g_c, x_c
        n_final = int(y.num_act.item())
        gpu_coords = y.coors[:n_final].cpu().numpy()
        gpu_feats = y.feats[:n_final].float().cpu().numpy() if dtype != torch.int8 else y.feats[:n_final].cpu().numpy()
        if args.pmc_copy_mib:
            src = torch.ones(args.pmc_copy_mib << 20, dtype=torch.uint8, device="cuda")
            dst = torch.empty_like(src)
            stream.synchronize()
            dst.copy_(src)
            stream.synchronize()

    # ---- rooflines ----
    es = ELEM[cfg["dtype"]]
    peak_mfma = PEAK_TFLOPS[cfg["dtype"]]
    meas_mfma = None
    meas_hbm = None
    if peaks:
        meas_mfma = {"float16": peaks.get("mfma_f16_tflops"), "bfloat16": peaks.get("mfma_bf16_tflops"),
                     "int8": peaks.get("mfma_i8_tops")}.get(cfg["dtype"])
        meas_hbm = peaks.get("hbm_copy_gbs")
    rooflines = []
    for li, spec in enumerate(specs[:len(layer_ms)]):
        key = spec["key"]
        kvol = int(np.prod(spec["ksize"]))
        secs = layer_ms[li] * 1e-3
        # compulsory bytes: input rows, output rows, weights, one table entry per (tap, output row)
        nbytes = (rows_in[key] * spec["cin"] * es + rows_out[key] * spec["cout"] * es +
                  kvol * spec["cin"] * spec["cout"] * es + 4 * kvol * rows_out[key])
        if spec["cin"] >= 32 and cfg["dtype"] != "float32":
            a = layer_flops[li] / secs / 1e12
            r = {"kernel": "SPConvMM %s (%d->%d, %d pairs)" % (spec["name"], spec["cin"], spec["cout"], pairs[key]),
                 "bound": "mfma", "achieved": round(a, 2), "peak": peak_mfma, "unit": "TFLOP/s" if es > 1 else "TOP/s",
                 "frac": round(a / peak_mfma, 4), "flops_per_launch": layer_flops[li]}
            if meas_mfma:
                r["frac_of_measured_peak"] = round(a / meas_mfma, 4)
        else:
            a = nbytes / secs / 1e9
            r = {"kernel": "SPConvMM %s (%d->%d, narrow)" % (spec["name"], spec["cin"], spec["cout"]),
                 "bound": "hbm", "achieved": round(a, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                 "frac": round(a / PEAK_HBM_GBS, 4), "bytes_per_launch": nbytes}
            if meas_hbm:
                r["frac_of_measured_peak"] = round(a / meas_hbm, 4)
        r.update(layer=spec["name"], avg_launch_ms=round(layer_ms[li], 4),
                 traffic=MEASURED_TRAFFIC.get((args.config, voxels, spec["name"])))
        rooflines.append(r)
    for key, li in first_of_key.items():
        spec = specs[li]
        kvol = int(np.prod(spec["ksize"]))
        nd1 = len(spec["ksize"]) + 1
        # coords in, one probe per (tap, input), three int32 per pair out, coords out (strided only)
        nbytes = (4 * nd1 * rows_in[key] + 4 * kvol * rows_in[key] + 12 * pairs[key] +
                  (0 if spec["subm"] else 4 * nd1 * rows_out[key]))
        a = nbytes / (rulebook_ms[key] * 1e-3) / 1e9
        r = {"kernel": "SPConvIdx%dd %s (%s, %d inputs, %d pairs; all launches of one build)" %
                       (nd1 - 1, key, "SubM" if spec["subm"] else "strided", rows_in[key], pairs[key]),
             "bound": "hbm", "achieved": round(a, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
             "frac": round(a / PEAK_HBM_GBS, 4), "bytes_per_launch": nbytes, "layer": key,
             "avg_launch_ms": round(rulebook_ms[key], 4), "traffic": None}
        if meas_hbm:
            r["frac_of_measured_peak"] = round(a / meas_hbm, 4)
        rooflines.append(r)
    # dominant kernel: the MFMA convolution with the largest device time; a configuration without one (config 1) is
    # judged on its slowest operator
    roofline = None
    if rooflines:
        mfma = [r for r in rooflines if r["bound"] == "mfma"]
        roofline = dict(max(mfma or rooflines, key=lambda r: r["avg_launch_ms"]))
        roofline["traffic_source"] = TRAFFIC_SOURCE if roofline.get("traffic") else None
        if meas_mfma and roofline["bound"] == "mfma":
            roofline["measured_peak"] = meas_mfma

    out = {
        "metric": METRIC, "value": round(ms, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": {"float16": "fp16", "float32": "fp32", "int8": "int8"}[cfg["dtype"]],
        "data": "synthetic",
        "config": {"workload": WORKLOAD[args.config] % n, "mode": mode,
                   "boundary": "C ABI; index tensors persistent (D3D_OPT_PERSISTENT_INDEX), convolutions linked to "
                               "their rulebook operators (d3d_link_rulebook)",
                   "stage_voxels": counts, "capacities": caps},
        "effective_tflops": round(total_flops / (ms * 1e-3) / 1e12, 2),
        "total_gflop": round(total_flops / 1e9, 2),
        "eager_ms_per_step": round(eager_ms, 4),
        "host_ms_per_graph_launch": None if host_ms is None else round(host_ms, 4),
        "outputs_match_warmup": same,
        "layer_ms": {s["name"]: round(t, 4) for s, t in zip(specs, layer_ms)},
        "rulebook_ms": {k: round(t, 4) for k, t in rulebook_ms.items()},
        "index_unused": fused,
        "native_schedule": sched,
        "reference_contract": extra.get("reference_contract"),
        "alternating_clouds": extra.get("alternating_clouds"),
        "capacity_1p5x": extra.get("capacity_1p5x"),
        "roofline": roofline,
        "rooflines": rooflines,
        "measured_peak": peaks,
    }

    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, gpu_coords, gpu_feats)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
