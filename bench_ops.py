"""Timing of the two operators on either side of the sparse backbone, on the shapes of the reference's own tests
and of the bench workload's tail:

    python3 bench_ops.py [--calls 200]

* SimpleMeanEncoder: 200 000 points, x y ~ N(0, 50), z ~ N(1, 2), grid [2, *, 41, 1536, 1536]
  (tests/voxel_encoder/test_simple_mean.py:8-15)
* BEVDensify: 10 000 rows x 128 channels into [2, 256, 128, 128] (tests/spconv/test_bev_densify.py:33-34), and
  38 000 rows x 128 fp16 channels into [1, 256, 180, 180], the map a CenterPoint-sized backbone ends in

Each operator is captured into a HIP graph (20 calls per graph) and replayed; one JSON line per case with the time
per call and the algorithmic bytes moved.  Inputs are synthetic and resident in HBM.
"""
import argparse
import json
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from deploy3d_amd.bev_densify import bev_densify  # noqa: E402
from deploy3d_amd.simple_mean import simple_mean_encoder  # noqa: E402

PER_GRAPH = 20


def _time(fn, calls):
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        fn()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(PER_GRAPH):
                fn()
    torch.cuda.synchronize()
    replays = max(1, calls // PER_GRAPH)
    graph.replay()
    t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0.record()
    for _ in range(replays):
        graph.replay()
    t1.record()
    torch.cuda.synchronize()
    return t0.elapsed_time(t1) * 1e3 / (replays * PER_GRAPH)


def voxelize_case(calls, n=200000):
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(1234)
    feats = torch.cat([torch.randn((n, 2), generator=g) * 50, torch.randn((n, 1), generator=g) * 2 + 1,
                       torch.randn((n, 1), generator=g)], dim=-1).to(dev)
    batch = torch.randint(0, 2, (n,), dtype=torch.int32, generator=g).to(dev)
    cfg = torch.tensor([-76.8, -76.8, -2.0, 0.1, 0.1, 0.15], device=dev)
    shape = torch.empty((2, 0, 41, 1536, 1536), dtype=torch.int32, device=dev)
    out = simple_mean_encoder(feats, batch, cfg, shape, n)
    voxels = int(out[2].item())
    us = _time(lambda: simple_mean_encoder(feats, batch, cfg, shape, n), calls)
    moved = n * (4 * 4 + 4) + voxels * (4 * 4 + 16)
    return dict(op="SimpleMeanEncoder", points=n, voxels=voxels, us_per_call=round(us, 2),
                mpoints_per_s=round(n / us, 1), algorithmic_mb=round(moved / 1e6, 2))


def densify_case(calls, rows, cap, shape, dtype):
    dev = torch.device("cuda:0")
    b, z, y, x = shape
    g = torch.Generator().manual_seed(7)
    cells = torch.randperm(b * z * y * x, generator=g)[:cap].sort().values
    coors = torch.stack([cells // (z * y * x), cells // (y * x) % z, cells // x % y, cells % x], dim=1).int().to(dev)
    feats = torch.randn((cap, 128), generator=g).to(dev).to(dtype)
    num = torch.tensor([rows], dtype=torch.int32, device=dev)
    shp = torch.empty((b, 0, z, y, x), dtype=torch.int32, device=dev)
    out = torch.empty((b, 128 * z, y, x), dtype=dtype, device=dev)
    us = _time(lambda: bev_densify(feats, coors, num, shp, 128 * z, out=out), calls)
    moved = out.numel() * out.element_size() + rows * 128 * out.element_size()
    return dict(op="BEVDensify", rows=rows, map=list(out.shape), dtype=str(dtype).replace("torch.", ""),
                us_per_call=round(us, 2), algorithmic_mb=round(moved / 1e6, 2),
                algorithmic_gb_per_s=round(moved / us / 1e3, 1))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--calls", type=int, default=200)
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("bench_ops.py needs a GPU")
    print(json.dumps(voxelize_case(args.calls)), flush=True)
    for rows, cap, shape, dtype in ((10000, 10000, (2, 2, 128, 128), torch.float32),
                                    (10000, 10000, (2, 2, 128, 128), torch.float16),
                                    (38000, 40000, (1, 2, 180, 180), torch.float16)):
        print(json.dumps(densify_case(args.calls, rows, cap, shape, dtype)), flush=True)


if __name__ == "__main__":
    main()
