"""The ONNX graph executor on the GPU: a graph of TRT_PluginV2 nodes run through deploy3d_amd.onnx_graph.GraphExecutor
gives, bit for bit, what deploy3d_amd.layers.SparseBackbone gives for the layer table the graph was written from,
and - the fixture graph and the config-3 graph - what the CPU oracle gives for that table (coordinates bit-exact
after sorting, features within 2e-2 * rms).  The graph FILE itself is parity unpinned by the reference, which has
no graph fixture."""
import os
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))


def _graph_inputs(x, grid, batch=1):
    shape = torch.empty((batch, 0) + tuple(grid), dtype=torch.int32, device="cuda")
    return dict(feats=x.feats, coors=x.coors, num_act=x.num_act, spatial_shape=shape)


def _same(y, out, model):
    feats, coors, num = (out[v.name] for v in model.outputs[:3])
    n = int(num.item())
    assert n == int(y.num_act.item())
    assert torch.equal(coors[:n], y.coors[:n])
    assert torch.equal(feats, y.feats)


def _against_the_oracle(out, model, cfg, last):
    """The executor's sparse outputs against the CPU oracle run over the layer table the graph was written from:
    the same coordinates (bit for bit after sorting both by coordinate), features within 2e-2 * rms (fp16 storage,
    fp32 accumulation on the GPU, fp64 in the oracle)."""
    import chain
    ref = chain.oracle_chain(cfg)[last]
    feats, coors, num = (out[v.name] for v in model.outputs[:3])
    n = int(num.item())
    assert n == len(ref["coords"])
    c_gpu, f_gpu = chain.sort_rows(coors[:n].cpu().numpy(), feats[:n].float().cpu().numpy())
    c_ref, f_ref = chain.sort_rows(ref["coords"], ref["feats"])
    assert np.array_equal(c_gpu, c_ref)
    rms = float(np.sqrt(np.mean(f_ref.astype(np.float64) ** 2)))
    assert rms > 0 and np.abs(f_gpu.astype(np.float64) - f_ref).max() <= 2e-2 * rms


def test_fixture_file_runs_like_the_layer_table(engine):
    import make_onnx_graph
    from deploy3d_amd import layers, onnx_graph, synth
    model, specs, weights, caps = make_onnx_graph.build()
    coords = synth.coords_lidar(synth.seed(0, 0), make_onnx_graph.GRID, make_onnx_graph.N)
    feats = synth.normal(synth.seed(0, 1), (len(coords), 5))
    x = layers.make_input(coords, feats, make_onnx_graph.GRID)
    y = layers.SparseBackbone(specs, weights, caps, overlap=False).forward(x)
    ex = onnx_graph.GraphExecutor(os.path.join(HERE, "golden", "backbone_head.onnx"))
    out = ex.run(**_graph_inputs(x, make_onnx_graph.GRID))
    torch.cuda.synchronize()
    _same(y, out, ex.model)
    # ... and like the CPU oracle on that table: the executor's result does not rest on the engine agreeing with itself
    cfg = dict(dtype="float16", coords=coords, feats=feats, grid=list(make_onnx_graph.GRID), layers=specs,
               weights=weights)
    _against_the_oracle(out, ex.model, cfg, specs[-1]["name"])


@pytest.mark.parametrize("config,n", [(3, 12000), (5, 20000)])
def test_whole_configurations_and_graph_capture(engine, config, n):
    """Config 3 (chain, four indice keys shared by three convolutions each, BEVDensify at the end) and config 5
    (two-branch residual block: an Add node, keys shared across branches).  Eager run, a second run with fewer live
    voxels in the same buffers, and HIP-graph replays all equal the layer runner."""
    from deploy3d_amd import layers, onnx_graph, synth
    cfg = (synth.config3 if config == 3 else synth.config5)(n)
    specs, weights = cfg["layers"], cfg["weights"]
    n = len(cfg["coords"])
    counts = layers.measure_output_counts(specs, cfg["coords"], cfg["grid"])
    caps = layers.plan_capacities(specs, n, counts)
    model = onnx_graph.backbone_model(specs, weights, caps, n, cfg["feats"].shape[1], cfg["grid"], densify=True)
    ex = onnx_graph.GraphExecutor(onnx_graph.write_model(model))
    net = layers.SparseBackbone(specs, weights, caps, overlap=False)
    x = layers.make_input(cfg["coords"], cfg["feats"], cfg["grid"])
    for live in (n, n // 2, n):
        x.num_act.fill_(live)
        y = net.forward(x)
        bev = layers.densify(y)
        out = ex.run(**_graph_inputs(x, cfg["grid"]))
        torch.cuda.synchronize()
        _same(y, out, ex.model)
        assert torch.equal(out["bev"], bev)
    if config == 3:  # the final tensor of the whole backbone against the CPU oracle
        _against_the_oracle(out, ex.model, cfg, specs[-1]["name"])
    # the same graph through the native schedule: one call per pass, rulebook nodes on lanes of their own
    if config == 3:
        for live in (n // 3, n):
            x.num_act.fill_(live)
            y = net.forward(x)
            bev = layers.densify(y)
            for name in ("bev", ex.model.outputs[0].name):
                ex._bound["values"][name].zero_()
            out = ex.run_scheduled(**_graph_inputs(x, cfg["grid"]))
            torch.cuda.synchronize()
            _same(y, out, ex.model)
            assert torch.equal(out["bev"], bev)
        assert len(ex._bound["schedule"]) == len(ex.nodes)
    else:
        with pytest.raises(NotImplementedError):
            ex.run_scheduled(**_graph_inputs(x, cfg["grid"]))
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        inputs = _graph_inputs(x, cfg["grid"])
        out = ex.run(**inputs)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            out = ex.run(**inputs)
        for _ in range(3):
            out[ex.model.outputs[0].name].zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            _same(y, out, ex.model)
            assert torch.equal(out["bev"], bev)


def test_points_to_dense_map_as_one_graph(engine):
    """All four operators in one graph: SimpleMeanEncoder -> Cast -> SPConvIdx / SPConvMM chain -> BEVDensify.  The
    graph's outputs equal, bit for bit, the same stages called one by one (which test_gpu_pipeline.py holds against
    the oracle) - eagerly, with fewer points in the same buffers, and from a HIP-graph replay; the native schedule
    refuses the Cast."""
    from deploy3d_amd import layers, onnx_graph, simple_mean_encoder, synth
    rng = np.random.default_rng(5)
    n_pts, max_vox = 40000, 20000
    grid = (16, 96, 96)
    vcfg = np.array([-9.6, -9.6, -1.0, 0.2, 0.2, 0.25], np.float32)
    pts = np.empty((n_pts, 5), np.float32)
    pts[:, 0:2] = rng.normal(0, 4.0, (n_pts, 2))
    pts[:, 2] = np.where(rng.random(n_pts) < 0.7, rng.uniform(-1.0, -0.4, n_pts), rng.normal(0.5, 0.8, n_pts))
    pts[:, 3:] = rng.random((n_pts, 2))
    batch = np.zeros(n_pts, np.int32)
    batch[rng.integers(0, n_pts, 300)] = -1
    specs = synth.voxelnet_layers()[:4]
    weights = [synth.layer_weights(0, i, s) for i, s in enumerate(specs)]
    caps = layers.plan_capacities(specs, max_vox)
    model = onnx_graph.backbone_model(specs, weights, caps, max_vox, 5, grid, densify=True, points=n_pts)
    assert [n.attrs.get("name", n.op_type.encode()) for n in model.nodes[:2]] == [b"SimpleMeanEncoder", b"Cast"]
    ex = onnx_graph.GraphExecutor(onnx_graph.write_model(model))
    net = layers.SparseBackbone(specs, weights, caps, overlap=False)
    d_pts, d_batch = torch.from_numpy(pts).cuda(), torch.from_numpy(batch).cuda()
    d_cfg = torch.from_numpy(vcfg).cuda()
    shape = torch.empty((1, 0) + grid, dtype=torch.int32, device="cuda")
    inputs = dict(points=d_pts, batch_indices=d_batch, voxel_config=d_cfg, spatial_shape=shape)

    def stage_by_stage(vals):
        """The voxeliser called on its own (coordinates and order exact; its means are sums of fp32 atomics, equal
        up to the order of addition), then the layer runner and the densifier on the graph's own voxels."""
        f, c, k = simple_mean_encoder(d_pts, d_batch, d_cfg, shape, max_vox)
        nv = int(k.item())
        assert nv == int(vals["num_act"].item()) and torch.equal(c[:nv], vals["coors"][:nv])
        torch.testing.assert_close(f[:nv], vals["voxel_means"][:nv], rtol=1e-5, atol=1e-6)
        y = net.forward(layers.SparseTensor(vals["voxel_means"].half(), vals["coors"], vals["num_act"], list(grid), 1))
        return y, layers.densify(y).clone()

    for drop in (0, n_pts // 2):
        d_batch.copy_(torch.from_numpy(batch))
        if drop:
            d_batch[:drop] = -1                          # fewer points, same buffers
        out = ex.run(**inputs)
        torch.cuda.synchronize()
        y, bev = stage_by_stage(ex._bound["values"])
        torch.cuda.synchronize()
        assert 1000 < int(y.num_act.item()) < max_vox
        _same(y, out, ex.model)
        assert torch.equal(out["bev"], bev)
    with pytest.raises(NotImplementedError):
        ex.run_scheduled(**inputs)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        out = ex.run(**inputs)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            out = ex.run(**inputs)
        for _ in range(2):
            out["bev"].zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            y, bev = stage_by_stage(ex._bound["values"])
            torch.cuda.synchronize()
            _same(y, out, ex.model)
            assert torch.equal(out["bev"], bev)
