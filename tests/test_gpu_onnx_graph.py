"""The ONNX graph executor on the GPU: a graph of TRT_PluginV2 nodes run through deploy3d_amd.onnx_graph.GraphExecutor
gives, bit for bit, what deploy3d_amd.layers.SparseBackbone gives for the layer table the graph was written from
(which the other GPU tests hold against the oracle).  Parity unpinned by the reference, which has no graph fixture."""
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
