#!/usr/bin/env python3
"""Writes tests/golden/backbone_head.onnx: the ONNX graph of the first four layers of the VoxelNet backbone of
BASELINE config 3 at 4 000 voxels (SubM 5->16, two SubM 16->16 sharing the indice key, strided 16->32), with the
node and attribute layout of the reference's exporter (TRT_PluginV2 nodes carrying name / data / namespace /
version; deploy3d/symfun/ops/spconv/spconv_index.py:94-105, spconv_mm.py:54-66).  The reference holds no graph
fixture and its exporter needs torch.onnx + TensorRT conventions that cannot run here, so the bytes are written by
deploy3d_amd.onnx_graph.write_model from the synthetic layer table; what the fixture pins is the reader and the
executor against a file on disk.  Run from the repository root:  python tests/golden/make_onnx_graph.py
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from deploy3d_amd import layers, onnx_graph, synth  # noqa: E402

N = 4000
GRID = (16, 96, 96)


def build():
    specs = synth.voxelnet_layers()[:4]
    weights = [synth.layer_weights(0, i, s) for i, s in enumerate(specs)]
    caps = layers.plan_capacities(specs, N)
    return onnx_graph.backbone_model(specs, weights, caps, N, 5, GRID), specs, weights, caps


if __name__ == "__main__":
    model, _, _, _ = build()
    path = os.path.join(HERE, "backbone_head.onnx")
    with open(path, "wb") as f:
        f.write(onnx_graph.write_model(model))
    print("wrote", path, os.path.getsize(path), "bytes")
