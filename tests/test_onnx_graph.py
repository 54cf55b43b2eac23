"""The ONNX reader / writer of deploy3d_amd.onnx_graph on the CPU: the bytes it writes are parsed by the real
protobuf runtime (google.protobuf) through message descriptors built here from the field numbers of the public
onnx.proto - an implementation that shares nothing with the module's own wire-format code - and the committed
fixture graph is read back node by node against the blobs of the layer table it was written from.
Parity unpinned by the reference: it holds no graph file (its exporter needs torch.onnx and TensorRT)."""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))


def _onnx_messages():
    """ModelProto and friends, restricted to the fields a TRT_PluginV2 graph uses (numbers from onnx.proto)."""
    from google.protobuf import descriptor_pb2, descriptor_pool, message_factory
    F = descriptor_pb2.FieldDescriptorProto
    fd = descriptor_pb2.FileDescriptorProto(name="onnx_subset_for_tests.proto", package="onnxsub", syntax="proto2")

    def msg(name, fields):
        m = fd.message_type.add(name=name)
        for fname, num, ftype, label, tname in fields:
            f = m.field.add(name=fname, number=num, type=ftype, label=label)
            if tname:
                f.type_name = ".onnxsub." + tname
    OPT, REP = F.LABEL_OPTIONAL, F.LABEL_REPEATED
    msg("AttributeProto", [("name", 1, F.TYPE_STRING, OPT, None), ("f", 2, F.TYPE_FLOAT, OPT, None),
                           ("i", 3, F.TYPE_INT64, OPT, None), ("s", 4, F.TYPE_BYTES, OPT, None),
                           ("type", 20, F.TYPE_INT32, OPT, None)])
    msg("NodeProto", [("input", 1, F.TYPE_STRING, REP, None), ("output", 2, F.TYPE_STRING, REP, None),
                      ("name", 3, F.TYPE_STRING, OPT, None), ("op_type", 4, F.TYPE_STRING, OPT, None),
                      ("attribute", 5, F.TYPE_MESSAGE, REP, "AttributeProto")])
    msg("Dimension", [("dim_value", 1, F.TYPE_INT64, OPT, None), ("dim_param", 2, F.TYPE_STRING, OPT, None)])
    msg("TensorShapeProto", [("dim", 1, F.TYPE_MESSAGE, REP, "Dimension")])
    msg("Tensor", [("elem_type", 1, F.TYPE_INT32, OPT, None), ("shape", 2, F.TYPE_MESSAGE, OPT, "TensorShapeProto")])
    msg("TypeProto", [("tensor_type", 1, F.TYPE_MESSAGE, OPT, "Tensor")])
    msg("ValueInfoProto", [("name", 1, F.TYPE_STRING, OPT, None), ("type", 2, F.TYPE_MESSAGE, OPT, "TypeProto")])
    msg("GraphProto", [("node", 1, F.TYPE_MESSAGE, REP, "NodeProto"), ("name", 2, F.TYPE_STRING, OPT, None),
                       ("input", 11, F.TYPE_MESSAGE, REP, "ValueInfoProto"),
                       ("output", 12, F.TYPE_MESSAGE, REP, "ValueInfoProto")])
    msg("OperatorSetIdProto", [("domain", 1, F.TYPE_STRING, OPT, None), ("version", 2, F.TYPE_INT64, OPT, None)])
    msg("ModelProto", [("ir_version", 1, F.TYPE_INT64, OPT, None), ("producer_name", 2, F.TYPE_STRING, OPT, None),
                       ("graph", 7, F.TYPE_MESSAGE, OPT, "GraphProto"),
                       ("opset_import", 8, F.TYPE_MESSAGE, REP, "OperatorSetIdProto")])
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    get = getattr(message_factory, "GetMessageClass", None)
    desc = pool.FindMessageTypeByName("onnxsub.ModelProto")
    return get(desc) if get else message_factory.MessageFactory(pool).GetPrototype(desc)


def _fixture():
    import make_onnx_graph
    return make_onnx_graph.build()


def test_written_bytes_parse_with_the_protobuf_runtime():
    from deploy3d_amd import onnx_graph
    model, specs, weights, caps = _fixture()
    data = onnx_graph.write_model(model)
    m = _onnx_messages()()
    m.ParseFromString(data)
    assert m.ir_version == 7 and m.opset_import[0].version == 11
    assert [n.op_type for n in m.graph.node] == ["TRT_PluginV2"] * 6          # 2 rulebooks + 4 convolutions
    names = [dict((a.name, a.s) for a in n.attribute)["name"] for n in m.graph.node]
    assert names == [b"SPConvIdx3d", b"SPConvMM", b"SPConvMM", b"SPConvMM", b"SPConvIdx3d", b"SPConvMM"]
    for n in m.graph.node:
        attrs = {a.name: a for a in n.attribute}
        assert set(attrs) == {"name", "data", "namespace", "version"}       # spconv_index.py:102-105
        assert all(a.type == 3 for a in attrs.values()) and attrs["version"].s == b"2.0"
    assert [i.name for i in m.graph.input] == ["feats", "coors", "num_act", "spatial_shape"]
    shape = [d.dim_value for d in m.graph.input[3].type.tensor_type.shape.dim]
    assert shape == [1, 0, 16, 96, 96]                                        # [B, 0, spatial...], a zero-element tensor
    # and the other way: bytes serialised by the protobuf runtime are read by the module's parser
    back = onnx_graph.read_model(m.SerializeToString())
    assert [n.attrs["data"] for n in back.nodes] == [n.attrs["data"] for n in model.nodes]


def test_reader_round_trip_and_blobs():
    from deploy3d_amd import onnx_graph
    from deploy3d_amd.spconv_index import index_blob
    from deploy3d_amd.spconv_mm import mm_blob
    model, specs, weights, caps = _fixture()
    back = onnx_graph.read_model(onnx_graph.write_model(model))
    assert len(back.nodes) == len(model.nodes)
    for a, b in zip(model.nodes, back.nodes):
        assert (a.op_type, a.inputs, a.outputs, a.name, a.attrs) == (b.op_type, b.inputs, b.outputs, b.name, b.attrs)
    assert [(v.name, v.elem_type, v.dims) for v in back.inputs] == [(v.name, v.elem_type, v.dims) for v in model.inputs]
    assert [(v.name, v.elem_type, v.dims) for v in back.outputs] == [(v.name, v.elem_type, v.dims) for v in model.outputs]
    # attribute blobs are the reference's packed layouts, byte for byte
    by_name = {n.name: n for n in back.nodes}
    s0, s3 = specs[0], specs[3]
    assert by_name[s0["key"]].attrs["data"] == index_blob(s0["ksize"], s0["stride"], s0["padding"], s0["dilation"],
                                                          (0, 0, 0), caps[0], True, False)
    assert by_name[s3["name"]].attrs["data"] == mm_blob(s3["ksize"], s3["cin"], s3["cout"], caps[3], False, False,
                                                        *weights[3], relu=s3.get("relu", False))
    # indice-key reuse: the three SubM convolutions of stage 1 read one index tensor
    idx_inputs = {by_name[s["name"]].inputs[3] for s in specs[:3]}
    assert idx_inputs == {specs[0]["key"] + "_index"}


def test_committed_fixture_matches_its_generator():
    from deploy3d_amd import onnx_graph
    model, _, _, _ = _fixture()
    with open(os.path.join(HERE, "golden", "backbone_head.onnx"), "rb") as f:
        data = f.read()
    assert data == onnx_graph.write_model(model)
    assert len(onnx_graph.read_model(data).nodes) == 6


def test_malformed_models_are_refused():
    from deploy3d_amd import onnx_graph
    with pytest.raises(ValueError):
        onnx_graph.read_model(b"\x0a\xff\xff\xff\xff\x0f")        # length runs past the message
    with pytest.raises(ValueError):
        onnx_graph.read_model(b"\x08\x07")                         # a model without a graph
    bad = onnx_graph.Model([onnx_graph.Node("Conv", ["feats"], ["y"])],
                           [onnx_graph.Value("feats", onnx_graph.FLOAT16, [4, 4])], [])
    with pytest.raises(NotImplementedError):
        onnx_graph.GraphExecutor.__new__(onnx_graph.GraphExecutor).__init__(bad)
