"""ONNX graphs of sparse-convolution plugin nodes: a reader, a writer and an executor.

The reference exports its sparse operators as ONNX nodes of type ``TRT_PluginV2`` whose attributes carry the
plugin name, version and packed attribute blob (deploy3d/symfun/ops/spconv/spconv_index.py:94-105,
spconv_mm.py:54-66, bev_densify.py:38-41) and hands the file to TensorRT, which deserialises one plugin per node
and runs them in graph order (deploy3d/symfun/trt_utils/trt_onnx_module.py:80-250).  This module plays that part for
the sparse section of such a graph:

* ``read_model`` parses the handful of ModelProto fields involved straight from the protobuf wire format (the
  ``onnx`` package is not needed): nodes with op_type / inputs / outputs / attributes, graph inputs and outputs with
  element type and dims;
* ``write_model`` emits the same subset (what the reference's ``symbolic()`` functions emit through torch.onnx);
* ``GraphExecutor`` creates one operator per ``TRT_PluginV2`` node through the C ABI, allocates every tensor once
  at its static capacity, links each SPConvMM to the SPConvIdx node that produces its index tensor (several
  convolutions may share one), and enqueues the nodes in topological order on the current stream - no host
  synchronisation, so a run can be captured in a HIP graph.  Besides plugin nodes it runs ``Cast`` (voxel means to
  the backbone's type) and ``Add`` (residual sums of two feature tensors); dense 2-D heads are outside its scope
  and any other op type is refused.
"""
import struct

import torch

from .plugin import OPT_INDEX_UNUSED, OPT_PERSISTENT_INDEX, EngineError, Plugin, Schedule, TensorDesc

# onnx.TensorProto.DataType
FLOAT, INT8, INT32, FLOAT16, BFLOAT16 = 1, 3, 6, 10, 16
_ELEM_TO_TORCH = {FLOAT: torch.float32, INT8: torch.int8, INT32: torch.int32, FLOAT16: torch.float16,
                  BFLOAT16: torch.bfloat16}
_TORCH_TO_ELEM = {v: k for k, v in _ELEM_TO_TORCH.items()}
# onnx.AttributeProto.AttributeType
_ATTR_FLOAT, _ATTR_INT, _ATTR_STRING = 1, 2, 3


# ---------------------------------------------------------------------------
# protobuf wire format
# ---------------------------------------------------------------------------
def _varint(buf, pos):
    shift = value = 0
    while True:
        if pos >= len(buf):
            raise ValueError("truncated varint")
        b = buf[pos]
        pos += 1
        value |= (b & 0x7F) << shift
        if not b & 0x80:
            return value, pos
        shift += 7
        if shift > 70:
            raise ValueError("varint too long")


def _fields(buf):
    """Yields (field number, wire type, value) of one message; value is an int or a memoryview."""
    buf = memoryview(buf)
    pos = 0
    while pos < len(buf):
        tag, pos = _varint(buf, pos)
        field, wire = tag >> 3, tag & 7
        if wire == 0:
            value, pos = _varint(buf, pos)
        elif wire == 1:
            value, pos = buf[pos:pos + 8], pos + 8
        elif wire == 2:
            n, pos = _varint(buf, pos)
            if pos + n > len(buf):
                raise ValueError("length-delimited field runs past the message")
            value, pos = buf[pos:pos + n], pos + n
        elif wire == 5:
            value, pos = buf[pos:pos + 4], pos + 4
        else:
            raise ValueError("wire type %d not supported" % wire)
        yield field, wire, value


def _enc_varint(v):
    out = bytearray()
    v &= (1 << 64) - 1
    while True:
        b = v & 0x7F
        v >>= 7
        out.append(b | (0x80 if v else 0))
        if not v:
            return bytes(out)


def _enc(field, wire, payload):
    if wire == 0:
        return _enc_varint(field << 3) + _enc_varint(payload)
    return _enc_varint(field << 3 | 2) + _enc_varint(len(payload)) + bytes(payload)


# ---------------------------------------------------------------------------
# model <-> plain Python
# ---------------------------------------------------------------------------
class Node:
    def __init__(self, op_type, inputs, outputs, attrs=None, name=""):
        self.op_type, self.inputs, self.outputs = op_type, list(inputs), list(outputs)
        self.attrs, self.name = dict(attrs or {}), name

    def __repr__(self):
        return "Node(%s %s -> %s)" % (self.attrs.get("name", self.op_type), self.inputs, self.outputs)


class Value:
    """A graph input or output: name, ONNX element type, dims (ints, or strings for symbolic dims)."""

    def __init__(self, name, elem_type, dims):
        self.name, self.elem_type, self.dims = name, elem_type, list(dims)


class Model:
    def __init__(self, nodes, inputs, outputs, name="graph"):
        self.nodes, self.inputs, self.outputs, self.name = list(nodes), list(inputs), list(outputs), name


def _read_attribute(buf):
    name, kind, value = "", 0, None
    vals = {}
    for field, _, v in _fields(buf):
        if field == 1:
            name = bytes(v).decode()
        elif field == 20:
            kind = v
        elif field == 2:
            vals[_ATTR_FLOAT] = struct.unpack("<f", bytes(v))[0]
        elif field == 3:
            vals[_ATTR_INT] = v - (1 << 64) if v >> 63 else v
        elif field == 4:
            vals[_ATTR_STRING] = bytes(v)
    if kind in vals:
        value = vals[kind]
    elif vals:  # writers that leave the type out
        value = next(iter(vals.values()))
    return name, value


def _read_node(buf):
    n = Node("", [], [])
    for field, _, v in _fields(buf):
        if field == 1:
            n.inputs.append(bytes(v).decode())
        elif field == 2:
            n.outputs.append(bytes(v).decode())
        elif field == 3:
            n.name = bytes(v).decode()
        elif field == 4:
            n.op_type = bytes(v).decode()
        elif field == 5:
            k, val = _read_attribute(v)
            n.attrs[k] = val
    return n


def _read_value_info(buf):
    name, elem, dims = "", 0, []
    for field, _, v in _fields(buf):
        if field == 1:
            name = bytes(v).decode()
        elif field == 2:  # TypeProto
            for f2, _, v2 in _fields(v):
                if f2 != 1:  # tensor_type
                    continue
                for f3, _, v3 in _fields(v2):
                    if f3 == 1:
                        elem = v3
                    elif f3 == 2:  # TensorShapeProto
                        for f4, _, v4 in _fields(v3):
                            if f4 != 1:
                                continue
                            dim = None
                            for f5, _, v5 in _fields(v4):
                                if f5 == 1:
                                    dim = v5
                                elif f5 == 2:
                                    dim = bytes(v5).decode()
                            dims.append(dim)
    return Value(name, elem, dims)


def read_model(data):
    """Parses ONNX ModelProto bytes (or a file path) into a Model."""
    if isinstance(data, str):
        with open(data, "rb") as f:
            data = f.read()
    graph = None
    for field, wire, v in _fields(data):
        if field == 7 and wire == 2:
            graph = v
    if graph is None:
        raise ValueError("not an ONNX model: no graph")
    model = Model([], [], [])
    initializers = set()
    for field, wire, v in _fields(graph):
        if field == 1:
            model.nodes.append(_read_node(v))
        elif field == 2:
            model.name = bytes(v).decode()
        elif field == 5:  # initializer: only its name matters here (it is not a runtime input)
            for f2, _, v2 in _fields(v):
                if f2 == 8:
                    initializers.add(bytes(v2).decode())
        elif field == 11:
            model.inputs.append(_read_value_info(v))
        elif field == 12:
            model.outputs.append(_read_value_info(v))
    model.inputs = [i for i in model.inputs if i.name not in initializers]
    return model


def _write_value_info(v):
    dims = b""
    for d in v.dims:
        dims += _enc(1, 2, _enc(2, 2, d.encode()) if isinstance(d, str) else _enc(1, 0, int(d)))
    tensor = _enc(1, 0, v.elem_type) + _enc(2, 2, dims)
    return _enc(1, 2, v.name.encode()) + _enc(2, 2, _enc(1, 2, tensor))


def write_model(model, producer="deploy3d_amd"):
    """ONNX ModelProto bytes of a Model (ir_version 7, opset 11, as the reference's exports)."""
    graph = b""
    for n in model.nodes:
        body = b"".join(_enc(1, 2, s.encode()) for s in n.inputs)
        body += b"".join(_enc(2, 2, s.encode()) for s in n.outputs)
        if n.name:
            body += _enc(3, 2, n.name.encode())
        body += _enc(4, 2, n.op_type.encode())
        for k, val in n.attrs.items():
            a = _enc(1, 2, k.encode())
            if isinstance(val, (bytes, bytearray)):
                a += _enc(4, 2, val) + _enc(20, 0, _ATTR_STRING)
            elif isinstance(val, float):
                a += _enc_varint(2 << 3 | 5) + struct.pack("<f", val) + _enc(20, 0, _ATTR_FLOAT)
            else:
                a += _enc(3, 0, int(val)) + _enc(20, 0, _ATTR_INT)
            body += _enc(5, 2, a)
        graph += _enc(1, 2, body)
    graph += _enc(2, 2, model.name.encode())
    graph += b"".join(_enc(11, 2, _write_value_info(v)) for v in model.inputs)
    graph += b"".join(_enc(12, 2, _write_value_info(v)) for v in model.outputs)
    opset = _enc(1, 2, b"") + _enc(2, 0, 11)
    return _enc(1, 0, 7) + _enc(2, 2, producer.encode()) + _enc(7, 2, graph) + _enc(8, 2, opset)


def plugin_node(name, blob, inputs, outputs, version="2.0", node_name=""):
    """The node the reference's ``symbolic()`` functions emit: g.op('TRT_PluginV2', ..., name_s=, data_s=,
    namespace_s=b'', version_s=b'2.0')."""
    return Node("TRT_PluginV2", inputs, outputs,
                dict(name=name.encode(), data=bytes(blob), namespace=b"", version=version.encode()), node_name)


def backbone_model(layers, weights, capacities, n_in, in_channels, grid, dtype=torch.float16, batch=1,
                   densify=False, points=0):
    """The graph the reference's exporter produces for a chain / small DAG of sparse convolutions described by a
    layer table (deploy3d_amd.synth): one SPConvIdx node per indice key, one SPConvMM node per layer, ``Add`` for a
    two-source layer, optionally a BEVDensify node at the end.  Inputs: feats, coors, num_act, spatial_shape - or,
    with ``points`` > 0 (the capacity of the point tensor), points [points, in_channels] float, batch_indices,
    voxel_config and spatial_shape: a SimpleMeanEncoder node then makes the voxels (n_in = its maxNumActOut) and a
    ``Cast`` brings its float means to the backbone's type (the reference's points -> voxels -> backbone graphs)."""
    from .spconv_index import index_blob
    from .spconv_mm import mm_blob
    elem = _TORCH_TO_ELEM[dtype]
    nd = len(grid)
    nodes = []
    if points:
        from .simple_mean import simple_mean_blob
        inputs = [Value("points", FLOAT, [points, in_channels]), Value("batch_indices", INT32, [points]),
                  Value("voxel_config", FLOAT, [6]), Value("spatial_shape", INT32, [batch, 0] + list(grid))]
        nodes.append(plugin_node("SimpleMeanEncoder", simple_mean_blob(n_in),
                                 ["points", "batch_indices", "voxel_config", "spatial_shape"],
                                 ["voxel_means", "coors", "num_act"], node_name="voxels"))
        if dtype == torch.float32:
            first = "voxel_means"
        else:
            nodes.append(Node("Cast", ["voxel_means"], ["feats"], dict(to=elem), name="voxel_cast"))
            first = "feats"
    else:
        inputs = [Value("feats", elem, [n_in, in_channels]), Value("coors", INT32, [n_in, nd + 1]),
                  Value("num_act", INT32, [1]), Value("spatial_shape", INT32, [batch, 0] + list(grid))]
        first = "feats"
    state = {"input": dict(feats=first, coors="coors", num="num_act", shape="spatial_shape", cap=n_in,
                           grid=list(grid))}
    keys = {}
    cur = state["input"]
    for spec, (w, b), cap in zip(layers, weights, capacities):
        name = spec["name"]
        src = spec.get("src")
        if src is None:
            x = cur
        elif "+" in src:
            p, q = (state[s] for s in src.split("+"))
            nodes.append(Node("Add", [p["feats"], q["feats"]], [name + "_sum"], name=name + "_add"))
            x = dict(p, feats=name + "_sum")
        else:
            x = state[src]
        key = spec["key"]
        if key not in keys:
            blob = index_blob(spec["ksize"], spec["stride"], spec["padding"], spec["dilation"], (0,) * nd, cap,
                              spec["subm"], spec.get("transpose", False))
            outs = [key + "_index", key + "_num_index"]
            if not spec["subm"]:
                outs += [key + "_coors", key + "_num_act", key + "_shape"]
            nodes.append(plugin_node("SPConvIdx%dd" % nd, blob, [x["coors"], x["num"], x["shape"]], outs,
                                     node_name=key))
            out_grid = x["grid"] if spec["subm"] else [
                (i + 2 * p - d * (kk - 1) - 1) // st + 1
                for i, kk, st, p, d in zip(x["grid"], spec["ksize"], spec["stride"], spec["padding"], spec["dilation"])]
            keys[key] = dict(index=outs[0], num_index=outs[1], inp=x,
                             out=x if spec["subm"] else dict(coors=outs[2], num=outs[3], shape=outs[4], cap=cap,
                                                             grid=out_grid))
        k = keys[key]
        inverse = bool(spec.get("inverse", False))
        tgt = k["inp"] if inverse else k["out"]
        num_in, num_out = (k["out"]["num"], k["inp"]["num"]) if inverse else (k["inp"]["num"], k["out"]["num"])
        blob = mm_blob(spec["ksize"], spec["cin"], spec["cout"], cap, spec["subm"], inverse, w, b,
                       relu=spec.get("relu", False), act_scale_in=float(spec.get("s_in", 1.0)),
                       act_scale_out=float(spec.get("s_out", 1.0)))
        nodes.append(plugin_node("SPConvMM", blob, [x["feats"], num_in, num_out, k["index"], k["num_index"]], [name],
                                 node_name=name))
        cur = dict(feats=name, coors=tgt["coors"], num=tgt["num"], shape=tgt["shape"], cap=cap, cout=spec["cout"],
                   grid=tgt["grid"])
        state[name] = cur
    outputs = [Value(cur["feats"], elem, [cur["cap"], cur["cout"]]), Value(cur["coors"], INT32, [cur["cap"], nd + 1]),
               Value(cur["num"], INT32, [1])]
    if densify:
        from .bev_densify import densify_blob
        nodes.append(plugin_node("BEVDensify", densify_blob(cur["cout"] * cur["grid"][0]),
                                 [cur["feats"], cur["coors"], cur["num"], cur["shape"]], ["bev"], node_name="bev"))
        outputs.append(Value("bev", elem, []))
    return Model(nodes, inputs, outputs, "sparse_backbone")


# ---------------------------------------------------------------------------
# executor
# ---------------------------------------------------------------------------
class GraphExecutor:
    """Runs the sparse section of an ONNX graph.  Tensors are allocated at the first ``run`` from the shapes of the
    inputs (static capacities) and reused afterwards; ``run`` only enqueues on the current stream."""

    def __init__(self, model, device="cuda"):
        if isinstance(model, (bytes, bytearray, memoryview, str)):
            model = read_model(model)
        self.model = model
        self.device = device
        self.nodes = self._toposort(model)
        self.plugins = {}
        for i, n in enumerate(self.nodes):
            if n.op_type == "TRT_PluginV2":
                name = n.attrs.get("name")
                blob = n.attrs.get("data")
                if not isinstance(name, (bytes, bytearray)) or not isinstance(blob, (bytes, bytearray)):
                    raise ValueError("%r: TRT_PluginV2 node without name / data attributes" % n)
                version = n.attrs.get("version", b"2.0")
                self.plugins[i] = Plugin(bytes(name).decode(), blob, bytes(version).decode())
            elif n.op_type == "Cast":
                if n.attrs.get("to") not in _ELEM_TO_TORCH:
                    raise NotImplementedError("Cast to ONNX element type %r (node %s)" % (n.attrs.get("to"), n.name))
            elif n.op_type != "Add":
                raise NotImplementedError("op type %s (node %s) is outside the sparse section this executor runs"
                                          % (n.op_type, n.name or n.outputs))
        # graph edges: an SPConvMM reads the index tensor that an SPConvIdx node writes
        producer = {out: (i, j) for i, n in enumerate(self.nodes) for j, out in enumerate(n.outputs)}
        linked = set()  # SPConvMM nodes whose link to the rulebook node was accepted
        for i, n in enumerate(self.nodes):
            p = self.plugins.get(i)
            if p is None:
                continue
            if p.name.startswith("SPConvIdx"):
                p.set_option(OPT_PERSISTENT_INDEX, 1)  # the executor owns the index tensor and nobody else writes it
                # a node on the coordinates a strided node wrote works from that node's occupancy map
                src = producer.get(n.inputs[0])
                if src is not None and src[1] == 2 and producer.get(n.inputs[1]) == (src[0], 3) and \
                        src[0] in self.plugins and self.plugins[src[0]].name == p.name:
                    try:
                        p.link_coords(self.plugins[src[0]])
                    except EngineError:
                        pass
            if p.name == "SPConvMM" and len(n.inputs) >= 5:
                src = producer.get(n.inputs[3])
                if src is not None and src[1] == 0 and src[0] in self.plugins and \
                        self.plugins[src[0]].name.startswith("SPConvIdx") and \
                        producer.get(n.inputs[4]) == (src[0], 1):
                    try:
                        p.link_rulebook(self.plugins[src[0]])
                        linked.add(i)
                    except EngineError:
                        pass  # kernel volume or maxNumActOut of the two nodes differ: this node derives its table
        # an index tensor that only linked forward convolutions read (not a graph output, no other consumer) need
        # not be written at all
        outputs = {v.name for v in model.outputs}
        for i, n in enumerate(self.nodes):
            p = self.plugins.get(i)
            if p is None or not p.name.startswith("SPConvIdx") or n.outputs[0] in outputs:
                continue
            readers = [(j, m) for j, m in enumerate(self.nodes) if n.outputs[0] in m.inputs]
            if readers and all(j in linked and self.plugins[j].name == "SPConvMM" and len(m.inputs) >= 5 and
                               m.inputs[3] == n.outputs[0] and m.inputs[4] == n.outputs[1] and
                               not self._inverse(m) for j, m in readers):
                p.set_option(OPT_INDEX_UNUSED, 1)
        self._bound = None

    @staticmethod
    def _inverse(node):
        """The `inverse` byte of an SPConvMM attribute blob (trt/spconv/mm_trt.cu:27-37: 4 x int32, subM, inverse)."""
        blob = node.attrs.get("data", b"")
        return len(blob) > 17 and blob[17] != 0

    @staticmethod
    def _toposort(model):
        known = {v.name for v in model.inputs}
        pending = list(model.nodes)
        order = []
        while pending:
            ready = [n for n in pending if all(i in known or i == "" for i in n.inputs)]
            if not ready:
                raise ValueError("graph has a cycle or reads undefined values: %r" % pending[0])
            for n in ready:
                order.append(n)
                known.update(n.outputs)
            pending = [n for n in pending if n not in ready]
        return order

    def _bind(self, inputs):
        """Descriptors, output tensors and workspaces of every node, from the shapes of the inputs."""
        values = dict(inputs)
        plan = []
        for i, n in enumerate(self.nodes):
            ins = [values[name] for name in n.inputs]
            if n.op_type == "Add":
                out = torch.empty_like(ins[0])
                values[n.outputs[0]] = out
                plan.append(("add", ins, out))
                continue
            if n.op_type == "Cast":
                out = torch.empty(ins[0].shape, dtype=_ELEM_TO_TORCH[n.attrs["to"]], device=self.device)
                values[n.outputs[0]] = out
                plan.append(("cast", ins, out))
                continue
            p = self.plugins[i]
            in_descs = [TensorDesc.of_tensor(t) for t in ins]
            out_descs = p.output_descs(in_descs)
            outs = [torch.empty(d.shape(), dtype=_dtype_of(d), device=self.device) for d in out_descs]
            p.configure(in_descs, out_descs)
            nbytes = p.workspace_size(in_descs, out_descs)
            ws = torch.empty(max(1, nbytes), dtype=torch.uint8, device=self.device) if nbytes else None
            for name, t in zip(n.outputs, outs):
                values[name] = t
            plan.append(("plugin", p, in_descs, out_descs, ins, outs, ws))
        self._bound = dict(shapes={k: (tuple(v.shape), v.dtype, v.data_ptr()) for k, v in inputs.items()},
                           values=values, plan=plan)

    def run(self, **inputs):
        """inputs: name -> device tensor for every graph input (a zero-element tensor for a spatial shape).
        Returns name -> tensor for every graph output (the executor's own buffers, overwritten by the next run)."""
        missing = [v.name for v in self.model.inputs if v.name not in inputs]
        if missing:
            raise ValueError("missing graph inputs: %s" % missing)
        sig = {k: (tuple(v.shape), v.dtype, v.data_ptr()) for k, v in inputs.items()}
        if self._bound is None or self._bound["shapes"] != sig:
            self._bind(inputs)
        for step in self._bound["plan"]:
            if step[0] == "add":
                torch.add(step[1][0], step[1][1], out=step[2])
            elif step[0] == "cast":
                step[2].copy_(step[1][0])
            else:
                _, p, in_descs, out_descs, ins, outs, ws = step
                p.enqueue(in_descs, out_descs, ins, outs, ws)
        return {v.name: self._bound["values"][v.name] for v in self.model.outputs}


    def run_scheduled(self, **inputs):
        """``run`` through a native schedule (d3d_schedule_*): every node becomes a step that waits for the steps
        its inputs come from; rulebook nodes get lanes of their own (strided 1, SubM 2), everything else runs on
        the current stream.  Graphs of plugin nodes only (an ``Add`` needs the step-by-step ``run``)."""
        sig = {k: (tuple(v.shape), v.dtype, v.data_ptr()) for k, v in inputs.items()}
        if self._bound is None or self._bound["shapes"] != sig:
            self.run(**inputs)  # binds, and brings every operator's buffers into being
        if "schedule" not in self._bound:
            if any(step[0] != "plugin" for step in self._bound["plan"]):
                raise NotImplementedError("a schedule holds plugin steps only")
            sched = Schedule(lanes=3)
            made = {}  # tensor name -> step that writes it
            plugin_nodes = [n for n in self.nodes if n.op_type == "TRT_PluginV2"]
            for n, (_, p, in_descs, out_descs, ins, outs, ws) in zip(plugin_nodes, self._bound["plan"]):
                lane = 0
                if p.name.startswith("SPConvIdx"):
                    lane = 2 if len(n.attrs["data"]) >= 2 and n.attrs["data"][-2] != 0 else 1   # the subM byte
                after = sorted({made[name] for name in n.inputs if name in made})
                step = sched.add(p, in_descs, out_descs, ins, outs, ws, lane=lane, after=after)
                for name in n.outputs:
                    made[name] = step
            self._bound["schedule"] = sched
        self._bound["schedule"].run()
        return {v.name: self._bound["values"][v.name] for v in self.model.outputs}


def _dtype_of(desc):
    from .plugin import torch_dtype
    return torch_dtype(desc.dtype)
