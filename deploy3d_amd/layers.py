"""Sparse-convolution layers wired the way the reference wires its plugins into a
network: one rulebook per indice key, shared by every convolution that names
the key (reference: InferSpConvModule, tests/cylinder/test_middle_encoder.py:8-96).

Tensors and workspaces are allocated once at their static capacities; a forward
pass only enqueues kernels on the current stream (no host synchronisation), so
it can be captured into a HIP graph.
"""
import numpy as np
import torch

from .plugin import OPT_INDEX_UNUSED, OPT_PERSISTENT_INDEX, Plugin, Schedule, TensorDesc
from .spconv_index import index_blob
from .spconv_mm import mm_blob


def _round_up(v, m):
    return (v + m - 1) // m * m


class SparseTensor:
    """Features + coordinates + live count + grid, all at static capacity."""

    def __init__(self, feats, coors, num_act, grid, batch=1, producer=None):
        self.feats, self.coors, self.num_act, self.grid, self.batch = feats, coors, num_act, list(grid), batch
        self.producer = producer  # the strided SPConvIdx operator that wrote coors / num_act, if one did

    @property
    def capacity(self):
        return self.coors.shape[0]


def densify(x):
    """[B, C*Z, Y, X] map of a SparseTensor (the step between a sparse backbone and a 2-D head,
    reference: deploy3d/symfun/ops/spconv/bev_densify.py:18-45)."""
    from .bev_densify import bev_densify
    z, y, xdim = x.grid
    shape = torch.empty((x.batch, 0, z, y, xdim), dtype=torch.int32, device=x.feats.device)
    return bev_densify(x.feats, x.coors, x.num_act, shape, x.feats.shape[1] * z)


class Rulebook:
    """Outputs of one SPConvIdx enqueue, cached under an indice key."""

    def __init__(self, index, num_index, out_coors, num_act_out, out_grid, in_tensor, plugin=None):
        self.index, self.num_index = index, num_index
        self.plugin = plugin  # the SPConvIdx operator that wrote it: convolutions of the key link to it
        self.out_coors, self.num_act_out, self.out_grid = out_coors, num_act_out, out_grid
        self.in_coors, self.num_act_in, self.in_grid = in_tensor.coors, in_tensor.num_act, in_tensor.grid
        self.in_producer = in_tensor.producer


class SparseConvLayer:
    """One convolution: an SPConvMM plugin plus (for the first user of a key) an SPConvIdx plugin."""

    def __init__(self, spec, weight, bias, max_num_act_out, dtype=torch.float16, device="cuda", extensions=True):
        self.spec = spec
        # extensions=False: the operators as a caller of the reference's plugins would use them - no links between
        # them, no persistent index tensor - so every enqueue fills its whole index tensor and every convolution
        # derives its table from the tensor it is handed
        self.extensions = extensions
        self.max_num_act_out = int(max_num_act_out)
        self.dtype = dtype
        self.device = device
        nd = len(spec["ksize"])
        self.idx_plugin = Plugin("SPConvIdx%dd" % nd, index_blob(
            spec["ksize"], spec["stride"], spec["padding"], spec["dilation"], (0,) * nd, self.max_num_act_out,
            spec["subm"], spec.get("transpose", False)))
        # the index tensor is allocated once below and written by this operator only
        if extensions:
            self.idx_plugin.set_option(OPT_PERSISTENT_INDEX, 1)
        self.mm_plugin = Plugin("SPConvMM", mm_blob(
            spec["ksize"], spec["cin"], spec["cout"], self.max_num_act_out, spec["subm"], spec.get("inverse", False),
            weight, bias, relu=spec.get("relu", False), act_scale_in=float(spec.get("s_in", 1.0)),
            act_scale_out=float(spec.get("s_out", 1.0))))
        self._idx_state = None
        self._mm_state = None

    # -- rulebook ---------------------------------------------------------------
    def build_rulebook(self, x):
        nd = len(self.spec["ksize"])
        if self._idx_state is None or self._idx_state["cap"] != x.capacity:
            in_descs = [TensorDesc.of_tensor(x.coors), TensorDesc.of_tensor(x.num_act),
                        TensorDesc.of((x.batch, 0) + tuple(x.grid), torch.int32)]
            out_descs = self.idx_plugin.output_descs(in_descs)
            outs = [torch.empty(d.shape(), dtype=torch.int32, device=self.device) if 0 not in d.shape() else None
                    for d in out_descs]
            ws = torch.empty(max(1, self.idx_plugin.workspace_size(in_descs, out_descs)), dtype=torch.uint8,
                             device=self.device)
            self._idx_state = dict(cap=x.capacity, in_descs=in_descs, out_descs=out_descs, outs=outs, ws=ws)
            # a SubM rulebook on the outputs of a strided one reuses that operator's occupancy map; a strided one
            # derives the occupancy of its own map from it
            if self.extensions and not self.spec.get("inverse", False):
                self.idx_plugin.link_coords(x.producer)
            self.idx_plugin.configure(in_descs, out_descs)  # reserves the maps an operator keeps between passes
        st = self._idx_state
        self.idx_plugin.enqueue(st["in_descs"], st["out_descs"], [x.coors, x.num_act, None], st["outs"], st["ws"])
        outs = st["outs"]
        if self.spec["subm"]:  # SubM: outputs sit on the input voxels (test_middle_encoder.py:68-69)
            return Rulebook(outs[0], outs[1], x.coors, x.num_act, x.grid, x, self.idx_plugin)
        out_grid = list(st["out_descs"][4].shape()[2:])
        return Rulebook(outs[0], outs[1], outs[2], outs[3], out_grid, x, self.idx_plugin)

    # -- convolution ------------------------------------------------------------
    def forward(self, x, rulebooks):
        key = self.spec["key"]
        rb = rulebooks.get(key)
        if rb is None:
            rb = rulebooks[key] = self.build_rulebook(x)
        feats = x.feats
        inverse = bool(self.spec.get("inverse", False))
        # an inverse convolution runs the rulebook backwards: its inputs sit on the rulebook's output sites and its
        # outputs on the rulebook's input sites (reference: SPConvMM `inverse`, trt/spconv/mm_trt.cu:171-176)
        num_in, num_out = (rb.num_act_out, rb.num_act_in) if inverse else (rb.num_act_in, rb.num_act_out)
        if self._mm_state is None or self._mm_state["in_rows"] != feats.shape[0] or self._mm_state["rb"] is not rb.plugin:
            in_descs = [TensorDesc.of_tensor(t) for t in (feats, num_in, num_out, rb.index, rb.num_index)]
            out_descs = self.mm_plugin.output_descs(in_descs)
            if self.extensions:
                self.mm_plugin.link_rulebook(rb.plugin)
            self.mm_plugin.configure(in_descs, out_descs)
            out = torch.empty(out_descs[0].shape(), dtype=self.dtype, device=self.device)
            self._mm_state = dict(in_rows=feats.shape[0], in_descs=in_descs, out_descs=out_descs, out=out, rb=rb.plugin)
        st = self._mm_state
        self.mm_plugin.enqueue(st["in_descs"], st["out_descs"], [feats, num_in, num_out, rb.index, rb.num_index],
                               [st["out"]])
        if inverse:
            return SparseTensor(st["out"], rb.in_coors, rb.num_act_in, rb.in_grid, x.batch, rb.in_producer)
        return SparseTensor(st["out"], rb.out_coors, rb.num_act_out, rb.out_grid, x.batch,
                            x.producer if self.spec["subm"] else rb.plugin)


class SparseBackbone:
    """A chain (or small DAG, via ``src``) of SparseConvLayers sharing rulebooks by indice key.

    Rulebooks depend on coordinates only, convolutions on features and on their rulebook.  With ``overlap``
    (the default) the strided rulebooks, which feed each other, are enqueued on a second HIP stream, the SubM
    rulebooks on a third, and every convolution waits for the event of its own rulebook: the latency-bound index
    kernels of later stages run beside the MFMA kernels of earlier ones.  A SubM rulebook is ordered behind the
    strided rulebook that wrote its coordinates through an event of the MAIN stream, recorded where the main
    stream waited for that rulebook (an event edge straight from one side stream to the other made
    hipStreamEndCapture crash in the runtime).  A strided rulebook in turn starts behind the SubM rulebook of the
    stage before it, which the convolutions need first.  The side streams fork from and join into the caller's current
    stream, so a forward pass can still be captured into one HIP graph (it then holds parallel branches).

    ``extensions=False`` runs the operators as the reference's contract alone describes them (no links, no options).

    ``index_tensors=False`` tells the rulebook operators that nothing outside this runner reads their index tensors
    (``Rulebook.index`` is then unspecified): they write the tables the convolutions read and skip the compaction.
    """

    def __init__(self, layers, weights, capacities, dtype=torch.float16, device="cuda", overlap=True,
                 index_tensors=True, extensions=True):
        self.specs = layers
        self.layers = [SparseConvLayer(s, w, b, cap, dtype=dtype, device=device, extensions=extensions)
                       for s, (w, b), cap in zip(layers, weights, capacities)]
        # every convolution reads the rulebook of the first layer that names its indice key: link them now, so
        # that already the first pass has the rulebook operators write the tables
        owner = {}
        for spec, lyr in zip(layers, self.layers):
            first = owner.setdefault(spec["key"], lyr)
            if extensions:
                lyr.mm_plugin.link_rulebook(first.idx_plugin)
        # index_tensors=False: this runner is the only reader of the index tensors and its convolutions read the
        # linked tables, so the rulebook operators may leave the tensors unwritten (D3D_OPT_INDEX_UNUSED) - except
        # for a key that an inverse convolution uses, which works from the tensor
        if not index_tensors and extensions:
            inverse_keys = {spec["key"] for spec in layers if spec.get("inverse", False)}
            for key, lyr in owner.items():
                if key not in inverse_keys:
                    lyr.idx_plugin.set_option(OPT_INDEX_UNUSED, 1)
        self.index_tensors = index_tensors
        self.overlap = overlap
        self._side = None

    def forward(self, x):
        main = side = None
        if self.overlap:
            if self._side is None:  # strided rulebooks feed each other; SubM rulebooks hang off them
                self._side = {False: torch.cuda.Stream(), True: torch.cuda.Stream()}
            main, side = torch.cuda.current_stream(), self._side
            fork = torch.cuda.Event()
            fork.record(main)
            for st in set(side.values()):
                st.wait_event(fork)
        rulebooks = {}
        inputs = {}
        pending = {}
        strided_coords = {}  # coordinate tensor written by a strided rulebook -> main-stream event after its wait
        subm_done = None     # main-stream event behind the wait for the latest SubM rulebook on strided coordinates
        outs = {"input": x}
        cur = x
        for spec, lyr in zip(self.specs, self.layers):
            src = spec.get("src")
            if src is None:
                inp = cur
            elif "+" in src:
                a, b = (outs[s] for s in src.split("+"))
                inp = SparseTensor(a.feats + b.feats, a.coors, a.num_act, a.grid, a.batch, a.producer)
            else:
                inp = outs[src]
            inputs[spec["name"]] = inp
            key = spec["key"]
            if side is not None and key not in rulebooks:
                subm = bool(spec["subm"])
                st = side[subm]
                if subm and id(inp.coors) in strided_coords:
                    # order behind the strided rulebook that wrote these coordinates, carried by an event of the
                    # main stream (recorded when the main stream waited for that rulebook)
                    st.wait_event(strided_coords[id(inp.coors)])
                if not subm and subm_done is not None:
                    # The SubM rulebook of the stage before (same input coordinates) is what the convolutions wait
                    # for next; this one is not needed before that stage's convolutions are through.  Running both at
                    # once stretches both, so this one starts when that one is done - again through an event of the
                    # main stream (0.75 -> 0.72 ms per pass of the VoxelNet backbone; making the FIRST strided
                    # rulebook wait for the input's SubM rulebook as well measured slower).
                    st.wait_event(subm_done)
                with torch.cuda.stream(st):
                    rb = rulebooks[key] = lyr.build_rulebook(inp)
                    pending[key] = torch.cuda.Event()
                    pending[key].record(st)
            if key in pending:
                main.wait_event(pending.pop(key))
                seen = torch.cuda.Event()
                seen.record(main)
                if not spec["subm"]:
                    strided_coords[id(rulebooks[key].out_coors)] = seen
                elif id(inp.coors) in strided_coords:
                    subm_done = seen
            cur = lyr.forward(inp, rulebooks)
            outs[spec["name"]] = cur
        self.rulebooks = rulebooks
        self.inputs = inputs    # layer name -> the SparseTensor it read
        self.outputs = outs
        return cur


    # -- the pass as one native call -------------------------------------------------------------------------
    def build_schedule(self, x):
        """Records the pass on ``x`` as a native schedule (d3d_schedule_*): convolutions on lane 0 (the caller's
        stream), strided rulebooks on lane 1, SubM rulebooks on lane 2; a convolution waits for its rulebook, a SubM
        rulebook for the strided rulebook that wrote its coordinates (directly - no detour through the main
        stream, which only stream capture needs).  Runs one ordinary pass first so that every buffer exists."""
        if any("+" in (spec.get("src") or "") for spec in self.specs):
            raise NotImplementedError("a schedule holds operator steps only; this chain adds feature maps in between")
        self.forward(x)
        sched = Schedule(lanes=3)
        rb_step, by_plugin = {}, {}
        for spec, lyr in zip(self.specs, self.layers):
            inp = self.inputs[spec["name"]]
            key = spec["key"]
            rb = self.rulebooks[key]
            if key not in rb_step:
                st = lyr._idx_state
                after = [by_plugin[id(inp.producer)]] if inp.producer is not None and id(inp.producer) in by_plugin else []
                rb_step[key] = sched.add(lyr.idx_plugin, st["in_descs"], st["out_descs"], [inp.coors, inp.num_act, None],
                                         st["outs"], st["ws"], lane=2 if spec["subm"] else 1, after=after)
                by_plugin[id(lyr.idx_plugin)] = rb_step[key]
            inverse = bool(spec.get("inverse", False))
            num_in, num_out = (rb.num_act_out, rb.num_act_in) if inverse else (rb.num_act_in, rb.num_act_out)
            st = lyr._mm_state
            sched.add(lyr.mm_plugin, st["in_descs"], st["out_descs"], [inp.feats, num_in, num_out, rb.index, rb.num_index],
                      [st["out"]], None, lane=0, after=[rb_step[key]])
        self._schedule = (sched, (x.feats.data_ptr(), x.coors.data_ptr(), x.num_act.data_ptr()))
        return sched

    def forward_scheduled(self, x):
        """The pass through the native schedule (recorded at the first call, and again when ``x`` is another set of
        buffers); same output tensors as ``forward``."""
        sig = (x.feats.data_ptr(), x.coors.data_ptr(), x.num_act.data_ptr())
        if getattr(self, "_schedule", None) is None or self._schedule[1] != sig:
            self.build_schedule(x)
        self._schedule[0].run()
        return self.outputs[self.specs[-1]["name"]]


def plan_capacities(layers, n_in, counts=None):
    """Static row capacity (maxNumActOut) of every layer's output.

    SubM layers keep the capacity of their input.  A strided layer's capacity is
    the measured output count rounded up to 1024 when ``counts[name]`` is given,
    else the safe bound 8x the input capacity.  An inverse layer outputs on the sites its key's
    rulebook was built from, so it takes that input's capacity.
    """
    caps = []
    cap_of = {"input": n_in}
    key_in_cap = {}  # capacity of the input a key's rulebook was built on: what an inverse layer of the key outputs
    cur = n_in
    for spec in layers:
        src = spec.get("src")
        if src is not None:
            cur = cap_of[src.split("+")[0]]
        key_in_cap.setdefault(spec["key"], cur)
        if spec.get("inverse", False):
            cap = key_in_cap[spec["key"]]
        elif spec["subm"]:
            cap = cur
        elif counts is not None and spec["name"] in counts:
            cap = _round_up(int(counts[spec["name"]]), 1024)
        else:
            cap = 8 * cur
        caps.append(cap)
        cap_of[spec["name"]] = cap
        cur = cap
    return caps


def measure_output_counts(layers, coords, grid, batch=1, device="cuda"):
    """Sizing pre-pass (set-up time, synchronises): live output count of every strided layer of a chain,
    found by running its rulebook at the safe capacity min(8 * inputs, output cells)."""
    from .spconv_index import spconv_index_nd
    counts = {}
    cur = torch.from_numpy(np.ascontiguousarray(coords)).to(device)
    cur_grid = list(grid)
    seen = set()
    for spec in layers:
        if spec["subm"] or spec["key"] in seen:
            continue
        seen.add(spec["key"])
        n = cur.shape[0]
        out_grid = [(i + 2 * p - d * (k - 1) - 1) // s + 1 for i, k, s, p, d in
                    zip(cur_grid, spec["ksize"], spec["stride"], spec["padding"], spec["dilation"])]
        cap_out = int(min(8 * n, batch * int(np.prod(out_grid))))
        num = torch.tensor([n], dtype=torch.int32, device=device)
        shape = torch.empty((batch, 0) + tuple(cur_grid), dtype=torch.int32, device=device)
        _, _, out_coors, num_out, _ = spconv_index_nd(cur, num, shape, spec["ksize"], spec["stride"], spec["padding"],
                                                      spec["dilation"], (0,) * len(out_grid), cap_out, False, False)
        m = int(num_out.item())
        counts[spec["name"]] = m
        cur = out_coors[:m].contiguous()
        cur_grid = out_grid
    return counts


def make_input(coords, feats, grid, dtype=torch.float16, device="cuda", capacity=None, batch=1):
    """Device tensors at capacity.  For torch.int8, ``feats`` must already be quantized int8 values."""
    n = len(coords)
    capacity = capacity or n
    c = torch.zeros((capacity, coords.shape[1]), dtype=torch.int32, device=device)
    c[:n] = torch.from_numpy(np.ascontiguousarray(coords)).to(device)
    f = torch.zeros((capacity, feats.shape[1]), dtype=dtype, device=device)
    f[:n] = torch.from_numpy(np.ascontiguousarray(feats)).to(device=device, dtype=dtype)
    num = torch.tensor([n], dtype=torch.int32, device=device)
    return SparseTensor(f, c, num, grid, batch)
