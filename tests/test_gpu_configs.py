"""The benchmark configurations end to end on the GPU, against the CPU oracle
at sizes it finishes in seconds, and through size-independent properties at
full size."""
import numpy as np
import pytest
import torch

import chain
from oracle import oracle

pytestmark = pytest.mark.gpu


def run_gpu_chain(cfg, counts=None):
    from deploy3d_amd import layers
    specs = cfg["layers"]
    n = len(cfg["coords"])
    if counts is None:
        counts = layers.measure_output_counts(specs, cfg["coords"], cfg["grid"])
    caps = layers.plan_capacities(specs, n, counts)
    dtype = chain.TORCH_DTYPE[cfg["dtype"]]
    net = layers.SparseBackbone(specs, cfg["weights"], caps, dtype=dtype)
    x = layers.make_input(cfg["coords"], cfg["feats"], cfg["grid"], dtype=dtype)
    y = net.forward(x)
    torch.cuda.synchronize()
    return net, x, y


def compare_chain(cfg, net, ref, tol_scale=1.0):
    """Every layer: same live count, same coordinate set, features within tolerance after sorting by coordinate."""
    for spec in cfg["layers"]:
        out = net.outputs[spec["name"]]
        want = ref[spec["name"]]
        n_out = int(out.num_act.item())
        assert n_out == len(want["coords"]), spec["name"]
        gc, gf = chain.sort_rows(out.coors[:n_out].cpu().numpy(), out.feats[:n_out].float().cpu().numpy())
        rc, rf = chain.sort_rows(want["coords"], want["exact"])
        np.testing.assert_array_equal(gc, rc, err_msg=spec["name"])
        rms = float(np.sqrt(np.mean(rf ** 2))) + 1e-30
        err = float(np.abs(gf - rf).max())
        if cfg["dtype"] == "float32":
            assert (np.abs(gf - rf) <= 1e-4 * (np.abs(rf) + rms)).all(), (spec["name"], err, rms)
        else:
            assert err <= 2e-2 * rms * tol_scale, (spec["name"], err, rms)


@pytest.mark.parametrize("config,n", [(3, 12000), (5, 20000), (1, 5000), (2, 8000)])
def test_unwritten_index_tensors_give_the_same_pass(engine, config, n):
    """D3D_OPT_INDEX_UNUSED (index_tensors=False): the rulebook operators write tables and tile masks in the probe
    pass and leave the index tensors unwritten.  Every layer's features, coordinates and live count must equal the
    full pass bit for bit - with rows in rank order and shuffled (config 1 and the first stage of config 3 feed
    unsorted voxels), with fewer live voxels in the same buffers, eager and under HIP-graph replay; numIndex is
    still written."""
    from deploy3d_amd import layers, synth
    cfg = {1: synth.config1, 2: synth.config2, 3: synth.config3, 5: synth.config5}[config](n)
    specs, weights = cfg["layers"], cfg["weights"]
    n = len(cfg["coords"])
    counts = layers.measure_output_counts(specs, cfg["coords"], cfg["grid"])
    caps = layers.plan_capacities(specs, n, counts)
    dtype = chain.TORCH_DTYPE[cfg["dtype"]]
    full = layers.SparseBackbone(specs, weights, caps, dtype=dtype, overlap=False)
    lean = layers.SparseBackbone(specs, weights, caps, dtype=dtype, overlap=False, index_tensors=False)
    x = layers.make_input(cfg["coords"], cfg["feats"], cfg["grid"], dtype=dtype)

    def same():
        for spec in specs:
            a, b = full.outputs[spec["name"]], lean.outputs[spec["name"]]
            m = int(a.num_act.item())
            assert m == int(b.num_act.item()), spec["name"]
            assert torch.equal(a.coors[:m], b.coors[:m]), spec["name"]
            assert torch.equal(a.feats, b.feats), spec["name"]
        for key, rb in full.rulebooks.items():
            assert int(rb.num_index.item()) == int(lean.rulebooks[key].num_index.item()), key

    for live in (n, n // 3, n):
        x.num_act.fill_(live)
        full.forward(x)
        lean.forward(x)
        torch.cuda.synchronize()
        same()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            y = lean.forward(x)
        for _ in range(3):
            y.feats.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            same()


@pytest.mark.parametrize("config,n,index_tensors", [(3, 12000, True), (3, 12000, False), (2, 20000, True)])
def test_native_schedule_equals_the_stream_runner(engine, config, n, index_tensors):
    """d3d_schedule_*: the pass recorded once and enqueued by one native call on three lanes gives, bit for bit,
    the features, coordinates and index tensors of the same runner enqueuing operator by operator - over passes of
    different live counts - and refuses to run on a capturing stream."""
    from deploy3d_amd import EngineError, layers, synth
    cfg = (synth.config3 if config == 3 else synth.config2)(n)
    specs, weights = cfg["layers"], cfg["weights"]
    n = len(cfg["coords"])
    counts = layers.measure_output_counts(specs, cfg["coords"], cfg["grid"])
    caps = layers.plan_capacities(specs, n, counts)
    plain = layers.SparseBackbone(specs, weights, caps, overlap=False, index_tensors=index_tensors)
    sched = layers.SparseBackbone(specs, weights, caps, overlap=False, index_tensors=index_tensors)
    x = layers.make_input(cfg["coords"], cfg["feats"], cfg["grid"])
    for live in (n, n // 3, n):
        x.num_act.fill_(live)
        plain.forward(x)
        y = sched.forward_scheduled(x)
        torch.cuda.synchronize()
        assert len(sched._schedule[0]) == len(specs) + len(sched.rulebooks)
        assert y is sched.outputs[specs[-1]["name"]]
        for spec in specs:
            a, b = plain.outputs[spec["name"]], sched.outputs[spec["name"]]
            k = int(a.num_act.item())
            assert k == int(b.num_act.item()), spec["name"]
            assert torch.equal(a.feats, b.feats) and torch.equal(a.coors[:k], b.coors[:k]), spec["name"]
        if index_tensors:
            for key, rb in plain.rulebooks.items():
                assert torch.equal(rb.index, sched.rulebooks[key].index), key
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            x.num_act.fill_(n)
            with pytest.raises(EngineError) as e:
                sched._schedule[0].run()
    assert e.value.status == -1


def test_schedule_on_one_lane_and_back_to_back_runs(engine):
    """A schedule built by hand on a single lane (the caller's stream only, no stream or event of its own), run
    several times back to back without a synchronisation in between on a non-default stream: every run gives the
    step-by-step result, and work enqueued behind a run on that stream sees the run's output."""
    from deploy3d_amd import layers, synth
    from deploy3d_amd.plugin import Schedule
    cfg = synth.config2(20000)
    specs, weights = cfg["layers"], cfg["weights"]
    n = len(cfg["coords"])
    caps = layers.plan_capacities(specs, n, layers.measure_output_counts(specs, cfg["coords"], cfg["grid"]))
    net = layers.SparseBackbone(specs, weights, caps, overlap=False)
    x = layers.make_input(cfg["coords"], cfg["feats"], cfg["grid"])
    y = net.forward(x)
    torch.cuda.synchronize()
    want = y.feats.clone()
    lyr, rb = net.layers[0], net.rulebooks[specs[0]["key"]]
    sched = Schedule(lanes=1)
    st = lyr._idx_state
    a = sched.add(lyr.idx_plugin, st["in_descs"], st["out_descs"], [x.coors, x.num_act, None], st["outs"], st["ws"])
    st = lyr._mm_state
    b = sched.add(lyr.mm_plugin, st["in_descs"], st["out_descs"],
                  [x.feats, rb.num_act_in, rb.num_act_out, rb.index, rb.num_index], [st["out"]], after=[a])
    assert (a, b) == (0, 1)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        copies = []
        for _ in range(4):
            y.feats.zero_()
            sched.run()
            copies.append(y.feats.clone())      # ordered behind the run on the same stream
    stream.synchronize()
    for c in copies:
        assert torch.equal(c, want)


def test_down_up_chain_with_inverse_convolution(engine):
    """An encoder-decoder wiring through the layer runner: strided down (key d), SubM at the lower resolution, then
    the inverse convolution of key d back onto the input sites, then a SubM that shares the first layer's key.  The
    inverse layer's outputs carry the coordinates, live count, grid and capacity of the rulebook's INPUT side
    (reference: SPConvMM `inverse`, trt/spconv/mm_trt.cu:171-176); every layer against the oracle chain."""
    from deploy3d_amd import synth
    grid, n = (16, 96, 96), 5000
    coords = synth.coords_lidar(synth.seed(0, 0), grid, n)
    n = len(coords)
    feats = synth.normal(synth.seed(0, 1), (n, 16))
    specs = [
        synth.layer("s0", "subm0", True, (3, 3, 3), 16, 16, padding=(1, 1, 1)),
        synth.layer("down", "d", False, (3, 3, 3), 16, 32, stride=(2, 2, 2), padding=(1, 1, 1)),
        synth.layer("mid", "subm1", True, (3, 3, 3), 32, 32, padding=(1, 1, 1)),
        dict(synth.layer("up", "d", False, (3, 3, 3), 32, 16, stride=(2, 2, 2), padding=(1, 1, 1)), inverse=True),
        synth.layer("s1", "subm0", True, (3, 3, 3), 16, 16, padding=(1, 1, 1)),
    ]
    cfg = dict(coords=coords, feats=feats, grid=grid, dtype="float16", layers=specs,
               weights=[synth.layer_weights(0, i, s) for i, s in enumerate(specs)])
    ref = chain.oracle_chain(cfg)
    net, x, y = run_gpu_chain(cfg, counts={"down": len(ref["down"]["coords"])})
    compare_chain(cfg, net, ref)
    up = net.outputs["up"]
    assert up.grid == list(grid) and up.coors.data_ptr() == x.coors.data_ptr() and up.feats.shape == (n, 16)
    assert int(y.num_act.item()) == n


def compare_rulebooks(cfg, net, ref):
    """Every rulebook of the pass against the oracle's, bit for bit in canonical form: output coordinates sorted,
    gather and scatter ids relabelled by the rank of their coordinate, triples (tap, gather, scatter) sorted."""
    for key, rb in net.rulebooks.items():
        name = next(s["name"] for s in cfg["layers"] if s["key"] == key)
        n_out = int(rb.num_act_out.item())
        ni = int(rb.num_index.item())
        c_got, t_got = chain.canonical_pairs(rb.index.cpu().numpy(), ni, rb.in_coors.cpu().numpy(),
                                             int(rb.num_act_in.item()), rb.out_coors.cpu().numpy(), n_out)
        orb = ref["_rulebooks"][key]
        c_ref, t_ref = chain.canonical_pairs(orb["index"], orb["num_index"], orb["in_coors"], len(orb["in_coors"]),
                                             orb["out_coors"], orb["num_act_out"])
        np.testing.assert_array_equal(c_got, c_ref, err_msg=key)
        np.testing.assert_array_equal(t_got, t_ref, err_msg=key)
        assert len(t_got) == ref[name]["pairs"], key
        assert ni % 128 == 0


def test_config1_subm_fp32_20k(engine):
    """BASELINE config 1 at full size: 20 000 voxels, SubM 3x3x3 16->16 fp32; index tensor bit-exact."""
    from deploy3d_amd import synth
    cfg = synth.config1()
    net, x, y = run_gpu_chain(cfg)
    ref = chain.oracle_chain(cfg)
    rb = net.rulebooks["subm"]
    orb = oracle.rulebook(cfg["coords"], 20000, [1] + list(cfg["grid"]), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1),
                          20000, True)
    np.testing.assert_array_equal(rb.index.cpu().numpy(), orb["index"])
    assert int(rb.num_index.item()) == orb["num_index"]
    compare_chain(cfg, net, ref)


def test_config2_strided_fp16_60k(engine):
    """BASELINE config 2 at full size: 60 000 voxels, SpConv k3 s2 p1 32->64 fp16."""
    from deploy3d_amd import synth
    cfg = synth.config2()
    net, x, y = run_gpu_chain(cfg)
    ref = chain.oracle_chain(cfg, threads=8)
    rb = net.rulebooks["down"]
    n_out = int(rb.num_act_out.item())
    orb = oracle.rulebook(cfg["coords"], 60000, [1, 21, 720, 720], (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1),
                          8 * 60000, False)
    assert rb.out_grid == [21, 720, 720]
    c_got, t_got = oracle.canonical(rb.index.cpu().numpy(), int(rb.num_index.item()), rb.out_coors.cpu().numpy(), n_out)
    c_ref, t_ref = oracle.canonical(orb["index"], orb["num_index"], orb["out_coors"], orb["num_act_out"])
    np.testing.assert_array_equal(c_got, c_ref)
    np.testing.assert_array_equal(t_got, t_ref)
    compare_chain(cfg, net, ref)


def test_config3_backbone_reduced(engine):
    """Config 3 wiring (13 convs over 8 rulebooks, shared indice keys, fused ReLU) at 12 000 voxels."""
    from deploy3d_amd import synth
    cfg = synth.config3(12000)
    net, x, y = run_gpu_chain(cfg)
    ref = chain.oracle_chain(cfg, threads=8)
    assert len(net.rulebooks) == 8
    compare_rulebooks(cfg, net, ref)
    compare_chain(cfg, net, ref, tol_scale=1.5)  # 13 layers of fp16 rounding drift between two chains


def _config4(n):
    """Config 4 = config 3 quantized: calibration activations from a floating-point oracle pass at the same size."""
    from deploy3d_amd import synth
    cfg3 = synth.config3(n)
    cfg3["dtype"] = "float32"
    ref = chain.oracle_chain(cfg3, threads=8, acc="f32")
    acts = {"input": cfg3["feats"]}
    acts.update({s["name"]: ref[s["name"]]["exact"] for s in cfg3["layers"]})
    return synth.config4(n, acts), ref


def test_config4_int8_backbone_bit_exact(engine):
    """Config 4 at 12 000 voxels: every layer's int8 output equals the oracle's (int32 accumulation + the written
    requantize rule), row for row after sorting by coordinate."""
    from deploy3d_amd import layers
    n = 12000
    cfg, ref = _config4(n)
    want = chain.oracle_chain_int8(cfg, ref)
    counts = layers.measure_output_counts(cfg["layers"], cfg["coords"], cfg["grid"])
    caps = layers.plan_capacities(cfg["layers"], n, counts)
    net = layers.SparseBackbone(cfg["layers"], cfg["weights"], caps, dtype=torch.int8)
    x = layers.make_input(cfg["coords"], cfg["feats_q"], cfg["grid"], dtype=torch.int8)
    net.forward(x)
    torch.cuda.synchronize()
    for spec in cfg["layers"]:
        out = net.outputs[spec["name"]]
        n_out = int(out.num_act.item())
        assert n_out == len(ref[spec["name"]]["coords"])
        gc, gf = chain.sort_rows(out.coors[:n_out].cpu().numpy(), out.feats[:n_out].cpu().numpy())
        rc, rf = chain.sort_rows(ref[spec["name"]]["coords"], want[spec["name"]])
        np.testing.assert_array_equal(gc, rc, err_msg=spec["name"])
        np.testing.assert_array_equal(gf, rf, err_msg=spec["name"])
        assert np.abs(rf.astype(np.int32)).max() >= 100, spec["name"]     # the calibrated range is in use


def test_config3_backbone_full_size_properties(engine):
    """Config 3 at 120 000 voxels: size-independent checks (no oracle pass over 138 GFLOP)."""
    from deploy3d_amd import synth
    cfg = synth.config3()
    net, x, y = run_gpu_chain(cfg)
    grids = {"subm1": [41, 1440, 1440], "down1": [21, 720, 720], "down2": [11, 360, 360], "down3": [5, 180, 180],
             "down4": [2, 180, 180]}
    for key, g in grids.items():
        assert net.rulebooks[key].out_grid == g
    for key, rb in net.rulebooks.items():
        ni = int(rb.num_index.item())
        idx = rb.index[:, :ni]
        live = idx[2] >= 0
        n_in, n_out = int(rb.num_act_in.item()), int(rb.num_act_out.item())
        assert ni % 128 == 0
        assert bool((idx[0][live] < n_in).all()) and bool((idx[1][live] < n_out).all())
        assert bool((rb.index[:, ni:] == -1).all())
        if key.startswith("subm"):
            kvol = 27
            # centre tap is the identity; tap k mirrors tap 26-k with the roles swapped (test_spconv.py:101-108)
            c = idx[:, idx[2] == 13]
            assert c.shape[1] == n_in and bool((c[0] == c[1]).all())
            cnt = torch.bincount(idx[2][live], minlength=kvol)
            assert bool((cnt == cnt.flip(0)).all())
        else:
            # every live output row is hit by at least one pair, coordinates unique and inside the grid
            hit = torch.zeros(n_out, dtype=torch.bool, device="cuda")
            hit[idx[1][live].long()] = True
            assert bool(hit.all())
            oc = rb.out_coors[:n_out].long()
            g = rb.out_grid
            lin = (oc[:, 1] * g[1] + oc[:, 2]) * g[2] + oc[:, 3]
            assert lin.unique().numel() == n_out
            assert bool((oc[:, 1:] >= 0).all()) and bool((oc[:, 1:] < torch.tensor(g, device="cuda")).all())
    # ReLU fused everywhere: no negative output; run-to-run bit reproducible
    first = y.feats.clone()
    assert bool((first >= 0).all()) and bool(torch.isfinite(first.float()).all())
    y2 = net.forward(x)
    torch.cuda.synchronize()
    assert torch.equal(first, y2.feats)
    # positive homogeneity of bias-free ReLU networks does not hold with biases, but per-layer linearity in the
    # input does: conv(2x) - conv(0) == 2 * (conv(x) - conv(0)) for one layer, checked on the widest layer
    lyr = net.layers[10]
    xin = net.outputs["down3"]
    from deploy3d_amd.layers import SparseTensor
    rbs = {"subm4": net.rulebooks["subm4"]}
    def f(feats):
        lyr._mm_state = None
        return lyr.forward(SparseTensor(feats, xin.coors, xin.num_act, xin.grid), rbs).feats.float().clone()
    # ReLU is fused in this layer, so linearity is checked where all three pre-activations are positive
    a, z, b2 = f(xin.feats), f(torch.zeros_like(xin.feats)), f(xin.feats * 2)
    pos = (a > 0) & (z > 0) & (b2 > 0)
    assert pos.float().mean() > 0.05
    lhs, rhs = (b2 - z)[pos], 2 * (a - z)[pos]
    assert float((lhs - rhs).abs().max()) <= 2e-2 * float(rhs.pow(2).mean().sqrt()) + 4e-3


def _bench_module():
    import os
    import sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench
    return bench


@pytest.mark.parametrize("config,min_pairs", [(3, 10_000_000), (5, 3_000_000)])
def test_backbones_at_full_size_against_the_oracle(engine, config, min_pairs):
    """Configs 3 and 5 at their stated sizes (120 000 voxels - the workload of the bench line - and 250 000) against
    one full pass of the CPU oracle with fp32 accumulation (the pass bench.py times as its CPU baseline): every
    rulebook bit for bit in canonical form (10.3 M pairs for config 3, 3.5 M for config 5) and the final features within 2e-2 * rms on
    identical coordinates."""
    import os
    bench = _bench_module()
    from deploy3d_amd import synth
    cfg = synth.config3() if config == 3 else synth.config5()
    net, x, y = run_gpu_chain(cfg)
    ref_rulebooks = {}
    _, _, ref_coords, ref_feats = bench.cpu_pass(cfg, min(16, os.cpu_count() or 1), ref_rulebooks)
    assert set(ref_rulebooks) == set(net.rulebooks)
    pairs = 0
    for key, rb in net.rulebooks.items():
        orb = ref_rulebooks[key]
        n_out = int(rb.num_act_out.item())
        assert n_out == orb["num_act_out"], key
        c_got, t_got = chain.canonical_pairs(rb.index.cpu().numpy(), int(rb.num_index.item()), rb.in_coors.cpu().numpy(),
                                             int(rb.num_act_in.item()), rb.out_coors.cpu().numpy(), n_out)
        c_ref, t_ref = chain.canonical_pairs(orb["index"], orb["num_index"], orb["in_coors"], len(orb["in_coors"]),
                                             orb["out_coors"], orb["num_act_out"])
        np.testing.assert_array_equal(c_got, c_ref, err_msg=key)
        np.testing.assert_array_equal(t_got, t_ref, err_msg=key)
        pairs += len(t_got)
    assert pairs > min_pairs
    n = int(y.num_act.item())
    gc, gf = chain.sort_rows(y.coors[:n].cpu().numpy(), y.feats[:n].float().cpu().numpy())
    rc, rf = chain.sort_rows(ref_coords, np.asarray(ref_feats, dtype=np.float32))
    assert np.array_equal(gc, rc)
    rms = float(np.sqrt(np.mean(rf.astype(np.float64) ** 2)))
    assert float(np.abs(gf - rf).max()) <= 2e-2 * rms


def test_config3_graph_replay_matches_eager(engine):
    """The whole backbone captured in a HIP graph: three replays, each equal to the eager result."""
    from deploy3d_amd import layers, synth
    cfg = synth.config3(30000)
    counts = layers.measure_output_counts(cfg["layers"], cfg["coords"], cfg["grid"])
    caps = layers.plan_capacities(cfg["layers"], 30000, counts)
    net = layers.SparseBackbone(cfg["layers"], cfg["weights"], caps)
    x = layers.make_input(cfg["coords"], cfg["feats"], cfg["grid"])
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        y = net.forward(x)
        y = net.forward(x)
        stream.synchronize()
        eager = y.feats.clone()
        n_eager = int(y.num_act.item())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            y = net.forward(x)
        for _ in range(3):
            y.feats.zero_()
            y.num_act.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert int(y.num_act.item()) == n_eager
            assert torch.equal(y.feats, eager)


def test_config5_cylinder_block_reduced(engine):
    """Config 5 wiring (asymmetric residual block, two shared keys, branch add, strided downsample) at 20 000 voxels."""
    from deploy3d_amd import synth
    cfg = synth.config5(20000)
    net, x, y = run_gpu_chain(cfg)
    ref = chain.oracle_chain(cfg, threads=8)
    assert set(net.rulebooks) == {"k313", "k133", "k333", "down"}
    compare_rulebooks(cfg, net, ref)
    compare_chain(cfg, net, ref, tol_scale=1.5)


def test_config5_full_size_runs(engine):
    from deploy3d_amd import synth
    cfg = synth.config5()
    net, x, y = run_gpu_chain(cfg)
    n_out = int(y.num_act.item())
    assert 0 < n_out <= y.feats.shape[0]
    assert bool(torch.isfinite(y.feats[:n_out].float()).all())
    rb = net.rulebooks["k313"]
    ni = int(rb.num_index.item())
    live = rb.index[2, :ni] >= 0
    cnt = torch.bincount(rb.index[2, :ni][live], minlength=9)
    assert bool((cnt == cnt.flip(0)).all()) and int(cnt[4]) == 250000


def _sampled_rows_reference(rb, rows, in_feats, w_tap_major, n_in):
    """For the output rows in ``rows``: the pairs that reach them, taken from the index tensor the GPU itself emitted
    (its rulebooks are checked against the oracle elsewhere), as (row position, tap, input row) arrays."""
    ni = int(rb.num_index.item())
    g, s, t = (rb.index[r, :ni] for r in range(3))
    pos = torch.full((int(rb.out_coors.shape[0]) + 1,), -1, dtype=torch.int64, device="cuda")
    pos[rows] = torch.arange(len(rows), device="cuda")
    live = t >= 0
    sel = live & (pos[s.clamp(min=0).long()] >= 0)
    return pos[s[sel].long()].cpu().numpy(), t[sel].cpu().numpy(), g[sel].cpu().numpy()


def test_config4_int8_backbone_full_size(engine):
    """Config 4 at its stated size (120 000 voxels, int8).  Activation scales are calibrated on this engine's own
    fp16 pass of config 3 (99.99th percentile, the rule of the reduced-size test).  Checked: the calibrated range is
    in use on every layer; two eager passes and three graph replays give the same bytes; and on 4 000 sampled output
    rows of three layers (16->32 strided, 64->64 SubM, 128->128 SubM) the int8 result equals int64 accumulation +
    the oracle's requantize rule applied to the pairs of the emitted index tensor, bit for bit."""
    from deploy3d_amd import layers, synth
    n = 120000
    cfg3 = synth.config3(n)
    net3, x3, _ = run_gpu_chain(cfg3)
    acts = {"input": cfg3["feats"]}
    acts.update({s["name"]: net3.outputs[s["name"]].feats[:int(net3.outputs[s["name"]].num_act.item())].float().cpu().numpy()
                 for s in cfg3["layers"]})
    counts = {s["name"]: int(net3.outputs[s["name"]].num_act.item()) for s in cfg3["layers"] if not s["subm"]}
    del net3, x3
    cfg = synth.config4(n, acts)
    caps = layers.plan_capacities(cfg["layers"], n, counts)
    net = layers.SparseBackbone(cfg["layers"], cfg["weights"], caps, dtype=torch.int8)
    x = layers.make_input(cfg["coords"], cfg["feats_q"], cfg["grid"], dtype=torch.int8)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        y = net.forward(x)
        stream.synchronize()
        first = {s["name"]: net.outputs[s["name"]].feats.clone() for s in cfg["layers"]}
        y = net.forward(x)
        stream.synchronize()
        for s in cfg["layers"]:
            assert torch.equal(net.outputs[s["name"]].feats, first[s["name"]]), s["name"]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            y = net.forward(x)
        for _ in range(3):
            y.feats.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y.feats, first[cfg["layers"][-1]["name"]])
    rng = np.random.default_rng(4)
    prev = "input"
    for spec, (w, b) in zip(cfg["layers"], cfg["weights"]):
        out = net.outputs[spec["name"]]
        n_out = int(out.num_act.item())
        q = first[spec["name"]][:n_out]
        assert int(q.abs().max()) >= 100, spec["name"]            # the calibrated range is in use
        if spec["name"] in ("down1", "conv3_1", "conv4_1"):
            rb = net.rulebooks[spec["key"]]
            rows = torch.from_numpy(rng.choice(n_out, size=min(4000, n_out), replace=False)).cuda()
            xin = x.feats if prev == "input" else first[prev]
            p, t, g = _sampled_rows_reference(rb, rows, xin, w, None)
            w_q, s_w = oracle.quantize_weights(w)
            xi = xin.cpu().numpy().astype(np.int64)
            acc = np.zeros((len(rows), spec["cout"]), dtype=np.int64)
            for tap in range(w_q.shape[0]):
                m_ = t == tap
                if m_.any():
                    np.add.at(acc, p[m_], xi[g[m_]] @ w_q[tap].astype(np.int64))
            assert np.abs(acc).max() < 2 ** 31
            m, bq = oracle.requant_params(spec["s_in"], s_w, spec["s_out"], b)
            want = oracle.requantize(acc.astype(np.int32), m, bq, bool(spec.get("relu")))
            np.testing.assert_array_equal(q[rows].cpu().numpy(), want, err_msg=spec["name"])
        prev = spec["name"]
    # and the whole pass against the oracle's int8 pass (int32 accumulation, the same requantize rule): the final
    # tensor of all 13 layers, every row, bit for bit
    import os
    _, _, ref_coords, ref_feats = _bench_module().cpu_pass(cfg, min(16, os.cpu_count() or 1))
    n_out = int(y.num_act.item())
    gc, gf = chain.sort_rows(y.coors[:n_out].cpu().numpy(), first[cfg["layers"][-1]["name"]][:n_out].cpu().numpy())
    rc, rf = chain.sort_rows(ref_coords, np.asarray(ref_feats))
    assert np.array_equal(gc, rc)
    np.testing.assert_array_equal(gf, rf)


def test_config5_full_size_first_layers_vs_oracle(engine):
    """Config 5 at its stated size (250 000 voxels): the two first-level layers of the block (SubM k(3,1,3) and
    k(1,3,3), 32->64) against the oracle: rulebooks bit-exact in canonical form, features within 2e-2*rms."""
    from deploy3d_amd import synth
    cfg = synth.config5()
    net, x, y = run_gpu_chain(cfg)
    two = dict(cfg, layers=[s for s in cfg["layers"] if s["name"] in ("a1", "b1")])
    two["weights"] = [cfg["weights"][cfg["layers"].index(s)] for s in two["layers"]]
    assert len(two["layers"]) == 2 and {s["key"] for s in two["layers"]} == {"k313", "k133"}
    ref = chain.oracle_chain(two, threads=8)
    for spec in two["layers"]:
        rb = net.rulebooks[spec["key"]]
        orb = ref["_rulebooks"][spec["key"]]
        np.testing.assert_array_equal(rb.index.cpu().numpy(), orb["index"], err_msg=spec["key"])
        out = net.outputs[spec["name"]]
        got = out.feats[:250000].float().cpu().numpy()
        want = ref[spec["name"]]["exact"]
        rms = float(np.sqrt(np.mean(want ** 2)))
        assert float(np.abs(got - want).max()) <= 2e-2 * rms, spec["name"]
