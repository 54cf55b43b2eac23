"""GPU rulebook parity: SPConvIdx{N}d through the C ABI vs the CPU oracle.

Bar: output coordinates and index pairs bit-exact after the canonical sort; for
SubM (where output ids are input rows) the whole index tensor is compared
bit for bit, padding included.
"""
import numpy as np
import pytest

from helpers import check_index_structure, gpu_rulebook, random_cloud
from oracle import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["blockmap", "blockmap-general", "blockmap-per-pair", "hash"])
def structure(request, monkeypatch):
    """Every case runs on every rulebook variant: the dense block map with one thread per input (default whenever
    the map fits and a kernel's reach is at most one brick; 3x3x3, 3x1x1, 3x1x3 and 1x3x3 kernels take a tap
    enumeration specialised at compile time, "general" switches that off), the block map with one thread per
    (tap, input) pair (long-reach kernels, 4-D) and the open-addressing hash (grids too large for the map)."""
    monkeypatch.setenv("D3D_RULEBOOK", request.param.split("-")[0])
    monkeypatch.setenv("D3D_RULEBOOK_NEAR", "0" if request.param.endswith("per-pair") else "1")
    monkeypatch.setenv("D3D_RULEBOOK_FIXED", "0" if request.param.endswith("general") else "1")
    return request.param

SUBM_CASES = [
    # (n, grid, batch, ksize, padding, dilation)
    (500, (9, 20, 18), 2, (3, 3, 3), (1, 1, 1), (1, 1, 1)),
    (3000, (12, 40, 33), 1, (3, 3, 3), (1, 1, 1), (1, 1, 1)),
    (2000, (12, 40, 33), 1, (3, 1, 3), (1, 0, 1), (1, 1, 1)),
    (2000, (12, 40, 33), 1, (1, 3, 3), (0, 1, 1), (1, 1, 1)),
    (2000, (16, 30, 30), 1, (3, 3, 3), (2, 2, 2), (2, 2, 2)),
    (1500, (10, 25, 25), 1, (5, 3, 1), (2, 1, 0), (1, 1, 1)),
    (700, (64, 64), 1, (3, 3), (1, 1), (1, 1)),
    (300, (500,), 2, (5,), (2,), (1,)),
    (1000, (6, 8, 10, 12), 1, (3, 3, 3, 3), (1, 1, 1, 1), (1, 1, 1, 1)),
    (20000, (41, 160, 140), 1, (3, 3, 3), (1, 1, 1), (1, 1, 1)),
]


@pytest.mark.parametrize("case", SUBM_CASES, ids=lambda c: "n%d_k%s" % (c[0], "x".join(map(str, c[3]))))
def test_subm_matches_oracle_bit_exact(engine, case):
    n, grid, batch, ksize, padding, dilation = case
    rng = np.random.default_rng(1000 + n)
    coords = random_cloud(rng, n, grid, batch)
    n = len(coords)
    stride = (1,) * len(ksize)
    ref = oracle.rulebook(coords, n, (batch,) + grid, ksize, stride, padding, dilation, n, True)
    got = gpu_rulebook(coords, n, grid, batch, ksize, stride, padding, dilation, n, True)
    assert got["num_index"] == ref["num_index"]
    np.testing.assert_array_equal(got["index"], ref["index"])
    check_index_structure(got["index"], got["num_index"], int(np.prod(ksize)), n)


CONV_CASES = [
    # (n, grid, batch, ksize, stride, padding, dilation, transpose)
    (500, (9, 20, 18), 2, (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), False),
    (3000, (12, 40, 33), 1, (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), False),
    (3000, (12, 40, 33), 1, (3, 3, 3), (2, 2, 2), (0, 1, 1), (1, 1, 1), False),
    (3000, (12, 40, 33), 1, (3, 1, 1), (2, 1, 1), (0, 0, 0), (1, 1, 1), False),
    (3000, (12, 40, 33), 1, (3, 3, 3), (2, 2, 1), (1, 1, 1), (1, 1, 1), False),
    (2000, (12, 40, 33), 1, (2, 2, 2), (2, 2, 2), (0, 0, 0), (1, 1, 1), False),
    (2000, (12, 40, 33), 1, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), False),
    (2000, (12, 40, 33), 1, (3, 3, 3), (3, 2, 1), (1, 0, 2), (2, 1, 1), False),
    (1000, (6, 20, 16), 1, (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), True),
    (1000, (6, 20, 16), 1, (2, 2, 2), (2, 2, 2), (0, 0, 0), (1, 1, 1), True),
    (700, (64, 64), 1, (3, 3), (2, 2), (1, 1), (1, 1), False),
    (300, (500,), 2, (3,), (2,), (1,), (1,), False),
    (800, (6, 8, 10, 12), 1, (3, 3, 3, 3), (2, 2, 2, 2), (1, 1, 1, 1), (1, 1, 1, 1), False),
    (20000, (41, 160, 140), 1, (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), False),
]


def _conv_case(case, max_out=None, cap=None):
    n, grid, batch, ksize, stride, padding, dilation, transpose = case
    rng = np.random.default_rng(2000 + n + 7 * int(transpose))
    coords = random_cloud(rng, n, grid, batch)
    n = len(coords)
    out_grid = oracle.out_shape(grid, ksize, stride, padding, dilation, None, transpose)
    kvol = int(np.prod(ksize))
    full = max_out is None
    max_out = n * kvol if full else max_out
    ref = oracle.rulebook(coords, n, [batch] + out_grid, ksize, stride, padding, dilation, max_out, False, transpose)
    got = gpu_rulebook(coords, n, grid, batch, ksize, stride, padding, dilation, max_out, False, transpose, cap=cap)
    return coords, out_grid, ref, got, kvol


@pytest.mark.parametrize("case", CONV_CASES,
                         ids=lambda c: "n%d_k%s_s%s%s" % (c[0], "x".join(map(str, c[3])), "x".join(map(str, c[4])),
                                                          "_T" if c[7] else ""))
def test_conv_matches_oracle_canonical(engine, case):
    coords, out_grid, ref, got, kvol = _conv_case(case)
    assert got["out_grid"] == out_grid
    assert got["num_act_out"] == ref["num_act_out"]
    assert got["num_index"] == ref["num_index"]
    c_ref, t_ref = oracle.canonical(ref["index"], ref["num_index"], ref["out_coors"], ref["num_act_out"])
    c_got, t_got = oracle.canonical(got["index"], got["num_index"], got["out_coors"], got["num_act_out"])
    np.testing.assert_array_equal(c_got, c_ref)
    np.testing.assert_array_equal(t_got, t_ref)
    check_index_structure(got["index"], got["num_index"], kvol, len(coords))


def test_conv_output_order_is_deterministic(engine):
    case = CONV_CASES[1]
    _, _, _, a, _ = _conv_case(case)
    _, _, _, b, _ = _conv_case(case)
    np.testing.assert_array_equal(a["index"], b["index"])
    np.testing.assert_array_equal(a["out_coors"][:a["num_act_out"]], b["out_coors"][:b["num_act_out"]])


@pytest.mark.parametrize("max_out", [1, 100, 1000])
def test_conv_truncation_keeps_a_consistent_subset(engine, max_out):
    """numActOut = min(total, maxNumActOut); survivors are unique members of the full output set and the
    pairs are exactly the full rulebook's pairs restricted to them (tests/spconv/test_spconv.py:72-124)."""
    case = CONV_CASES[1]
    coords, out_grid, full_ref, _, kvol = _conv_case(case)
    _, _, _, got, _ = _conv_case(case, max_out=max_out)
    total = full_ref["num_act_out"]
    assert got["num_act_out"] == min(total, max_out)
    full_set = {tuple(c): i for i, c in enumerate(full_ref["out_coors"][:total].tolist())}
    kept = [tuple(c) for c in got["out_coors"][:got["num_act_out"]].tolist()]
    assert len(set(kept)) == len(kept) and all(k in full_set for k in kept)
    # pairs of the full rulebook restricted to survivors, in coordinate terms
    ni = full_ref["num_index"]
    g, s, t = full_ref["index"][:, :ni]
    live = t >= 0
    ref_pairs = {(int(tt), int(gg), tuple(full_ref["out_coors"][ss])) for gg, ss, tt in
                 zip(g[live], s[live], t[live]) if tuple(full_ref["out_coors"][ss]) in set(kept)}
    ni = got["num_index"]
    g, s, t = got["index"][:, :ni]
    live = t >= 0
    got_pairs = {(int(tt), int(gg), tuple(got["out_coors"][ss])) for gg, ss, tt in zip(g[live], s[live], t[live])}
    assert got_pairs == ref_pairs
    check_index_structure(got["index"], got["num_index"], kvol, len(coords))


def test_capacity_larger_than_live_count(engine):
    """cap > numActIn: rows beyond the live count are ignored (test_spconv.py:167-168 uses 20000 of 40000)."""
    case = CONV_CASES[1]
    coords, out_grid, ref, got, kvol = _conv_case(case, cap=2 * case[0])
    c_ref, t_ref = oracle.canonical(ref["index"], ref["num_index"], ref["out_coors"], ref["num_act_out"])
    c_got, t_got = oracle.canonical(got["index"], got["num_index"], got["out_coors"], got["num_act_out"])
    np.testing.assert_array_equal(c_got, c_ref)
    np.testing.assert_array_equal(t_got, t_ref)
    assert got["index"].shape[1] == kvol * (2 * case[0] + 128)


def test_empty_input(engine):
    """numActIn = 0 => numIndex = 0 and numActOut = 0 (trt/spconv/index.cu:271-275, :414-417)."""
    coords = np.zeros((256, 4), dtype=np.int32)
    got = gpu_rulebook(coords, 0, (8, 8, 8), 1, (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), 100, False)
    assert got["num_index"] == 0 and got["num_act_out"] == 0
    got = gpu_rulebook(coords, 0, (8, 8, 8), 1, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 256, True)
    assert got["num_index"] == 0
    assert (got["index"] == -1).all()


def test_single_voxel_and_full_block(engine):
    one = np.array([[0, 2, 3, 4]], dtype=np.int32)
    got = gpu_rulebook(one, 1, (5, 6, 7), 1, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, True)
    assert got["num_index"] == 128
    live = got["index"][2] >= 0
    assert live.sum() == 1 and got["index"][2][live][0] == 13 and got["index"][0][live][0] == 0
    # a full dense block: every interior voxel has all 27 neighbours
    zz, yy, xx = np.meshgrid(np.arange(4), np.arange(5), np.arange(6), indexing="ij")
    block = np.stack([np.zeros(120, dtype=np.int64), zz.ravel(), yy.ravel(), xx.ravel()], 1).astype(np.int32)
    got = gpu_rulebook(block, 120, (4, 5, 6), 1, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 120, True)
    live = got["index"][2] >= 0
    expected = sum((4 - abs(dz)) * (5 - abs(dy)) * (6 - abs(dx)) for dz in (-1, 0, 1) for dy in (-1, 0, 1)
                   for dx in (-1, 0, 1))
    assert live.sum() == expected


def test_submanifold_on_a_strided_operators_map(engine):
    """d3d_link_coords: a SubM operator on the outputs of a strided operator takes over that operator's occupancy map
    (no clearing, marking, scanning, no permutation).  Its index tensor must equal, bit for bit, the oracle's for
    those coordinates and what the same operator builds on its own - also when the strided operator truncated its
    outputs (the map then holds cells whose rows were dropped) and when the tensors handed over are not the ones
    the strided operator wrote (the link must not be used)."""
    import torch
    from deploy3d_amd import spconv_index_nd
    from deploy3d_amd.spconv_index import index_plugin
    grid, n = (12, 40, 33), 3000
    rng = np.random.default_rng(99)
    coords = random_cloud(rng, n, grid, 1)
    c = torch.from_numpy(coords).cuda()
    num = torch.tensor([n], dtype=torch.int32, device="cuda")
    shape = torch.empty((1, 0) + grid, dtype=torch.int32, device="cuda")
    down = ((3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), (0, 0, 0))
    same = ((3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), (0, 0, 0))
    for max_out in (8 * n, 700):
        producer = index_plugin(*down, max_out, False, False)
        subm = index_plugin(*same, max_out, True, False)
        results = []
        for linked in (True, False, True):
            subm.link_coords(producer if linked else None)
            _, _, out_coors, num_out, out_shape = spconv_index_nd(c, num, shape, *down, max_out, False, False)
            index, num_index = spconv_index_nd(out_coors, num_out, out_shape, *same, max_out, True, False)
            torch.cuda.synchronize()
            results.append(index.cpu().numpy())
            m = int(num_out.item())
            ref = oracle.rulebook(out_coors.cpu().numpy(), m, (1,) + tuple(out_shape.shape[2:]), *same[:4], max_out, True)
            assert int(num_index.item()) == ref["num_index"]
            np.testing.assert_array_equal(results[-1], ref["index"])
        np.testing.assert_array_equal(results[0], results[1])
        # other coordinates in a tensor the producer did not write: the link is there, the map must not be used
        subm.link_coords(producer)
        other = torch.zeros_like(out_coors)
        m2 = min(500, max_out)
        other[:m2] = torch.from_numpy(random_cloud(rng, m2, tuple(out_shape.shape[2:]), 1)).cuda()
        num2 = torch.tensor([m2], dtype=torch.int32, device="cuda")
        index, num_index = spconv_index_nd(other, num2, out_shape, *same, max_out, True, False)
        torch.cuda.synchronize()
        ref = oracle.rulebook(other.cpu().numpy(), m2, (1,) + tuple(out_shape.shape[2:]), *same[:4], max_out, True)
        np.testing.assert_array_equal(index.cpu().numpy(), ref["index"])
        subm.link_coords(None)


@pytest.mark.parametrize("second", [((3, 3, 3), (2, 2, 2), (1, 1, 1)), ((3, 3, 3), (2, 2, 2), (0, 1, 1)),
                                    ((3, 1, 1), (2, 1, 1), (0, 0, 0)), ((3, 3, 3), (2, 2, 2), (0, 0, 0))])
def test_strided_operator_on_a_strided_operators_map(engine, second):
    """d3d_link_coords with a strided consumer: for the kernel shapes it knows it derives the occupancy of its output
    grid from the producer's map instead of marking it input by input (the last parameter set is a shape it does not
    know: the link is there and changes nothing).  Odd grid extents (bricks cut by the edge on both levels), two
    samples, a producer that truncates its outputs (its map then holds cells whose rows were dropped), changing
    clouds (the producer's two maps take turns); checked against the oracle on the producer's coordinates and
    against the same operator without the link."""
    import torch
    from deploy3d_amd import spconv_index_nd
    from deploy3d_amd.spconv_index import index_plugin
    grid, batch, n = (13, 45, 38), 2, 4000
    rng = np.random.default_rng(123)
    first = ((3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), (0, 0, 0))
    nxt = second + ((1, 1, 1), (0, 0, 0))
    shape = torch.empty((batch, 0) + grid, dtype=torch.int32, device="cuda")
    for max1 in (8 * n, 900):
        max2 = 8 * max1
        producer = index_plugin(*first, max1, False, False)
        consumer = index_plugin(*nxt, max2, False, False)
        for m in (n, 2500, n):
            coords = random_cloud(rng, m, grid, batch)
            c = torch.from_numpy(coords).cuda()
            num = torch.tensor([len(coords)], dtype=torch.int32, device="cuda")
            canon = []
            for linked in (True, False):
                consumer.link_coords(producer if linked else None)
                _, _, oc, no, osh = spconv_index_nd(c, num, shape, *first, max1, False, False)
                index, num_index, oc2, no2, osh2 = spconv_index_nd(oc, no, osh, *nxt, max2, False, False)
                torch.cuda.synchronize()
                got = oracle.canonical(index.cpu().numpy(), int(num_index.item()), oc2.cpu().numpy(), int(no2.item()))
                canon.append(got)
                if linked:
                    live = int(no.item())
                    assert live == min(max1, live) and (max1 > 900 or live == 900)
                    ref = oracle.rulebook(oc.cpu().numpy(), live, (batch,) + tuple(osh2.shape[2:]), *nxt[:4], max2, False)
                    want = oracle.canonical(ref["index"], ref["num_index"], ref["out_coors"], ref["num_act_out"])
                    assert int(num_index.item()) == ref["num_index"] and int(no2.item()) == ref["num_act_out"]
                    np.testing.assert_array_equal(got[0], want[0])
                    np.testing.assert_array_equal(got[1], want[1])
            np.testing.assert_array_equal(canon[0][0], canon[1][0])
            np.testing.assert_array_equal(canon[0][1], canon[1][1])
        consumer.link_coords(None)


def test_ordered_scan_variant(engine, monkeypatch):
    """D3D_RULEBOOK_ORDERED_SCAN=1 selects acquire-release tickets in the scan pass of the block map: same results."""
    monkeypatch.setenv("D3D_RULEBOOK_ORDERED_SCAN", "1")
    test_subm_matches_oracle_bit_exact(engine, SUBM_CASES[9])
    coords, out_grid, ref, got, kvol = _conv_case(CONV_CASES[1])
    c_ref, t_ref = oracle.canonical(ref["index"], ref["num_index"], ref["out_coors"], ref["num_act_out"])
    c_got, t_got = oracle.canonical(got["index"], got["num_index"], got["out_coors"], got["num_act_out"])
    np.testing.assert_array_equal(c_got, c_ref)
    np.testing.assert_array_equal(t_got, t_ref)


def test_persistent_index_tensor(engine):
    """D3D_OPT_PERSISTENT_INDEX: one handle, one index tensor, passes of different sizes.  After every enqueue the
    whole tensor equals the oracle's (every unused slot -1) although only the first pass fills it at capacity.
    The documented limit of the promise: a value the caller writes past the used part is not the library's to
    clean (it is wiped without the option)."""
    import torch
    from deploy3d_amd.plugin import OPT_PERSISTENT_INDEX, Plugin, TensorDesc
    from deploy3d_amd.spconv_index import index_blob
    from deploy3d_amd.spconv_mm import get_plugin, mm_blob
    grid, cap = (12, 40, 33), 4000
    rng = np.random.default_rng(77)
    for subm, stride, with_table in ((True, (1, 1, 1), True), (False, (2, 2, 2), True), (True, (1, 1, 1), False)):
        max_out = cap if subm else 8 * cap
        args = ((3, 3, 3), stride, (1, 1, 1), (1, 1, 1))
        plugin = Plugin("SPConvIdx3d", index_blob(*args, (0, 0, 0), max_out, subm, False))
        plugin.set_option(OPT_PERSISTENT_INDEX, 1)
        if with_table:
            get_plugin(mm_blob((3, 3, 3), 1, 1, max_out, subm, False, np.zeros(27, np.float32))).link_rulebook(plugin)
        coors = torch.zeros((cap, 4), dtype=torch.int32, device="cuda")
        num = torch.zeros(1, dtype=torch.int32, device="cuda")
        in_descs = [TensorDesc.of_tensor(coors), TensorDesc.of_tensor(num), TensorDesc.of((1, 0) + grid, torch.int32)]
        out_descs = plugin.output_descs(in_descs)
        outs = [torch.empty(d.shape(), dtype=torch.int32, device="cuda") for d in out_descs]
        outs[0].fill_(12345)  # the first pass must not rely on what the buffer held
        ws = torch.empty(max(1, plugin.workspace_size(in_descs, out_descs)), dtype=torch.uint8, device="cuda")
        out_grid = (1,) + (grid if subm else tuple(out_descs[4].shape()[2:]))
        for n in (3000, 500, 0, 4000, 1200):
            coords = random_cloud(rng, n, grid, 1) if n else np.zeros((0, 4), np.int32)
            coors.zero_()
            coors[:n] = torch.from_numpy(coords).cuda()
            num.fill_(n)
            plugin.enqueue(in_descs, out_descs, [coors, num, None], outs, ws)
            torch.cuda.synchronize()
            ref = oracle.rulebook(coors.cpu().numpy(), n, out_grid, *args, max_out, subm)
            index = outs[0].cpu().numpy()
            ni = int(outs[1].item())
            assert ni == ref["num_index"]
            if subm:
                np.testing.assert_array_equal(index, ref["index"])
            else:
                assert (index[:, ni:] == -1).all()
                c_ref, t_ref = oracle.canonical(ref["index"], ref["num_index"], ref["out_coors"], ref["num_act_out"])
                c_got, t_got = oracle.canonical(index, ni, outs[2].cpu().numpy(), int(outs[3].item()))
                np.testing.assert_array_equal(c_got, c_ref)
                np.testing.assert_array_equal(t_got, t_ref)
            check_index_structure(index, ni, 27, cap)
        # a caller's write past the used part survives the next pass of a persistent tensor ...
        outs[0][1, -1] = 777
        plugin.enqueue(in_descs, out_descs, [coors, num, None], outs, ws)
        torch.cuda.synchronize()
        assert int(outs[0][1, -1].item()) == 777
        # ... and not that of an ordinary one
        plugin.set_option(OPT_PERSISTENT_INDEX, 0)
        plugin.enqueue(in_descs, out_descs, [coors, num, None], outs, ws)
        torch.cuda.synchronize()
        assert int(outs[0][1, -1].item()) == -1
        # switching the option on again starts with a full fill
        plugin.set_option(OPT_PERSISTENT_INDEX, 1)
        outs[0][2, -2] = 778
        plugin.enqueue(in_descs, out_descs, [coors, num, None], outs, ws)
        torch.cuda.synchronize()
        assert int(outs[0][2, -2].item()) == -1
        plugin.close()


def test_configured_operator_captures_without_an_eager_pass(engine):
    """An operator that keeps its occupancy map between passes (persistent index tensor) reserves its two maps at
    configure: captured in a graph without ever having been enqueued eagerly, every replay - the maps take turns
    from replay to replay - on changing clouds gives the oracle's rulebook."""
    import torch
    from deploy3d_amd.plugin import OPT_PERSISTENT_INDEX, Plugin, TensorDesc
    from deploy3d_amd.spconv_index import index_blob
    grid, cap = (12, 40, 33), 4000
    rng = np.random.default_rng(78)
    for subm, stride in ((True, (1, 1, 1)), (False, (2, 2, 2))):
        max_out = cap if subm else 8 * cap
        args = ((3, 3, 3), stride, (1, 1, 1), (1, 1, 1))
        plugin = Plugin("SPConvIdx3d", index_blob(*args, (0, 0, 0), max_out, subm, False))
        plugin.set_option(OPT_PERSISTENT_INDEX, 1)
        coors = torch.zeros((cap, 4), dtype=torch.int32, device="cuda")
        num = torch.zeros(1, dtype=torch.int32, device="cuda")
        in_descs = [TensorDesc.of_tensor(coors), TensorDesc.of_tensor(num), TensorDesc.of((1, 0) + grid, torch.int32)]
        out_descs = plugin.output_descs(in_descs)
        outs = [torch.empty(d.shape(), dtype=torch.int32, device="cuda") for d in out_descs]
        ws = torch.empty(max(1, plugin.workspace_size(in_descs, out_descs)), dtype=torch.uint8, device="cuda")
        plugin.configure(in_descs, out_descs)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            plugin.enqueue(in_descs, out_descs, [coors, num, None], outs, ws)
        out_grid = (1,) + (grid if subm else tuple(out_descs[4].shape()[2:]))
        for n in (3000, 700, 4000, 1500):
            coords = random_cloud(rng, n, grid, 1)
            coors.zero_()
            coors[:n] = torch.from_numpy(coords).cuda()
            num.fill_(n)
            graph.replay()
            torch.cuda.synchronize()
            ref = oracle.rulebook(coors.cpu().numpy(), n, out_grid, *args, max_out, subm)
            index, ni = outs[0].cpu().numpy(), int(outs[1].item())
            assert ni == ref["num_index"]
            if subm:
                np.testing.assert_array_equal(index[:, :ni], ref["index"][:, :ni])
            else:
                c_ref, t_ref = oracle.canonical(ref["index"], ref["num_index"], ref["out_coors"], ref["num_act_out"])
                c_got, t_got = oracle.canonical(index, ni, outs[2].cpu().numpy(), int(outs[3].item()))
                np.testing.assert_array_equal(c_got, c_ref)
                np.testing.assert_array_equal(t_got, t_ref)
        plugin.close()


def _random_geometry(rng):
    """A random but valid layer: 1 to 4 dims, kernel 1..5, stride 1..3, padding 0..2, dilation 1..2."""
    nd = int(rng.integers(1, 5))
    budget = 4096 if nd < 4 else 1500            # cells of the grid: keeps the oracle and the brute force quick
    side = max(3, int(round(budget ** (1.0 / nd))))
    grid = tuple(int(rng.integers(max(3, side // 2), side + 3)) for _ in range(nd))
    ksize = tuple(int(rng.integers(1, 6 if nd < 3 else 4)) for _ in range(nd))
    dilation = tuple(int(rng.integers(1, 3)) for _ in range(nd))
    stride = tuple(int(rng.integers(1, 4)) for _ in range(nd))
    padding = tuple(int(rng.integers(0, 3)) for _ in range(nd))
    batch = int(rng.integers(1, 4))
    return nd, grid, ksize, stride, padding, dilation, batch


def test_random_geometries(engine):
    """Seeded sweep over random layer geometries (all three kinds: SubM, strided, transposed), each compared with
    the oracle: SubM bit for bit, the others after the canonical sort."""
    rng = np.random.default_rng(20240611)
    done = 0
    while done < 36:
        nd, grid, ksize, stride, padding, dilation, batch = _random_geometry(rng)
        kind = ("subm", "conv", "transpose")[done % 3]
        cells = batch * int(np.prod(grid))
        n = int(rng.integers(1, max(2, min(1500, cells // 2))))
        coords = random_cloud(rng, n, grid, batch)
        n = len(coords)
        kvol = int(np.prod(ksize))
        if kind == "subm":
            stride1 = (1,) * nd
            ref = oracle.rulebook(coords, n, (batch,) + grid, ksize, stride1, padding, dilation, n, True)
            got = gpu_rulebook(coords, n, grid, batch, ksize, stride1, padding, dilation, n, True)
            assert got["num_index"] == ref["num_index"], (grid, ksize, padding, dilation)
            np.testing.assert_array_equal(got["index"], ref["index"])
        else:
            transpose = kind == "transpose"
            out_pad = tuple(int(rng.integers(0, s)) for s in stride) if transpose else None
            out_grid = oracle.out_shape(grid, ksize, stride, padding, dilation, out_pad, transpose)
            if min(out_grid) < 1 or batch * int(np.prod(out_grid)) > 200000:
                continue
            max_out = min(n * kvol, batch * int(np.prod(out_grid)))
            ref = oracle.rulebook(coords, n, [batch] + out_grid, ksize, stride, padding, dilation, max_out, False,
                                  transpose)
            got = gpu_rulebook(coords, n, grid, batch, ksize, stride, padding, dilation, max_out, False, transpose,
                               out_padding=out_pad)
            where = (kind, grid, ksize, stride, padding, dilation, out_pad)
            assert got["out_grid"] == out_grid, where
            assert got["num_act_out"] == ref["num_act_out"], where
            assert got["num_index"] == ref["num_index"], where
            c_ref, t_ref = oracle.canonical(ref["index"], ref["num_index"], ref["out_coors"], ref["num_act_out"])
            c_got, t_got = oracle.canonical(got["index"], got["num_index"], got["out_coors"], got["num_act_out"])
            np.testing.assert_array_equal(c_got, c_ref, err_msg=str(where))
            np.testing.assert_array_equal(t_got, t_ref, err_msg=str(where))
        check_index_structure(got["index"], got["num_index"], kvol, n)
        done += 1
