"""d3d_enqueue_static, the entry point that allocates nothing: the operators that take a workspace run with the
library's fixed scratch array instead, and must give exactly what d3d_enqueue gives with a caller's workspace -
on two calls in a row, the second on a smaller input (the array keeps the first call's contents)."""
import numpy as np
import pytest
import torch

from helpers import random_cloud

pytestmark = pytest.mark.gpu


def _index_outputs(plugin, coords, cap, grid, workspace):
    from deploy3d_amd import TensorDesc
    c = torch.zeros((cap, 4), dtype=torch.int32, device="cuda")
    c[:len(coords)] = torch.from_numpy(coords).cuda()
    num = torch.tensor([len(coords)], dtype=torch.int32, device="cuda")
    ins = [TensorDesc.of_tensor(c), TensorDesc.of_tensor(num), TensorDesc.of((1, 0) + tuple(grid), torch.int32)]
    outs = plugin.output_descs(ins)
    bufs = [torch.full(d.shape(), 7, dtype=torch.int32, device="cuda") if 0 not in d.shape() else None for d in outs]
    if workspace is None:
        workspace = torch.empty(max(1, plugin.workspace_size(ins, outs)), dtype=torch.uint8, device="cuda")
    plugin.enqueue(ins, outs, [c, num, None], bufs, workspace)
    torch.cuda.synchronize()
    return bufs


@pytest.mark.parametrize("subm", [True, False])
def test_static_scratch_rulebook_equals_workspace_rulebook(engine, subm):
    from deploy3d_amd import Plugin
    from deploy3d_amd.spconv_index import index_blob
    grid = (12, 96, 96)
    rng = np.random.default_rng(70 + subm)
    for n in (20000, 3000):          # the second call is smaller and finds the first call's data in the array
        coords = random_cloud(rng, n, grid, 1)
        max_out = n if subm else 4 * n
        blob = index_blob((3, 3, 3), (1, 1, 1) if subm else (2, 2, 2), (1, 1, 1), (1, 1, 1), (0, 0, 0), max_out, subm,
                          False)
        want = _index_outputs(Plugin("SPConvIdx3d", blob), coords, n, grid, None)
        got = _index_outputs(Plugin("SPConvIdx3d", blob), coords, n, grid, "static")
        n_out = n if subm else int(want[3].item())
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])       # index tensor, numIndex
        if not subm:
            assert int(got[3].item()) == n_out and 0 < n_out <= max_out
            assert torch.equal(got[2][:n_out], want[2][:n_out])                    # outCoors of the live rows


def test_static_scratch_densify_and_voxelize(engine):
    from deploy3d_amd import Plugin, TensorDesc
    from deploy3d_amd.bev_densify import densify_blob
    from deploy3d_amd.simple_mean import simple_mean_blob
    rng = np.random.default_rng(72)
    for n, grid in ((5000, (4, 64, 64)), (700, (2, 32, 48))):
        coords = random_cloud(rng, n, grid, 1)
        feats = torch.from_numpy(rng.standard_normal((n, 16)).astype(np.float32)).cuda().half()
        c = torch.from_numpy(coords).cuda()
        num = torch.tensor([n], dtype=torch.int32, device="cuda")
        ins = [TensorDesc.of_tensor(feats), TensorDesc.of_tensor(c), TensorDesc.of_tensor(num),
               TensorDesc.of((1, 0) + grid, torch.int32)]
        res = []
        for ws in (None, "static"):
            p = Plugin("BEVDensify", densify_blob(16 * grid[0]))
            outs = p.output_descs(ins)
            out = torch.full(outs[0].shape(), 3.0, dtype=torch.float16, device="cuda")
            w = ws or torch.empty(p.workspace_size(ins, outs), dtype=torch.uint8, device="cuda")
            p.enqueue(ins, outs, [feats, c, num, None], [out], w)
            torch.cuda.synchronize()
            res.append(out)
        assert torch.equal(res[0], res[1])
    for n in (30000, 2000):
        pts = torch.from_numpy((rng.random((n, 4)) * [40, 40, 4, 1]).astype(np.float32)).cuda()
        bidx = torch.zeros(n, dtype=torch.int32, device="cuda")
        conf = torch.tensor([0, 0, 0, 0.5, 0.5, 0.5], dtype=torch.float32, device="cuda")
        ins = [TensorDesc.of_tensor(pts), TensorDesc.of_tensor(bidx), TensorDesc.of_tensor(conf),
               TensorDesc.of((1, 0, 8, 80, 80), torch.int32)]
        res = []
        for ws in (None, "static"):
            p = Plugin("SimpleMeanEncoder", simple_mean_blob(n))
            outs = p.output_descs(ins)
            bufs = [torch.zeros(d.shape(), dtype=torch.float32 if i == 0 else torch.int32, device="cuda")
                    for i, d in enumerate(outs)]
            w = ws or torch.empty(p.workspace_size(ins, outs), dtype=torch.uint8, device="cuda")
            p.enqueue(ins, outs, [pts, bidx, conf, None], bufs, w)
            torch.cuda.synchronize()
            res.append(bufs)
        m = int(res[0][2].item())
        assert m == int(res[1][2].item()) and m > 0
        assert torch.equal(res[0][1][:m], res[1][1][:m])                          # voxel coordinates: deterministic
        torch.testing.assert_close(res[0][0][:m], res[1][0][:m], rtol=1e-5, atol=2e-5)  # means add in atomic order


def test_static_scratch_limits(engine):
    """Beyond the array's size the call is refused with D3D_ERR_WORKSPACE; SPConvMM is not served at all."""
    from deploy3d_amd import EngineError, Plugin, TensorDesc
    from deploy3d_amd.plugin import STATIC_SCRATCH_BYTES
    from deploy3d_amd.spconv_index import index_blob
    from deploy3d_amd.spconv_mm import mm_blob
    cap = 700000
    p = Plugin("SPConvIdx3d", index_blob((3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), (0, 0, 0), cap, True, False))
    c = torch.zeros((cap, 4), dtype=torch.int32, device="cuda")
    num = torch.zeros(1, dtype=torch.int32, device="cuda")
    ins = [TensorDesc.of_tensor(c), TensorDesc.of_tensor(num), TensorDesc.of((1, 0, 41, 1440, 1440), torch.int32)]
    outs = p.output_descs(ins)
    assert p.workspace_size(ins, outs) > STATIC_SCRATCH_BYTES
    bufs = [torch.empty(d.shape(), dtype=torch.int32, device="cuda") for d in outs]
    with pytest.raises(EngineError) as e:
        p.enqueue(ins, outs, [c, num, None], bufs, "static")
    assert e.value.status == -5 and "workspace" in str(e.value)
    mm = Plugin("SPConvMM", mm_blob((1, 1, 1), 16, 16, 64, True, False, np.zeros((1, 16, 16), np.float32)))
    x = torch.zeros((64, 16), dtype=torch.float16, device="cuda")
    idx = torch.full((3, 192), -1, dtype=torch.int32, device="cuda")
    ins = [TensorDesc.of_tensor(t) for t in (x, num, num, idx, num)]
    outs = mm.output_descs(ins)
    with pytest.raises(EngineError) as e:
        mm.enqueue(ins, outs, [x, num, num, idx, num], [torch.empty((64, 16), dtype=torch.float16, device="cuda")],
                   "static")
    assert e.value.status == -1


def test_static_enqueue_allocates_nothing(engine):
    """The entry point's promise itself: free device memory is the same before and after static calls (operators made
    and tensors allocated beforehand), also for a strided operator that keeps a map for a linked submanifold
    operator and has the persistent-index option set (both would otherwise make the library allocate on first use);
    and the calls can be recorded into a HIP graph in the capture mode that refuses allocation, and replayed."""
    from deploy3d_amd import Plugin, TensorDesc
    from deploy3d_amd.plugin import OPT_PERSISTENT_INDEX
    from deploy3d_amd.spconv_index import index_blob
    grid, n = (12, 96, 96), 6000
    rng = np.random.default_rng(75)
    coords = random_cloud(rng, n, grid, 1)
    strided = Plugin("SPConvIdx3d", index_blob((3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), (0, 0, 0), 4 * n, False, False))
    subm = Plugin("SPConvIdx3d", index_blob((3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), (0, 0, 0), 4 * n, True, False))
    strided.set_option(OPT_PERSISTENT_INDEX, 1)
    subm.link_coords(strided)
    c = torch.from_numpy(coords).cuda()
    num = torch.tensor([n], dtype=torch.int32, device="cuda")
    ins = [TensorDesc.of_tensor(c), TensorDesc.of_tensor(num), TensorDesc.of((1, 0) + grid, torch.int32)]
    outs = strided.output_descs(ins)
    bufs = [torch.full(d.shape(), 7, dtype=torch.int32, device="cuda") if 0 not in d.shape() else None for d in outs]
    ins2 = [TensorDesc.of_tensor(bufs[2]), TensorDesc.of_tensor(bufs[3]), TensorDesc.of((1, 0, 6, 48, 48), torch.int32)]
    outs2 = subm.output_descs(ins2)
    bufs2 = [torch.full(d.shape(), 7, dtype=torch.int32, device="cuda") for d in outs2]
    want = _index_outputs(Plugin("SPConvIdx3d", index_blob((3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), (0, 0, 0),
                                                           4 * n, False, False)), coords, n, grid, None)

    def both():
        strided.enqueue(ins, outs, [c, num, None], bufs, "static")
        subm.enqueue(ins2, outs2, [bufs[2], bufs[3], None], bufs2, "static")

    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    both()
    both()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(bufs[0], want[0]) and torch.equal(bufs[1], want[1])
    first = [b.clone() for b in bufs2]
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream, capture_error_mode="global"):
            both()
        for b in bufs2:
            b.fill_(7)
        graph.replay()
        graph.replay()
    stream.synchronize()
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(first, bufs2))
