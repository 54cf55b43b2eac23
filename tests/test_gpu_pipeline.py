"""Points -> voxels -> sparse layers -> dense map, every stage on the GPU through the C ABI, against the same chain
on the CPU oracle.  The voxeliser's row order differs between the two (first appearance here, hash-slot order in
the reference's algorithm), so stages are compared after sorting rows by coordinate; the dense map has no row order
and is compared directly."""
import numpy as np
import pytest
import torch

import chain
from oracle import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_points_to_dense_map(engine):
    from deploy3d_amd import layers, simple_mean_encoder, synth
    rng = np.random.default_rng(3)
    n_pts = 60000
    shape = (1, 16, 96, 96)                                  # (B, Z, Y, X)
    cfg = np.array([-9.6, -9.6, -1.0, 0.2, 0.2, 0.25], np.float32)
    # ground shell plus clusters, five features (x y z intensity time); a few NaN rows and padding rows
    pts = np.empty((n_pts, 5), np.float32)
    pts[:, 0:2] = rng.normal(0, 4.0, (n_pts, 2))
    pts[:, 2] = np.where(rng.random(n_pts) < 0.7, rng.uniform(-1.0, -0.4, n_pts), rng.normal(0.5, 0.8, n_pts))
    pts[:, 3:] = rng.random((n_pts, 2))
    pts[rng.integers(0, n_pts, 50)] = np.nan
    batch = np.zeros(n_pts, np.int32)
    batch[rng.integers(0, n_pts, 500)] = -1
    # snap away from cell boundaries so that both sides agree on every cell whatever the last bit of the division
    q = (pts[:, :3] - cfg[:3]) / cfg[3:]
    near = np.abs(q - np.round(q)).min(axis=1) < 1e-3
    batch[near] = -1

    max_vox = 30000
    ref_f, ref_c, ref_n = oracle.simple_mean(pts, batch, cfg, shape, max_vox)
    assert 5000 < ref_n < max_vox
    feats_g, coors_g, num_g = simple_mean_encoder(torch.from_numpy(pts).to(DEV), torch.from_numpy(batch).to(DEV),
                                                  torch.from_numpy(cfg).to(DEV),
                                                  torch.empty((1, 0) + shape[1:], dtype=torch.int32, device=DEV), max_vox)
    n_vox = int(num_g.item())
    assert n_vox == ref_n
    gc, gf = chain.sort_rows(coors_g[:n_vox].cpu().numpy(), feats_g[:n_vox].cpu().numpy())
    rc, rf = chain.sort_rows(ref_c[:ref_n], ref_f[:ref_n])
    assert np.array_equal(gc, rc)
    np.testing.assert_allclose(gf, rf, rtol=1e-5, atol=2e-5)

    # sparse layers: SubM 5->16, SubM 16->16 (shared key), strided 16->32, on the GPU's own voxels
    specs = synth.voxelnet_layers()[:4]
    weights = [synth.layer_weights(0, i, s) for i, s in enumerate(specs)]
    vox_coords = coors_g[:n_vox].cpu().numpy()
    vox_feats = feats_g[:n_vox].cpu().numpy()
    cfg_chain = dict(coords=vox_coords, feats=vox_feats, grid=list(shape[1:]), dtype="float16", layers=specs,
                     weights=weights)
    ref = chain.oracle_chain(cfg_chain)
    caps = layers.plan_capacities(specs, max_vox)
    net = layers.SparseBackbone(specs, weights, caps)
    x = layers.SparseTensor(feats_g.half(), coors_g, num_g, list(shape[1:]), 1)   # capacity rows, live count on device
    y = net.forward(x)
    torch.cuda.synchronize()
    n_out = int(y.num_act.item())
    want = ref[specs[-1]["name"]]
    assert n_out == len(want["coords"])
    yc, yf = chain.sort_rows(y.coors[:n_out].cpu().numpy(), y.feats[:n_out].float().cpu().numpy())
    wc, wf = chain.sort_rows(want["coords"], want["exact"])
    assert np.array_equal(yc, wc)
    rms = float(np.sqrt(np.mean(wf ** 2)))
    assert float(np.abs(yf - wf).max()) <= 2e-2 * rms

    # dense map of the GPU's rows vs the oracle's map of the same rows: bytes only
    dense = layers.densify(y)
    torch.cuda.synchronize()
    want_dense = oracle.bev_densify(y.feats.cpu().view(torch.int16).numpy(), y.coors.cpu().numpy(), n_out,
                                    [1] + list(y.grid))
    assert tuple(dense.shape) == (1, y.feats.shape[1] * y.grid[0], y.grid[1], y.grid[2])
    assert np.array_equal(dense.cpu().view(torch.int16).numpy(), want_dense)
    # and against the oracle chain's own values, cell by cell (fp16 tolerance)
    ref_dense = oracle.bev_densify(want["feats"].astype(np.float32), want["coords"], n_out, [1] + list(y.grid))
    assert float(np.abs(dense.float().cpu().numpy() - ref_dense).max()) <= 2e-2 * rms
