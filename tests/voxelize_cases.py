"""Inputs and ground truth of the reference's voxeliser test (tests/voxel_encoder/test_simple_mean.py:8-33):
200 000 points with x, y ~ N(0, 50), z ~ N(1, 2), one more N(0, 1) feature, batch index 0 or 1, grid
[B=2, *, 41, 1536, 1536], voxels of 0.1 x 0.1 x 0.15 from (-76.8, -76.8, -2); points within 1e-3 of a cell
boundary are dropped (:22-25) so that the grouping does not hang on the last bit of a float division; the ground
truth groups the points with torch.unique and averages them (the reference uses torch_scatter.scatter_mean, which
is not installed here: index_add_ and bincount do the same)."""
import numpy as np
import torch

SHAPE = (2, 41, 1536, 1536)   # (B, Z, Y, X)
CONFIG = [-76.8, -76.8, -2.0, 0.1, 0.1, 0.15]


def make_points(seed, n=200000, shape=SHAPE, config=CONFIG, extra=1):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((n, 1), generator=g) * 50
    y = torch.randn((n, 1), generator=g) * 50
    z = torch.randn((n, 1), generator=g) * 2 + 1
    other = torch.randn((n, extra), generator=g)
    feats = torch.cat([x, y, z, other], dim=-1)
    batch = torch.randint(0, shape[0], (n,), dtype=torch.int32, generator=g)
    cfg = torch.tensor(config, dtype=torch.float32)
    coors_f = (feats[:, :3] - cfg[:3]) / cfg[3:]
    keep = (coors_f - coors_f.round()).abs().amin(-1) > 1e-3
    return feats[keep].contiguous(), batch[keep].contiguous(), cfg


def ground_truth(feats, batch, cfg, shape=SHAPE):
    """(coords [V, 4] sorted, mean feats [V, C] float32, point counts [V]) of the valid points."""
    size = torch.tensor([shape[3], shape[2], shape[1]])
    finite = torch.isfinite(feats).all(dim=-1)
    coors_f = (feats[:, :3] - cfg[:3]) / cfg[3:]
    coors = torch.nan_to_num(coors_f, nan=0.0, posinf=3e9, neginf=-3e9).clamp(-2147483648.0, 2147483520.0).int()
    valid = coors.lt(size.unsqueeze(0)).logical_and(coors.ge(0)).all(dim=-1)
    valid &= finite & batch.ge(0) & batch.lt(shape[0])
    full = torch.cat([batch.unsqueeze(-1), coors[:, [2, 1, 0]]], dim=-1)[valid]
    uniq, inverse = full.unique(sorted=True, return_inverse=True, dim=0)
    sums = torch.zeros((len(uniq), feats.shape[1]), dtype=torch.float64)
    sums.index_add_(0, inverse, feats[valid].double())
    counts = torch.bincount(inverse, minlength=len(uniq))
    return uniq.numpy().astype(np.int32), (sums / counts.unsqueeze(-1)).float().numpy(), counts.numpy()


def check_against_truth(out_feats, out_coors, num_act_out, truth, max_num_act_out, rtol=1e-5, atol=1e-4):
    """The reference test's assertions (test_simple_mean.py:41-56): unique rows, count = min(max, voxels), every row
    one of the true voxels with its mean - at rtol 1e-5 / atol 1e-4 where the reference asks 1e-3 / 1e-3."""
    t_coors, t_feats, _ = truth
    n = int(num_act_out)
    assert n == min(max_num_act_out, len(t_coors)), (n, len(t_coors))
    got_c = np.asarray(out_coors)[:n]
    assert len({tuple(r) for r in got_c.tolist()}) == n, "duplicate voxel rows"
    lut = {tuple(r): i for i, r in enumerate(t_coors.tolist())}
    rows = [lut.get(tuple(r), -1) for r in got_c.tolist()]
    assert min(rows, default=0) >= 0, "a row that is no voxel of the input"
    want = t_feats[np.asarray(rows, dtype=np.int64)] if n else np.zeros((0, t_feats.shape[1]), np.float32)
    np.testing.assert_allclose(np.asarray(out_feats)[:n], want, rtol=rtol, atol=atol)
    return np.asarray(rows, dtype=np.int64)
