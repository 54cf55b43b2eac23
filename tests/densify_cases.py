"""The six parameterisations of the reference's sparse-to-dense test (tests/spconv/test_bev_densify.py:33-54):
128 channels, capacity 10 000 rows, grid [B=2, *, Z=2, Y=128, X=128], 10 000 / 100 / 0 live rows, fp32 and fp16,
and the way that test builds its input (unique random coordinates, :10-17) and its ground truth (dense indexing,
:19-23)."""
import numpy as np
import torch

REFERENCE_CASES = [(n, dt) for dt in ("float32", "float16") for n in (10000, 100, 0)]
CAP, CHANNELS, SHAPE = 10000, 128, (2, 2, 128, 128)   # (B, Z, Y, X)


def unique_coords(rng, n, shape):
    b, z, y, x = shape
    cells = rng.choice(b * z * y * x, size=n, replace=False)
    out = np.stack(np.unravel_index(cells, shape), axis=1).astype(np.int32)
    return out


def make_case(seed, num_act, dtype, cap=CAP, channels=CHANNELS, shape=SHAPE):
    rng = np.random.default_rng(seed)
    feats = torch.from_numpy(rng.standard_normal((cap, channels)).astype(np.float32)).to(getattr(torch, dtype))
    coords = np.zeros((cap, 4), dtype=np.int32)
    coords[:num_act] = unique_coords(rng, num_act, shape)
    # rows past the live count hold in-range garbage that must not show up in the map
    coords[num_act:] = unique_coords(rng, cap - num_act, shape) if cap - num_act <= np.prod(shape) else 0
    return feats, coords


def dense_indexing(feats, coords, num_act, shape):
    """Ground truth as the reference's test writes it: gt[b, :, z, y, x] = feats, then merge C and Z."""
    b, z, y, x = shape
    c = feats.shape[1]
    gt = torch.zeros((b, c, z, y, x), dtype=feats.dtype)
    _b, _z, _y, _x = torch.from_numpy(coords[:num_act]).long().T
    gt[_b, :, _z, _y, _x] = feats[:num_act]
    return gt.reshape(b, c * z, y, x)
