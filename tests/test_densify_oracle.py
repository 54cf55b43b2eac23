"""Pins the sparse-to-dense oracle (d3d_oracle_bev_densify) against torch's dense indexing - the ground truth the
reference's own test uses (tests/spconv/test_bev_densify.py:19-23) - on that test's six cases and on ragged shapes.
A transposed (c, z) merge, a swapped y/x, or a missing clear each fail."""
import numpy as np
import pytest
import torch

from densify_cases import CAP, CHANNELS, REFERENCE_CASES, SHAPE, dense_indexing, make_case
from oracle import oracle


def _as_numpy(t):
    return t.view(torch.int16).numpy() if t.dtype in (torch.float16, torch.bfloat16) else t.numpy()


@pytest.mark.parametrize("num_act,dtype", REFERENCE_CASES)
def test_reference_cases_match_dense_indexing(num_act, dtype):
    feats, coords = make_case(5 + num_act, num_act, dtype)
    want = dense_indexing(feats, coords, num_act, SHAPE)
    got = oracle.bev_densify(_as_numpy(feats), coords, num_act, SHAPE)
    assert got.shape == (2, CHANNELS * 2, 128, 128)
    assert np.array_equal(got, _as_numpy(want))
    if num_act == 0:
        assert not got.any()


@pytest.mark.parametrize("shape,channels,dtype", [((1, 1, 5, 7), 3, "float32"), ((3, 4, 9, 5), 10, "float16"),
                                                  ((2, 3, 1, 33), 17, "int8"), ((1, 2, 6, 6), 64, "bfloat16")])
def test_ragged_shapes(shape, channels, dtype):
    rng = np.random.default_rng(11)
    n = int(np.prod(shape) * 0.4)
    cap = n + 13
    if dtype == "int8":
        feats = torch.from_numpy(rng.integers(-128, 128, (cap, channels), dtype=np.int8))
        _, coords = make_case(3, n, "float32", cap=cap, channels=1, shape=shape)
    else:
        feats, coords = make_case(3, n, dtype, cap=cap, channels=channels, shape=shape)
    want = dense_indexing(feats, coords, n, shape)
    got = oracle.bev_densify(_as_numpy(feats), coords, n, shape)
    assert np.array_equal(got, _as_numpy(want))


def test_marker_values_land_where_the_layout_says():
    """out viewed as [B, C, Z, Y, X]: each cell carries a value that encodes its own address."""
    shape, c = (2, 3, 4, 5), 6
    cells = np.stack(np.meshgrid(*[np.arange(s) for s in shape], indexing="ij"), -1).reshape(-1, 4).astype(np.int32)
    perm = np.random.default_rng(2).permutation(len(cells))
    cells = cells[perm]
    code = ((cells[:, 0] * 3 + cells[:, 1]) * 4 + cells[:, 2]) * 5 + cells[:, 3]
    feats = (code[:, None] * 10 + np.arange(c)[None, :]).astype(np.float32)
    got = oracle.bev_densify(feats, cells, len(cells), shape).reshape(2, c, 3, 4, 5)
    for b, ch, z, y, x in [(0, 0, 0, 0, 0), (1, 5, 2, 3, 4), (1, 2, 0, 3, 1), (0, 4, 2, 0, 4)]:
        assert got[b, ch, z, y, x] == (((b * 3 + z) * 4 + y) * 5 + x) * 10 + ch
