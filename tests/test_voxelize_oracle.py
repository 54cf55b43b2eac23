"""Pins the voxeliser oracle (d3d_oracle_simple_mean) against a torch.unique / index_add scatter-mean - the
formulation of the reference's own test (tests/voxel_encoder/test_simple_mean.py:17-33) - on that test's two cases
(maxNumActOut 200 000 and 100), plus the rules a plausible mistake would break: conversion toward zero (a point up
to one cell below the grid's minimum lands in cell 0), rows with NaN / inf or a negative batch index are skipped,
features beyond x y z are averaged too, rows past numActOut stay zero."""
import numpy as np
import pytest
import torch

from oracle import oracle
from voxelize_cases import CONFIG, SHAPE, check_against_truth, ground_truth, make_points


@pytest.mark.parametrize("max_out", [200000, 100])
def test_reference_cases(max_out):
    feats, batch, cfg = make_points(1234)
    truth = ground_truth(feats, batch, cfg)
    out_feats, out_coors, n = oracle.simple_mean(feats.numpy(), batch.numpy(), cfg.numpy(), SHAPE, max_out)
    check_against_truth(out_feats, out_coors, n, truth, max_out)
    assert not out_feats[n:].any()
    if max_out >= len(truth[0]):   # every voxel present: the sorted rows are the truth's rows
        order = np.lexsort(out_coors[:n].T[::-1])
        assert np.array_equal(out_coors[:n][order], truth[0])


def test_truncation_toward_zero_and_skipped_rows():
    cfg = np.array([0.0, 0.0, 0.0, 1.0, 1.0, 1.0], np.float32)
    pts = np.array([
        [-0.5, 0.5, 0.5, 7.0],      # (x - min) / size = -0.5 -> int 0: cell (0, 0, 0), not out of range
        [0.25, 0.75, 0.25, 9.0],    # same cell
        [-1.0, 0.5, 0.5, 1.0],      # -1 -> out
        [3.5, 1.5, 0.5, 2.0],       # cell z0 y1 x3
        [4.0, 0.5, 0.5, 3.0],       # x = 4 == X -> out
        [np.nan, 0.5, 0.5, 1.0],    # skipped
        [0.5, 0.5, 0.5, np.inf],    # a non-finite feature anywhere skips the row
        [1.5, 0.5, 1.5, 5.0],       # batch -1 -> skipped
        [1.5, 0.5, 1.5, 6.0],       # batch 1: cell (1, 1, 0, 1)
        [1.5, 0.5, 1.5, 8.0],       # batch 2 == B -> out
    ], np.float32)
    batch = np.array([0, 0, 0, 0, 0, 0, 0, -1, 1, 2], np.int32)
    out_feats, out_coors, n = oracle.simple_mean(pts, batch, cfg, (2, 2, 2, 4), 8)
    assert n == 3
    got = {tuple(c): f for c, f in zip(out_coors[:n].tolist(), out_feats[:n])}
    assert set(got) == {(0, 0, 0, 0), (0, 0, 1, 3), (1, 1, 0, 1)}
    np.testing.assert_allclose(got[(0, 0, 0, 0)], [-0.125, 0.625, 0.375, 8.0])
    np.testing.assert_allclose(got[(0, 0, 1, 3)], [3.5, 1.5, 0.5, 2.0])
    np.testing.assert_allclose(got[(1, 1, 0, 1)], [1.5, 0.5, 1.5, 6.0])
    assert not out_feats[n:].any()


def test_empty_and_zero_capacity():
    cfg = np.array(CONFIG, np.float32)
    out_feats, out_coors, n = oracle.simple_mean(np.zeros((0, 4), np.float32), np.zeros(0, np.int32), cfg, SHAPE, 16)
    assert n == 0 and not out_feats.any()
    feats, batch, cfg_t = make_points(5, n=1000)
    _, _, n = oracle.simple_mean(feats.numpy(), batch.numpy(), cfg_t.numpy(), SHAPE, 0)
    assert n == 0


def test_many_points_per_voxel_mean():
    """Closed form: k points at the same cell with features 0..k-1 average to (k-1)/2."""
    k = 1000
    pts = np.zeros((k, 5), np.float32)
    pts[:, 0] = 0.3
    pts[:, 1] = 0.6
    pts[:, 2] = 0.1
    pts[:, 3] = np.arange(k)
    pts[:, 4] = -2.0 * np.arange(k)
    out_feats, out_coors, n = oracle.simple_mean(pts, np.zeros(k, np.int32), np.array([0, 0, 0, 1, 1, 1], np.float32),
                                                 (1, 1, 1, 1), 4)
    assert n == 1 and out_coors[0].tolist() == [0, 0, 0, 0]
    np.testing.assert_allclose(out_feats[0, 3:], [(k - 1) / 2, -(k - 1)], rtol=1e-6)
