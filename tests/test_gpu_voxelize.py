"""SimpleMeanEncoder on the GPU, through the C ABI: the two parameterisations of the reference's test
(tests/voxel_encoder/test_simple_mean.py:59-64) with its assertions, then against the CPU oracle after sorting both
by coordinate (coordinates and the live count bit-exact; means within rtol 1e-5 / atol 2e-5 - both sides add in
fp32, in different orders), the row order this engine promises (first appearance among the points), and the
edge cases: conversion toward zero, skipped rows, empty input, zero capacity, one crowded voxel."""
import numpy as np
import pytest
import torch

from oracle import oracle
from voxelize_cases import CONFIG, SHAPE, check_against_truth, ground_truth, make_points

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _run(feats, batch, cfg, shape, max_out):
    from deploy3d_amd import simple_mean_encoder
    b, z, y, x = shape
    f = torch.as_tensor(feats).to(DEV)
    out = simple_mean_encoder(f, torch.as_tensor(batch).to(DEV), torch.as_tensor(cfg).to(DEV),
                              torch.empty((b, 0, z, y, x), dtype=torch.int32, device=DEV), max_out)
    torch.cuda.synchronize()
    return out[0].cpu().numpy(), out[1].cpu().numpy(), int(out[2].item())


def _first_appearance(feats, batch, cfg, shape):
    """Cells of the valid points in the order in which they first occur (numpy restatement of the validity rule)."""
    feats = np.asarray(feats, np.float32)
    cfg = np.asarray(cfg, np.float32)
    with np.errstate(all="ignore"):
        q = ((feats[:, :3] - cfg[:3]) / cfg[3:]).astype(np.float32)
        ok = np.isfinite(feats).all(axis=1) & (np.asarray(batch) >= 0) & (np.asarray(batch) < shape[0])
        q = np.where(np.isfinite(q), q, -1.0)
        c = np.trunc(q).astype(np.int64)
    ok &= (c[:, 0] >= 0) & (c[:, 0] < shape[3]) & (c[:, 1] >= 0) & (c[:, 1] < shape[2]) & (c[:, 2] >= 0) & (c[:, 2] < shape[1])
    cells = np.stack([np.asarray(batch, np.int64), c[:, 2], c[:, 1], c[:, 0]], axis=1)[ok]
    key = ((cells[:, 0] * shape[1] + cells[:, 1]) * shape[2] + cells[:, 2]) * shape[3] + cells[:, 3]
    _, first = np.unique(key, return_index=True)
    return cells[np.sort(first)].astype(np.int32)


@pytest.mark.parametrize("max_out", [200000, 100])
def test_reference_cases(engine, max_out):
    feats, batch, cfg = make_points(1234)
    truth = ground_truth(feats, batch, cfg)
    got_f, got_c, n = _run(feats, batch, cfg, SHAPE, max_out)
    check_against_truth(got_f, got_c, n, truth, max_out)                 # the reference's assertions
    assert not got_f[n:].any()                                           # simple_mean_trt.cu:142
    order = _first_appearance(feats.numpy(), batch.numpy(), cfg.numpy(), SHAPE)
    assert np.array_equal(got_c[:n], order[:n])                          # row order, and which voxels survive a cut
    ref_f, ref_c, ref_n = oracle.simple_mean(feats.numpy(), batch.numpy(), cfg.numpy(), SHAPE, 200000)
    assert min(ref_n, max_out) == n
    lut = {tuple(r): i for i, r in enumerate(ref_c[:ref_n].tolist())}
    rows = np.array([lut[tuple(r)] for r in got_c[:n].tolist()])
    np.testing.assert_allclose(got_f[:n], ref_f[rows], rtol=1e-5, atol=2e-5)
    if max_out >= ref_n:
        assert np.array_equal(got_c[:n][np.lexsort(got_c[:n].T[::-1])], ref_c[:ref_n][np.lexsort(ref_c[:ref_n].T[::-1])])


def test_deterministic_rows(engine):
    feats, batch, cfg = make_points(77, n=50000)
    a = _run(feats, batch, cfg, SHAPE, 60000)
    b = _run(feats, batch, cfg, SHAPE, 60000)
    assert a[2] == b[2] and np.array_equal(a[1][:a[2]], b[1][:b[2]])
    np.testing.assert_allclose(a[0], b[0], rtol=1e-5, atol=2e-5)


def test_truncation_toward_zero_and_skipped_rows(engine):
    cfg = np.array([0.0, 0.0, 0.0, 1.0, 1.0, 1.0], np.float32)
    pts = np.array([[-0.5, 0.5, 0.5, 7.0], [0.25, 0.75, 0.25, 9.0], [-1.0, 0.5, 0.5, 1.0], [3.5, 1.5, 0.5, 2.0],
                    [4.0, 0.5, 0.5, 3.0], [np.nan, 0.5, 0.5, 1.0], [0.5, 0.5, 0.5, np.inf], [1.5, 0.5, 1.5, 5.0],
                    [1.5, 0.5, 1.5, 6.0], [1.5, 0.5, 1.5, 8.0]], np.float32)
    batch = np.array([0, 0, 0, 0, 0, 0, 0, -1, 1, 2], np.int32)
    got_f, got_c, n = _run(pts, batch, cfg, (2, 2, 2, 4), 8)
    assert n == 3
    assert got_c[:3].tolist() == [[0, 0, 0, 0], [0, 0, 1, 3], [1, 1, 0, 1]]
    np.testing.assert_allclose(got_f[:3], [[-0.125, 0.625, 0.375, 8.0], [3.5, 1.5, 0.5, 2.0], [1.5, 0.5, 1.5, 6.0]])
    assert not got_f[3:].any()
    ref_f, ref_c, ref_n = oracle.simple_mean(pts, batch, cfg, (2, 2, 2, 4), 8)
    assert ref_n == 3 and {tuple(r) for r in ref_c[:3].tolist()} == {tuple(r) for r in got_c[:3].tolist()}


def test_huge_and_degenerate_values(engine):
    """Quotients that overflow to +-inf or past int32 convert to the saturated value and fall outside the grid."""
    cfg = np.array([0.0, 0.0, 0.0, 1e-30, 1.0, 1.0], np.float32)
    pts = np.array([[1e10, 0.5, 0.5], [-1e10, 0.5, 0.5], [0.0, 0.5, 0.5], [1e-30, 0.5, 0.5]], np.float32)
    batch = np.zeros(4, np.int32)
    got_f, got_c, n = _run(pts, batch, cfg, (1, 1, 1, 4), 4)
    ref_f, ref_c, ref_n = oracle.simple_mean(pts, batch, cfg, (1, 1, 1, 4), 4)
    assert n == ref_n == 2
    assert sorted(map(tuple, got_c[:n].tolist())) == sorted(map(tuple, ref_c[:n].tolist())) == [(0, 0, 0, 0), (0, 0, 0, 1)]


def test_empty_input_and_zero_capacity(engine):
    cfg = np.array(CONFIG, np.float32)
    got_f, got_c, n = _run(np.zeros((0, 4), np.float32), np.zeros(0, np.int32), cfg, SHAPE, 16)
    assert n == 0 and not got_f.any()
    feats, batch, cfg_t = make_points(5, n=1000)
    _, _, n = _run(feats, batch, cfg_t, SHAPE, 0)
    assert n == 0
    # every point skipped
    got_f, _, n = _run(feats, torch.full_like(batch, -1), cfg_t, SHAPE, 64)
    assert n == 0 and not got_f.any()


@pytest.mark.parametrize("channels", [3, 5, 9])
def test_crowded_voxels_and_channel_counts(engine, channels):
    rng = np.random.default_rng(channels)
    n = 30000
    pts = rng.uniform(0, 4, (n, channels)).astype(np.float32)        # 4 x 4 x 4 cells: ~470 points per voxel
    batch = rng.integers(0, 2, n).astype(np.int32)
    cfg = np.array([0, 0, 0, 1, 1, 1], np.float32)
    got_f, got_c, got_n = _run(pts, batch, cfg, (2, 4, 4, 4), 200)
    ref_f, ref_c, ref_n = oracle.simple_mean(pts, batch, cfg, (2, 4, 4, 4), 200)
    assert got_n == ref_n == 128
    go, ro = np.lexsort(got_c[:128].T[::-1]), np.lexsort(ref_c[:128].T[::-1])
    assert np.array_equal(got_c[:128][go], ref_c[:128][ro])
    np.testing.assert_allclose(got_f[:128][go], ref_f[:128][ro], rtol=2e-5, atol=2e-5)


def test_wrong_dtype_is_unsupported(engine):
    from deploy3d_amd import EngineError, Plugin, TensorDesc
    from deploy3d_amd.simple_mean import simple_mean_blob
    p = Plugin("SimpleMeanEncoder", simple_mean_blob(8))
    ins = [TensorDesc.of((4, 4), torch.float16), TensorDesc.of((4,), torch.int32), TensorDesc.of((6,), torch.float16),
           TensorDesc.of((1, 0, 2, 2, 2), torch.int32)]
    outs = p.output_descs(ins)
    t = torch.zeros(64, device=DEV)
    with pytest.raises(EngineError) as e:
        p.enqueue(ins, outs, [t, t, t, None], [t, t, t], torch.zeros(1 << 16, dtype=torch.uint8, device=DEV))
    assert e.value.status == -1
