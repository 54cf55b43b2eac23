"""BEVDensify on the GPU, through the C ABI, against the CPU oracle - bit-exact (the operator only moves bytes).
Covers the six parameterisations of the reference's test (tests/spconv/test_bev_densify.py:33-54) with its own
assertion (dense indexing, :19-26), ragged shapes that exercise every store variant, bf16 / int8 rows, stale
coordinates past the live count, rows outside the grid, and the tail of the CenterPoint-sized backbone."""
import numpy as np
import pytest
import torch

from densify_cases import CHANNELS, REFERENCE_CASES, SHAPE, dense_indexing, make_case, unique_coords
from oracle import oracle

pytestmark = pytest.mark.gpu


def _bits(t):
    t = t.cpu()
    return t.view(torch.int16).numpy() if t.dtype in (torch.float16, torch.bfloat16) else t.numpy()


def _run(feats, coords, num_act, shape, poison=True):
    from deploy3d_amd import bev_densify
    b, z, y, x = shape
    dev = torch.device("cuda:0")
    c = feats.shape[1]
    out = torch.empty((b, c * z, y, x), dtype=feats.dtype, device=dev)
    if poison:   # every byte of the map must be written by the operator
        out.view(torch.int8).fill_(0x5a)
    got = bev_densify(feats.to(dev), torch.from_numpy(coords).to(dev),
                      torch.tensor([num_act], dtype=torch.int32, device=dev),
                      torch.empty((b, 0, z, y, x), dtype=torch.int32, device=dev), c * z, out=out)
    torch.cuda.synchronize()
    return got


@pytest.mark.parametrize("num_act,dtype", REFERENCE_CASES)
def test_reference_cases(engine, num_act, dtype):
    feats, coords = make_case(5 + num_act, num_act, dtype)
    got = _run(feats, coords, num_act, SHAPE)
    assert tuple(got.shape) == (2, CHANNELS * 2, 128, 128) and got.dtype == feats.dtype
    want = oracle.bev_densify(_bits(feats), coords, num_act, SHAPE)
    assert np.array_equal(_bits(got), want)
    assert torch.allclose(dense_indexing(feats, coords, num_act, SHAPE), got.cpu())   # the reference's assertion


@pytest.mark.parametrize("shape,channels,dtype", [
    ((1, 1, 5, 7), 3, "float32"),       # odd plane, scalar loads
    ((3, 4, 9, 5), 10, "float16"),      # odd plane: one cell per store
    ((2, 3, 6, 33), 24, "float16"),     # even plane, rows of 48 bytes (vector loads, short chunk)
    ((1, 2, 37, 41), 200, "float32"),   # seven channel chunks, last one short
    ((2, 1, 7, 12), 17, "int8"),        # four cells per store, scalar loads
    ((2, 2, 5, 13), 32, "int8"),        # odd plane, vector loads
    ((1, 2, 64, 64), 64, "bfloat16"),
    ((1, 1, 1, 1), 1, "float32"),
])
def test_ragged_shapes_and_types(engine, shape, channels, dtype):
    rng = np.random.default_rng(17)
    n = max(1, int(np.prod(shape) * 0.4))
    cap = n + 13
    if dtype == "int8":
        feats = torch.from_numpy(rng.integers(-128, 128, (cap, channels), dtype=np.int8))
        _, coords = make_case(3, n, "float32", cap=cap, channels=1, shape=shape)
    else:
        feats, coords = make_case(3, n, dtype, cap=cap, channels=channels, shape=shape)
    got = _run(feats, coords, n, shape)
    assert np.array_equal(_bits(got), oracle.bev_densify(_bits(feats), coords, n, shape))


def test_full_grid_and_empty_grid(engine):
    shape = (2, 2, 16, 24)
    n = int(np.prod(shape))
    feats, coords = make_case(9, n, "float16", cap=n, channels=40, shape=shape)
    got = _run(feats, coords, n, shape)
    assert np.array_equal(_bits(got), oracle.bev_densify(_bits(feats), coords, n, shape))
    got = _run(feats, coords, 0, shape)
    assert not _bits(got).any()


def test_rows_outside_the_grid_are_skipped(engine):
    """The reference would write out of bounds (bev_densify_trt.cu:33); here such rows are dropped."""
    shape = (1, 2, 8, 8)
    feats, coords = make_case(4, 20, "float32", cap=24, channels=8, shape=shape)
    coords[3] = (0, 2, 0, 0)
    coords[7] = (-1, 0, 0, 0)
    coords[11] = (0, 0, 8, 1)
    coords[12] = (0, 1, 3, -5)
    keep = np.array([i for i in range(20) if i not in (3, 7, 11, 12)])
    got = _run(feats, coords, 20, shape)
    want = oracle.bev_densify(feats[keep].numpy(), coords[keep], len(keep), shape)
    assert np.array_equal(got.cpu().numpy(), want)


def test_repeated_cell_keeps_the_last_row(engine):
    shape = (1, 1, 4, 4)
    feats, coords = make_case(6, 10, "float32", cap=10, channels=4, shape=shape)
    coords[8] = coords[2]
    got = _run(feats, coords, 10, shape)
    want = oracle.bev_densify(feats.numpy(), coords, 10, shape)
    assert np.array_equal(got.cpu().numpy(), want)
    b, z, y, x = coords[2]
    assert np.array_equal(got.cpu().numpy().reshape(1, 4, 1, 4, 4)[b, :, z, y, x], feats[8].numpy())


def test_backbone_tail_shape(engine):
    """The map a CenterPoint-sized backbone hands to its 2-D head: [1, 128*2, 180, 180] fp16 from about 38 000 rows."""
    shape = (1, 2, 180, 180)
    rng = np.random.default_rng(23)
    n, cap = 38000, 40000
    feats = torch.from_numpy(rng.standard_normal((cap, 128)).astype(np.float32)).half()
    coords = np.zeros((cap, 4), dtype=np.int32)
    coords[:n] = unique_coords(rng, n, shape)
    got = _run(feats, coords, n, shape)
    assert np.array_equal(_bits(got), oracle.bev_densify(_bits(feats), coords, n, shape))
    # linearity of the scatter: the map's sum is the sum of the live rows
    assert abs(float(got.float().sum()) - float(feats[:n].float().sum())) < 1e-2 * n ** 0.5


def test_wrong_out_channels_is_an_error(engine):
    from deploy3d_amd import EngineError, bev_densify
    dev = torch.device("cuda:0")
    with pytest.raises(EngineError) as e:
        bev_densify(torch.zeros((8, 16), device=dev), torch.zeros((8, 4), dtype=torch.int32, device=dev),
                    torch.zeros(1, dtype=torch.int32, device=dev),
                    torch.empty((1, 0, 2, 4, 4), dtype=torch.int32, device=dev), 16)
    assert e.value.status == -3
