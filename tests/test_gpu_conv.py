"""GPU convolution parity: SPConvMM through the C ABI vs the CPU oracle
(out = bias; for tap: out[scatter] += in[gather] @ W[tap], fp64 accumulation
on operands rounded to the storage type).

Tolerances (stated by the task): fp32 within 1e-4 relative (|err| <= 1e-4 * (|ref| + rms(ref)));
fp16 within 2e-2 * rms(ref) absolute; bf16 (an extension) within 8 * 2e-2 * rms(ref), its ulp being 8x fp16's.
"""
import numpy as np
import pytest
import torch

from helpers import gpu_rulebook, random_cloud
from oracle import oracle

pytestmark = pytest.mark.gpu

TORCH_DTYPE = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}


def round_to(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(TORCH_DTYPE[dtype]).float().numpy()


def check_close(got, ref, dtype):
    rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2))) + 1e-30
    err = np.abs(got.astype(np.float64) - ref)
    if dtype == "float32":
        bound = 1e-4 * (np.abs(ref) + rms)
        assert (err <= bound).all(), "fp32: max err %g (rms %g)" % (err.max(), rms)
    else:
        tol = 2e-2 * rms * (8 if dtype == "bfloat16" else 1)
        assert err.max() <= tol, "%s: max err %g > %g (rms %g)" % (dtype, err.max(), tol, rms)


def run_case(n, grid, ksize, stride, padding, cin, cout, dtype, subm, with_bias=True, relu=False, inverse=False,
             seed=0, cap_extra=0, link=True):
    """link: the convolution is linked to the rulebook operator and reads the table that operator wrote (an inverse
    convolution never does); otherwise it derives the table from the index tensor, as an unlinked node does."""
    from deploy3d_amd import spconv_mm
    rng = np.random.default_rng(seed + n + cin * 7 + cout)
    coords = random_cloud(rng, n, grid, 1)
    n = len(coords)
    kvol = int(np.prod(ksize))
    dil = (1,) * len(ksize)
    max_out = n if subm else n * 8
    rb = gpu_rulebook(coords, n, grid, 1, ksize, stride, padding, dil, max_out, subm, cap=n + cap_extra, link=link)
    n_out = n if subm else rb["num_act_out"]
    in_rows, out_rows = (n + cap_extra, max_out) if not inverse else (max_out, n + cap_extra)
    feats = round_to(rng.standard_normal((in_rows, cin)), dtype)
    w = round_to(rng.standard_normal((kvol, cin, cout)) / np.sqrt(kvol * cin), dtype)
    b = round_to(rng.standard_normal(cout), dtype) if with_bias else None
    if inverse:
        cin_, cout_ = cin, cout
    ref = oracle.conv(feats, w, b, rb["index"], rb["num_index"], out_rows, inverse=inverse, acc="f64")
    if relu:
        ref = np.maximum(ref, 0.0)
    idx_dev, num_index_dev = rb["dev"][0], rb["dev"][1]
    num_in = rb["num_act_in"]
    num_out = num_in if subm else rb["dev"][3]
    if inverse:
        num_in, num_out = num_out, num_in
    x = torch.from_numpy(feats).to(device="cuda", dtype=TORCH_DTYPE[dtype])
    y = spconv_mm(x, num_in, num_out, idx_dev, num_index_dev, ksize, cin, cout, out_rows, subm, inverse, w, b,
                  relu=relu, rulebook=rb["plugin"] if link else None)
    torch.cuda.synchronize()
    got = y.float().cpu().numpy()
    live = n if (subm or inverse) else n_out
    check_close(got[:live], ref[:live], dtype)
    # rows beyond the live outputs hold the (activated) bias, as after the reference's biasInit (trt/spconv/mm.h:51-56)
    if out_rows > live:
        tail = np.zeros(cout) if b is None else b.astype(np.float64)
        if relu:
            tail = np.maximum(tail, 0)
        np.testing.assert_allclose(got[live:], np.broadcast_to(round_to(tail, dtype), got[live:].shape), rtol=0, atol=0)
    return got, ref


@pytest.mark.parametrize("cin,cout", [(16, 16), (16, 32), (32, 32), (32, 64), (64, 64), (64, 128), (128, 128),
                                      (128, 16), (16, 128)])
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_mfma_subm(engine, cin, cout, dtype):
    run_case(3000, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), cin, cout, dtype, True, relu=(cin == 32))


@pytest.mark.parametrize("cin,cout", [(16, 32), (32, 64), (64, 128), (128, 128)])
def test_mfma_strided(engine, cin, cout):
    run_case(3000, (10, 36, 30), (3, 3, 3), (2, 2, 2), (1, 1, 1), cin, cout, "float16", False, relu=True)


@pytest.mark.parametrize("cin,cout,dtype", [(5, 16, "float16"), (16, 16, "float32"), (3, 7, "float32"),
                                            (32, 64, "float32"), (40, 24, "float16"), (70, 130, "float32"),
                                            (5, 16, "bfloat16"), (1, 1, "float32")])
def test_narrow_subm(engine, cin, cout, dtype):
    run_case(2500, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), cin, cout, dtype, True, relu=(cout == 16))


@pytest.mark.parametrize("cin,cout,dtype", [(5, 16, "float16"), (16, 16, "float32"), (3, 7, "float32"), (24, 32, "float32"),
                                            (32, 20, "bfloat16")])
def test_narrow_tile_kernel_still_matches(engine, monkeypatch, cin, cout, dtype):
    """Layers of at most 32 x 32 channels take the rows-per-wavefront kernel; D3D_CONV_NARROW_ROWS=0 keeps them on the
    tile kernel that serves every other shape.  Both against the oracle."""
    monkeypatch.setenv("D3D_CONV_NO_PAD", "1")  # keep 2-byte layers off the MFMA path
    run_case(2500, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), cin, cout, dtype, True, seed=41)
    run_case(2500, (10, 36, 30), (3, 3, 3), (2, 2, 2), (1, 1, 1), cin, cout, dtype, False, seed=42, relu=True)
    monkeypatch.setenv("D3D_CONV_NARROW_ROWS", "0")
    run_case(2500, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), cin, cout, dtype, True, seed=41)


def test_narrow_strided_fp32(engine):
    run_case(2500, (10, 36, 30), (3, 3, 3), (2, 2, 2), (1, 1, 1), 16, 16, "float32", False)


@pytest.mark.parametrize("ksize,padding", [((3, 1, 3), (1, 0, 1)), ((1, 3, 3), (0, 1, 1)), ((1, 1, 1), (0, 0, 0)),
                                           ((5, 5, 5), (2, 2, 2))])
def test_kernel_shapes(engine, ksize, padding):
    run_case(2500, (10, 36, 30), ksize, (1, 1, 1), padding, 32, 64, "float16", True)


def test_large_kernel_volume_falls_back(engine):
    """7x7x7 at 128 channels fits no MFMA instantiation (343 taps of index rows and weights exceed LDS): the narrow
    kernel takes over instead of an error status; the reference accepts any kernel volume."""
    run_case(400, (12, 16, 16), (7, 7, 7), (1, 1, 1), (3, 3, 3), 128, 128, "float16", True, seed=31)
    run_case(400, (12, 16, 16), (7, 7, 7), (1, 1, 1), (3, 3, 3), 16, 128, "bfloat16", True, seed=32, link=False)


def test_mirrored_neighbour_table(engine, monkeypatch):
    """SubM with 'same' padding: the compaction writes the output-major table from the mirrored twin of every pair
    instead of scattering; D3D_RULEBOOK_MIRROR=0 selects the scatter, and an unlinked convolution derives the table
    from the index tensor.  All three must give the same features bit for bit, for shuffled rows and for rows in
    rank order; a SubM geometry without the symmetry (padding (1, 1, 0)) takes the scatter by itself and must still
    match the oracle."""
    for ksize, padding in (((3, 3, 3), (1, 1, 1)), ((3, 1, 3), (1, 0, 1)), ((5, 5, 5), (2, 2, 2))):
        monkeypatch.delenv("D3D_RULEBOOK_MIRROR", raising=False)
        a, _ = run_case(3000, (10, 36, 30), ksize, (1, 1, 1), padding, 32, 64, "float16", True, seed=5)
        monkeypatch.setenv("D3D_RULEBOOK_MIRROR", "0")
        b, _ = run_case(3000, (10, 36, 30), ksize, (1, 1, 1), padding, 32, 64, "float16", True, seed=5)
        c, _ = run_case(3000, (10, 36, 30), ksize, (1, 1, 1), padding, 32, 64, "float16", True, seed=5, link=False)
        assert np.array_equal(a, b) and np.array_equal(a, c)
    monkeypatch.delenv("D3D_RULEBOOK_MIRROR", raising=False)
    run_case(3000, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 0), 32, 64, "float16", True, seed=6)
    run_case(3000, (10, 36, 30), (3, 3, 2), (1, 1, 1), (1, 1, 0), 16, 32, "float16", True, seed=7)


@pytest.mark.parametrize("subm,stride", [(True, (1, 1, 1)), (False, (2, 2, 2))])
@pytest.mark.parametrize("cin,cout,dtype", [(64, 64, "float16"), (16, 32, "float16"), (5, 16, "float32")])
def test_unlinked_convolution_derives_its_table(engine, subm, stride, cin, cout, dtype):
    """A node nobody linked works from the index tensor alone, like the reference's (trt/spconv/mm_trt.cu:166-170)."""
    a, _ = run_case(3000, (10, 36, 30), (3, 3, 3), stride, (1, 1, 1), cin, cout, dtype, subm, link=False, seed=11)
    b, _ = run_case(3000, (10, 36, 30), (3, 3, 3), stride, (1, 1, 1), cin, cout, dtype, subm, link=True, seed=11)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("structure,near", [("blockmap", "1"), ("blockmap", "0"), ("hash", "1")])
def test_rows_outside_the_grid(engine, monkeypatch, structure, near):
    """Live rows whose coordinate lies outside the grid are out of contract in the reference (its hash keys alias
    into other cells, trt/spconv/index.cu:174-182); this engine ignores them: they take part in no pair.  The
    mirrored table a linked convolution reads and the table an unlinked one derives from the index tensor agree
    on that, in-grid rows get what the oracle gives for the in-grid cloud alone, and the ignored rows hold the
    bias."""
    from deploy3d_amd import spconv_mm
    monkeypatch.setenv("D3D_RULEBOOK", structure)
    monkeypatch.setenv("D3D_RULEBOOK_NEAR", near)
    rng = np.random.default_rng(21)
    grid, cin, cout = (10, 36, 30), 32, 64
    inside = random_cloud(rng, 2500, grid, 1)
    n_in = len(inside)
    bad = np.array([[0, -1, 5, 5], [0, 3, 36, 2], [0, 3, 4, 30], [1, 2, 2, 2], [0, 10, 0, 0], [-1, 1, 1, 1]], np.int32)
    where = np.sort(rng.choice(n_in + len(bad), size=len(bad), replace=False))
    coords = np.zeros((n_in + len(bad), 4), np.int32)
    is_bad = np.zeros(len(coords), bool)
    is_bad[where] = True
    coords[is_bad] = bad
    coords[~is_bad] = inside
    n = len(coords)
    feats = round_to(rng.standard_normal((n, cin)), "float16")
    w = round_to(rng.standard_normal((27, cin, cout)) / np.sqrt(27 * cin), "float16")
    b = round_to(rng.standard_normal(cout), "float16")
    geom = ((3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1))
    ref_rb = oracle.rulebook(inside, n_in, (1,) + grid, *geom, n_in, True)
    ref = oracle.conv(feats[~is_bad], w, b, ref_rb["index"], ref_rb["num_index"], n_in, acc="f64")
    got = {}
    for link in (True, False):
        rb = gpu_rulebook(coords, n, grid, 1, *geom, n, True, link=link)
        x = torch.from_numpy(feats).cuda().half()
        y = spconv_mm(x, rb["num_act_in"], rb["num_act_in"], rb["dev"][0], rb["dev"][1], (3, 3, 3), cin, cout, n,
                      True, False, w, b, rulebook=rb["plugin"] if link else None)
        torch.cuda.synchronize()
        got[link] = y.float().cpu().numpy()
        g, s, t = rb["index"][:, :rb["num_index"]]
        live = t >= 0
        assert not is_bad[g[live]].any() and not is_bad[s[live]].any()
    assert np.array_equal(got[True], got[False])
    check_close(got[True][~is_bad], ref, "float16")
    np.testing.assert_array_equal(got[True][is_bad], np.broadcast_to(b, (len(bad), cout)))


def _mm_on_index(index_np, num_index, n, cin, cout, feats, w, rulebook=None, index_dev=None):
    from deploy3d_amd import spconv_mm
    one = torch.tensor([n], dtype=torch.int32, device="cuda")
    idx = index_dev if index_dev is not None else torch.from_numpy(index_np).cuda()
    ni = torch.tensor([num_index], dtype=torch.int32, device="cuda")
    y = spconv_mm(torch.from_numpy(feats).cuda().half(), one, one, idx, ni, (3, 3, 3), cin, cout, n, True, False, w,
                  rulebook=rulebook)
    torch.cuda.synchronize()
    return y.float().cpu().numpy()


def test_foreign_and_edited_index_tensors(engine):
    """The index tensor is the contract: (a) a tensor uploaded from the CPU oracle, which this library never wrote;
    (b) a library-written tensor overwritten in place with another rulebook, fed to an unlinked node; (c) a linked
    node handed a tensor at another address than the one its rulebook operator wrote.  Each must give the result
    of the pairs the tensor holds."""
    rng = np.random.default_rng(42)
    grid, n, cin, cout = (10, 36, 30), 2000, 32, 32
    coords_a = random_cloud(rng, n, grid, 1)
    coords_b = random_cloud(rng, n, grid, 1)
    feats = round_to(rng.standard_normal((n, cin)), "float16")
    w = round_to(rng.standard_normal((27, cin, cout)) / np.sqrt(27 * cin), "float16")
    geom = ((3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1))
    ref = {}
    for name, c in (("a", coords_a), ("b", coords_b)):
        r = oracle.rulebook(c, n, (1,) + grid, *geom, n, True)
        ref[name] = (r["index"], r["num_index"], oracle.conv(feats, w, None, r["index"], r["num_index"], n, acc="f64"))
    # (a) oracle-written tensor
    got = _mm_on_index(ref["a"][0], ref["a"][1], n, cin, cout, feats, w)
    check_close(got, ref["a"][2], "float16")
    # (b) library-written, then edited in place
    rb = gpu_rulebook(coords_a, n, grid, 1, *geom, n, True, link=True)
    got = _mm_on_index(None, rb["num_index"], n, cin, cout, feats, w, rulebook=rb["plugin"], index_dev=rb["dev"][0])
    check_close(got, ref["a"][2], "float16")
    rb["dev"][0].copy_(torch.from_numpy(ref["b"][0]).cuda())
    got = _mm_on_index(None, ref["b"][1], n, cin, cout, feats, w, index_dev=rb["dev"][0])
    check_close(got, ref["b"][2], "float16")
    # (c) linked node, tensor at another address
    other = torch.from_numpy(ref["b"][0]).cuda()
    got = _mm_on_index(None, ref["b"][1], n, cin, cout, feats, w, rulebook=rb["plugin"], index_dev=other)
    check_close(got, ref["b"][2], "float16")


def test_duplicate_pairs_keep_the_highest_input(engine):
    """An index tensor that names two inputs for one (tap, output) - what duplicate input coordinates produce - is
    outside what the output-stationary convolution accumulates: it keeps one input per (tap, output), the highest
    row, on every run (the reference adds both; parity unpinned by the reference's tests, which never feed
    duplicates)."""
    n, cin, cout = 256, 32, 32
    rng = np.random.default_rng(3)
    feats = round_to(rng.standard_normal((n, cin)), "float16")
    w = round_to(rng.standard_normal((27, cin, cout)) / np.sqrt(27 * cin), "float16")
    row_len = 27 * (n + 128)
    index = np.full((3, row_len), -1, np.int32)
    # tap 13 (the centre): inputs 5 and 9 both feed output 5; input 7 feeds output 7
    index[0, :3] = (5, 7, 9)
    index[1, :3] = (5, 7, 5)
    index[2, :3] = 13
    keep = index.copy()
    keep[:, 0] = -1  # the pair (5 -> 5) loses against (9 -> 5)
    ref = oracle.conv(feats, w, None, keep, 128, n, acc="f64")
    for _ in range(3):
        got = _mm_on_index(index, 128, n, cin, cout, feats, w)
        check_close(got, ref, "float16")


@pytest.mark.parametrize("cin,cout", [(32, 32), (128, 128), (16, 16)])
def test_gather_rows_outside_the_input_are_no_neighbours(engine, cin, cout):
    """A foreign index tensor whose gather row names no input row - negative other than -1, at or past the row
    count, or so large that a row offset computed in 32 bits would wrap back inside the feature buffer (2^24 rows of
    256 bytes) - contributes nothing: the derived table keeps -1 or existing rows only."""
    n = 256
    rng = np.random.default_rng(11)
    feats = round_to(rng.standard_normal((n, cin)), "float16")
    w = round_to(rng.standard_normal((27, cin, cout)) / np.sqrt(27 * cin), "float16")
    row_len = 27 * (n + 128)
    index = np.full((3, row_len), -1, np.int32)
    bad = [n, n + 7, -5, (1 << 24) + 3, (1 << 25) + 1, np.iinfo(np.int32).max]
    index[0, :3] = (5, 7, 9)
    index[1, :3] = (5, 7, 5 + 64)
    index[2, :3] = 13
    index[0, 3:3 + len(bad)] = bad            # under the same tap, each feeding an output row of its own
    index[1, 3:3 + len(bad)] = np.arange(100, 100 + len(bad))
    index[2, 3:3 + len(bad)] = 13
    keep = index.copy()
    keep[:, 3:3 + len(bad)] = -1
    ref = oracle.conv(feats, w, None, keep, 128, n, acc="f64")
    got = _mm_on_index(index, 128, n, cin, cout, feats, w)
    check_close(got, ref, "float16")


@pytest.mark.parametrize("tile_rows", [128, 256, 512])
@pytest.mark.parametrize("cin,cout", [(32, 64), (64, 64), (64, 128), (128, 128)])
def test_mfma_tile_sizes(engine, monkeypatch, tile_rows, cin, cout):
    """Every workgroup tile height of the MFMA kernel (the launcher normally picks one from the row count)."""
    monkeypatch.setenv("D3D_CONV_TILE_ROWS", str(tile_rows))
    monkeypatch.setenv("D3D_CONV_STAGED", "off")
    run_case(3001, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), cin, cout, "float16", True, relu=True)


@pytest.mark.parametrize("shape", ["32,8", "32,6", "32,4", "48,4"])
@pytest.mark.parametrize("cin,cout,dtype", [(32, 128, "float16"), (64, 128, "float16"), (128, 128, "float16"),
                                            (128, 128, "bfloat16")])
def test_pipelined_tile_shapes_of_wide_layers(engine, monkeypatch, shape, cin, cout, dtype):
    """The four workgroup shapes (rows per wavefront, wavefronts) the pipelined kernel chooses from for 128 output
    channels by row count - 48-row wavefronts (three 16-row groups: the register sets alternate across steps) among
    them - each forced on a SubM layer (tile masks) and a strided one, and once on a layer with more tiles than
    workgroups, where the pipeline runs across tiles."""
    monkeypatch.setenv("D3D_CONV_PIPE_SHAPE", shape)
    run_case(9001, (12, 48, 40), (3, 3, 3), (1, 1, 1), (1, 1, 1), cin, cout, dtype, True, relu=True, cap_extra=50)
    if cin == 64:
        run_case(5000, (12, 48, 40), (3, 3, 3), (2, 2, 2), (1, 1, 1), cin, cout, dtype, False)
        run_case(70000, (16, 200, 200), (3, 3, 3), (1, 1, 1), (1, 1, 1), cin, cout, dtype, True, relu=True)


@pytest.mark.parametrize("cfg", ["off", "4,8,2", "2,8,3", "2,8,2", "4,4,2", "4,4,3", "4,8,3,1", "2,8,3,1"])
@pytest.mark.parametrize("cin,cout", [(16, 32), (32, 32), (32, 64), (64, 64), (64, 128), (128, 128), (128, 16)])
def test_staged_configurations(engine, monkeypatch, cfg, cin, cout):
    """Every configuration of the LDS-staged MFMA kernel (rows per wavefront, wavefronts, stage depth, resident
    weights), and the register-gather kernels behind "off"; a configuration a layer does not support falls back."""
    monkeypatch.setenv("D3D_CONV_STAGED", cfg)
    run_case(3001, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), cin, cout, "float16", True, relu=True)
    if cfg in ("4,8,2", "2,8,3", "off"):
        run_case(2100, (10, 36, 30), (3, 1, 1), (2, 1, 1), (0, 0, 0), cin, cout, "bfloat16", False)


@pytest.mark.parametrize("cin,cout", [(5, 16), (3, 32), (20, 32), (40, 64), (100, 128)])
@pytest.mark.parametrize("padded", [True, False])
def test_widened_input_channels(engine, monkeypatch, cin, cout, padded):
    """A layer whose output channels fit the MFMA path but whose input channels do not runs on rows widened with
    zero channels (weights widened with zero rows); D3D_CONV_NO_PAD keeps it on the narrow-channel kernel."""
    if not padded:
        monkeypatch.setenv("D3D_CONV_NO_PAD", "1")
    run_case(3000, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), cin, cout, "float16", True, relu=True, cap_extra=77)


def test_no_bias_no_relu(engine):
    run_case(2500, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), 32, 32, "float16", True, with_bias=False)


@pytest.mark.parametrize("subm", [True, False])
@pytest.mark.parametrize("dtype", ["float16", "float32"])
def test_inverse(engine, subm, dtype):
    """inverse swaps the gather and scatter rows of the same rulebook (trt/spconv/mm_trt.cu:174-177)."""
    stride = (1, 1, 1) if subm else (2, 2, 2)
    run_case(2500, (10, 36, 30), (3, 3, 3), stride, (1, 1, 1), 32, 16, dtype, subm, inverse=True)


def test_capacity_rows_beyond_live(engine):
    run_case(2500, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), 32, 32, "float16", True, cap_extra=777)


def test_bit_reproducible(engine):
    a, _ = run_case(3000, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), 64, 64, "float16", True)
    b, _ = run_case(3000, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), 64, 64, "float16", True)
    np.testing.assert_array_equal(a, b)


def test_unsupported_dtype_returns_minus_one(engine):
    """The reference returns -1 from enqueue for a dtype it does not implement (trt/spconv/mm_trt.cu:204)."""
    from deploy3d_amd import EngineError, spconv_mm
    x = torch.zeros((128, 16), dtype=torch.int32, device="cuda")
    idx = torch.full((3, 27 * 256), -1, dtype=torch.int32, device="cuda")
    one = torch.zeros(1, dtype=torch.int32, device="cuda")
    with pytest.raises((EngineError, KeyError)) as e:
        spconv_mm(x, one, one, idx, one, (3, 3, 3), 16, 16, 128, True, False, np.zeros(27 * 16 * 16, np.float32))
    if isinstance(e.value, EngineError):
        assert e.value.status == -1


def test_random_layers(engine):
    """Seeded sweep over random layers: channel counts on and off the MFMA shapes, all storage types, SubM and
    strided, kernel shapes, bias / ReLU / inverse, live rows short of the capacity - each against the fp64 oracle."""
    rng = np.random.default_rng(977)
    channels = [1, 3, 5, 8, 16, 20, 32, 48, 64, 96, 128]
    kernels = [((3, 3, 3), (1, 1, 1)), ((3, 1, 3), (1, 0, 1)), ((1, 3, 3), (0, 1, 1)), ((1, 1, 1), (0, 0, 0)),
               ((2, 2, 2), (0, 0, 0)), ((3, 3, 1), (1, 1, 0))]
    for i in range(30):
        cin, cout = (int(rng.choice(channels)) for _ in range(2))
        dtype = ("float16", "bfloat16", "float32")[int(rng.integers(0, 3))]
        ksize, padding = kernels[int(rng.integers(0, len(kernels)))]
        subm = bool(rng.integers(0, 2))
        stride = (1, 1, 1) if subm else tuple(int(rng.integers(1, 3)) for _ in range(3))
        inverse = (not subm) and bool(rng.integers(0, 4) == 0)
        run_case(int(rng.integers(200, 2500)), (10, 30, 28), ksize, stride, padding, cin, cout, dtype, subm,
                 with_bias=bool(rng.integers(0, 2)), relu=bool(rng.integers(0, 2)), inverse=inverse, seed=100 + i,
                 cap_extra=int(rng.integers(0, 3)) * 37)


def test_an_unprepared_node_is_refused_under_capture(engine):
    """Under stream capture an enqueue neither allocates nor synchronises.  A node that was never configured (its
    weights are not on the device, its derived table not reserved) reports UNSUPPORTED there; a node configured from
    its descriptors captures without ever having been enqueued, and so does the first one after an eager enqueue;
    replays give the eager result."""
    from deploy3d_amd import EngineError
    from deploy3d_amd.plugin import Plugin, TensorDesc
    from deploy3d_amd.spconv_mm import mm_blob, run_mm
    rng = np.random.default_rng(77)
    grid, ksize = (10, 36, 30), (3, 3, 3)
    coords = random_cloud(rng, 2000, grid, 1)
    n = len(coords)
    rb = gpu_rulebook(coords, n, grid, 1, ksize, (1, 1, 1), (1, 1, 1), (1, 1, 1), n, True)
    w = round_to(rng.standard_normal((27, 32, 32)) / 30.0, "float16")
    b = round_to(rng.standard_normal(32), "float16")
    x = torch.from_numpy(round_to(rng.standard_normal((n, 32)), "float16")).to(device="cuda", dtype=torch.float16)
    out = torch.empty((n, 32), dtype=torch.float16, device="cuda")
    args = (x, rb["num_act_in"], rb["num_act_in"], rb["dev"][0], rb["dev"][1])
    ref = oracle.conv(x.float().cpu().numpy(), w, b, rb["index"], rb["num_index"], n, acc="f64")

    def captured(plugin):
        graph, err = torch.cuda.CUDAGraph(), None
        with torch.cuda.graph(graph):
            try:
                run_mm(plugin, *args, out=out)
            except EngineError as e:
                err = e
        return graph, err

    def replayed(graph):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        return out.clone()

    fresh = Plugin("SPConvMM", mm_blob(ksize, 32, 32, n, True, False, w, b))
    _, err = captured(fresh)
    assert err is not None and err.status == -1 and "capture" in str(err)
    configured = Plugin("SPConvMM", mm_blob(ksize, 32, 32, n, True, False, w, b))
    in_descs = [TensorDesc.of_tensor(t) for t in args]
    configured.configure(in_descs, configured.output_descs(in_descs))
    graph, err = captured(configured)
    assert err is None
    check_close(replayed(graph).float().cpu().numpy(), ref, "float16")
    eager = run_mm(fresh, *args, out=out).clone()      # one eager enqueue reserves everything
    torch.cuda.synchronize()
    check_close(eager.float().cpu().numpy(), ref, "float16")
    graph, err = captured(fresh)
    assert err is None
    assert torch.equal(replayed(graph), eager)
