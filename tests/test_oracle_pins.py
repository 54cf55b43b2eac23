"""Pins the CPU oracle (oracle/spconv_oracle.cpp) with checks that do not restate its formulas:
published known answers, torch's dense convolutions, an independent brute-force rulebook that walks from the
OUTPUT side, closed forms, and the structural invariants the reference's own test asserts
(tests/spconv/test_spconv.py:72-124)."""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import bruteforce_rulebook, check_index_structure, dense_from_sparse, dense_weight, random_cloud
from oracle import oracle


# ---- hash finaliser --------------------------------------------------------------------------------------
def test_fmix32_known_answers():
    """MurmurHash3 fmix32 (trt/include/common/hash32.h:23-33): published answers, plus bijectivity on a sample
    (fmix32 is invertible, so distinct inputs never collide) - a dropped xor-shift or a wrong constant fails."""
    assert oracle.fmix32(0) == 0
    assert oracle.fmix32(1) == 0x514E28B7
    assert oracle.fmix32(2) == 0x30F4C306
    outs = {oracle.fmix32(i) for i in range(20000)}
    assert len(outs) == 20000


# ---- output shape ----------------------------------------------------------------------------------------
@pytest.mark.parametrize("k,s,p,d", [(3, 1, 1, 1), (3, 2, 1, 1), (3, 2, 0, 1), (2, 2, 0, 1), (5, 3, 2, 1), (3, 1, 2, 2),
                                     (1, 1, 0, 1), (4, 3, 1, 2)])
def test_out_shape_matches_torch_conv(k, s, p, d):
    for n in (7, 16, 41):
        if n + 2 * p - d * (k - 1) < 1:
            continue
        want = F.conv1d(torch.zeros(1, 1, n), torch.zeros(1, 1, k), stride=s, padding=p, dilation=d).shape[-1]
        assert oracle.out_shape([n], [k], [s], [p], [d]) == [want]
        for op in range(s):
            wt = F.conv_transpose1d(torch.zeros(1, 1, n), torch.zeros(1, 1, k), stride=s, padding=p, dilation=d,
                                    output_padding=op).shape[-1]
            assert oracle.out_shape([n], [k], [s], [p], [d], [op], transpose=True) == [wt]


def test_out_shape_config3_grids():
    """The stage grids of the VoxelNet backbone are fixed numbers any SECOND implementation reproduces."""
    g = [41, 1440, 1440]
    g = oracle.out_shape(g, (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1)); assert g == [21, 720, 720]
    g = oracle.out_shape(g, (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1)); assert g == [11, 360, 360]
    g = oracle.out_shape(g, (3, 3, 3), (2, 2, 2), (0, 1, 1), (1, 1, 1)); assert g == [5, 180, 180]
    g = oracle.out_shape(g, (3, 1, 1), (2, 1, 1), (0, 0, 0), (1, 1, 1)); assert g == [2, 180, 180]


# ---- rulebook vs brute force -----------------------------------------------------------------------------
RB_CASES = [
    # grid, batch, n, k, s, p, d, subm, transpose
    ((6, 10, 9), 2, 300, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), True, False),
    ((6, 10, 9), 1, 200, (3, 1, 3), (1, 1, 1), (1, 0, 1), (1, 1, 1), True, False),
    ((8, 8, 8), 1, 200, (3, 3, 3), (1, 1, 1), (2, 2, 2), (2, 2, 2), True, False),
    ((6, 10, 9), 2, 300, (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), False, False),
    ((6, 10, 9), 1, 300, (3, 3, 3), (2, 2, 1), (1, 0, 1), (1, 2, 1), False, False),
    ((7, 9, 11), 1, 250, (2, 2, 2), (2, 2, 2), (0, 0, 0), (1, 1, 1), False, False),
    ((7, 9, 11), 1, 250, (3, 3, 3), (3, 2, 1), (1, 0, 2), (1, 1, 1), False, False),
    ((5, 6, 7), 1, 100, (3, 2, 3), (2, 2, 2), (1, 0, 1), (1, 1, 1), False, True),
    ((5, 6, 7), 2, 100, (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), False, True),
    ((30, 40), 1, 300, (3, 3), (2, 2), (1, 1), (1, 1), False, False),
    ((200,), 2, 120, (5,), (1,), (2,), (1,), True, False),
    ((4, 5, 6, 7), 1, 200, (3, 3, 3, 3), (2, 2, 2, 2), (1, 1, 1, 1), (1, 1, 1, 1), False, False),
]


@pytest.mark.parametrize("case", RB_CASES, ids=lambda c: "%s_k%s_s%s%s%s" % (
    "x".join(map(str, c[0])), "".join(map(str, c[3])), "".join(map(str, c[4])), "_subm" if c[7] else "",
    "_T" if c[8] else ""))
def test_rulebook_matches_bruteforce(case):
    grid, batch, n, k, s, p, d, subm, transpose = case
    rng = np.random.default_rng(hash(case) & 0xFFFF)
    coords = random_cloud(rng, n, grid, batch)
    n = len(coords)
    out_grid = list(grid) if subm else oracle.out_shape(grid, k, s, p, d, None, transpose)
    kvol = int(np.prod(k))
    rb = oracle.rulebook(coords, n, [batch] + out_grid, k, s, p, d, n * kvol, subm, transpose)
    out_coords = coords if subm else rb["out_coors"]
    n_out = n if subm else rb["num_act_out"]
    got_c, got_t = oracle.canonical(rb["index"], rb["num_index"], out_coords, n_out)
    want_c, want_t = bruteforce_rulebook(coords, [batch] + out_grid, k, s, p, d, subm, transpose)
    np.testing.assert_array_equal(got_c, want_c)
    np.testing.assert_array_equal(got_t, want_t)
    check_index_structure(rb["index"], rb["num_index"], kvol, n)


def test_subm_symmetry_and_identity():
    """Reference-held invariants (test_spconv.py:101-108): centre tap is the identity, tap k mirrors tap 26-k."""
    rng = np.random.default_rng(5)
    coords = random_cloud(rng, 2000, (10, 30, 30), 1)
    rb = oracle.rulebook(coords, 2000, [1, 10, 30, 30], (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 2000, True)
    g, s, t = rb["index"][:, :rb["num_index"]]
    c = t == 13
    assert c.sum() == 2000 and (g[c] == s[c]).all()
    for k in range(13):
        a = {(int(x), int(y)) for x, y in zip(g[t == k], s[t == k])}
        b = {(int(y), int(x)) for x, y in zip(g[t == 26 - k], s[t == 26 - k])}
        assert a == b


def test_truncation_subset():
    """test_spconv.py:72-78: with maxNumActOut below the true count exactly that many unique outputs survive."""
    rng = np.random.default_rng(6)
    coords = random_cloud(rng, 1500, (10, 30, 30), 1)
    args = ([1, 5, 15, 15], (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1))
    full = oracle.rulebook(coords, 1500, *args, 100000, False)
    cut = oracle.rulebook(coords, 1500, *args, 200, False)
    assert cut["num_act_out"] == 200 < full["num_act_out"]
    kept = {tuple(c) for c in cut["out_coors"][:200].tolist()}
    assert len(kept) == 200 and kept <= {tuple(c) for c in full["out_coors"][:full["num_act_out"]].tolist()}
    live = cut["index"][2, :cut["num_index"]] >= 0
    assert (cut["index"][1, :cut["num_index"]][live] < 200).all()


def test_empty_and_single():
    coords = np.zeros((8, 4), dtype=np.int32)
    rb = oracle.rulebook(coords, 0, [1, 4, 4, 4], (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), 8, False)
    assert rb["num_index"] == 0 and rb["num_act_out"] == 0
    one = np.array([[0, 2, 3, 4]], dtype=np.int32)
    rb = oracle.rulebook(one, 1, [1, 5, 6, 7], (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, True)
    assert rb["num_index"] == 128 and (rb["index"][:, 0] == [0, 0, 13]).all()


# ---- convolution vs dense torch --------------------------------------------------------------------------
CONV_CASES = [
    ((6, 7, 8), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), True),
    ((6, 7, 8), (3, 1, 3), (1, 1, 1), (1, 0, 1), (1, 1, 1), True),
    ((6, 7, 8), (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), False),
    ((6, 7, 8), (3, 3, 3), (2, 1, 2), (0, 1, 1), (1, 1, 1), False),
    ((6, 7, 8), (2, 2, 2), (2, 2, 2), (0, 0, 0), (1, 1, 1), False),
    ((8, 8, 8), (3, 3, 3), (1, 1, 1), (2, 2, 2), (2, 2, 2), False),
]


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "k%s_s%s_p%s%s" % (
    "".join(map(str, c[1])), "".join(map(str, c[2])), "".join(map(str, c[3])), "_subm" if c[5] else ""))
def test_conv_equals_dense_conv3d(case):
    """Sparse conv == torch conv3d on the densified input, sampled at the active outputs; every dense output
    outside the active set equals the bias alone (no input reaches it).  A transposed tap order, a sign error in
    the offset or a swapped weight axis all fail this."""
    grid, k, s, p, d, subm = case
    rng = np.random.default_rng(11)
    batch, cin, cout, n = 2, 5, 7, 150
    coords = random_cloud(rng, n, grid, batch)
    feats = rng.standard_normal((n, cin)).astype(np.float32)
    w = rng.standard_normal((int(np.prod(k)), cin, cout)).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    dense = F.conv3d(dense_from_sparse(coords, feats, grid, batch), dense_weight(w, k), torch.as_tensor(b).double(),
                     stride=s, padding=p, dilation=d)
    out_grid = list(grid) if subm else oracle.out_shape(grid, k, s, p, d)
    assert list(dense.shape[2:]) == out_grid
    rb = oracle.rulebook(coords, n, [batch] + out_grid, k, s, p, d, n * 27, subm)
    n_out = n if subm else rb["num_act_out"]
    oc = coords if subm else rb["out_coors"][:n_out]
    y = oracle.conv(feats, w, b, rb["index"], rb["num_index"], n_out, acc="f64")
    want = dense[oc[:, 0], :, oc[:, 1], oc[:, 2], oc[:, 3]].numpy()
    np.testing.assert_allclose(y, want, rtol=1e-9, atol=1e-9)
    if not subm:
        mask = torch.ones(dense.shape[0], *dense.shape[2:], dtype=torch.bool)
        mask[oc[:, 0], oc[:, 1], oc[:, 2], oc[:, 3]] = False
        rest = dense.permute(0, 2, 3, 4, 1)[mask]
        np.testing.assert_allclose(rest.numpy(), np.broadcast_to(b.astype(np.float64), rest.shape), atol=1e-9)


def test_conv_transposed_equals_conv_transpose3d():
    grid, k, s, p = (4, 5, 6), (3, 3, 3), (2, 2, 2), (1, 1, 1)
    rng = np.random.default_rng(12)
    cin, cout, n = 4, 3, 60
    coords = random_cloud(rng, n, grid, 1)
    feats = rng.standard_normal((n, cin)).astype(np.float32)
    w = rng.standard_normal((27, cin, cout)).astype(np.float32)
    out_grid = oracle.out_shape(grid, k, s, p, (1, 1, 1), (0, 0, 0), transpose=True)
    rb = oracle.rulebook(coords, n, [1] + out_grid, k, s, p, (1, 1, 1), n * 27, False, True)
    y = oracle.conv(feats, w, None, rb["index"], rb["num_index"], rb["num_act_out"], acc="f64")
    wt = torch.as_tensor(w, dtype=torch.float64).reshape(3, 3, 3, cin, cout).permute(3, 4, 0, 1, 2)  # [I, O, kz, ky, kx]
    dense = F.conv_transpose3d(dense_from_sparse(coords, feats, grid, 1), wt.contiguous(), stride=s, padding=p)
    oc = rb["out_coors"][:rb["num_act_out"]]
    np.testing.assert_allclose(y, dense[oc[:, 0], :, oc[:, 1], oc[:, 2], oc[:, 3]].numpy(), rtol=1e-9, atol=1e-9)
    assert abs(dense.abs().sum().item() - np.abs(y).sum()) < 1e-6  # nothing lands outside the emitted outputs


def test_conv_special_cases():
    rng = np.random.default_rng(13)
    n, cin, cout = 100, 6, 4
    coords = random_cloud(rng, n, (5, 6, 7), 1)
    feats = rng.standard_normal((n, cin)).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    # 1x1x1 kernel is a plain matrix product
    w1 = rng.standard_normal((1, cin, cout)).astype(np.float32)
    rb = oracle.rulebook(coords, n, [1, 5, 6, 7], (1, 1, 1), (1, 1, 1), (0, 0, 0), (1, 1, 1), n, True)
    y = oracle.conv(feats, w1, b, rb["index"], rb["num_index"], n, acc="f64")
    np.testing.assert_allclose(y, feats.astype(np.float64) @ w1[0] + b, rtol=1e-12)
    # a single voxel: the output at its own site is x @ W[centre]
    w = rng.standard_normal((27, cin, cout)).astype(np.float32)
    one = coords[:1]
    rb = oracle.rulebook(one, 1, [1, 5, 6, 7], (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, True)
    y = oracle.conv(feats[:1], w, None, rb["index"], rb["num_index"], 1, acc="f64")
    np.testing.assert_allclose(y[0], feats[0].astype(np.float64) @ w[13], rtol=1e-12)
    # inverse: gather and scatter rows swapped (trt/spconv/mm_trt.cu:174-177) == the adjoint pairing
    rb = oracle.rulebook(coords, n, [1, 3, 3, 4], (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), 27 * n, False)
    m = rb["num_act_out"]
    g = rng.standard_normal((m, cin)).astype(np.float32)
    winv = rng.standard_normal((27, cin, cout)).astype(np.float32)
    y = oracle.conv(g, winv, None, rb["index"], rb["num_index"], n, inverse=True, acc="f64")
    want = np.zeros((n, cout))
    gi, si, ti = rb["index"][:, :rb["num_index"]]
    for a, c, t in zip(gi, si, ti):
        if t >= 0:
            want[a] += g[c].astype(np.float64) @ winv[t]
    np.testing.assert_allclose(y, want, rtol=1e-10, atol=1e-10)
    # fp32 accumulation stays within fp32 rounding of fp64 accumulation; threads do not change the result
    rb = oracle.rulebook(coords, n, [1, 5, 6, 7], (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), n, True)
    y64 = oracle.conv(feats, w, b, rb["index"], rb["num_index"], n, acc="f64")
    y32 = oracle.conv(feats, w, b, rb["index"], rb["num_index"], n, acc="f32")
    np.testing.assert_allclose(y32, y64, rtol=1e-4, atol=1e-5)
    np.testing.assert_array_equal(oracle.conv(feats, w, b, rb["index"], rb["num_index"], n, acc="f64", threads=4), y64)


def test_int8_conv_and_requantize_exact():
    """The int8 path is this build's extension (the reference accepts fp16 only, trt/spconv/mm_trt.cu:184):
    parity unpinned by the reference.  Integer accumulation is checked against numpy int64; the requantize rule
    against a float64 evaluation wherever that is not within 1e-3 of a rounding tie."""
    rng = np.random.default_rng(14)
    n, cin, cout = 200, 16, 8
    coords = random_cloud(rng, n, (5, 8, 8), 1)
    rb = oracle.rulebook(coords, n, [1, 5, 8, 8], (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), n, True)
    x = rng.integers(-128, 128, (n, cin)).astype(np.int8)
    w = rng.integers(-127, 128, (27, cin, cout)).astype(np.int8)
    acc = oracle.conv_i8(x, w, rb["index"], rb["num_index"], n)
    want = np.zeros((n, cout), dtype=np.int64)
    gi, si, ti = rb["index"][:, :rb["num_index"]]
    for a, c, t in zip(gi, si, ti):
        if t >= 0:
            want[c] += x[a].astype(np.int64) @ w[t].astype(np.int64)
    np.testing.assert_array_equal(acc, want)
    m = (rng.random(cout) * 1e-3 + 1e-4).astype(np.float32)
    bq = rng.standard_normal(cout).astype(np.float32)
    for relu in (False, True):
        q = oracle.requantize(acc, m, bq, relu)
        exact = acc.astype(np.float64) * m.astype(np.float64) + bq.astype(np.float64)
        ref = np.clip(np.rint(exact), 0 if relu else -128, 127)
        safe = np.abs(exact - np.floor(exact) - 0.5) > 1e-3
        np.testing.assert_array_equal(q[safe], ref[safe].astype(np.int8))
    assert oracle.requantize(np.array([[5]], np.int32), np.array([0.5], np.float32), np.array([0.0], np.float32),
                             False)[0, 0] == 2      # 2.5 rounds to even
    assert oracle.requantize(np.array([[7]], np.int32), np.array([0.5], np.float32), np.array([0.0], np.float32),
                             False)[0, 0] == 4      # 3.5 rounds to even
    assert oracle.requantize(np.array([[10 ** 9]], np.int32), np.array([1.0], np.float32),
                             np.array([0.0], np.float32), False)[0, 0] == 127
    assert oracle.requantize(np.array([[-10 ** 9]], np.int32), np.array([1.0], np.float32),
                             np.array([0.0], np.float32), True)[0, 0] == 0


def test_quantize_weights_per_output_channel():
    """oracle.quantize_weights (no counterpart in the reference: it has no int8 path, trt/spconv/mm_trt.cu:184).
    Pinned by what symmetric per-OUTPUT-channel quantization means, not by its formula: every channel's largest
    magnitude sits in a different (tap, input channel) and must land on +-127 with a scale that reproduces it; an
    all-zero channel gets scale 1; every weight is reproduced to within half a quantum.  Taking the maximum over
    the wrong axes, a per-tensor scale, 128 levels or truncation instead of rounding each fail one of these."""
    rng = np.random.default_rng(21)
    kvol, cin, cout = 27, 16, 8
    w = (rng.standard_normal((kvol, cin, cout)) * 0.01).astype(np.float32)
    peaks = np.array([0.5, 3.0, 0.125, 7.5, 1.0, 0.75, 2.25, 0.0], dtype=np.float32)
    where = [(c * 3 % kvol, (5 * c + 1) % cin) for c in range(cout)]
    for c, (t, ci) in enumerate(where):
        w[t, ci, c] = peaks[c] * (-1 if c % 2 else 1)
    w[:, :, 7] = 0.0                                     # a dead channel
    q, s_w = oracle.quantize_weights(w)
    assert q.dtype == np.int8 and q.shape == w.shape and s_w.shape == (cout,)
    for c, (t, ci) in enumerate(where[:7]):
        assert q[t, ci, c] == (-127 if c % 2 else 127), c
        assert abs(float(s_w[c]) * 127.0 - float(peaks[c])) <= 1e-12 * float(peaks[c]), c
        assert np.abs(q[:, :, c]).max() == 127
    assert s_w[7] == 1.0 and not q[:, :, 7].any()
    err = np.abs(w.astype(np.float64) - q.astype(np.float64) * s_w[None, None, :])
    assert (err <= s_w[None, None, :] * (0.5 + 1e-9)).all()
    assert np.abs(q).max() <= 127 and q.min() >= -127    # symmetric: -128 is never produced
    # an exact tie between two levels rounds to the even one: 2.5 quanta -> 2, 3.5 quanta -> 4
    t = np.zeros((1, 4, 1), dtype=np.float32)
    t[0, :, 0] = [127.0, 2.5, 3.5, -2.5]
    qt, st = oracle.quantize_weights(t)
    assert st[0] == 1.0 and qt[0, :, 0].tolist() == [127, 2, 4, -2]


def test_requant_params_mean_what_requantization_needs():
    """oracle.requant_params: with activations x = q_x * s_in, weights w = q_w * s_w[c] and outputs in quanta of
    s_out, the real pre-activation of an accumulator a is a * s_in * s_w[c] + bias[c], so the output level is
    rint((a * s_in * s_w[c] + bias[c]) / s_out).  m and bq are checked (1) against exact rational arithmetic,
    correctly rounded to fp32 up to the double rounding of one division, and (2) end to end through
    oracle.requantize against that definition evaluated in rationals, away from rounding ties.  A swapped
    quotient, a missing scale or a bias left in real units fails both."""
    from fractions import Fraction
    rng = np.random.default_rng(22)
    cout = 6
    s_in, s_out = np.float32(0.0371), np.float32(0.0519)
    s_w = (rng.random(cout) * 0.01 + 1e-4).astype(np.float64)
    bias = rng.standard_normal(cout).astype(np.float32)
    m, bq = oracle.requant_params(s_in, s_w, s_out, bias)
    assert m.dtype == np.float32 and bq.dtype == np.float32
    for c in range(cout):
        m_exact = Fraction(float(s_in)) * Fraction(float(s_w[c])) / Fraction(float(s_out))
        b_exact = Fraction(float(bias[c])) / Fraction(float(s_out))
        for got, exact in ((m[c], m_exact), (bq[c], b_exact)):
            ulp = float(np.spacing(np.float32(abs(float(exact)))))
            assert abs(Fraction(float(got)) - exact) <= Fraction(ulp) * Fraction(501, 1000), (c, got, float(exact))
    m0, bq0 = oracle.requant_params(s_in, s_w, s_out, None)
    assert np.array_equal(m0, m) and not bq0.any()
    acc = rng.integers(-40000, 40000, (300, cout)).astype(np.int32)
    for relu in (False, True):
        q = oracle.requantize(acc, m, bq, relu)
        for r in range(acc.shape[0]):
            for c in range(cout):
                real = (Fraction(int(acc[r, c])) * Fraction(float(s_in)) * Fraction(float(s_w[c])) +
                        Fraction(float(bias[c]))) / Fraction(float(s_out))
                frac = real - (real.numerator // real.denominator)
                if abs(frac - Fraction(1, 2)) < Fraction(1, 100):
                    continue                                 # fp32 evaluation may fall on the other side of a tie
                level = int(round(real))
                level = max(0 if relu else -128, min(127, level))
                assert q[r, c] == level, (r, c, float(real))
