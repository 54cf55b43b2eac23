#!/usr/bin/env python3
"""Writes tests/golden/spconv_cases.npz: small fixed cases with expected results that come from neither the
oracle nor the GPU engine.

The reference holds no vectors for this path (its test draws unseeded inputs and compares with the spconv package
at run time, tests/spconv/test_spconv.py:37-48,165-197), so each expected value here is computed by a route that
shares no code with either implementation under test:
  * rulebooks  - the brute force of tests/helpers.py (walks OUTPUT sites, dictionary look-ups);
  * features   - torch's dense conv3d / conv_transpose3d in float64 on the densified cloud, sampled at the
                 brute-force output sites (fp16-rounded operands, so fp16 engines see exact inputs).
Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from helpers import bruteforce_rulebook, dense_from_sparse, dense_weight  # noqa: E402
from deploy3d_amd import synth  # noqa: E402

# name, grid, batch, n, ksize, stride, padding, dilation, subm, transpose, cin, cout
CASES = [
    ("subm333", (8, 24, 20), 2, 900, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), True, False, 16, 32),
    ("subm313", (8, 24, 20), 1, 600, (3, 1, 3), (1, 1, 1), (1, 0, 1), (1, 1, 1), True, False, 32, 32),
    ("down333", (8, 24, 20), 2, 900, (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), False, False, 16, 32),
    ("down221", (9, 24, 8), 2, 900, (3, 3, 3), (2, 2, 1), (1, 1, 1), (1, 1, 1), False, False, 16, 32),
    ("down311", (9, 12, 12), 1, 500, (3, 1, 1), (2, 1, 1), (0, 0, 0), (1, 1, 1), False, False, 64, 64),
    ("dil2", (10, 12, 12), 1, 400, (3, 3, 3), (1, 1, 1), (2, 2, 2), (2, 2, 2), True, False, 5, 16),
    ("up333", (4, 10, 9), 1, 200, (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), False, True, 16, 16),
]


def out_extent(i, k, s, p, d, transpose):
    return (i - 1) * s - 2 * p + d * (k - 1) + 1 if transpose else (i + 2 * p - d * (k - 1) - 1) // s + 1


def r16(a):
    return np.asarray(a, dtype=np.float32).astype(np.float16).astype(np.float32)


def main():
    blob = {}
    for ci, (name, grid, batch, n, k, s, p, d, subm, transpose, cin, cout) in enumerate(CASES):
        sd = synth.seed(15, 1000 + 16 * ci)
        coords = synth.coords_uniform(sd, grid, n, batch)
        feats = r16(synth.normal(sd + 1, (n, cin)))
        kvol = int(np.prod(k))
        w = r16(synth.normal(sd + 2, (kvol, cin, cout), 0.0, (1.0 / (kvol * cin)) ** 0.5))
        b = r16(synth.normal(sd + 3, (cout,)))
        og = list(grid) if subm else [out_extent(i, kk, ss, pp, dd, transpose) for i, kk, ss, pp, dd in
                                      zip(grid, k, s, p, d)]
        out_coords, triples = bruteforce_rulebook(coords, [batch] + og, k, s, p, d, subm, transpose)
        x = dense_from_sparse(coords, feats, grid, batch)
        if transpose:
            wt = torch.as_tensor(w, dtype=torch.float64).reshape(tuple(k) + (cin, cout)).permute(3, 4, 0, 1, 2)
            dense = F.conv_transpose3d(x, wt.contiguous(), torch.as_tensor(b).double(), stride=s, padding=p,
                                       dilation=d)
        else:
            dense = F.conv3d(x, dense_weight(w, k), torch.as_tensor(b).double(), stride=s, padding=p, dilation=d)
        assert list(dense.shape[2:]) == og, (name, dense.shape, og)
        oc = torch.as_tensor(out_coords)
        y = dense[oc[:, 0], :, oc[:, 1], oc[:, 2], oc[:, 3]].numpy()
        meta = np.array(list(grid) + [batch] + list(k) + list(s) + list(p) + list(d) + [subm, transpose, cin, cout],
                        dtype=np.int32)
        blob[name + ".meta"] = meta
        blob[name + ".coords"] = coords.astype(np.int32)
        blob[name + ".feats"] = feats.astype(np.float16)
        blob[name + ".weight"] = w.astype(np.float16)
        blob[name + ".bias"] = b.astype(np.float16)
        blob[name + ".out_coords"] = out_coords.astype(np.int32)      # sorted lexicographically
        blob[name + ".triples"] = triples.astype(np.int32)            # sorted (tap, input row, output rank)
        blob[name + ".out_feats"] = y.astype(np.float32)              # rows follow out_coords
        print("%-8s n=%d outputs=%d pairs=%d" % (name, len(coords), len(out_coords), len(triples)))
    path = os.path.join(HERE, "spconv_cases.npz")
    np.savez_compressed(path, **blob)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
