"""Loader of tests/golden/spconv_cases.npz (written by tests/golden/make_golden.py)."""
import os

import numpy as np

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "spconv_cases.npz")


def load():
    z = np.load(PATH)   # plain arrays only; pickles stay disabled
    names = sorted({k.split(".")[0] for k in z.files})
    cases = []
    for name in names:
        m = z[name + ".meta"].tolist()
        c = dict(name=name, grid=tuple(m[0:3]), batch=m[3], ksize=tuple(m[4:7]), stride=tuple(m[7:10]),
                 padding=tuple(m[10:13]), dilation=tuple(m[13:16]), subm=bool(m[16]), transpose=bool(m[17]),
                 cin=m[18], cout=m[19])
        for f in ("coords", "feats", "weight", "bias", "out_coords", "triples", "out_feats"):
            c[f] = z[name + "." + f]
        cases.append(c)
    return cases


def canonical_features(out_coords, feats):
    """Rows reordered so that their coordinates ascend lexicographically (the fixtures' row order)."""
    order = np.lexsort(np.asarray(out_coords).T[::-1])
    return np.asarray(feats)[order]
