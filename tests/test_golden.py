"""The CPU oracle against the committed fixtures, whose expected values come from a brute-force rulebook and
torch's dense convolutions (tests/golden/make_golden.py), never from the oracle itself."""
import numpy as np
import pytest

import golden_cases
from oracle import oracle

CASES = golden_cases.load()


@pytest.mark.parametrize("case", CASES, ids=lambda c: c["name"])
def test_oracle_matches_golden(case):
    c = case
    n = len(c["coords"])
    kvol = int(np.prod(c["ksize"]))
    og = list(c["grid"]) if c["subm"] else oracle.out_shape(c["grid"], c["ksize"], c["stride"], c["padding"],
                                                           c["dilation"], None, c["transpose"])
    rb = oracle.rulebook(c["coords"], n, [c["batch"]] + og, c["ksize"], c["stride"], c["padding"], c["dilation"],
                         n * kvol, c["subm"], c["transpose"])
    oc = c["coords"] if c["subm"] else rb["out_coors"]
    n_out = n if c["subm"] else rb["num_act_out"]
    got_c, got_t = oracle.canonical(rb["index"], rb["num_index"], oc, n_out)
    np.testing.assert_array_equal(got_c, c["out_coords"])
    np.testing.assert_array_equal(got_t, c["triples"])
    y = oracle.conv(c["feats"].astype(np.float32), c["weight"].astype(np.float32), c["bias"].astype(np.float32),
                    rb["index"], rb["num_index"], n_out, acc="f64")
    np.testing.assert_allclose(golden_cases.canonical_features(oc[:n_out], y), c["out_feats"], rtol=2e-6, atol=2e-6)
