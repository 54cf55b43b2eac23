"""The HIP engine, through the C ABI, against the committed fixtures (expected values from a brute-force rulebook
and torch's dense convolutions).  Coordinates and pairs bit-exact after the canonical sort; fp16 features within
2e-2 of the output rms, fp32 within 1e-4 relative."""
import numpy as np
import pytest
import torch

import golden_cases
from helpers import gpu_rulebook
from oracle import oracle

pytestmark = pytest.mark.gpu
CASES = golden_cases.load()


@pytest.mark.parametrize("dtype", ["float16", "float32"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: c["name"])
def test_engine_matches_golden(engine, case, dtype):
    from deploy3d_amd import spconv_mm
    c = case
    n = len(c["coords"])
    kvol = int(np.prod(c["ksize"]))
    max_out = n if c["subm"] else n * kvol
    rb = gpu_rulebook(c["coords"], n, c["grid"], c["batch"], c["ksize"], c["stride"], c["padding"], c["dilation"],
                      max_out, c["subm"], c["transpose"])
    oc = c["coords"] if c["subm"] else rb["out_coors"]
    n_out = n if c["subm"] else rb["num_act_out"]
    got_c, got_t = oracle.canonical(rb["index"], rb["num_index"], oc, n_out)
    np.testing.assert_array_equal(got_c, c["out_coords"])
    np.testing.assert_array_equal(got_t, c["triples"])

    tdt = {"float16": torch.float16, "float32": torch.float32}[dtype]
    x = torch.from_numpy(c["feats"]).to(device="cuda", dtype=tdt)
    num_in = rb["num_act_in"]
    num_out = num_in if c["subm"] else rb["dev"][3]
    y = spconv_mm(x, num_in, num_out, rb["dev"][0], rb["dev"][1], c["ksize"], c["cin"], c["cout"], max_out,
                  c["subm"], False, c["weight"].astype(np.float32), c["bias"].astype(np.float32))
    torch.cuda.synchronize()
    got = golden_cases.canonical_features(oc[:n_out], y[:n_out].float().cpu().numpy())
    ref = c["out_feats"].astype(np.float64)
    rms = float(np.sqrt(np.mean(ref ** 2)))
    err = np.abs(got - ref)
    if dtype == "float32":
        assert (err <= 1e-4 * (np.abs(ref) + rms)).all(), err.max()
    else:
        assert err.max() <= 2e-2 * rms, (err.max(), rms)
