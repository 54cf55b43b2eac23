"""Runs a layer table (deploy3d_amd.synth) through the CPU oracle, mirroring the
wiring of deploy3d_amd.layers.SparseBackbone: one rulebook per indice key, bias
and weights rounded to the storage type, fp64 accumulation, one rounding of the
output to the storage type, ReLU where the layer fuses it.
"""
import numpy as np
import torch

from oracle import oracle

TORCH_DTYPE = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}


def round_to(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(TORCH_DTYPE[dtype]).float().numpy()


def oracle_chain(cfg, threads=1, acc="f64"):
    """Returns dict name -> dict(feats [n, C] float32 (storage-rounded), coords [n, 4], grid, pairs P)."""
    dtype = cfg["dtype"]
    coords = cfg["coords"]
    outs = {"input": dict(feats=round_to(cfg["feats"], dtype), coords=coords, grid=list(cfg["grid"]))}
    rulebooks = {}
    cur = outs["input"]
    for spec, (w, b) in zip(cfg["layers"], cfg["weights"]):
        src = spec.get("src")
        if src is None:
            x = cur
        elif "+" in src:
            a, c = (outs[s] for s in src.split("+"))
            x = dict(feats=round_to(a["feats"] + c["feats"], dtype), coords=a["coords"], grid=a["grid"])
        else:
            x = outs[src]
        n = len(x["coords"])
        rb = rulebooks.get(spec["key"])
        if rb is None:
            if spec["subm"]:
                rb = oracle.rulebook(x["coords"], n, [1] + x["grid"], spec["ksize"], spec["stride"], spec["padding"],
                                     spec["dilation"], n, True)
                rb.update(out_coors=x["coords"], num_act_out=n, out_grid=x["grid"])
            else:
                og = oracle.out_shape(x["grid"], spec["ksize"], spec["stride"], spec["padding"], spec["dilation"])
                rb = oracle.rulebook(x["coords"], n, [1] + og, spec["ksize"], spec["stride"], spec["padding"],
                                     spec["dilation"], 8 * n, False)
                rb["out_coors"] = rb["out_coors"][:rb["num_act_out"]].copy()
                rb["out_grid"] = og
            rb["pairs"] = int((rb["index"][2, :rb["num_index"]] >= 0).sum())
            rb["in_coors"] = x["coords"]
            rb["in_grid"] = x["grid"]
            rulebooks[spec["key"]] = rb
        # an inverse layer runs its key's rulebook backwards: outputs on the sites the rulebook was built from
        inverse = bool(spec.get("inverse", False))
        n_out = len(rb["in_coors"]) if inverse else rb["num_act_out"]
        y = oracle.conv(x["feats"], round_to(w, dtype), round_to(b, dtype), rb["index"], rb["num_index"], n_out,
                        inverse=inverse, acc=acc, threads=threads)
        if spec.get("relu"):
            y = np.maximum(y, 0)
        cur = dict(feats=round_to(y, dtype), exact=y, coords=rb["in_coors"] if inverse else rb["out_coors"],
                   grid=rb["in_grid"] if inverse else rb["out_grid"], pairs=rb["pairs"], key=spec["key"])
        outs[spec["name"]] = cur
    outs["_rulebooks"] = rulebooks
    return outs


def oracle_chain_int8(cfg, rulebook_chain):
    """Config-4 style chain in int8: ``cfg`` from synth.config4, ``rulebook_chain`` the result of oracle_chain on the
    floating-point configuration (its rulebooks are reused: coordinates do not depend on the values).
    Returns name -> int8 features [n, C] in the row order of rulebook_chain[name]["coords"]."""
    outs = {"input": cfg["feats_q"]}
    cur = outs["input"]
    for spec, (w, b) in zip(cfg["layers"], cfg["weights"]):
        rb = rulebook_chain["_rulebooks"][spec["key"]]
        w_q, s_w = oracle.quantize_weights(w)
        m, bq = oracle.requant_params(spec["s_in"], s_w, spec["s_out"], b)
        acc = oracle.conv_i8(cur, w_q, rb["index"], rb["num_index"], rb["num_act_out"])
        cur = oracle.requantize(acc, m, bq, bool(spec.get("relu")))
        outs[spec["name"]] = cur
    return outs


def canonical_pairs(index, num_index, in_coors, num_act_in, out_coors, num_act_out):
    """Canonical form of a rulebook inside a chain, where the row numbering of the INPUT voxels is as arbitrary as
    that of the outputs (they are the outputs of an earlier strided layer): both sides are relabelled by the rank
    of their coordinate, then the triples (tap, gather, scatter) are sorted.  Returns (sorted output coordinates,
    triples) as int64 arrays."""
    def ranks(coords, n):
        c = np.asarray(coords)[:n].astype(np.int64)
        order = np.lexsort(c.T[::-1])
        r = np.empty(n, dtype=np.int64)
        r[order] = np.arange(n)
        return c[order], r
    _, rin = ranks(in_coors, num_act_in)
    cout, rout = ranks(out_coors, num_act_out)
    g, s, t = (np.asarray(index)[r, :num_index].astype(np.int64) for r in range(3))
    live = t >= 0
    tri = np.stack([t[live], rin[g[live]], rout[s[live]]], axis=1)
    return cout, tri[np.lexsort((tri[:, 2], tri[:, 1], tri[:, 0]))]


def sort_rows(coords, feats):
    order = np.lexsort(np.asarray(coords).T[::-1])
    return np.asarray(coords)[order], np.asarray(feats)[order]
