"""Shared test helpers: an independent brute-force rulebook (the check that pins
the oracle), dense-convolution equivalents, and GPU run wrappers."""
import itertools

import numpy as np


# ---------------------------------------------------------------------------
# brute force: dict of coordinates, plain Python loops.  Written from the
# definition of a sparse convolution (output o reads input o*s - p + tap*d),
# not from the oracle's code: it walks OUTPUT sites and looks inputs up, the
# opposite direction to the reference's input-side tap walk.
# ---------------------------------------------------------------------------
def bruteforce_rulebook(coords, out_grid, ksize, stride, padding, dilation, subm=False, transpose=False):
    """coords [n, nd+1]; out_grid (B, spatial...).  Returns (sorted out coords [m, nd+1],
    sorted triples [P, 3] = (tap, input row, rank of output coordinate))."""
    coords = np.asarray(coords)
    nd = coords.shape[1] - 1
    rows = {tuple(int(v) for v in c): i for i, c in enumerate(coords)}
    taps = list(itertools.product(*[range(k) for k in ksize]))  # row-major tap order
    pairs = []  # (tap, in_row, out_coord)
    if subm:
        cand = list(rows.keys())
    else:
        # every output site that any input can reach
        cand = set()
        for c in rows:
            for t in taps:
                o = []
                ok = True
                for dim in range(nd):
                    if transpose:
                        v = c[1 + dim] * stride[dim] - padding[dim] + t[dim] * dilation[dim]
                    else:
                        num = c[1 + dim] + padding[dim] - t[dim] * dilation[dim]
                        if num % stride[dim] != 0:  # Python floor-mod: exact-division test, sign-safe
                            ok = False
                            break
                        v = num // stride[dim]
                    if v < 0 or v >= out_grid[1 + dim]:
                        ok = False
                        break
                    o.append(v)
                if ok and 0 <= c[0] < out_grid[0]:
                    cand.add((c[0],) + tuple(o))
        cand = list(cand)
    for o in cand:
        for ti, t in enumerate(taps):
            if transpose:
                # input i with i*s - p + t*d == o
                src = []
                ok = True
                for dim in range(nd):
                    num = o[1 + dim] + padding[dim] - t[dim] * dilation[dim]
                    if num % stride[dim] != 0:
                        ok = False
                        break
                    src.append(num // stride[dim])
                if not ok:
                    continue
                src = (o[0],) + tuple(src)
            else:
                src = (o[0],) + tuple(o[1 + dim] * stride[dim] - padding[dim] + t[dim] * dilation[dim]
                                      for dim in range(nd))
            if any(o[1 + dim] < 0 or o[1 + dim] >= out_grid[1 + dim] for dim in range(nd)):
                continue
            i = rows.get(src)
            if i is not None:
                pairs.append((ti, i, o))
    outs = sorted(set(p[2] for p in pairs)) if not subm else sorted(rows.keys())
    if subm:
        # SubM output ids are input rows; canonical rank = rank of the coordinate
        pass
    rank = {o: r for r, o in enumerate(outs)}
    tri = sorted((t, i, rank[o]) for t, i, o in pairs)
    return (np.array(outs, dtype=np.int64).reshape(-1, nd + 1),
            np.array(tri, dtype=np.int64).reshape(-1, 3))


def random_cloud(rng, n, grid, batch=1):
    """n unique rows (b, spatial...) uniform over [batch, *grid], numpy Generator."""
    cells = batch * int(np.prod(grid))
    n = min(n, cells)
    offs = rng.choice(cells, size=n, replace=False)
    cols = []
    for extent in reversed(grid):
        cols.append(offs % extent)
        offs = offs // extent
    cols.append(offs)
    return np.stack(cols[::-1], axis=1).astype(np.int32)


def check_index_structure(index, num_index, kvol, cap):
    """Structural invariants the reference's own test asserts (tests/spconv/test_spconv.py:82-91)."""
    gather, scatter, tap = index
    assert index.shape == (3, kvol * (cap + 128))
    assert num_index % 128 == 0
    live = tap >= 0
    assert not live[num_index:].any()
    assert (tap[live] < kvol).all()
    assert (gather[~live] == -1).all() and (scatter[~live] == -1).all() and (tap[~live] == -1).all()
    pos = 0
    for k in range(kvol):
        where = np.nonzero(tap == k)[0]
        if len(where) == 0:
            continue
        assert where[0] % 128 == 0, "tap segment must start on a multiple of 128"
        assert where[0] == pos and where[-1] - where[0] + 1 == len(where), "segments are contiguous and tap-major"
        assert (np.diff(gather[where]) > 0).all(), "input rows ascend inside a tap"
        pos = (where[-1] + 1 + 127) // 128 * 128
    assert num_index == pos


def dense_from_sparse(coords, feats, grid, batch):
    """[B, C, *grid] dense tensor (torch, float64) from sparse rows."""
    import torch
    c = feats.shape[1]
    dense = torch.zeros((batch, c) + tuple(grid), dtype=torch.float64)
    idx = (torch.as_tensor(coords[:, 0]).long(),) + tuple(torch.as_tensor(coords[:, 1 + d]).long()
                                                           for d in range(len(grid)))
    dense[(idx[0], slice(None)) + idx[1:]] = torch.as_tensor(feats, dtype=torch.float64)
    return dense


def dense_weight(weight, ksize):
    """W[tap, I, O] -> torch conv weight [O, I, *ksize] (tap row-major over the kernel dims)."""
    import torch
    kvol, cin, cout = weight.shape
    w = torch.as_tensor(weight, dtype=torch.float64).reshape(tuple(ksize) + (cin, cout))
    nd = len(ksize)
    return w.permute(nd + 1, nd, *range(nd)).contiguous()


# ---------------------------------------------------------------------------
# GPU wrappers (through the C ABI via deploy3d_amd)
# ---------------------------------------------------------------------------
def gpu_rulebook(coords, num_act_in, grid, batch, ksize, stride, padding, dilation, max_num_act_out, subm,
                 transpose=False, out_padding=None, cap=None, link=False):
    """link=True: a placeholder convolution is linked to the operator first, so that this enqueue also writes the
    neighbour table and tile masks (res["plugin"] is what spconv_mm(..., rulebook=) takes)."""
    import torch
    from deploy3d_amd import spconv_index_nd
    from deploy3d_amd.spconv_index import index_plugin
    from deploy3d_amd.spconv_mm import get_plugin, mm_blob
    nd = len(ksize)
    plugin = index_plugin(ksize, stride, padding, dilation, out_padding or (0,) * nd, max_num_act_out, subm, transpose)
    if link:
        get_plugin(mm_blob(ksize, 1, 1, max_num_act_out, subm, False,
                           np.zeros(int(np.prod(ksize)), np.float32))).link_rulebook(plugin)
    cap = cap or len(coords)
    c = torch.zeros((cap, nd + 1), dtype=torch.int32, device="cuda")
    c[:len(coords)] = torch.from_numpy(np.ascontiguousarray(coords)).cuda()
    num = torch.tensor([num_act_in], dtype=torch.int32, device="cuda")
    shape = torch.empty((batch, 0) + tuple(grid), dtype=torch.int32, device="cuda")
    out = spconv_index_nd(c, num, shape, ksize, stride, padding, dilation, out_padding or (0,) * nd, max_num_act_out,
                          subm, transpose)
    torch.cuda.synchronize()
    res = dict(index=out[0].cpu().numpy(), num_index=int(out[1].item()), dev=out, in_coors=c, num_act_in=num,
               plugin=plugin)
    if not subm:
        res.update(out_coors=out[2].cpu().numpy(), num_act_out=int(out[3].item()),
                   out_grid=list(out[4].shape[2:]))
    return res
