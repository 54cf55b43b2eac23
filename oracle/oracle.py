"""ctypes front end of the CPU oracle (TEST INFRASTRUCTURE, not product code).

Loads ``oracle/libd3d_oracle.so`` (built by ``make -C oracle`` or
``__graft_entry__.build()``) and wraps its entry points with numpy.  Only
tests, the smoke check and the benchmark's cpu_baseline leg import this.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libd3d_oracle.so")
_lib = None

_i32p = ctypes.POINTER(ctypes.c_int32)


def build():
    subprocess.check_call(["make", "-C", _HERE, "-B", "libd3d_oracle.so"], stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.d3d_oracle_fmix32.restype = ctypes.c_uint32
        _lib.d3d_oracle_fmix32.argtypes = [ctypes.c_uint32]
        _lib.d3d_oracle_rulebook.restype = ctypes.c_int
    return _lib


def _p(a, ty=None):
    return a.ctypes.data_as(ctypes.c_void_p)


def _i32(seq):
    return np.ascontiguousarray(np.asarray(seq, dtype=np.int32))


def fmix32(k):
    return int(lib().d3d_oracle_fmix32(ctypes.c_uint32(k & 0xFFFFFFFF)))


def out_shape(in_shape, ksize, stride, padding, dilation, out_padding=None, transpose=False):
    """Spatial output shape (reference: trt/spconv/geometry.h:118-169)."""
    nd = len(ksize)
    out_padding = [0] * nd if out_padding is None else out_padding
    out = np.zeros(nd, dtype=np.int32)
    lib().d3d_oracle_out_shape(ctypes.c_int(nd), _p(_i32(in_shape)), _p(_i32(ksize)), _p(_i32(stride)),
                               _p(_i32(padding)), _p(_i32(dilation)), _p(_i32(out_padding)),
                               ctypes.c_int(int(transpose)), _p(out))
    return [int(v) for v in out]


def rulebook(coors, num_act_in, out_grid, ksize, stride, padding, dilation, max_num_act_out, subm, transpose=False):
    """Rulebook of SPConvIdx{N}d (reference: trt/spconv/index.cu:253-476).

    coors: int32 [cap, nd+1]; out_grid: (B, spatial...) of the output grid (for
    SubM the input grid).  Returns dict(index [3, kVol*(cap+128)], num_index,
    out_coors [max_num_act_out, nd+1] | None, num_act_out | None).
    """
    coors = np.ascontiguousarray(coors, dtype=np.int32)
    cap, cw = coors.shape
    nd = cw - 1
    kvol = int(np.prod(ksize))
    row_len = kvol * (cap + 128)
    index = np.full((3, row_len), -1, dtype=np.int32)
    num_index = np.zeros(1, dtype=np.int32)
    out_coors = np.zeros((max_num_act_out, cw), dtype=np.int32)
    num_act_out = np.zeros(1, dtype=np.int32)
    rc = lib().d3d_oracle_rulebook(ctypes.c_int(nd), _p(coors), ctypes.c_int32(int(num_act_in)), ctypes.c_int32(cap),
                                   _p(_i32(out_grid)), _p(_i32(ksize)), _p(_i32(stride)), _p(_i32(padding)),
                                   _p(_i32(dilation)), ctypes.c_int32(int(max_num_act_out)), ctypes.c_int(int(subm)),
                                   ctypes.c_int(int(transpose)), _p(index), _p(num_index), _p(out_coors),
                                   _p(num_act_out))
    if rc != 0:
        raise RuntimeError("oracle rulebook: hash table full")
    if subm:
        return dict(index=index, num_index=int(num_index[0]), out_coors=None, num_act_out=None)
    return dict(index=index, num_index=int(num_index[0]), out_coors=out_coors, num_act_out=int(num_act_out[0]))


def conv(in_feats, weight, bias, index, num_index, max_num_act_out, inverse=False, acc="f64", threads=1):
    """out = bias; for tap: out[scatter] += in[gather] @ W[tap]
    (reference: tests/spconv/test_spconv.py:152-161, trt/spconv/mm.h:35-71).

    in_feats float32 [capIn, Cin]; weight float32 [kVol, Cin, Cout]; bias float32 [Cout] or None.
    acc: "f64" (parity target) or "f32" (the timed CPU baseline).
    """
    in_feats = np.ascontiguousarray(in_feats, dtype=np.float32)
    weight = np.ascontiguousarray(weight, dtype=np.float32)
    index = np.ascontiguousarray(index, dtype=np.int32)
    kvol, cin, cout = weight.shape
    assert in_feats.shape[1] == cin
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    out = np.empty((max_num_act_out, cout), dtype=np.float64 if acc == "f64" else np.float32)
    fn = lib().d3d_oracle_conv_f64 if acc == "f64" else lib().d3d_oracle_conv_f32
    fn(_p(in_feats), _p(weight), _p(b) if b is not None else None, _p(index), ctypes.c_int64(index.shape[1]),
       ctypes.c_int32(int(num_index)), ctypes.c_int(cin), ctypes.c_int(cout), ctypes.c_int32(int(max_num_act_out)),
       ctypes.c_int(int(inverse)), ctypes.c_int(int(threads)), _p(out))
    return out


def conv_i8(in_q, w_q, index, num_index, max_num_act_out, inverse=False, threads=1):
    """int8 x int8 -> int32 accumulators (this build's extension; no reference counterpart)."""
    in_q = np.ascontiguousarray(in_q, dtype=np.int8)
    w_q = np.ascontiguousarray(w_q, dtype=np.int8)
    index = np.ascontiguousarray(index, dtype=np.int32)
    kvol, cin, cout = w_q.shape
    out = np.empty((max_num_act_out, cout), dtype=np.int32)
    lib().d3d_oracle_conv_i8(_p(in_q), _p(w_q), _p(index), ctypes.c_int64(index.shape[1]),
                             ctypes.c_int32(int(num_index)), ctypes.c_int(cin), ctypes.c_int(cout),
                             ctypes.c_int32(int(max_num_act_out)), ctypes.c_int(int(inverse)),
                             ctypes.c_int(int(threads)), _p(out))
    return out


def requantize(acc, m, bq, relu):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    m = np.ascontiguousarray(m, dtype=np.float32)
    bq = np.ascontiguousarray(bq, dtype=np.float32)
    rows, cout = acc.shape
    out = np.empty((rows, cout), dtype=np.int8)
    lib().d3d_oracle_requantize(_p(acc), _p(m), _p(bq), ctypes.c_int64(rows), ctypes.c_int(cout),
                                ctypes.c_int(int(relu)), _p(out))
    return out


def quantize_weights(w):
    """Per-output-channel symmetric int8: s_w[c] = max|W[:,:,c]| / 127, q = clamp(rint(w / s_w))."""
    w = np.asarray(w, dtype=np.float32)
    s_w = (np.abs(w).max(axis=(0, 1)).astype(np.float64) / 127.0)
    s_w = np.where(s_w == 0.0, 1.0, s_w)
    q = np.clip(np.rint(w.astype(np.float64) / s_w[None, None, :]), -127, 127).astype(np.int8)
    return q, s_w


def requant_params(s_in, s_w, s_out, bias):
    m = (np.float64(s_in) * s_w.astype(np.float64) / np.float64(s_out)).astype(np.float32)
    b = np.zeros_like(s_w) if bias is None else np.asarray(bias, dtype=np.float64)
    bq = (b / np.float64(s_out)).astype(np.float32)
    return m, bq


def simple_mean(point_feats, batch_indices, voxel_config, spatial_shape, max_num_act_out):
    """Voxel means in the reference's (hash-slot) order; spatial_shape = (B, Z, Y, X).
    Returns (out_feats [max, C] float32, out_coors [max, 4] int32 (-1 past the live rows), num_act_out)."""
    point_feats = np.ascontiguousarray(point_feats, dtype=np.float32)
    batch_indices = np.ascontiguousarray(batch_indices, dtype=np.int32)
    voxel_config = np.ascontiguousarray(voxel_config, dtype=np.float32)
    n, c = point_feats.shape
    b, z, y, x = (int(v) for v in spatial_shape)
    out_feats = np.empty((max_num_act_out, c), dtype=np.float32)
    out_coors = np.empty((max_num_act_out, 4), dtype=np.int32)
    num = np.zeros(1, dtype=np.int32)
    lib().d3d_oracle_simple_mean.restype = ctypes.c_int
    rc = lib().d3d_oracle_simple_mean(_p(point_feats), _p(batch_indices), _p(voxel_config), ctypes.c_int64(n),
                                      ctypes.c_int(c), ctypes.c_int(b), ctypes.c_int(z), ctypes.c_int(y), ctypes.c_int(x),
                                      ctypes.c_int32(int(max_num_act_out)), _p(out_feats), _p(out_coors), _p(num))
    if rc != 0:
        raise RuntimeError("oracle simple_mean: hash table full")
    return out_feats, out_coors, int(num[0])


def bev_densify(in_feats, in_coors, num_act_in, spatial_shape):
    """Dense map [B, C*Z, Y, X] of the first num_act_in rows; spatial_shape = (B, Z, Y, X).
    in_feats may be any 1/2/4-byte numpy dtype (fp16 as np.float16, bf16 as its uint16 bits)."""
    in_feats = np.ascontiguousarray(in_feats)
    in_coors = np.ascontiguousarray(in_coors, dtype=np.int32)
    b, z, y, x = (int(v) for v in spatial_shape)
    c = in_feats.shape[1]
    out = np.empty((b, c * z, y, x), dtype=in_feats.dtype)
    lib().d3d_oracle_bev_densify(_p(in_feats), _p(in_coors), ctypes.c_int32(int(num_act_in)), ctypes.c_int(c),
                                 ctypes.c_int(in_feats.dtype.itemsize), ctypes.c_int(b), ctypes.c_int(z),
                                 ctypes.c_int(y), ctypes.c_int(x), _p(out))
    return out


def canonical(index, num_index, out_coors, num_act_out):
    """Canonical form of a rulebook: output coordinates sorted lexicographically,
    scatter ids relabelled by that rank, triples (tap, gather, scatter) sorted.
    out_coors are the live output coordinates (for SubM: the input coordinates).
    Returns (coords [n, nd+1], triples [P, 3]) as int64 arrays.
    """
    index = np.asarray(index)
    coords = np.asarray(out_coors)[:num_act_out].astype(np.int64)
    order = np.lexsort(coords.T[::-1])
    rank = np.empty(len(order), dtype=np.int64)
    rank[order] = np.arange(len(order))
    g, s, t = (index[r, :num_index].astype(np.int64) for r in range(3))
    live = t >= 0
    g, s, t = g[live], s[live], t[live]
    tri = np.stack([t, g, rank[s]], axis=1)
    tri = tri[np.lexsort((tri[:, 2], tri[:, 1], tri[:, 0]))]
    return coords[order], tri
