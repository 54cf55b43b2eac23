"""Seeded synthetic workloads: voxel clouds, features, weights and the layer
tables of the five benchmark configurations.

All random numbers come from ``libs/libd3d_synth.so`` (splitmix64; uniforms
from the top 53 bits; Box-Muller normals in fp64), so the GPU harness, the CPU
oracle and the committed fixtures see identical bits on every machine.  One
stream per tensor: seed = 0xD3D00000 + 16*config + tensor_id, with tensor ids
0 = coordinates, 1 = features and, for layer L (0-based), 256*(L+1) + j with
j = 0 weight, 1 BN gamma, 2 BN beta, 3 BN mean, 4 BN variance.
"""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SYNTH_LIB = os.path.join(HERE, "libs", "libd3d_synth.so")
SEED_BASE = 0xD3D00000
_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(SYNTH_LIB):
            raise ImportError("%s is missing: build it with deploy3d_amd/build.py" % SYNTH_LIB)
        _lib = ctypes.CDLL(SYNTH_LIB)
        for fn in ("d3d_synth_coords_uniform", "d3d_synth_coords_lidar", "d3d_synth_coords_cylinder"):
            getattr(_lib, fn).restype = ctypes.c_int64
        _lib.d3d_synth_splitmix64.restype = ctypes.c_uint64
    return _lib


def seed(config, tensor_id):
    return SEED_BASE + 16 * config + tensor_id


def layer_tensor_id(layer, j):
    return 256 * (layer + 1) + j


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def splitmix64(seed_value, nth=0):
    return int(_load().d3d_synth_splitmix64(ctypes.c_uint64(seed_value), ctypes.c_int64(nth)))


def normal(seed_value, shape, mean=0.0, std=1.0):
    out = np.empty(shape, dtype=np.float32)
    _load().d3d_synth_normal_f32(ctypes.c_uint64(seed_value), _ptr(out), ctypes.c_int64(out.size),
                                 ctypes.c_double(mean), ctypes.c_double(std))
    return out


def uniform(seed_value, shape, lo=0.0, hi=1.0):
    out = np.empty(shape, dtype=np.float32)
    _load().d3d_synth_uniform_f32(ctypes.c_uint64(seed_value), _ptr(out), ctypes.c_int64(out.size),
                                  ctypes.c_double(lo), ctypes.c_double(hi))
    return out


def _grid(grid):
    return np.ascontiguousarray(np.asarray(grid, dtype=np.int32))


def coords_uniform(seed_value, grid, n, batch=1):
    """n unique (b, z, y, x) rows, linear offset uniform over [batch, *grid]; draw order kept."""
    out = np.empty((n, 4), dtype=np.int32)
    got = _load().d3d_synth_coords_uniform(ctypes.c_uint64(seed_value), ctypes.c_int32(batch), _ptr(_grid(grid)),
                                           ctypes.c_int64(n), _ptr(out))
    return out[:got]


def coords_lidar(seed_value, grid, n):
    """70 % ground shell (z in 0..3) + 30 % in 200 Gaussian clusters (sigma 3 / 8 / 8); batch 1."""
    out = np.empty((n, 4), dtype=np.int32)
    _load().d3d_synth_coords_lidar(ctypes.c_uint64(seed_value), _ptr(_grid(grid)), ctypes.c_int64(n), _ptr(out))
    return out


def coords_cylinder(seed_value, grid, n):
    """(b, rho, phi, z): rho ~ floor(Exp(120)), phi uniform, z ~ round(N(8, 4)), clipped to the grid."""
    out = np.empty((n, 4), dtype=np.int32)
    got = _load().d3d_synth_coords_cylinder(ctypes.c_uint64(seed_value), _ptr(_grid(grid)), ctypes.c_int64(n),
                                            _ptr(out))
    return out[:got]


# ---------------------------------------------------------------------------
# layers
# ---------------------------------------------------------------------------
def conv_out_shape(in_shape, ksize, stride, padding, dilation=(1, 1, 1)):
    """Reference: outSize, trt/spconv/geometry.h:118-136."""
    return [(i + 2 * p - d * (k - 1) - 1) // s + 1 for i, k, s, p, d in zip(in_shape, ksize, stride, padding, dilation)]


def layer(name, key, subm, ksize, cin, cout, stride=(1, 1, 1), padding=(0, 0, 0), relu=True, src=None):
    return dict(name=name, key=key, subm=subm, ksize=tuple(ksize), stride=tuple(stride), padding=tuple(padding),
                dilation=(1, 1, 1), cin=cin, cout=cout, relu=relu, src=src)


def voxelnet_layers():
    """SECOND / CenterPoint-style sparse backbone: 13 convolutions over 8 rulebooks."""
    p1 = (1, 1, 1)
    L = []
    L.append(layer("conv_input", "subm1", True, (3, 3, 3), 5, 16, padding=p1))
    L.append(layer("conv1_0", "subm1", True, (3, 3, 3), 16, 16, padding=p1))
    L.append(layer("conv1_1", "subm1", True, (3, 3, 3), 16, 16, padding=p1))
    L.append(layer("down1", "down1", False, (3, 3, 3), 16, 32, stride=(2, 2, 2), padding=p1))
    L.append(layer("conv2_0", "subm2", True, (3, 3, 3), 32, 32, padding=p1))
    L.append(layer("conv2_1", "subm2", True, (3, 3, 3), 32, 32, padding=p1))
    L.append(layer("down2", "down2", False, (3, 3, 3), 32, 64, stride=(2, 2, 2), padding=p1))
    L.append(layer("conv3_0", "subm3", True, (3, 3, 3), 64, 64, padding=p1))
    L.append(layer("conv3_1", "subm3", True, (3, 3, 3), 64, 64, padding=p1))
    L.append(layer("down3", "down3", False, (3, 3, 3), 64, 128, stride=(2, 2, 2), padding=(0, 1, 1)))
    L.append(layer("conv4_0", "subm4", True, (3, 3, 3), 128, 128, padding=p1))
    L.append(layer("conv4_1", "subm4", True, (3, 3, 3), 128, 128, padding=p1))
    L.append(layer("conv_out", "down4", False, (3, 1, 1), 128, 128, stride=(2, 1, 1), padding=(0, 0, 0)))
    return L


def cylinder_block_layers():
    """Cylinder3D asymmetric residual block + downsample (wiring: tests/cylinder/test_cylinder3d.py:125-154).

    `src` names the layer whose output feeds this one ("input" = block input); the
    outputs of a2 and b2 are added before c.  Two (3,1,3) convs share key k313, two (1,3,3) share k133.
    """
    L = []
    L.append(layer("a1", "k313", True, (3, 1, 3), 32, 64, padding=(1, 0, 1), src="input"))
    L.append(layer("a2", "k133", True, (1, 3, 3), 64, 64, padding=(0, 1, 1), src="a1"))
    L.append(layer("b1", "k133", True, (1, 3, 3), 32, 64, padding=(0, 1, 1), src="input"))
    L.append(layer("b2", "k313", True, (3, 1, 3), 64, 64, padding=(1, 0, 1), src="b1"))
    L.append(layer("c", "k333", True, (3, 3, 3), 64, 64, padding=(1, 1, 1), src="a2+b2"))
    L.append(layer("down", "down", False, (3, 3, 3), 64, 128, stride=(2, 2, 2), padding=(1, 1, 1), relu=False,
                   src="c"))
    return L


def layer_weights(config, layer_index, spec, with_bn=True):
    """W ~ N(0, 1/(kVol*Cin)) [kVol, Cin, Cout]; synthetic BN folded with the reference's formula
    (tests/cylinder/test_middle_encoder.py:22-34: w / sqrt(var) * gamma, beta - mean / sqrt(var) * gamma, no eps).
    Returns fp32 (weight, bias)."""
    kvol = int(np.prod(spec["ksize"]))
    cin, cout = spec["cin"], spec["cout"]
    w = normal(seed(config, layer_tensor_id(layer_index, 0)), (kvol, cin, cout), 0.0, (1.0 / (kvol * cin)) ** 0.5)
    if not with_bn:
        return w, np.zeros(cout, dtype=np.float32)
    gamma = uniform(seed(config, layer_tensor_id(layer_index, 1)), (cout,), 0.5, 1.5)
    beta = normal(seed(config, layer_tensor_id(layer_index, 2)), (cout,), 0.0, 0.1)
    mean = normal(seed(config, layer_tensor_id(layer_index, 3)), (cout,), 0.0, 0.1)
    var = uniform(seed(config, layer_tensor_id(layer_index, 4)), (cout,), 0.5, 1.5)
    std = np.sqrt(var)
    w = (w / std[None, None, :] * gamma[None, None, :]).astype(np.float32)
    b = (beta - mean / std * gamma).astype(np.float32)
    return w, b


# ---------------------------------------------------------------------------
# configurations
# ---------------------------------------------------------------------------
def config1(n=20000):
    """Single SubM 3x3x3, 16 -> 16, fp32."""
    grid = (41, 1600, 1408)
    coords = coords_uniform(seed(1, 0), grid, n)
    feats = normal(seed(1, 1), (n, 16))
    spec = layer("subm", "subm", True, (3, 3, 3), 16, 16, padding=(1, 1, 1), relu=False)
    w, b = layer_weights(1, 0, spec, with_bn=False)
    return dict(config=1, grid=grid, coords=coords, feats=feats, dtype="float32", layers=[spec], weights=[(w, b)])


def config2(n=60000):
    """Single strided SpConv 3x3x3 s2 p1, 32 -> 64, fp16."""
    grid = (41, 1440, 1440)
    coords = coords_lidar(seed(2, 0), grid, n)
    feats = normal(seed(2, 1), (n, 32))
    spec = layer("down", "down", False, (3, 3, 3), 32, 64, stride=(2, 2, 2), padding=(1, 1, 1), relu=False)
    w, b = layer_weights(2, 0, spec, with_bn=False)
    return dict(config=2, grid=grid, coords=coords, feats=feats, dtype="float16", layers=[spec], weights=[(w, b)])


def config3(n=120000):
    """VoxelNet sparse backbone, fp16, 5 input channels."""
    grid = (41, 1440, 1440)
    coords = coords_lidar(seed(3, 0), grid, n)
    feats = normal(seed(3, 1), (n, 5))
    layers = voxelnet_layers()
    weights = [layer_weights(3, i, s) for i, s in enumerate(layers)]
    return dict(config=3, grid=grid, coords=coords, feats=feats, dtype="float16", layers=layers, weights=weights)


def activation_scale(a):
    """Per-tensor symmetric int8 scale: the 99.99th percentile of |a| over 127, as float32."""
    a = np.abs(np.asarray(a, dtype=np.float64)).reshape(-1)
    s = np.percentile(a, 99.99) / 127.0 if a.size else 1.0
    return np.float32(s if s > 0 else 1.0)


def quantize_activations(a, scale):
    return np.clip(np.rint(np.asarray(a, dtype=np.float64) / np.float64(scale)), -128, 127).astype(np.int8)


def config4(n=120000, activations=None):
    """Config 3 quantized to int8.  ``activations`` maps "input" and every layer name to that tensor's values
    from a floating-point pass of config 3 at the same size (the calibration data); each layer gets the scales of
    its input and output tensors as ``s_in`` / ``s_out``.  Weights stay fp32 in the blob: the engine derives the
    per-output-channel weight scales itself."""
    cfg = config3(n)
    if activations is None:
        raise ValueError("config4 needs the activations of a floating-point pass for calibration")
    scales = {name: activation_scale(a) for name, a in activations.items()}
    layers = []
    prev = "input"
    for spec in cfg["layers"]:
        spec = dict(spec, s_in=scales[prev], s_out=scales[spec["name"]])
        layers.append(spec)
        prev = spec["name"]
    cfg.update(config=4, dtype="int8", layers=layers, scales=scales,
               feats_q=quantize_activations(cfg["feats"], scales["input"]))
    return cfg


def config5(n=250000):
    """Cylinder3D-style block on a cylindrical grid [rho, phi, z], fp16."""
    grid = (480, 360, 32)
    coords = coords_cylinder(seed(5, 0), grid, n)
    feats = normal(seed(5, 1), (len(coords), 32))
    layers = cylinder_block_layers()
    weights = [layer_weights(5, i, s) for i, s in enumerate(layers)]
    return dict(config=5, grid=grid, coords=coords, feats=feats, dtype="float16", layers=layers, weights=weights)
