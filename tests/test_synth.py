"""The seeded synthetic-data generator: published splitmix64 answers, determinism, and the shape of the clouds."""
import numpy as np

from deploy3d_amd import synth


def test_splitmix64_published_vectors():
    """First outputs of splitmix64 seeded with 1234567 (Vigna's reference implementation)."""
    want = [6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431,
            16408922859458223821]
    assert [synth.splitmix64(1234567, i) for i in range(5)] == want


def test_streams_are_deterministic_and_distinct():
    a = synth.normal(synth.seed(3, 1), (1000, 5))
    b = synth.normal(synth.seed(3, 1), (1000, 5))
    c = synth.normal(synth.seed(3, 2), (1000, 5))
    np.testing.assert_array_equal(a, b)
    assert not np.array_equal(a, c)
    assert abs(float(a.mean())) < 0.06 and abs(float(a.std()) - 1.0) < 0.05
    u = synth.uniform(7, (4000,), 0.5, 1.5)
    assert 0.5 <= u.min() and u.max() < 1.5 and abs(float(u.mean()) - 1.0) < 0.03


def test_clouds_are_unique_and_in_grid():
    for coords, grid in ((synth.coords_uniform(synth.seed(1, 0), (41, 1600, 1408), 20000), (41, 1600, 1408)),
                         (synth.coords_lidar(synth.seed(2, 0), (41, 1440, 1440), 60000), (41, 1440, 1440)),
                         (synth.coords_cylinder(synth.seed(5, 0), (480, 360, 32), 50000), (480, 360, 32))):
        assert coords.dtype == np.int32 and coords.shape[1] == 4
        assert (coords[:, 0] == 0).all()
        assert (coords[:, 1:] >= 0).all() and (coords[:, 1:] < np.array(grid)).all()
        assert len(np.unique(coords, axis=0)) == len(coords)
    lidar = synth.coords_lidar(synth.seed(2, 0), (41, 1440, 1440), 60000)
    assert (lidar[:42000, 1] < 4).all()            # the first 70 % sit on the ground shell
    assert (lidar[42000:, 1] >= 4).any()


def test_layer_tables():
    layers = synth.voxelnet_layers()
    assert len(layers) == 13 and len({l["key"] for l in layers}) == 8
    assert [l["cout"] for l in layers] == [16, 16, 16, 32, 32, 32, 64, 64, 64, 128, 128, 128, 128]
    w, b = synth.layer_weights(3, 0, layers[0])
    assert w.shape == (27, 5, 16) and b.shape == (16,) and w.dtype == np.float32
    cyl = synth.cylinder_block_layers()
    assert [l["key"] for l in cyl] == ["k313", "k133", "k133", "k313", "k333", "down"]


def test_bn_fold_matches_batchnorm_eval():
    """The fold w/sqrt(var)*gamma, beta - mean/sqrt(var)*gamma (tests/cylinder/test_middle_encoder.py:22-34, no eps)
    equals conv followed by an eval-mode BatchNorm whose eps is negligible."""
    import torch
    spec = synth.layer("x", "x", True, (1, 1, 1), 6, 4)
    w_raw = synth.normal(synth.seed(9, synth.layer_tensor_id(0, 0)), (1, 6, 4), 0.0, (1.0 / 6) ** 0.5)
    w, b = synth.layer_weights(9, 0, spec)
    bn = torch.nn.BatchNorm1d(4, eps=1e-12).eval()  # torch refuses 0; 1e-12 vanishes beside var >= 0.5 in fp32
    with torch.no_grad():
        bn.weight.copy_(torch.from_numpy(synth.uniform(synth.seed(9, synth.layer_tensor_id(0, 1)), (4,), 0.5, 1.5)))
        bn.bias.copy_(torch.from_numpy(synth.normal(synth.seed(9, synth.layer_tensor_id(0, 2)), (4,), 0.0, 0.1)))
        bn.running_mean.copy_(torch.from_numpy(synth.normal(synth.seed(9, synth.layer_tensor_id(0, 3)), (4,), 0.0, 0.1)))
        bn.running_var.copy_(torch.from_numpy(synth.uniform(synth.seed(9, synth.layer_tensor_id(0, 4)), (4,), 0.5, 1.5)))
    x = torch.randn(50, 6)
    want = bn(x @ torch.from_numpy(w_raw[0]))
    got = x @ torch.from_numpy(w[0]) + torch.from_numpy(b)
    assert torch.allclose(got, want, atol=1e-5)


def test_int8_calibration_helpers():
    a = np.linspace(-2.0, 2.0, 100001)
    s = synth.activation_scale(a)
    assert s.dtype == np.float32 and abs(float(s) - np.percentile(np.abs(a), 99.99) / 127) < 1e-7
    s = np.float32(0.25)                                # exact in binary, so the ties below are exact ties
    q = synth.quantize_activations(np.array([0.0, 0.125, 0.375, 0.625, -75.0, 75.0]), s)
    assert q.tolist() == [0, 0, 2, 2, -128, 127]        # ties to even, clamp to the int8 range
    assert synth.activation_scale(np.zeros(5)) == np.float32(1.0)
