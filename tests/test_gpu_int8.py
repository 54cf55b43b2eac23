"""int8 convolution (this build's extension: the reference accepts fp16 only, trt/spconv/mm_trt.cu:184) through the
C ABI against the CPU oracle: int32 accumulation of int8 products and the requantize rule
q = clamp(rint(float(acc) * m[c] + bq[c])), bit-exact.  Parity is pinned by that written rule, not by the reference."""
import numpy as np
import pytest
import torch

from chain import oracle_chain
from helpers import gpu_rulebook, random_cloud
from oracle import oracle

pytestmark = pytest.mark.gpu


def run_int8(n, grid, ksize, stride, padding, cin, cout, subm, relu, with_bias=True, seed=0):
    from deploy3d_amd import spconv_mm
    rng = np.random.default_rng(seed + 31 * cin + cout + n)
    coords = random_cloud(rng, n, grid, 1)
    n = len(coords)
    kvol = int(np.prod(ksize))
    max_out = n if subm else 8 * n
    rb = gpu_rulebook(coords, n, grid, 1, ksize, stride, padding, (1,) * len(ksize), max_out, subm)
    n_out = n if subm else rb["num_act_out"]
    x_q = rng.integers(-128, 128, (n, cin)).astype(np.int8)
    w = (rng.standard_normal((kvol, cin, cout)) / np.sqrt(kvol * cin)).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32) if with_bias else None
    s_in, s_out = np.float32(0.043), np.float32(0.057)
    w_q, s_w = oracle.quantize_weights(w)
    m, bq = oracle.requant_params(s_in, s_w, s_out, b)
    acc = oracle.conv_i8(x_q, w_q, rb["index"], rb["num_index"], max_out)
    want = oracle.requantize(acc, m, bq, relu)
    num_in = rb["num_act_in"]
    num_out = num_in if subm else rb["dev"][3]
    y = spconv_mm(torch.from_numpy(x_q).cuda(), num_in, num_out, rb["dev"][0], rb["dev"][1], ksize, cin, cout, max_out,
                  subm, False, w, b, relu=relu, act_scale_in=float(s_in), act_scale_out=float(s_out))
    torch.cuda.synchronize()
    assert y.dtype == torch.int8
    got = y.cpu().numpy()
    np.testing.assert_array_equal(got[:n_out], want[:n_out])
    # rows past the live outputs hold the requantized bias alone
    if max_out > n_out:
        tail = oracle.requantize(np.zeros((1, cout), np.int32), m, bq, relu)
        np.testing.assert_array_equal(got[n_out:], np.broadcast_to(tail, got[n_out:].shape))
    assert np.abs(got[:n_out].astype(np.int32)).max() > 30      # the case exercises the value range


@pytest.mark.parametrize("cin,cout", [(5, 16), (16, 16), (16, 32), (32, 32), (32, 64), (64, 64), (64, 128), (128, 128),
                                      (128, 16), (20, 64), (100, 32)])
@pytest.mark.parametrize("relu", [False, True])
def test_int8_subm_bit_exact(engine, cin, cout, relu):
    run_int8(3000, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), cin, cout, True, relu)


@pytest.mark.parametrize("cin,cout", [(16, 32), (32, 64), (64, 128), (128, 128)])
def test_int8_strided_bit_exact(engine, cin, cout):
    run_int8(3000, (10, 36, 30), (3, 3, 3), (2, 2, 2), (1, 1, 1), cin, cout, False, True)
    run_int8(2000, (10, 36, 30), (3, 1, 1), (2, 1, 1), (0, 0, 0), cin, cout, False, False, with_bias=False)


@pytest.mark.parametrize("cfg", ["4,8,2", "2,8,3", "2,8,2", "4,4,2", "4,4,3"])
def test_int8_staged_configurations(engine, monkeypatch, cfg):
    monkeypatch.setenv("D3D_CONV_STAGED", cfg)
    run_int8(3001, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), 64, 64, True, True)
    run_int8(3001, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), 128, 32, True, False)


@pytest.mark.parametrize("shape", ["32,8", "32,6", "32,4", "48,4"])
@pytest.mark.parametrize("cin,cout", [(64, 128), (128, 128)])
def test_int8_pipelined_tile_shapes(engine, monkeypatch, shape, cin, cout):
    """Layers with rows of 64 bytes and more run the software-pipelined kernel; for 128 output channels it chooses
    among four workgroup shapes by row count.  Each forced on a SubM layer with spare capacity and a strided one, and
    once on a layer with more tiles than workgroups, where the pipeline runs across tiles."""
    monkeypatch.setenv("D3D_CONV_PIPE_SHAPE", shape)
    run_int8(9001, (12, 48, 40), (3, 3, 3), (1, 1, 1), (1, 1, 1), cin, cout, True, True)
    if cin == 64:
        run_int8(5000, (12, 48, 40), (3, 3, 3), (2, 2, 2), (1, 1, 1), cin, cout, False, False)
        run_int8(70000, (16, 200, 200), (3, 3, 3), (1, 1, 1), (1, 1, 1), cin, cout, True, True)


@pytest.mark.parametrize("cin,cout", [(64, 32), (64, 64), (128, 64), (128, 128)])
def test_int8_pipelined_and_barrier_per_tap_kernels_agree_with_the_oracle(engine, monkeypatch, cin, cout):
    """The same layer on the pipelined kernel (the default from 64 input channels up), across several tiles per
    workgroup, and with the pipelined kernel switched off, which leaves the barrier-per-tap kernel."""
    run_int8(40000, (16, 120, 120), (3, 3, 3), (1, 1, 1), (1, 1, 1), cin, cout, True, True)
    monkeypatch.setenv("D3D_CONV_PIPE", "0")
    run_int8(3001, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), cin, cout, True, False)


def test_int8_unsupported_channels_report_status(engine):
    from deploy3d_amd import EngineError
    with pytest.raises(EngineError) as e:
        run_int8(500, (10, 36, 30), (3, 3, 3), (1, 1, 1), (1, 1, 1), 16, 24, True, True)
    assert e.value.status == -1
