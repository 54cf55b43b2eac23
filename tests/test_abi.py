"""The C-ABI library without a GPU: it loads, exports every symbol the header declares, parses and round-trips
the reference's attribute blobs, infers shapes like the reference's plugins, and reports errors as status codes.
No kernel is launched here."""
import ctypes
import os
import re
import struct

import numpy as np
import pytest
import torch

import deploy3d_amd
from deploy3d_amd import EngineError, Plugin, TensorDesc
from deploy3d_amd.plugin import EXPORTS
from deploy3d_amd.bev_densify import densify_blob
from deploy3d_amd.simple_mean import simple_mean_blob
from deploy3d_amd.spconv_index import index_blob
from deploy3d_amd.spconv_mm import mm_blob

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    lib = deploy3d_amd.load_library()
    header = open(os.path.join(ROOT, "include", "d3d_spconv.h")).read()
    declared = set(re.findall(r"\b(d3d_[a-z_0-9]+)\s*\(", header))
    assert declared, "no declarations found"
    assert declared == set(EXPORTS)
    for name in declared:
        assert getattr(lib, name) is not None
    assert [lib.d3d_op_name(i).decode() for i in range(lib.d3d_num_ops())] == [
        "SPConvIdx1d", "SPConvIdx2d", "SPConvIdx3d", "SPConvIdx4d", "SPConvMM", "BEVDensify", "SimpleMeanEncoder"]


def test_index_blob_layout_and_round_trip():
    """SPConvIdxPluginParam<3> is 66 packed bytes (trt/spconv/index_trt.cu:39-50; writer spconv_index.py:94-101)."""
    blob = index_blob((3, 1, 3), (2, 1, 2), (1, 0, 1), (1, 1, 1), (0, 0, 0), 4096, False, False)
    assert len(blob) == 66
    assert struct.unpack("<16i", blob[:64]) == (3, 1, 3, 2, 1, 2, 1, 0, 1, 1, 1, 1, 0, 0, 0, 4096)
    assert blob[64:] == b"\x00\x00"
    p = Plugin("SPConvIdx3d", blob)
    assert p.plugin_type == "SPConvIdx3d" and p.plugin_version == "2.0"
    assert p.serialize() == blob and p.num_outputs == 5
    assert p.clone().serialize() == blob
    assert Plugin("SPConvIdx3d", index_blob((3,) * 3, (1,) * 3, (1,) * 3, (1,) * 3, (0,) * 3, 7, True, False)).num_outputs == 2
    for nd in (1, 2, 4):
        b = index_blob((3,) * nd, (2,) * nd, (1,) * nd, (1,) * nd, (0,) * nd, 10, False, False)
        assert len(b) == 20 * nd + 6
        assert Plugin("SPConvIdx%dd" % nd, b).serialize() == b


def test_index_shape_inference():
    """getOutputDimensions (trt/spconv/index_trt.cu:102-151)."""
    p = Plugin("SPConvIdx3d", index_blob((3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), (0, 0, 0), 5000, False, False))
    ins = [TensorDesc.of((20000, 4), torch.int32), TensorDesc.of((1,), torch.int32),
           TensorDesc.of((2, 0, 41, 1440, 1440), torch.int32)]
    outs = p.output_descs(ins)
    assert [o.shape() for o in outs] == [(3, 27 * 20128), (1,), (5000, 4), (1,), (2, 0, 21, 720, 720)]
    assert all(o.dtype == 3 for o in outs)
    assert p.workspace_size(ins, outs) > 0
    assert p.supports_format(0, ins + outs, 3, 5)
    t = Plugin("SPConvIdx3d", index_blob((3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), (1, 1, 1), 5000, False, True))
    assert t.output_descs(ins)[4].shape() == (2, 0, 82, 2880, 2880)


def test_mm_blob_layout_and_round_trip():
    """SPConvMMPluginParam is 19 packed bytes + fp32 W + fp32 bias (trt/spconv/mm_trt.cu:27-37, :61-74)."""
    w = np.arange(27 * 4 * 8, dtype=np.float32)
    b = np.arange(8, dtype=np.float32)
    blob = mm_blob((3, 3, 3), 4, 8, 1000, True, False, w, b)
    assert len(blob) == 19 + 4 * (27 * 4 * 8 + 8)
    assert struct.unpack("<4i3?", blob[:19]) == (27, 4, 8, 1000, True, False, True)
    p = Plugin("SPConvMM", blob)
    assert p.serialize() == blob and p.num_outputs == 1
    ins = [TensorDesc.of((500, 4), torch.float16), TensorDesc.of((1,), torch.int32), TensorDesc.of((1,), torch.int32),
           TensorDesc.of((3, 27 * 628), torch.int32), TensorDesc.of((1,), torch.int32)]
    out = p.output_descs(ins)[0]
    assert out.shape() == (1000, 8) and out.dtype == 1      # dtype of input 0 (mm_trt.cu:104-106)
    assert p.workspace_size(ins, [out]) == 0                # mm_trt.cu:143-148
    assert p.supports_format(0, ins + [out], 5, 1) and p.supports_format(5, ins + [out], 5, 1)
    bad = list(ins)
    bad[0] = TensorDesc.of((500, 4), torch.int32)
    assert not p.supports_format(0, bad + [out], 5, 1)
    q = list(ins)
    q[0] = TensorDesc.of((500, 4), torch.int8)          # int8 features: this build's extension
    assert p.supports_format(0, q + [out], 5, 1) and not p.supports_format(5, q + [out], 5, 1)
    assert p.output_descs(q)[0].dtype == 2
    ext = mm_blob((3, 3, 3), 4, 8, 1000, True, False, w, b, relu=True)
    assert len(ext) == len(blob) + 20 and Plugin("SPConvMM", ext).serialize() == ext


def test_densify_blob_and_shape_inference():
    """BEVDensifyPluginParam is one int32 (trt/spconv/bev_densify_trt.cu:43-47; writer bev_densify.py:38);
    getOutputDimensions gives [B, outChannels, Y, X] (bev_densify_trt.cu:86-97)."""
    blob = densify_blob(256)
    assert blob == struct.pack("<i", 256)
    p = Plugin("BEVDensify", blob)
    assert p.plugin_type == "BEVDensify" and p.plugin_version == "2.0" and p.num_outputs == 1
    assert p.serialize() == blob and p.clone().serialize() == blob
    for dtype, code in ((torch.float32, 0), (torch.float16, 1)):
        ins = [TensorDesc.of((10000, 128), dtype), TensorDesc.of((10000, 4), torch.int32),
               TensorDesc.of((1,), torch.int32), TensorDesc.of((2, 0, 2, 128, 128), torch.int32)]
        outs = p.output_descs(ins)
        assert [o.shape() for o in outs] == [(2, 256, 128, 128)] and outs[0].dtype == code
        assert all(p.supports_format(i, ins + outs, 4, 1) for i in range(5))
        assert p.workspace_size(ins, outs) == 2 * 2 * 128 * 128 * 4
    bad = [TensorDesc.of((10, 128), torch.int32)] + ins[1:] + outs
    assert not p.supports_format(0, bad, 4, 1)


def test_simple_mean_blob_and_shape_inference():
    """SimpleMeanEncoderPluginParam is one int32 (trt/voxel_encoder/simple_mean_trt.cu:176-180; writer
    simple_mean.py:44); outputs [max, C] float, [max, 4] int32, [1] int32 (simple_mean_trt.cu:221-244)."""
    blob = simple_mean_blob(30000)
    assert blob == struct.pack("<i", 30000)
    p = Plugin("SimpleMeanEncoder", blob)
    assert p.plugin_type == "SimpleMeanEncoder" and p.plugin_version == "2.0" and p.num_outputs == 3
    assert p.serialize() == blob and p.clone().serialize() == blob
    ins = [TensorDesc.of((200000, 5), torch.float32), TensorDesc.of((200000,), torch.int32),
           TensorDesc.of((6,), torch.float32), TensorDesc.of((2, 0, 41, 1536, 1536), torch.int32)]
    outs = p.output_descs(ins)
    assert [o.shape() for o in outs] == [(30000, 5), (30000, 4), (1,)]
    assert [o.dtype for o in outs] == [0, 3, 3]
    assert all(p.supports_format(i, ins + outs, 4, 3) for i in range(7))
    assert p.workspace_size(ins, outs) >= 2 * 200000 * 8
    half = [TensorDesc.of((200000, 5), torch.float16)] + ins[1:] + outs
    assert not p.supports_format(0, half, 4, 3)


@pytest.mark.parametrize("name,blob,status", [
    ("SPConvIdx3d", b"\x00" * 10, -2),
    ("SPConvMM", b"\x00" * 5, -2),
    ("SPConvMM", mm_blob((3, 3, 3), 4, 8, 10, True, False, np.zeros(27 * 32, np.float32))[:-40], -2),
    ("SPConvIdx3d", index_blob((0, 3, 3), (1,) * 3, (1,) * 3, (1,) * 3, (0,) * 3, 10, True, False), -2),
    ("BEVDensify", b"\x00\x00", -2),
    ("SimpleMeanEncoder", b"\x01", -2),
    ("CylinderEncoder", b"", -4),
])
def test_bad_blobs_and_unknown_ops_return_status(name, blob, status):
    with pytest.raises(EngineError) as e:
        Plugin(name, blob)
    assert e.value.status == status and str(e.value)


def test_wrong_version_is_unknown_op():
    with pytest.raises(EngineError) as e:
        Plugin("SPConvMM", mm_blob((1, 1, 1), 1, 1, 1, True, False, np.zeros(1, np.float32)), version="1.0")
    assert e.value.status == -4


def test_header_is_c_and_a_c_client_works(tmp_path):
    """include/d3d_spconv.h compiles as C99 and a plain C program drives the library through it (no GPU work)."""
    import shutil
    import subprocess
    from deploy3d_amd.build import ENGINE_LIB
    gcc = shutil.which("gcc")
    assert gcc, "gcc is part of the image"
    exe = tmp_path / "abi_check"
    src = os.path.join(ROOT, "tests", "abi_c", "abi_check.c")
    subprocess.check_call([gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"),
                           src, "-o", str(exe), "-ldl"])
    deploy3d_amd.load_library()  # builds the library if it is not there yet
    res = subprocess.run([str(exe), ENGINE_LIB], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert res.returncode == 0 and "abi_check ok" in res.stdout, res.stdout


def test_short_workspace_is_refused_before_any_launch():
    """enqueue with a workspace smaller than d3d_workspace_size() returns D3D_ERR_WORKSPACE (-5) for every operator
    that takes one (the reference sizes it in getWorkspaceSize, trt/spconv/index_trt.cu:178-187, and trusts the
    caller).  The check comes before the first kernel launch, so host tensors stand in for device memory here."""
    def enqueue(p, in_descs, out_descs, ins, outs, ws_bytes):
        ws = torch.zeros(max(1, ws_bytes), dtype=torch.uint8)
        with pytest.raises(EngineError) as e:
            p.enqueue(in_descs, out_descs, ins, outs, ws[:ws_bytes] if ws_bytes else None, stream=0)
        return e.value

    cap = 1000
    for subm in (True, False):
        p = Plugin("SPConvIdx3d", index_blob((3, 3, 3), (1, 1, 1) if subm else (2, 2, 2), (1, 1, 1), (1, 1, 1),
                                             (0, 0, 0), cap, subm, False))
        coors = torch.zeros((cap, 4), dtype=torch.int32)
        num = torch.zeros(1, dtype=torch.int32)
        ins = [TensorDesc.of_tensor(coors), TensorDesc.of_tensor(num), TensorDesc.of((1, 0, 8, 16, 16), torch.int32)]
        outs = p.output_descs(ins)
        need = p.workspace_size(ins, outs)
        assert need > 0
        bufs = [torch.zeros(d.shape(), dtype=torch.int32) if 0 not in d.shape() else None for d in outs]
        # d3d_workspace_size() covers whichever occupancy structure is chosen; the smaller one may fit in less,
        # so the refusal is forced with sizes below either
        for have in (0, 16, 4096):
            err = enqueue(p, ins, outs, [coors, num, None], bufs, have)
            assert err.status == -5 and "workspace" in str(err)

    p = Plugin("BEVDensify", densify_blob(16 * 4))
    feats = torch.zeros((10, 16), dtype=torch.float16)
    coors = torch.zeros((10, 4), dtype=torch.int32)
    num = torch.zeros(1, dtype=torch.int32)
    ins = [TensorDesc.of_tensor(feats), TensorDesc.of_tensor(coors), TensorDesc.of_tensor(num),
           TensorDesc.of((1, 0, 4, 8, 8), torch.int32)]
    outs = p.output_descs(ins)
    need = p.workspace_size(ins, outs)
    assert need == 4 * 4 * 8 * 8
    out = torch.zeros(outs[0].shape(), dtype=torch.float16)
    assert enqueue(p, ins, outs, [feats, coors, num, None], [out], need - 4).status == -5

    p = Plugin("SimpleMeanEncoder", simple_mean_blob(50))
    pts = torch.zeros((100, 4), dtype=torch.float32)
    bidx = torch.zeros(100, dtype=torch.int32)
    conf = torch.zeros(6, dtype=torch.float32)
    ins = [TensorDesc.of_tensor(pts), TensorDesc.of_tensor(bidx), TensorDesc.of_tensor(conf),
           TensorDesc.of((1, 0, 4, 8, 8), torch.int32)]
    outs = p.output_descs(ins)
    need = p.workspace_size(ins, outs)
    bufs = [torch.zeros(d.shape(), dtype=torch.float32 if i == 0 else torch.int32) for i, d in enumerate(outs)]
    assert enqueue(p, ins, outs, [pts, bidx, conf, None], bufs, need - 1).status == -5


def test_schedule_bookkeeping_without_a_gpu():
    """d3d_schedule_*: a one-lane schedule needs no HIP object, so its bookkeeping is testable here - step indices,
    refused steps (wrong output count, a wait for a step that does not precede, a lane outside the schedule)."""
    from deploy3d_amd.plugin import Schedule
    lib = deploy3d_amd.load_library()
    h = ctypes.c_void_p()
    assert lib.d3d_schedule_create(0, ctypes.byref(h)) == -3 and lib.d3d_schedule_create(9, ctypes.byref(h)) == -3
    assert lib.d3d_schedule_size(None) == -3 and lib.d3d_schedule_run(None, None) == -3
    lib.d3d_schedule_destroy(None)
    p = Plugin("SPConvIdx3d", index_blob((3,) * 3, (1,) * 3, (1,) * 3, (1,) * 3, (0,) * 3, 64, True, False))
    ins = [TensorDesc.of((64, 4), torch.int32), TensorDesc.of((1,), torch.int32),
           TensorDesc.of((1, 0, 8, 8, 8), torch.int32)]
    outs = p.output_descs(ins)
    coors, num = torch.zeros((64, 4), dtype=torch.int32), torch.zeros(1, dtype=torch.int32)
    index, num_index = torch.empty(outs[0].shape(), dtype=torch.int32), torch.zeros(1, dtype=torch.int32)
    s = Schedule(lanes=1)
    assert len(s) == 0
    assert s.add(p, ins, outs, [coors, num, None], [index, num_index]) == 0
    assert s.add(p, ins, outs, [coors, num, None], [index, num_index], after=[0]) == 1
    assert len(s) == 2
    with pytest.raises(EngineError) as e:
        s.add(p, ins, outs[:1], [coors, num, None], [index])           # the operator has two outputs
    assert e.value.status == -3
    with pytest.raises(EngineError) as e:
        s.add(p, ins[:2], outs, [coors, num], [index, num_index])      # the operator reads three inputs
    assert e.value.status == -3 and "reads 3 inputs" in str(e.value)
    with pytest.raises(EngineError):
        s.add(p, ins, outs, [coors, num, None], [index, num_index], after=[2])   # itself
    with pytest.raises(EngineError):
        s.add(p, ins, outs, [coors, num, None], [index, num_index], lane=1)
    assert len(s) == 2


def test_a_link_between_nodes_of_different_sizes_is_refused():
    """d3d_link_rulebook: the table a rulebook operator writes has maxNumActOut rows of ITS attribute blob
    (reference: two independent blob fields, spconv_index.py:99 and spconv_mm.py:57).  A forward convolution with
    another maxNumActOut could never use that table, so the link is refused; an inverse convolution, which always
    derives its table from the index tensor, may link whatever the sizes; and so is one with another kernel volume."""
    import numpy as np
    from deploy3d_amd.spconv_mm import mm_blob
    idx = Plugin("SPConvIdx3d", index_blob((3,) * 3, (2,) * 3, (1,) * 3, (1,) * 3, (0,) * 3, 512, False, False))
    w = np.zeros((27, 4, 4), np.float32)
    same = Plugin("SPConvMM", mm_blob((3, 3, 3), 4, 4, 512, False, False, w))
    other = Plugin("SPConvMM", mm_blob((3, 3, 3), 4, 4, 256, False, False, w))
    inverse = Plugin("SPConvMM", mm_blob((3, 3, 3), 4, 4, 256, False, True, w))
    volume = Plugin("SPConvMM", mm_blob((1, 3, 3), 4, 4, 512, False, False, np.zeros((9, 4, 4), np.float32)))
    for p in (other, volume):
        with pytest.raises(EngineError) as e:
            p.link_rulebook(idx)
        assert e.value.status == -3
    assert "maxNumActOut 256" in str(pytest.raises(EngineError, other.link_rulebook, idx).value)
    # accepted links reserve device memory for the table: without a GPU they get as far as that (status -6), with
    # one they succeed
    for p in (same, inverse):
        try:
            p.link_rulebook(idx)
        except EngineError as err:
            assert err.status == -6
