"""ctypes binding of the C ABI declared in include/d3d_spconv.h.

``Plugin`` plays the part TensorRT plays for the reference's plugins
(deploy3d/symfun/trt_utils/trt_module.py:99-140): it deserialises an operator
from (name, version, attribute blob), negotiates shapes, sizes the workspace
and enqueues on the current HIP stream.  torch is used for device memory and
streams only.
"""
import ctypes
import os

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ENGINE_LIB = os.path.join(HERE, "libs", "libdeploy3d_amd.so")

D3D_MAX_DIMS = 8
FLOAT, HALF, INT8, INT32, BOOL, BF16 = 0, 1, 2, 3, 4, 7
_TORCH_TO_D3D = {torch.float32: FLOAT, torch.float16: HALF, torch.int8: INT8, torch.int32: INT32,
                 torch.bool: BOOL, torch.bfloat16: BF16}
_D3D_TO_TORCH = {v: k for k, v in _TORCH_TO_D3D.items()}

STATUS_NAMES = {0: "OK", -1: "UNSUPPORTED", -2: "BAD_BLOB", -3: "BAD_ARG", -4: "UNKNOWN_OP", -5: "WORKSPACE",
                -6: "DEVICE"}

EXPORTS = [
    "d3d_create", "d3d_clone", "d3d_destroy", "d3d_plugin_type", "d3d_plugin_version", "d3d_serialize_size",
    "d3d_serialize", "d3d_num_outputs", "d3d_output_dims", "d3d_output_dtype", "d3d_supports_format",
    "d3d_configure", "d3d_workspace_size", "d3d_enqueue", "d3d_last_error", "d3d_num_ops", "d3d_op_name",
    "d3d_enqueue_static", "d3d_link_rulebook", "d3d_link_coords", "d3d_set_option",
    "d3d_schedule_create", "d3d_schedule_add", "d3d_schedule_size", "d3d_schedule_run", "d3d_schedule_destroy",
]
OPT_PERSISTENT_INDEX = 1
OPT_INDEX_UNUSED = 2


class EngineError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("d3d status %d (%s): %s" % (status, STATUS_NAMES.get(status, "?"), message))
        self.status = status


class TensorDesc(ctypes.Structure):
    _fields_ = [("dtype", ctypes.c_int32), ("format", ctypes.c_int32), ("nb_dims", ctypes.c_int32),
                ("dims", ctypes.c_int32 * D3D_MAX_DIMS)]

    @classmethod
    def of(cls, dims, dtype):
        d = cls()
        d.dtype = _TORCH_TO_D3D[dtype] if isinstance(dtype, torch.dtype) else int(dtype)
        d.format = 0
        d.nb_dims = len(dims)
        for i, v in enumerate(dims):
            d.dims[i] = int(v)
        return d

    @classmethod
    def of_tensor(cls, t):
        return cls.of(tuple(t.shape), t.dtype)

    def shape(self):
        return tuple(self.dims[i] for i in range(self.nb_dims))


_lib = None


def load_library(path=None):
    """Loads the engine; raises if the HIP library has not been built (there is no fallback path)."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    path = path or ENGINE_LIB
    if not os.path.exists(path):
        raise ImportError("%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                          "(hipcc --offload-arch=gfx950) first" % path)
    lib = ctypes.CDLL(path)
    vp, i32, sz = ctypes.c_void_p, ctypes.c_int32, ctypes.c_size_t
    descp = ctypes.POINTER(TensorDesc)
    lib.d3d_create.restype = i32
    lib.d3d_create.argtypes = [ctypes.c_char_p, ctypes.c_char_p, vp, sz, ctypes.POINTER(vp)]
    lib.d3d_clone.restype = i32
    lib.d3d_clone.argtypes = [vp, ctypes.POINTER(vp)]
    lib.d3d_destroy.restype = None
    lib.d3d_destroy.argtypes = [vp]
    lib.d3d_plugin_type.restype = ctypes.c_char_p
    lib.d3d_plugin_type.argtypes = [vp]
    lib.d3d_plugin_version.restype = ctypes.c_char_p
    lib.d3d_plugin_version.argtypes = [vp]
    lib.d3d_serialize_size.restype = sz
    lib.d3d_serialize_size.argtypes = [vp]
    lib.d3d_serialize.restype = i32
    lib.d3d_serialize.argtypes = [vp, vp, sz]
    lib.d3d_num_outputs.restype = i32
    lib.d3d_num_outputs.argtypes = [vp]
    lib.d3d_output_dims.restype = i32
    lib.d3d_output_dims.argtypes = [vp, i32, descp, i32, descp]
    lib.d3d_output_dtype.restype = i32
    lib.d3d_output_dtype.argtypes = [vp, i32, ctypes.POINTER(i32), i32]
    lib.d3d_supports_format.restype = i32
    lib.d3d_supports_format.argtypes = [vp, i32, descp, i32, i32]
    lib.d3d_configure.restype = i32
    lib.d3d_configure.argtypes = [vp, descp, i32, descp, i32]
    lib.d3d_workspace_size.restype = sz
    lib.d3d_workspace_size.argtypes = [vp, descp, i32, descp, i32]
    lib.d3d_enqueue.restype = i32
    lib.d3d_enqueue.argtypes = [vp, descp, descp, ctypes.POINTER(vp), ctypes.POINTER(vp), vp, sz, vp]
    lib.d3d_enqueue_static.restype = i32
    lib.d3d_enqueue_static.argtypes = [vp, descp, descp, ctypes.POINTER(vp), ctypes.POINTER(vp), vp]
    lib.d3d_last_error.restype = ctypes.c_char_p
    lib.d3d_num_ops.restype = i32
    lib.d3d_op_name.restype = ctypes.c_char_p
    lib.d3d_op_name.argtypes = [i32]
    lib.d3d_link_rulebook.restype = i32
    lib.d3d_link_rulebook.argtypes = [vp, vp]
    lib.d3d_link_coords.restype = i32
    lib.d3d_link_coords.argtypes = [vp, vp]
    lib.d3d_set_option.restype = i32
    lib.d3d_set_option.argtypes = [vp, i32, ctypes.c_int64]
    lib.d3d_schedule_create.restype = i32
    lib.d3d_schedule_create.argtypes = [i32, ctypes.POINTER(vp)]
    lib.d3d_schedule_add.restype = i32
    lib.d3d_schedule_add.argtypes = [vp, vp, descp, i32, descp, i32, ctypes.POINTER(vp), ctypes.POINTER(vp), vp, sz,
                                     i32, ctypes.POINTER(i32), i32]
    lib.d3d_schedule_size.restype = i32
    lib.d3d_schedule_size.argtypes = [vp]
    lib.d3d_schedule_run.restype = i32
    lib.d3d_schedule_run.argtypes = [vp, vp]
    lib.d3d_schedule_destroy.restype = None
    lib.d3d_schedule_destroy.argtypes = [vp]
    _lib = lib
    return lib


def _check(status):
    if status != 0:
        raise EngineError(status, load_library().d3d_last_error().decode())


def _desc_array(descs):
    arr = (TensorDesc * max(1, len(descs)))()
    for i, d in enumerate(descs):
        arr[i] = d
    return arr


class Plugin:
    """One operator instance (``d3d_plugin*``)."""

    def __init__(self, name, blob, version="2.0", _handle=None):
        self._lib = load_library()
        self.name = name
        if _handle is not None:
            self._h = _handle
            return
        h = ctypes.c_void_p()
        buf = ctypes.create_string_buffer(bytes(blob), len(blob))
        _check(self._lib.d3d_create(name.encode(), version.encode() if version is not None else None, buf, len(blob),
                                    ctypes.byref(h)))
        self._h = h

    def clone(self):
        h = ctypes.c_void_p()
        _check(self._lib.d3d_clone(self._h, ctypes.byref(h)))
        return Plugin(self.name, None, _handle=h)

    def close(self):
        if getattr(self, "_h", None):
            self._lib.d3d_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def plugin_type(self):
        return self._lib.d3d_plugin_type(self._h).decode()

    @property
    def plugin_version(self):
        return self._lib.d3d_plugin_version(self._h).decode()

    def serialize(self):
        n = self._lib.d3d_serialize_size(self._h)
        buf = ctypes.create_string_buffer(n)
        _check(self._lib.d3d_serialize(self._h, buf, n))
        return buf.raw

    @property
    def num_outputs(self):
        return self._lib.d3d_num_outputs(self._h)

    def output_descs(self, in_descs):
        ins = _desc_array(in_descs)
        in_types = (ctypes.c_int32 * len(in_descs))(*[d.dtype for d in in_descs])
        outs = []
        for i in range(self.num_outputs):
            d = TensorDesc()
            _check(self._lib.d3d_output_dims(self._h, i, ins, len(in_descs), ctypes.byref(d)))
            d.dtype = self._lib.d3d_output_dtype(self._h, i, in_types, len(in_descs))
            outs.append(d)
        return outs

    def supports_format(self, pos, descs, nb_in, nb_out):
        return bool(self._lib.d3d_supports_format(self._h, pos, _desc_array(descs), nb_in, nb_out))

    def configure(self, in_descs, out_descs):
        _check(self._lib.d3d_configure(self._h, _desc_array(in_descs), len(in_descs), _desc_array(out_descs),
                                       len(out_descs)))

    def workspace_size(self, in_descs, out_descs):
        return self._lib.d3d_workspace_size(self._h, _desc_array(in_descs), len(in_descs), _desc_array(out_descs),
                                            len(out_descs))

    def link_rulebook(self, idx_plugin):
        """SPConvMM only: this node's index tensor is the output of ``idx_plugin`` (None removes the link), so the
        rulebook operator writes the neighbour table and tile masks itself and this node uses them."""
        _check(self._lib.d3d_link_rulebook(self._h, None if idx_plugin is None else idx_plugin._h))

    def link_coords(self, producer):
        """SPConvIdx only: the coordinates it is handed are the output of the strided SPConvIdx ``producer`` (None
        removes the link).  A submanifold operator then reuses that operator's occupancy map instead of building its
        own; a strided one derives the occupancy of its output grid from it instead of marking it input by input."""
        _check(self._lib.d3d_link_coords(self._h, None if producer is None else producer._h))

    def set_option(self, option, value):
        _check(self._lib.d3d_set_option(self._h, int(option), int(value)))

    def enqueue(self, in_descs, out_descs, inputs, outputs, workspace=None, stream=None):
        """inputs / outputs: torch tensors (or None for shape-only tensors); returns the raw status check."""
        def ptrs(ts):
            arr = (ctypes.c_void_p * max(1, len(ts)))()
            for i, t in enumerate(ts):
                arr[i] = None if t is None or t.numel() == 0 else t.data_ptr()
            return arr
        static = isinstance(workspace, str)
        ws_ptr = None if workspace is None or static else workspace.data_ptr()
        ws_bytes = 0 if workspace is None or static else workspace.numel() * workspace.element_size()
        if stream is None:
            stream = torch.cuda.current_stream().cuda_stream
        if static:  # workspace="static" -> d3d_enqueue_static: the library's own fixed scratch array, no allocation
            _check(self._lib.d3d_enqueue_static(self._h, _desc_array(in_descs), _desc_array(out_descs), ptrs(inputs),
                                                ptrs(outputs), ctypes.c_void_p(stream)))
            return
        _check(self._lib.d3d_enqueue(self._h, _desc_array(in_descs), _desc_array(out_descs), ptrs(inputs),
                                     ptrs(outputs), ws_ptr, ws_bytes, ctypes.c_void_p(stream)))


class Schedule:
    """A pass recorded once and enqueued by one native call (d3d_schedule_*): steps are operator enqueues with their
    descriptors, tensors and workspace, each on a lane (lane 0 = the stream of ``run``; the others are streams the
    schedule owns) and behind the earlier steps it names.  Keeps the tensors and operators it was given alive."""

    def __init__(self, lanes=1):
        self._lib = load_library()
        h = ctypes.c_void_p()
        _check(self._lib.d3d_schedule_create(int(lanes), ctypes.byref(h)))
        self._h = h
        self.lanes = int(lanes)
        self._keep = []

    def add(self, plugin, in_descs, out_descs, inputs, outputs, workspace=None, lane=0, after=()):
        """Appends ``plugin.enqueue(in_descs, out_descs, inputs, outputs, workspace)``; returns the step's index."""
        def ptrs(ts):
            arr = (ctypes.c_void_p * max(1, len(ts)))()
            for i, t in enumerate(ts):
                arr[i] = None if t is None or t.numel() == 0 else t.data_ptr()
            return arr
        ws_ptr = None if workspace is None else workspace.data_ptr()
        ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
        dep = (ctypes.c_int32 * max(1, len(after)))(*[int(a) for a in after])
        rc = self._lib.d3d_schedule_add(self._h, plugin._h, _desc_array(in_descs), len(in_descs),
                                        _desc_array(out_descs), len(out_descs), ptrs(inputs), ptrs(outputs), ws_ptr,
                                        ws_bytes, int(lane), dep, len(after))
        if rc < 0:
            _check(rc)
        self._keep.append((plugin, list(inputs), list(outputs), workspace))
        return rc

    def __len__(self):
        return int(self._lib.d3d_schedule_size(self._h))

    def run(self, stream=None):
        if stream is None:
            stream = torch.cuda.current_stream().cuda_stream
        _check(self._lib.d3d_schedule_run(self._h, ctypes.c_void_p(stream)))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.d3d_schedule_destroy(h)


STATIC_SCRATCH_BYTES = 64 << 20


def torch_dtype(d3d_dtype):
    return _D3D_TO_TORCH[d3d_dtype]
