"""Rulebook operator with the calling convention of the reference's
``spconv_index`` (deploy3d/symfun/ops/spconv/spconv_index.py:6-108), executed
by the HIP engine instead of being exported to a TensorRT graph.
"""
import hashlib

import numpy as np
import torch

from .plugin import Plugin, TensorDesc

_plugins = {}
_workspaces = {}


def index_blob(kernel_size, stride, padding, dilation, out_padding, max_num_act_out, subm, transpose):
    """Packed SPConvIdxPluginParam<N> (trt/spconv/index_trt.cu:39-50; writer: spconv_index.py:94-101)."""
    data = b"".join(np.array(v, dtype=np.int32).tobytes()
                    for v in (kernel_size, stride, padding, dilation, out_padding))
    data += np.array([max_num_act_out], dtype=np.int32).tobytes()
    data += np.array([bool(subm)], dtype=np.bool_).tobytes()
    data += np.array([bool(transpose)], dtype=np.bool_).tobytes()
    return data


def _plugin(name, blob):
    key = (name, hashlib.sha1(blob).digest())
    p = _plugins.get(key)
    if p is None:
        p = _plugins[key] = Plugin(name, blob)
    return p


def _workspace(nbytes, device):
    key = (str(device), torch.cuda.current_stream().cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = _workspaces[key] = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
    return ws


def index_plugin(kernel_size, stride, padding, dilation, out_padding, max_num_act_out, subm, transpose):
    """The operator instance ``spconv_index_nd`` runs for these attributes (one per distinct attribute blob); what
    ``spconv_mm(..., rulebook=...)`` links a convolution to."""
    blob = index_blob(kernel_size, stride, padding, dilation, out_padding, max_num_act_out, subm, transpose)
    return _plugin("SPConvIdx%dd" % len(kernel_size), blob)


def spconv_index_nd(in_coors, num_act_in, in_spatial_shape, kernel_size, stride, padding, dilation, out_padding,
                    max_num_act_out, subm, transpose):
    """SPConvIdx{N}d for N = len(kernel_size) in 1..4.

    in_coors          int32 [cap, N+1] rows (b, spatial...), device
    num_act_in        int32 [1], device (never read on the host)
    in_spatial_shape  zero-element tensor of shape [B, 0, spatial...]
    Returns (index [3, kVol*(cap+128)], num_index [1]) for SubM, else also
    (out_coors [max_num_act_out, N+1], num_act_out [1], out_spatial_shape).
    """
    nd = len(kernel_size)
    if in_coors.dtype != torch.int32 or num_act_in.dtype != torch.int32:
        raise TypeError("coordinates and counts must be int32")
    in_coors = in_coors.contiguous()
    plugin = index_plugin(kernel_size, stride, padding, dilation, out_padding, max_num_act_out, subm, transpose)
    in_descs = [TensorDesc.of_tensor(in_coors), TensorDesc.of_tensor(num_act_in),
                TensorDesc.of(tuple(in_spatial_shape.shape), torch.int32)]
    out_descs = plugin.output_descs(in_descs)
    dev = in_coors.device
    outs = []
    for i, d in enumerate(out_descs):
        outs.append(torch.empty(d.shape(), dtype=torch.int32, device=dev))
    ws = _workspace(plugin.workspace_size(in_descs, out_descs), dev)
    plugin.enqueue(in_descs, out_descs, [in_coors, num_act_in, None], outs, ws)
    return tuple(outs)


def spconv_index(in_coors, num_act_in, in_spatial_shape, kernel_size, stride, padding, dilation, out_padding,
                 max_num_act_out, subm, transpose):
    """3-D rulebook; same positional arguments as the reference's ``spconv_index``."""
    return spconv_index_nd(in_coors, num_act_in, in_spatial_shape, kernel_size, stride, padding, dilation,
                           out_padding, max_num_act_out, subm, transpose)


class SPConvIdx3d:
    """Name-compatible handle: ``SPConvIdx3d.apply(...)`` as in the reference."""
    apply = staticmethod(spconv_index)
