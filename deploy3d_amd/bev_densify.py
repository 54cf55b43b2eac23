"""Sparse-to-dense operator with the calling convention of the reference's
``bev_densify`` (deploy3d/symfun/ops/spconv/bev_densify.py:18-45), executed by
the HIP engine: the reference's torch-side ``forward`` returns zeros of the
right shape, this one returns the map.
"""
import numpy as np
import torch

from .plugin import Plugin, TensorDesc

_plugins = {}
_workspaces = {}


def densify_blob(out_channels):
    """BEVDensifyPluginParam (trt/spconv/bev_densify_trt.cu:43-47; writer: bev_densify.py:38)."""
    return np.array([out_channels], dtype=np.int32).tobytes()


def _workspace(nbytes, device):
    key = (str(device), torch.cuda.current_stream().cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = _workspaces[key] = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
    return ws


def bev_densify(in_feats, in_coors, num_act_in, in_spatial_shape, out_channels, out=None):
    """out[B, C*Z, Y, X]: zero everywhere except out[b, c*Z + z, y, x] = in_feats[i, c] for the live rows.

    in_feats          [cap, C] float32 / float16 / bfloat16 / int8, device
    in_coors          int32 [cap, 4] rows (b, z, y, x), device
    num_act_in        int32 [1], device (never read on the host)
    in_spatial_shape  zero-element tensor of shape [B, 0, Z, Y, X]
    out_channels      C*Z
    """
    if in_coors.dtype != torch.int32 or num_act_in.dtype != torch.int32:
        raise TypeError("coordinates and counts must be int32")
    in_feats = in_feats.contiguous()
    in_coors = in_coors.contiguous()
    plugin = _plugins.get(int(out_channels))
    if plugin is None:
        plugin = _plugins[int(out_channels)] = Plugin("BEVDensify", densify_blob(out_channels))
    in_descs = [TensorDesc.of_tensor(in_feats), TensorDesc.of_tensor(in_coors), TensorDesc.of_tensor(num_act_in),
                TensorDesc.of(tuple(in_spatial_shape.shape), torch.int32)]
    out_descs = plugin.output_descs(in_descs)
    if out is None:
        out = torch.empty(out_descs[0].shape(), dtype=in_feats.dtype, device=in_feats.device)
    ws = _workspace(plugin.workspace_size(in_descs, out_descs), in_feats.device)
    plugin.enqueue(in_descs, out_descs, [in_feats, in_coors, num_act_in, None], [out], ws)
    return out


class BEVDensify:
    """Name-compatible handle: ``BEVDensify.apply(...)`` as in the reference."""
    apply = staticmethod(bev_densify)
