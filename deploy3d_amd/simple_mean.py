"""Voxeliser with the calling convention of the reference's ``simple_mean_encoder``
(deploy3d/symfun/ops/voxel_encoder/simple_mean.py:6-52), executed by the HIP
engine: the reference's torch-side ``forward`` returns zero tensors of the right
shape, this one returns the voxels.
"""
import numpy as np
import torch

from .plugin import Plugin, TensorDesc

_plugins = {}
_workspaces = {}


def simple_mean_blob(max_num_act_out):
    """SimpleMeanEncoderPluginParam (trt/voxel_encoder/simple_mean_trt.cu:176-180; writer: simple_mean.py:44)."""
    return np.array([max_num_act_out], dtype=np.int32).tobytes()


def _workspace(nbytes, device):
    key = (str(device), torch.cuda.current_stream().cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = _workspaces[key] = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
    return ws


def simple_mean_encoder(batch_point_feats, batch_indices, voxel_config, in_spatial_shape, max_num_act_out):
    """Points to voxels: mean of the features of the points in every occupied cell.

    batch_point_feats  float32 [N, C], x y z first; rows with a non-finite feature are skipped
    batch_indices      int32 [N]; negative = skip the point
    voxel_config       float32 [6] on the device: xMin yMin zMin xSize ySize zSize
    in_spatial_shape   zero-element tensor of shape [B, 0, Z, Y, X]
    Returns (out_feats [max_num_act_out, C], out_coors int32 [max_num_act_out, 4] rows (b, z, y, x),
    num_act_out int32 [1]); voxels come in order of first appearance among the points.
    """
    if batch_point_feats.dtype != torch.float32 or voxel_config.dtype != torch.float32:
        raise TypeError("point features and voxel config must be float32")
    if batch_indices.dtype != torch.int32:
        raise TypeError("batch indices must be int32")
    batch_point_feats = batch_point_feats.contiguous()
    batch_indices = batch_indices.contiguous()
    dev = batch_point_feats.device
    voxel_config = voxel_config.to(dev).contiguous()
    plugin = _plugins.get(int(max_num_act_out))
    if plugin is None:
        plugin = _plugins[int(max_num_act_out)] = Plugin("SimpleMeanEncoder", simple_mean_blob(max_num_act_out))
    in_descs = [TensorDesc.of_tensor(batch_point_feats), TensorDesc.of_tensor(batch_indices),
                TensorDesc.of_tensor(voxel_config), TensorDesc.of(tuple(in_spatial_shape.shape), torch.int32)]
    out_descs = plugin.output_descs(in_descs)
    out_feats = torch.empty(out_descs[0].shape(), dtype=torch.float32, device=dev)
    out_coors = torch.empty(out_descs[1].shape(), dtype=torch.int32, device=dev)
    num_act_out = torch.empty(out_descs[2].shape(), dtype=torch.int32, device=dev)
    ws = _workspace(plugin.workspace_size(in_descs, out_descs), dev)
    plugin.enqueue(in_descs, out_descs, [batch_point_feats, batch_indices, voxel_config, None],
                   [out_feats, out_coors, num_act_out], ws)
    return out_feats, out_coors, num_act_out


class SimpleMeanEncoder:
    """Name-compatible handle: ``SimpleMeanEncoder.apply(...)`` as in the reference."""
    apply = staticmethod(simple_mean_encoder)
