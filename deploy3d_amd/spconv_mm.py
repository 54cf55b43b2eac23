"""Gather-GEMM-scatter operator with the calling convention of the reference's
``spconv_mm`` (deploy3d/symfun/ops/spconv/spconv_mm.py:6-70), executed by the
HIP engine.  ``relu`` (fused ReLU) and the activation scales are this build's
extensions, carried in an extension record after the reference's blob.
"""
import hashlib
import struct

import numpy as np
import torch

from .plugin import Plugin, TensorDesc

_plugins = {}
EXT_MAGIC = 0x58443344  # "D3DX"


def mm_blob(kernel_size, in_channels, out_channels, max_num_act_out, subm, inverse, weight, bias=None, relu=False,
            act_scale_in=1.0, act_scale_out=1.0):
    """Packed SPConvMMPluginParam + fp32 payload (trt/spconv/mm_trt.cu:27-37; writer: spconv_mm.py:54-63)."""
    kvol = int(np.prod(kernel_size)) if not np.isscalar(kernel_size) else int(kernel_size)
    weight = np.ascontiguousarray(weight, dtype=np.float32).reshape(-1)
    assert weight.size == kvol * in_channels * out_channels
    data = np.array([kvol, in_channels, out_channels, max_num_act_out], dtype=np.int32).tobytes()
    data += np.array([bool(subm), bool(inverse), bias is not None], dtype=np.bool_).tobytes()
    data += weight.tobytes()
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=np.float32).reshape(-1)
        assert bias.size == out_channels
        data += bias.tobytes()
    if relu or act_scale_in != 1.0 or act_scale_out != 1.0:
        data += struct.pack("<IIIff", EXT_MAGIC, 1, 1 if relu else 0, act_scale_in, act_scale_out)
    return data


def get_plugin(blob):
    key = hashlib.sha1(blob).digest()
    p = _plugins.get(key)
    if p is None:
        p = _plugins[key] = Plugin("SPConvMM", blob)
    return p


def run_mm(plugin, in_feats, num_act_in, num_act_out, index, num_index, out=None):
    in_descs = [TensorDesc.of_tensor(t) for t in (in_feats, num_act_in, num_act_out, index, num_index)]
    out_descs = plugin.output_descs(in_descs)
    if out is None:
        out = torch.empty(out_descs[0].shape(), dtype=in_feats.dtype, device=in_feats.device)
    plugin.enqueue(in_descs, out_descs, [in_feats, num_act_in, num_act_out, index, num_index], [out])
    return out


def spconv_mm(in_feats, num_act_in, num_act_out, index, num_index, kernel_size, in_channels, out_channels,
              max_num_act_out, subm, inverse, weight, bias=None, relu=False, act_scale_in=1.0, act_scale_out=1.0,
              rulebook=None):
    """out[maxNumActOut, Cout] = bias + sum over taps of in[gather] @ W[tap] scattered to out rows.

    Same positional arguments as the reference's ``spconv_mm``; ``weight`` is the
    flat fp32 [kVol, Cin, Cout] array, ``bias`` fp32 [Cout] or None.  The keyword arguments are this
    build's extensions: a fused ReLU; for int8 features, the activation scales of input and output; and
    ``rulebook``, the SPConvIdx operator instance that wrote ``index`` (``spconv_index.index_plugin``): the
    convolution is linked to it and reads the neighbour table that operator wrote instead of deriving one from the
    index tensor (which is what happens without it, and for any tensor that operator did not write last).
    """
    blob = mm_blob(kernel_size, in_channels, out_channels, max_num_act_out, subm, inverse, weight, bias, relu,
                   act_scale_in, act_scale_out)
    plugin = get_plugin(blob)
    plugin.link_rulebook(rulebook)
    return run_mm(plugin, in_feats.contiguous(), num_act_in, num_act_out, index, num_index)


class SPConvMM:
    """Name-compatible handle: ``SPConvMM.apply(...)`` as in the reference."""
    apply = staticmethod(spconv_mm)
