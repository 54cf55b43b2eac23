"""MI355X-native sparse-convolution engine with the operator surface of
deploy3d's SPConvIdx{1..4}d / SPConvMM / BEVDensify / SimpleMeanEncoder
TensorRT plugins.

The compute path is the in-tree HIP library ``libs/libdeploy3d_amd.so`` reached
through the C ABI of ``include/d3d_spconv.h``; there is no CPU fallback.
"""
from .plugin import Plugin, TensorDesc, EngineError, load_library  # noqa: F401
from .spconv_index import SPConvIdx3d, spconv_index, spconv_index_nd  # noqa: F401
from .spconv_mm import SPConvMM, spconv_mm  # noqa: F401
from .bev_densify import BEVDensify, bev_densify  # noqa: F401
from .simple_mean import SimpleMeanEncoder, simple_mean_encoder  # noqa: F401
