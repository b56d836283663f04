"""swin3d_amd: MI355X (gfx950) sparse window attention (forward and backward), window index and KNN for Swin3D.

The compute lives in libswin3d_amd.so (hand-written HIP behind a C ABI, see
include/swin3d_amd.h); this package is the host side that mirrors the
reference's operator surface (Swin3D/sparse_dl) on top of it.
"""
from . import _lib
from .sparse_dl.attn.attn_coff import (IndexMode, PosEmb, PrecisionMode, SelfAttnAIOFunction,
                                       TableDims, window_attention_backward, window_attention_forward)
from .sparse_dl.knn import KNN, KNNInterpolate, knn_interpolate, knn_query
from .window_index import (WindowIndex, build_window_index, build_window_indices, get_index01, sparse_self_attention,
                           window_signals)
from .crse import crse_table_rows, crse_table_sizes, scale_crse_coords
from .fused_norm import add_layernorm

__version__ = "0.1.0"

__all__ = [
    "IndexMode", "PosEmb", "PrecisionMode", "SelfAttnAIOFunction", "TableDims",
    "window_attention_forward", "window_attention_backward", "KNN", "KNNInterpolate", "knn_interpolate", "knn_query", "WindowIndex", "build_window_index",
    "build_window_indices", "window_signals",
    "get_index01", "sparse_self_attention", "crse_table_rows", "crse_table_sizes",
    "scale_crse_coords", "add_layernorm",
]
