"""`Swin3D.sparse_dl.attn.attn_coff` (the names Swin3D/modules/swin3d_layers.py:16-22 imports)."""
from swin3d_amd.sparse_dl.attn.attn_coff import (  # noqa: F401
    IndexMode, PosEmb, PrecisionMode, SelfAttnAIOFunction, TableDims)
