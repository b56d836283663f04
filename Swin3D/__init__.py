"""Import-path alias: `Swin3D.sparse_dl.*` served by the swin3d_amd HIP library.

The reference's modules import their operators as `Swin3D.sparse_dl.attn.attn_coff` and
`Swin3D.sparse_dl.knn` (Swin3D/modules/swin3d_layers.py:16-24).  With this directory's parent on
sys.path ahead of the reference's checkout, those imports resolve to swin3d_amd without any edit of
the calling module, while the rest of the reference's package (`Swin3D.modules`, `Swin3D.models`)
is still found in the reference's own directory: the package path is extended over every `Swin3D`
directory on sys.path, this one first.  Nothing else of the reference's package lives here.
"""
from pkgutil import extend_path

__path__ = extend_path(__path__, __name__)
