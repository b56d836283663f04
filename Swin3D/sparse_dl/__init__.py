"""`Swin3D.sparse_dl`: the operator package of the reference, served by swin3d_amd.sparse_dl."""
from . import attn, knn  # noqa: F401
