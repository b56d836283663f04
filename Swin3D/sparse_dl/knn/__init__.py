"""`Swin3D.sparse_dl.knn` (Swin3D/modules/swin3d_layers.py:23-24 imports KNN from here)."""
from swin3d_amd.sparse_dl.knn import KNN  # noqa: F401
