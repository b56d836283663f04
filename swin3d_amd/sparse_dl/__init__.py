"""Operator surface mirroring Swin3D/sparse_dl (attention and KNN autograd functions)."""
from . import attn, knn
