"""K-nearest-neighbour operator on the swin3d_amd HIP library.

Same Python surface as Swin3D/sparse_dl/knn/knn.py:9-26: KNN.apply(K, src_xyz, query_xyz,
src_offset, query_offset) -> (idx int32 [Nq,K], euclidean dist fp32 [Nq,K]); offsets are
cumulative END positions of the batch segments.  Result order: ascending (distance, source
row); segments with fewer than K sources are padded with row -1.
"""
import torch
from torch.autograd.function import Function

from ... import _lib


def knn_query(K, src_xyz, query_xyz, src_offset, query_offset, cell_size=0.0):
    """-> (idx int32 [Nq,K], SQUARED distances fp32 [Nq,K]).  cell_size <= 0: chosen from the data."""
    K = int(K)
    if not 1 <= K <= _lib.KNN_KMAX:
        raise ValueError(f"K must be in 1..{_lib.KNN_KMAX}, got {K}")
    for name, t in (("src_xyz", src_xyz), ("query_xyz", query_xyz)):
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be a CUDA (HIP) tensor")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
        if t.dtype != torch.float32 or t.dim() != 2 or t.shape[1] != 3:
            raise ValueError(f"{name} must be float32 [n,3], got {t.dtype} {tuple(t.shape)}")
    dev = query_xyz.device
    if src_xyz.device != dev:
        raise RuntimeError("src_xyz and query_xyz must be on the same device")
    offs = []
    for name, t in (("src_offset", src_offset), ("query_offset", query_offset)):
        if not isinstance(t, torch.Tensor):
            t = torch.as_tensor(t)
        if t.dtype not in (torch.int32, torch.int64) or t.dim() != 1:
            raise TypeError(f"{name} must be a 1-D int32/int64 tensor")
        offs.append(t.to(device=dev, dtype=torch.int32).contiguous())
    src_offset, query_offset = offs
    if src_offset.numel() != query_offset.numel() or src_offset.numel() == 0:
        raise ValueError("src_offset and query_offset must have the same non-zero length")
    ns, nq, b = src_xyz.shape[0], query_xyz.shape[0], src_offset.numel()
    idx = torch.empty((nq, K), dtype=torch.int32, device=dev)
    dist2 = torch.empty((nq, K), dtype=torch.float32, device=dev)
    lib = _lib.lib()
    with torch.cuda.device(dev):
        ws_bytes = lib.s3d_knn_workspace_bytes(ns, nq, b)
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        stream = torch.cuda.current_stream(dev).cuda_stream
        status = lib.s3d_knn(K, src_xyz.data_ptr(), ns, query_xyz.data_ptr(), nq,
                             src_offset.data_ptr(), query_offset.data_ptr(), b, idx.data_ptr(),
                             dist2.data_ptr(), float(cell_size), workspace.data_ptr(), ws_bytes,
                             stream)
    _lib.check(status, "s3d_knn")
    return idx, dist2


class KNN(Function):
    # edge of the bucketing grid in xyz units; 0 lets the library choose from the data
    cell_size = 0.0

    @staticmethod
    def forward(ctx, K, src_xyz, query_xyz, src_offset, query_offset):
        idx, dist2 = knn_query(K, src_xyz, query_xyz, src_offset, query_offset, KNN.cell_size)
        dist = torch.sqrt(dist2)
        ctx.mark_non_differentiable(idx, dist)
        return idx, dist
