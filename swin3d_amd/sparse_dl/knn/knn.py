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


_FEAT_DTYPE = {torch.float32: 0, torch.float16: 1}


def knn_interpolate(idx, dist2, src_feat):
    """Inverse-distance interpolation of src_feat [Ns,C] at the queries of a knn_query result
    (idx int32 [Nq,K], SQUARED distances fp32 [Nq,K]) -> [Nq,C] in the dtype of src_feat
    (Swin3D/modules/swin3d_layers.py:65-72 in one kernel; padded slots carry no weight)."""
    if not (idx.is_cuda and dist2.is_cuda and src_feat.is_cuda):
        raise RuntimeError("idx, dist2 and src_feat must be CUDA (HIP) tensors")
    if idx.dtype != torch.int32 or dist2.dtype != torch.float32 or idx.shape != dist2.shape or idx.dim() != 2:
        raise ValueError("idx must be int32 [Nq,K] and dist2 float32 [Nq,K]")
    if src_feat.dim() != 2 or src_feat.dtype not in _FEAT_DTYPE:
        raise ValueError(f"src_feat must be float16/float32 [Ns,C], got {src_feat.dtype} {tuple(src_feat.shape)}")
    idx, dist2, src_feat = idx.contiguous(), dist2.contiguous(), src_feat.contiguous()
    nq, k = idx.shape
    ns, c = src_feat.shape
    out = torch.empty((nq, c), dtype=src_feat.dtype, device=src_feat.device)
    with torch.cuda.device(src_feat.device):
        stream = torch.cuda.current_stream(src_feat.device).cuda_stream
        status = _lib.lib().s3d_knn_interpolate(idx.data_ptr(), dist2.data_ptr(), k, nq, src_feat.data_ptr(), ns, c,
                                                _FEAT_DTYPE[src_feat.dtype], out.data_ptr(), stream)
    _lib.check(status, "s3d_knn_interpolate")
    return out


def knn_max_pool(idx, src_feat):
    """Channel-wise maximum of src_feat [Ns,C] over the K nearest sources of every query (idx int32 [Nq,K] of a
    knn_query result) -> [Nq,C] in the dtype of src_feat: the gather + max of the KNN downsample
    (Swin3D/modules/swin3d_layers.py:292-312) without the [Nq,K,C] intermediate.  Padded slots (row -1) read
    row 0, as the clamped gather does.  No autograd (inference)."""
    if not (idx.is_cuda and src_feat.is_cuda):
        raise RuntimeError("idx and src_feat must be CUDA (HIP) tensors")
    if idx.dtype != torch.int32 or idx.dim() != 2:
        raise ValueError("idx must be int32 [Nq,K]")
    if src_feat.dim() != 2 or src_feat.dtype not in _FEAT_DTYPE:
        raise ValueError(f"src_feat must be float16/float32 [Ns,C], got {src_feat.dtype} {tuple(src_feat.shape)}")
    idx, src_feat = idx.contiguous(), src_feat.contiguous()
    nq, k = idx.shape
    ns, c = src_feat.shape
    out = torch.empty((nq, c), dtype=src_feat.dtype, device=src_feat.device)
    with torch.cuda.device(src_feat.device):
        stream = torch.cuda.current_stream(src_feat.device).cuda_stream
        status = _lib.lib().s3d_knn_max_pool(idx.data_ptr(), k, nq, src_feat.data_ptr(), ns, c,
                                             _FEAT_DTYPE[src_feat.dtype], out.data_ptr(), stream)
    _lib.check(status, "s3d_knn_max_pool")
    return out


class KNNInterpolate(Function):
    """Differentiable (w.r.t. the features) inverse-distance interpolation; the forward is the fused
    HIP kernel, the backward scatters the weighted output gradient back with torch's index_add_."""

    @staticmethod
    def forward(ctx, idx, dist2, src_feat):
        ctx.save_for_backward(idx, dist2)
        ctx.num_src = src_feat.shape[0]
        return knn_interpolate(idx, dist2, src_feat)

    @staticmethod
    def backward(ctx, grad_out):
        idx, dist2 = ctx.saved_tensors
        valid = idx >= 0
        weight = torch.where(valid, 1.0 / (torch.sqrt(dist2) + 1e-8), torch.zeros_like(dist2))
        weight = weight / weight.sum(dim=1, keepdim=True).clamp_min(1e-30)
        grad_src = torch.zeros((ctx.num_src, grad_out.shape[1]), dtype=torch.float32, device=grad_out.device)
        rows = idx.clamp(min=0).long()
        for i in range(idx.shape[1]):
            grad_src.index_add_(0, rows[:, i], grad_out.float() * weight[:, i:i + 1])
        return None, None, grad_src.to(grad_out.dtype)
