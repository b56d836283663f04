"""Swin3D encoder on the swin3d_amd operators, without MinkowskiEngine (inference path).

The sparse voxel set is a pair of tensors (`SparseVoxels`); dense math (Linear, GELU, the 27-offset stem
convolution as one GEMM) goes to hipBLASLt through torch.  Window attention runs through
`SelfAttnAIOFunction`, the window index through `build_window_indices` / `window_signals`, neighbour
gathering through `KNN` / `knn_max_pool`.  On the GPU the coordinate work runs on the library's kernels too
(coarse cells and their representatives from the window sort, the stem's neighbour rows by binary search in
sorted packed keys, the fused add + LayerNorm); the same functions have a tensor statement for host tensors,
against which the kernels are tested.  The geometry of all stages is computed first (`plan_stages`): it
needs no features and is the only place where the host waits for the device.

What each piece mirrors in the reference (semantics, not code):
  sparse_conv3x3x3 + BatchNorm + ReLU   MinkConvBNRelu stem            Swin3D/modules/mink_layers.py:50-80
  pool_coordinates                      MinkowskiMaxPooling on coords  Swin3D/modules/swin3d_layers.py:284-286
  pick_cell_representatives             GridCoordsDown                 :179-231
  pool_and_pick                         the two above on the GPU (window sort + one kernel over the cells)
  segment_offsets                       get_offset                     :234-241
  GridKNNDownsample                     same name                      :272-315
  WindowAttention / SwinBlock / Stage   WindowAttention, SwinTransformerBlock, BasicLayer  :382-871
  Swin3DEncoder                         same name                      Swin3D/models/Swin3D.py:185-269
  query_knn_feature, knn_linear_interpolation, Upsample   same names   Swin3D/modules/swin3d_layers.py:27-73, 318-379
  Swin3DUNet, load_state_with_same_shape                  same names   Swin3D/models/Swin3D.py:12-183
MinkowskiEngine's output ORDER of pooled coordinates and its tie-breaking are not pinned by
anything in the reference; here pooled voxels are sorted by (batch, x, y, z) and ties go to
the lower row.  Stochastic depth is inference-time identity.
"""
from dataclasses import dataclass

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _lib
from .crse import crse_num_axes, crse_table_sizes, scale_crse_coords
from .fused_norm import add_layernorm
from .sparse_dl.attn.attn_coff import IndexMode, PosEmb, PrecisionMode, SelfAttnAIOFunction, TableDims
from .sparse_dl.knn import KNN, KNNInterpolate, knn_max_pool, knn_query
from .window_index import build_window_indices, get_index01, index_arguments, window_signals


@dataclass
class SparseVoxels:
    """coords int32 [N,4] = (batch, x, y, z), x/y/z multiples of `stride`, batches contiguous and
    ascending; feats [N,C]."""
    coords: torch.Tensor
    feats: torch.Tensor
    stride: int = 1

    def with_feats(self, feats):
        return SparseVoxels(self.coords, feats, self.stride)


_FIELD = 19            # bits per coordinate in a packed key
_BIAS = 1 << (_FIELD - 1)


def pack_coords(coords):
    """int64 key, order-preserving for (batch, x, y, z) with |x|,|y|,|z| < 2^18 and batch < 64."""
    c = coords.long()
    key = c[:, 0]
    for axis in (1, 2, 3):
        key = (key << _FIELD) + (c[:, axis] + _BIAS)
    return key


def lookup_rows(sorted_keys, order, query_keys):
    """row of every query key in the voxel set described by (sorted_keys, order); -1 if absent."""
    pos = torch.searchsorted(sorted_keys, query_keys).clamp_(max=sorted_keys.numel() - 1)
    hit = sorted_keys[pos] == query_keys
    return torch.where(hit, order[pos], torch.full_like(pos, -1))


def conv3x3x3_neighbours(coords, stride):
    """[N, 27] long: the row of every voxel's 27 lattice neighbours (offsets ordered x-major), N where the
    neighbour is missing.  Depends on the coordinates only.  A packed key is linear in the coordinates, so a
    neighbour's key is the voxel's key plus a constant per offset; taken in sorted key order the 27 query lists are
    sorted themselves, which keeps the binary searches local."""
    n = coords.shape[0]
    sorted_keys, order = torch.sort(pack_coords(coords))
    deltas = torch.tensor([((dx << _FIELD) + dy << _FIELD) + dz for dx in (-1, 0, 1) for dy in (-1, 0, 1)
                           for dz in (-1, 0, 1)], dtype=torch.long, device=coords.device) * stride
    if coords.is_cuda:
        out = torch.empty((n, 27), dtype=torch.long, device=coords.device)
        with torch.cuda.device(coords.device):
            status = _lib.lib().s3d_key_neighbours(sorted_keys.data_ptr(), order.data_ptr(), n, deltas.data_ptr(), 27,
                                                   out.data_ptr(), torch.cuda.current_stream(coords.device).cuda_stream)
        _lib.check(status, "s3d_key_neighbours")
        return out
    queries = sorted_keys.unsqueeze(0) + deltas.unsqueeze(1)                    # [27, N], rows ascending
    pos = torch.searchsorted(sorted_keys, queries).clamp_(max=n - 1)
    rows = torch.where(sorted_keys[pos] == queries, order[pos], torch.full_like(pos, n))
    out = torch.empty((n, 27), dtype=torch.long, device=coords.device)
    out[order] = rows.t()
    return out


def sparse_conv3x3x3(voxels, weight, neighbours=None):
    """Submanifold-style 3x3x3 convolution (outputs on the input voxels; missing neighbours are
    zeros).  weight [27, Cin, Cout], offsets ordered x-major.  One gather + one GEMM."""
    feats = voxels.feats
    n, cin = feats.shape
    if neighbours is None:
        neighbours = conv3x3x3_neighbours(voxels.coords, voxels.stride)
    padded = torch.cat([feats, feats.new_zeros(1, cin)], 0)   # row n = zeros for missing neighbours
    gathered = padded[neighbours.reshape(-1)].view(n, 27 * cin)
    return gathered @ weight.reshape(27 * cin, -1).to(gathered.dtype)


def pool_coordinates(coords, stride, factor):
    """coarse voxel coordinates (floor to the coarse lattice), unique and sorted by (b,x,y,z);
    also the coarse row of every fine voxel."""
    step = stride * factor
    if coords.is_cuda and 1 <= factor <= 10:
        # on the GPU a coarse cell is a window of `factor` voxels per side: the window sort gives the cells in the
        # same ascending (batch, x, y, z) order, one host wait, a third of the time of unique + scatter
        try:
            index = build_window_indices(coords, stride, factor, (0,))[0]
        except ValueError:          # coordinates outside the window sort's range
            index = None
        if index is not None:
            n = coords.shape[0]
            rows = index.n2n.long()
            members = coords[rows[index.w2n.long()]]            # one voxel of every cell
            members[:, 1:] = torch.div(members[:, 1:], step, rounding_mode="floor") * step
            cell_of_sorted = torch.repeat_interleave(torch.arange(index.num_windows, device=coords.device),
                                                     index.w_sizes.long(), output_size=n)
            inverse = torch.empty(n, dtype=torch.long, device=coords.device)
            inverse[rows] = cell_of_sorted
            return members, inverse
    coarse = coords.clone()
    coarse[:, 1:] = torch.div(coords[:, 1:], step, rounding_mode="floor") * step
    keys = pack_coords(coarse)
    uniq, inverse = torch.unique(keys, sorted=True, return_inverse=True)
    first = torch.full((uniq.numel(),), coords.shape[0], dtype=torch.long, device=coords.device)
    first.scatter_reduce_(0, inverse, torch.arange(coords.shape[0], device=coords.device), reduce="amin")
    return coarse[first], inverse


def pool_and_pick(coords, stride, factor, signals, index=None):
    """(coarse coordinates, representative fine row of every coarse voxel).  On the GPU both come from one window
    sort at window = factor (a coarse cell is a window; `index`, when the caller has built it already) and one
    kernel over the cells; elsewhere from pool_coordinates and pick_cell_representatives."""
    sig = signals.float()
    if coords.is_cuda and 1 <= factor <= 10 and 1 <= sig.shape[1] <= 16:
        if index is None:
            try:
                index = build_window_indices(coords, stride, factor, (0,))[0]
            except ValueError:          # coordinates outside the window sort's range
                index = None
        if index is not None:
            step = stride * factor
            members = coords[index.n2n.long()[index.w2n.long()]]            # one voxel of every cell
            members[:, 1:] = torch.div(members[:, 1:], step, rounding_mode="floor") * step
            if sig.stride(1) != 1:
                sig = sig.contiguous()
            pick = torch.empty(index.num_windows, dtype=torch.long, device=coords.device)
            with torch.cuda.device(coords.device):
                status = _lib.lib().s3d_cell_representatives(
                    index.n2n.data_ptr(), index.w2n.data_ptr(), index.w_sizes.data_ptr(), index.num_windows,
                    sig.data_ptr(), sig.stride(0), sig.shape[1], pick.data_ptr(),
                    torch.cuda.current_stream(coords.device).cuda_stream)
            _lib.check(status, "s3d_cell_representatives")
            return members, pick
    coarse, cell_of_row = pool_coordinates(coords, stride, factor)
    return coarse, pick_cell_representatives(signals, cell_of_row, coarse.shape[0])


def pick_cell_representatives(signals, cell_of_row, num_cells):
    """For every coarse cell the fine row whose signal vector (all columns of the coordinate
    features) is nearest to the cell mean; ties go to the lower row."""
    sig = signals.float()
    sums = sig.new_zeros(num_cells, sig.shape[1]).index_add_(0, cell_of_row, sig)
    counts = sig.new_zeros(num_cells).index_add_(0, cell_of_row, sig.new_ones(sig.shape[0]))
    mean = sums / counts.unsqueeze(1)
    dist = (sig - mean[cell_of_row]).pow(2).sum(1).sqrt()
    best = dist.new_full((num_cells,), float("inf")).scatter_reduce_(0, cell_of_row, dist, reduce="amin")
    rows = torch.arange(sig.shape[0], device=sig.device)
    cand = torch.where(dist == best[cell_of_row], rows, torch.full_like(rows, sig.shape[0]))
    pick = torch.full((num_cells,), sig.shape[0], dtype=torch.long, device=sig.device)
    pick.scatter_reduce_(0, cell_of_row, cand, reduce="amin")
    return pick


def segment_offsets(batch_column, num_batches=None):
    """cumulative END row of every batch element, int32 (what the KNN op takes).  With `num_batches` given the
    host does not wait for the device (batch ids are ascending: the end of batch b is a binary search)."""
    if num_batches is not None:
        ids = torch.arange(num_batches, dtype=batch_column.dtype, device=batch_column.device)
        return torch.searchsorted(batch_column.contiguous(), ids, right=True).to(torch.int32)
    counts = torch.bincount(batch_column.long())
    return torch.cumsum(counts, 0).to(torch.int32)


class _ConvKernel(nn.Module):
    """Holds the stem convolution's weight under the name MinkowskiConvolution gives it: `kernel`
    [27, Cin, Cout] (kernel volume, in, out)."""

    def __init__(self, in_channels, out_channels):
        super().__init__()
        self.kernel = nn.Parameter(torch.empty(27, in_channels, out_channels))
        nn.init.kaiming_normal_(self.kernel.view(27 * in_channels, out_channels).t())


class _BatchNorm(nn.Module):
    """BatchNorm1d under the name MinkowskiBatchNorm gives it: `bn`."""

    def __init__(self, channels):
        super().__init__()
        self.bn = nn.BatchNorm1d(channels)

    def forward(self, x):
        return self.bn(x)


class StemConv(nn.Module):
    """3x3x3 sparse convolution + BatchNorm + ReLU (MinkConvBNRelu, Swin3D/modules/mink_layers.py:50-80).  The
    parameters carry the reference's checkpoint names: `conv_layers.0.kernel` and `conv_layers.1.bn.*`.  The
    27 kernel offsets are ordered x-major here; which order MinkowskiEngine uses for its kernel rows is not
    pinned by anything available offline, so a stem loaded from a published checkpoint is parity unpinned."""

    def __init__(self, in_channels, out_channels):
        super().__init__()
        self.conv_layers = nn.Sequential(_ConvKernel(in_channels, out_channels), _BatchNorm(out_channels))

    @property
    def weight(self):
        return self.conv_layers[0].kernel

    def forward(self, voxels, neighbours=None):
        out = sparse_conv3x3x3(voxels, self.weight, neighbours)
        return voxels.with_feats(F.relu(self.conv_layers[1](out.float())))


# Inference-time copies of parameters (autocast-dtype weights, scaled projections, flat tables) are kept on their
# layers and checked against the parameters' addresses and version counters.  An update through `param.data` (EMA
# helpers, some optimizer and init code) changes values without touching the version counter, so every copy also
# carries the number of forward passes with autograd enabled that the process had seen when it was made: any
# training forward in between renews it.  What this does not catch is a `.data` update with no grad-enabled forward
# between two inference passes; call `drop_inference_copies(model)` after such an update.
_GRAD_FORWARDS = [0]


def _cache_epoch():
    if torch.is_grad_enabled():
        _GRAD_FORWARDS[0] += 1
    return _GRAD_FORWARDS[0]


def drop_inference_copies(model):
    """Forget the inference-time copies of parameters that the layers of `model` keep (see above)."""
    for m in model.modules():
        if hasattr(m, "_s3d_cast"):
            del m._s3d_cast
        if isinstance(m, WindowAttention):
            m._cache = None


def _linear(layer, x):
    """layer(x) for an nn.Linear.  Inference under autocast keeps the parameters' copies in the autocast dtype on
    the layer (per parameter version) instead of casting them in every forward: autocast's own cache lives only as
    long as its context, and the encoder has about seventy such layers."""
    epoch = _cache_epoch()
    if torch.is_grad_enabled() or not torch.is_autocast_enabled() or not x.is_cuda:
        return layer(x)
    dtype = torch.get_autocast_dtype("cuda")
    w, b = layer.weight, layer.bias
    key = (epoch, dtype, w.data_ptr(), w._version, None if b is None else (b.data_ptr(), b._version))
    kept = getattr(layer, "_s3d_cast", None)
    if kept is None or kept[0] != key:
        kept = (key, w.detach().to(dtype), None if b is None else b.detach().to(dtype))
        layer._s3d_cast = kept
    return F.linear(x, kept[1], kept[2])


class Mlp(nn.Module):
    """fc1 -> GELU -> fc2 with the reference's attribute names (Swin3D/modules/swin3d_layers.py:153-176);
    dropout is 0 in every shipped configuration and left out."""

    def __init__(self, in_features, hidden_features):
        super().__init__()
        self.fc1 = nn.Linear(in_features, hidden_features)
        self.act = nn.GELU()
        self.fc2 = nn.Linear(hidden_features, in_features)

    def forward(self, x):
        return _linear(self.fc2, self.act(_linear(self.fc1, x)))


def _fused_norm_applies(feats):
    """Inference under fp16 autocast on an fp32 residual stream: the fused add + LayerNorm kernel can stand in for
    torch's LayerNorm (it has no autograd)."""
    return (not torch.is_grad_enabled() and feats.is_cuda and feats.dtype == torch.float32
            and torch.is_autocast_enabled() and torch.get_autocast_dtype("cuda") == torch.float16
            and feats.shape[1] % 4 == 0 and feats.shape[1] <= 1024)


class GridKNNDownsample(nn.Module):
    """Coarse voxel = stride-2 cell; its feature = max over the K=16 nearest fine points of
    Linear(LayerNorm(feature)); its coordinate signals = those of the picked representative."""

    def __init__(self, in_channels, out_channels, stride=2, k=16):
        super().__init__()
        self.factor, self.k = stride, k
        self.norm = nn.LayerNorm(in_channels)
        self.linear = nn.Linear(in_channels, out_channels, bias=False)

    def plan(self, coords, stride, signals, num_batches=None, cell_index=None):
        """The part that depends on coordinates and signals only: (coarse coordinates, coarse signals, the K
        nearest fine rows of every coarse voxel).  cell_index: the window index at window = stride factor, when
        the caller built it along with its own."""
        coarse, pick = pool_and_pick(coords, stride, self.factor, signals, cell_index)
        coarse_signals = signals[pick]
        src_xyz = signals[:, 1:4].contiguous().float()
        qry_xyz = coarse_signals[:, 1:4].contiguous().float()
        idx, _ = KNN.apply(self.k, src_xyz, qry_xyz, segment_offsets(coords[:, 0], num_batches),
                           segment_offsets(coarse[:, 0], num_batches))
        return coarse, coarse_signals, idx

    def forward(self, voxels, signals, plan=None, pending=None):
        """pending: a term still to be added to voxels.feats (the last block's MLP output on the fused inference
        path): the add runs inside the LayerNorm kernel and voxels.feats is updated in place.  Returns (coarse
        voxels, coarse signals)."""
        coarse, coarse_signals, idx = plan if plan is not None else self.plan(voxels.coords, voxels.stride, signals)
        # LayerNorm and Linear act on single rows, so they commute with the gather: project the Ns fine rows once
        # instead of the K * Nq gathered copies (the reference statement, swin3d_layers.py:292-312, gathers first)
        if _fused_norm_applies(voxels.feats):
            _, normed = add_layernorm(voxels.feats, pending, self.norm, inplace=True)
        else:
            if pending is not None:
                voxels.feats += pending
            normed = self.norm(voxels.feats)
        projected = _linear(self.linear, normed)
        if not torch.is_grad_enabled() and projected.is_cuda and projected.dtype in (torch.float16, torch.float32):
            feats = knn_max_pool(idx, projected)      # one kernel, no [Nq, K, C] intermediate
        else:
            rows = idx.view(-1).long().clamp_(min=0)
            feats = projected[rows].view(coarse.shape[0], self.k, projected.shape[1]).amax(dim=1)
        return SparseVoxels(coarse, feats.float(), voxels.stride * self.factor), coarse_signals


class WindowAttention(nn.Module):
    """Window multi-head self-attention with cRSE tables on the fused HIP operator."""

    def __init__(self, dim, window_size, quant_size, num_heads, cRSE="XYZ_RGB", fp16_mode=0):
        super().__init__()
        self.dim, self.num_heads, self.window_size, self.quant_size = dim, num_heads, window_size, quant_size
        self.head_dim = dim // num_heads
        self.scale = self.head_dim ** -0.5
        self.cRSE, self.fp16_mode = cRSE, fp16_mode
        self.table_sizes = crse_table_sizes(window_size, quant_size, num_heads, self.head_dim, cRSE)
        rows = [sz // dim for sz in self.table_sizes]
        for kind in ("query", "key", "value"):
            for group, name in enumerate(("xyz", "rgb", "norm")[: crse_num_axes(cRSE) // 3]):
                table = nn.Parameter(torch.zeros(3, rows[3 * group], num_heads, self.head_dim))
                nn.init.trunc_normal_(table, std=0.02)
                setattr(self, f"{kind}_{name}_table", table)
        self.qkv = nn.Linear(dim, dim * 3)
        self.proj = nn.Linear(dim, dim)
        self._cache = None   # inference-time copies of the scaled projection and the flat tables

    def _flat_table(self, kind):
        names = ("xyz", "rgb", "norm")[: crse_num_axes(self.cRSE) // 3]
        return torch.cat([getattr(self, f"{kind}_{n}_table").reshape(-1) for n in names])

    def _prepared(self):
        """(qkv weight with the q scale folded in, its bias, the three flat tables).  Without autograd (inference)
        they are built once per parameter version, in the autocast dtype when autocast is on, instead of on every
        call: the scaling, three concatenations and the casts are a dozen small kernels per block otherwise."""
        caching = not torch.is_grad_enabled()
        dtype = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled() else self.qkv.weight.dtype
        names = ("xyz", "rgb", "norm")[: crse_num_axes(self.cRSE) // 3]
        params = [self.qkv.weight, self.qkv.bias] + [getattr(self, f"{k}_{n}_table") for k in ("query", "key", "value")
                                                     for n in names]
        key = (_cache_epoch(), dtype) + tuple((p.data_ptr(), p._version) for p in params if p is not None)
        if caching and self._cache is not None and self._cache[0] == key:
            return self._cache[1]
        # q scale folded into the projection (a C x C multiply instead of an N x C one)
        scale = torch.ones(3 * self.dim, dtype=self.qkv.weight.dtype, device=self.qkv.weight.device)
        scale[: self.dim] = self.scale
        weight = self.qkv.weight * scale.unsqueeze(1)
        bias = None if self.qkv.bias is None else self.qkv.bias * scale
        tables = [self._flat_table(kind) for kind in ("query", "key", "value")]
        if caching:
            weight, tables = weight.to(dtype), [t.to(dtype) for t in tables]
            bias = None if bias is None else bias.to(dtype)
            self._cache = (key, (weight, bias, tables))
        return weight, bias, tables

    def forward(self, feats, attn_args):
        n = feats.shape[0]
        _, _, m2w, w_sizes, w2n, n2n, w2m, n_coords = attn_args[:8]
        weight, bias, tables = self._prepared()
        # q, k, v stay slices of the [N, 3C] projection output, which the attention kernels read in place
        qkv = F.linear(feats, weight, bias).view(n, 3, self.num_heads, self.head_dim)
        query, key, value = qkv[:, 0], qkv[:, 1], qkv[:, 2]
        # the scaled signals of the index set, when the caller prepared them once for all blocks that share it
        n_crse = attn_args[8] if len(attn_args) > 8 else scale_crse_coords(n_coords, self.quant_size, self.cRSE)
        precision = (PrecisionMode.HALF_NONE, PrecisionMode.HALF_FORWARD, PrecisionMode.HALF_ALL)[self.fp16_mode]
        out = SelfAttnAIOFunction.apply(
            query, key, value, *tables, self.table_sizes, [m2w, w_sizes, w2m, w2n, n2n, n_crse], PosEmb.SEPARATE,
            TableDims.D0, IndexMode.INDIRECT, precision)
        out = out.reshape(n, self.dim)
        return _linear(self.proj, out if torch.is_autocast_enabled() else out.to(feats.dtype))


class SwinBlock(nn.Module):
    def __init__(self, dim, num_heads, window_size, quant_size, mlp_ratio=4.0, cRSE="XYZ_RGB", fp16_mode=0):
        super().__init__()
        self.norm1 = nn.LayerNorm(dim)
        self.attn = WindowAttention(dim, window_size, quant_size, num_heads, cRSE, fp16_mode)
        self.norm2 = nn.LayerNorm(dim)
        hidden = int(dim * mlp_ratio)
        self.mlp = Mlp(dim, hidden)

    def forward(self, feats, attn_args):
        if self._fused_path(feats):
            feats, pending = self.forward_fused(feats, None, attn_args)
            return feats + pending
        feats = feats + self.attn(self.norm1(feats), attn_args)      # fp32 + fp16 promotes to fp32
        return feats + self.mlp(self.norm2(feats))

    def forward_fused(self, feats, pending, attn_args):
        """Inference under fp16 autocast: (feats, pending) stands for the residual stream feats + pending, where
        pending is the previous block's MLP output (or None).  The residual adds and LayerNorms run as fused
        kernels that write the normalised rows in fp16, the dtype the following GEMM reads; the block's own MLP
        output is handed on as the new pending term instead of being added here."""
        feats, normed = add_layernorm(feats, pending, self.norm1)
        feats, normed = add_layernorm(feats, self.attn(normed, attn_args), self.norm2, inplace=pending is not None)
        return feats, self.mlp(normed)

    def _fused_path(self, feats):
        return _fused_norm_applies(feats)


class Stage(nn.Module):
    """`depth` Swin blocks on one resolution (regular / shifted windows alternate), then an
    optional KNN downsample."""

    def __init__(self, dim, depth, num_heads, window_size, quant_size, out_channels=None, down_stride=2,
                 downsample=True, cRSE="XYZ_RGB", fp16_mode=0):
        super().__init__()
        self.window_size = window_size
        self.blocks = nn.ModuleList(
            [SwinBlock(dim, num_heads, window_size, quant_size, cRSE=cRSE, fp16_mode=fp16_mode) for _ in range(depth)])
        self.downsample = GridKNNDownsample(dim, out_channels or dim * 2, stride=down_stride) if downsample else None

    def plan(self, coords, stride, signals, num_batches=None, rows_in_window_order=False):
        """Everything of the stage that depends on coordinates and signals only: the two window index sets
        (regular and shifted windows) with their scaled signals, and the downsample's geometry.  This is where
        the host waits for the device (window counts, unique cells); `forward` with a plan does not.

        rows_in_window_order: the caller has put the rows into the order of this stage's regular windows (the
        window sort's n2n applied to coordinates, signals and features alike).  The row map of the regular set is
        then the identity and is handed to the attention op as None: its kernels read and write the rows in place,
        without the indirection."""
        local = (signals[:, 1:4].float() - coords[:, 1:].float()) / stride
        extra = signals[:, 4:].float()
        # both window sets (one, for a single block) are enqueued before the host waits for their window counts
        shifts = list((0, self.window_size // 2)[:max(1, min(2, len(self.blocks)))])
        pooled = self.downsample is not None and coords.is_cuda and 1 <= self.downsample.factor <= 10
        if pooled:
            shifts.append((self.downsample.factor, 0))      # the downsample's cells: the same host wait
        indices = build_window_indices(coords, stride, self.window_size, shifts)
        cell_index = indices.pop() if pooled else None
        args = [index_arguments(index, local, extra) for index in indices]
        if rows_in_window_order and args:
            args[0] = args[0][:5] + (None,) + args[0][6:]      # (.., w2n, n2n, w2m, ..): no row map
        if len(self.blocks) > 0:
            # the quantiser scaling of the signals is the same for every block of the stage: once per index set,
            # fused with the gather into window order
            attn = self.blocks[0].attn
            args = [tuple(a) + (window_signals(index, local, extra, crse_num_axes(attn.cRSE) - 3, attn.quant_size,
                                               2 * attn.quant_size),) for a, index in zip(args, indices)]
        down = (self.downsample.plan(coords, stride, signals, num_batches, cell_index)
                if self.downsample is not None else None)
        return args, down

    def forward(self, voxels, signals, plan=None):
        """signals [N, 4|7|10] float = (batch, xyz in voxel units, rgb, normal) of the point kept
        in every voxel.  Returns (features at this resolution, next voxels, next signals)."""
        args, down_plan = plan if plan is not None else self.plan(voxels.coords, voxels.stride, signals)
        feats = voxels.feats
        pending = None
        if len(self.blocks) > 0 and self.blocks[0]._fused_path(feats):
            for i, block in enumerate(self.blocks):
                feats, pending = block.forward_fused(feats, pending, args[i % len(args)])
            if self.downsample is None or not feats.is_contiguous():
                feats, pending = feats + pending, None
            # else: the downsample's LayerNorm kernel adds the last MLP output, in place
        else:
            for i, block in enumerate(self.blocks):
                feats = block(feats, args[i % len(args)])
        voxels = voxels.with_feats(feats)
        if self.downsample is None:
            return voxels, voxels, signals
        down, down_signals = self.downsample(voxels, signals, down_plan, pending)
        return voxels, down, down_signals


def window_order(coords, stride, window_size):
    """long [N]: the rows of `coords` in the order of the regular windows of `window_size` voxels (the n2n of the
    window sort), without waiting for the device; None where the window sort does not apply (CPU tensors)."""
    if not coords.is_cuda or not 1 <= window_size <= 10 or coords.shape[0] == 0:
        return None
    n = coords.shape[0]
    dev = coords.device
    coords = coords.to(torch.int32).contiguous()
    n2n, wwid, w_sizes, w2n = (torch.empty(n, dtype=torch.int32, device=dev) for _ in range(4))
    counts = torch.empty(4, dtype=torch.int64, device=dev)
    lib = _lib.lib()
    with torch.cuda.device(dev):
        ws_bytes = lib.s3d_window_index_workspace_bytes(n)
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        status = lib.s3d_window_index(coords.data_ptr(), n, int(stride), int(window_size), 0, n2n.data_ptr(),
                                      wwid.data_ptr(), w_sizes.data_ptr(), w2n.data_ptr(), counts.data_ptr(),
                                      workspace.data_ptr(), ws_bytes, torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(status, "s3d_window_index")
    return n2n.long()      # coordinates out of the sort's range are reported by the stage's own index build


def geometry_steps(stem_coords, stride, signals, layers, window_ordered=False):
    """Generator over the geometry of a forward pass, in the order the feature pass needs it: with window_ordered
    the permutation of the input rows (or None), then the stem convolution's neighbour rows, then the plan of every
    stage (finest first).  None of it depends on features.

    window_ordered: the voxels of every level are put into the order of that level's regular windows (each
    window's voxels contiguous) before anything else is derived from them: the window index of the regular blocks
    is then the identity and that of the shifted blocks a near-local permutation, so the attention kernels read
    the rows of a window from neighbouring memory instead of through a scattered gather."""
    coords = stem_coords
    ordered = False      # the current level's rows are in the order of its regular windows
    if window_ordered:
        order = window_order(coords, stride, layers[0].window_size) if len(layers) else None
        if order is not None:
            coords, signals = coords[order], signals[order]
            ordered = True
        yield order, coords, signals
    yield conv3x3x3_neighbours(coords, stride)
    num_batches = int(coords[-1, 0]) + 1 if coords.shape[0] else 0    # batch ids are ascending: one read
    for level, layer in enumerate(layers):
        plan = layer.plan(coords, stride, signals, num_batches, rows_in_window_order=ordered)
        ordered = False
        if plan[1] is not None:
            coarse, coarse_signals, idx = plan[1]
            coarse_stride = stride * layer.downsample.factor
            if window_ordered and level + 1 < len(layers):
                order = window_order(coarse, coarse_stride, layers[level + 1].window_size)
                if order is not None:
                    coarse, coarse_signals, idx = coarse[order], coarse_signals[order], idx[order]
                    plan = (plan[0], (coarse, coarse_signals, idx))
                    ordered = True
        yield plan
        if plan[1] is not None:
            coords, signals = plan[1][0], plan[1][1]
            stride = stride * layer.downsample.factor


def plan_stages(stem_coords, stride, signals, layers):
    """(stem neighbours, [stage plans]) computed up front on the current stream."""
    steps = list(geometry_steps(stem_coords, stride, signals, layers))
    return steps[0], steps[1:]


def plan_stages_window_ordered(voxels, signals, layers):
    """As plan_stages, with every level in the order of its regular windows: -> (input voxels and signals in
    that order, the permutation applied to the input rows (long [N], or None), stem neighbours, [stage plans])."""
    steps = list(geometry_steps(voxels.coords, voxels.stride, signals, layers, window_ordered=True))
    order, coords, signals = steps[0]
    if order is not None:
        voxels = SparseVoxels(coords, voxels.feats[order], voxels.stride)
    return voxels, signals, order, steps[1], steps[2:]


class Swin3DEncoder(nn.Module):
    """stem -> `num_layers` stages; returns the per-stage SparseVoxels (finest first)."""

    def __init__(self, depths, channels, num_heads, window_sizes, quant_size, num_layers=5, first_down_stride=2,
                 in_channels=6, cRSE="XYZ_RGB", fp16_mode=0, window_ordered=False):
        super().__init__()
        # window_ordered: every level's voxels are kept in the order of its regular windows (geometry_steps); the
        # returned SparseVoxels are in that order (they carry their coordinates), `last_input_order` maps the rows
        # of the finest level back to the input rows.  Off by default: the attention kernels read q, k, v in place
        # from the [N, 3C] projection output, where every (row, head) slice is a cache line of its own whatever the
        # row order, and the extra sort and gathers per level cost what the ordering saves (Swin3D-L, 2 x 300k
        # voxels: 32.7 ms against 32.0 ms).  With dense [N, H, D] operands the ordering is worth 10 % of a call.
        self.window_ordered = window_ordered
        self.last_input_order = None
        self.stem_layer = StemConv(in_channels, channels[0])
        self.layers = nn.ModuleList([
            Stage(channels[i], depths[i], num_heads[i], window_sizes[i], quant_size,
                  out_channels=channels[i + 1] if i < num_layers - 1 else None,
                  down_stride=first_down_stride if i == 0 else 2, downsample=i < num_layers - 1,
                  cRSE=cRSE, fp16_mode=fp16_mode)
            for i in range(num_layers)])
        for m in self.modules():
            if isinstance(m, nn.Linear):
                nn.init.trunc_normal_(m.weight, std=0.02)
                if m.bias is not None:
                    nn.init.zeros_(m.bias)

    def forward(self, voxels, signals):
        # geometry first (it needs no features, and it is where the host waits for the device), then the
        # feature pass in one uninterrupted run of launches
        if self.window_ordered:
            voxels, signals, self.last_input_order, neighbours, plans = plan_stages_window_ordered(voxels, signals,
                                                                                                   self.layers)
        else:
            neighbours, plans = plan_stages(voxels.coords, voxels.stride, signals, self.layers)
            self.last_input_order = None
        voxels = self.stem_layer(voxels, neighbours)
        outputs = []
        for layer, plan in zip(self.layers, plans):
            here, voxels, signals = layer(voxels, signals, plan)
            outputs.append(here)
        return outputs


def query_knn_feature(K, src_xyz, query_xyz, src_feat, src_offset, query_offset, return_idx=False):
    """Features of the K nearest sources of every query, [Nq,K,C] (swin3d_layers.py:27-50).  Slots
    of segments with fewer than K sources repeat source row 0 of the gather (index clamped)."""
    if query_xyz is None:
        query_xyz, query_offset = src_xyz, src_offset
    idx, _ = KNN.apply(K, src_xyz, query_xyz, src_offset, query_offset)
    grouped = src_feat[idx.view(-1).long().clamp_(min=0)].view(query_xyz.shape[0], K, src_feat.shape[1])
    return (grouped, idx) if return_idx else grouped


def knn_linear_interpolation(src_xyz, query_xyz, src_feat, src_offset, query_offset, K=3):
    """Inverse-distance interpolation of src_feat at the queries (swin3d_layers.py:53-73): one KNN
    call and one fused gather kernel; differentiable w.r.t. src_feat."""
    idx, dist2 = knn_query(K, src_xyz.contiguous(), query_xyz.contiguous(), src_offset, query_offset, KNN.cell_size)
    return KNNInterpolate.apply(idx, dist2, src_feat.contiguous())


class Upsample(nn.Module):
    """Coarse features interpolated onto the finer voxel set and added to its projected skip features,
    optionally followed by one attention block (swin3d_layers.py:318-379)."""

    def __init__(self, in_channels, out_channels, num_heads, window_size, quant_size, attn=True, up_k=3,
                 cRSE="XYZ_RGB", fp16_mode=0):
        super().__init__()
        self.linear1 = nn.Sequential(nn.LayerNorm(out_channels), nn.Linear(out_channels, out_channels))
        self.linear2 = nn.Sequential(nn.LayerNorm(in_channels), nn.Linear(in_channels, out_channels))
        self.up_k = up_k
        self.attn = attn and window_size > 0
        if self.attn:
            self.block = Stage(out_channels, 1, num_heads, window_size, quant_size, downsample=False, cRSE=cRSE,
                               fp16_mode=fp16_mode)

    @staticmethod
    def _norm_linear(block, feats):
        """LayerNorm + Linear; for inference under fp16 autocast the norm is the fused kernel that writes fp16."""
        if _fused_norm_applies(feats):
            _, normed = add_layernorm(feats, None, block[0])
            return block[1](normed)
        return block(feats)

    def forward(self, voxels, signals, voxels_up, signals_up, plan_up=None):
        """(voxels, signals): the coarse level; (voxels_up, signals_up): the finer level it feeds.  plan_up: a
        stage plan of the finer level's voxel set with the same window size (the encoder's, whose regular window
        set is the one this level's attention block needs), so that the index is not built a second time."""
        xyz = signals[:, 1:4].detach().contiguous().float()
        support_xyz = signals_up[:, 1:4].detach().contiguous().float()
        feats = self._norm_linear(self.linear1, voxels_up.feats) + knn_linear_interpolation(
            xyz, support_xyz, self._norm_linear(self.linear2, voxels.feats).float(),
            segment_offsets(voxels.coords[:, 0]), segment_offsets(voxels_up.coords[:, 0]), K=self.up_k)
        voxels_up = voxels_up.with_feats(feats.float())
        if self.attn:
            if plan_up is not None:
                plan_up = (plan_up[0][:1], None)      # the regular window set; nothing to downsample here
            voxels_up, _, _ = self.block(voxels_up, signals_up, plan_up)
        return voxels_up


def load_state_with_same_shape(model, weights, skip_first_conv=False, verbose=True):
    """The subset of a checkpoint's state dict that this model can take (Swin3D/models/Swin3D.py:12-40):
    a `module.` prefix is stripped, decoder (`upsamples`) and `classifier` entries are dropped, so is
    `stem_layer` on request, and so is every entry whose name or shape the model does not have."""
    if weights and next(iter(weights)).startswith("module."):
        weights = {k.partition("module.")[2]: v for k, v in weights.items()}
    model_state = model.state_dict()
    wanted = {k: v for k, v in weights.items()
              if "upsamples" not in k and "classifier" not in k and not (skip_first_conv and "stem_layer" in k)}
    filtered = {k: v for k, v in wanted.items() if k in model_state and v.size() == model_state[k].size()}
    if verbose:
        print("checkpoint entries left out:", ", ".join(sorted(set(weights) - set(filtered))) or "none")
        print("model entries without a checkpoint value:", ", ".join(k for k in model_state if k not in filtered) or "none")
    return filtered


def unmatched_encoder_parameters(model, matched):
    """Parameters and buffers of the encoder stages (`layers.*`) that a filtered checkpoint leaves at their
    initial values; `num_batches_tracked` counters aside."""
    return [k for k in model.state_dict()
            if k.startswith("layers.") and k not in matched and not k.endswith("num_batches_tracked")]


class Swin3DUNet(nn.Module):
    """Encoder stages, the Upsample decoder and the per-voxel classifier (Swin3D/models/Swin3D.py:42-183,
    stem_transformer=True layout)."""

    def __init__(self, depths, channels, num_heads, window_sizes, quant_size, up_k=3, num_layers=5, num_classes=13,
                 first_down_stride=2, upsample="linear", in_channels=6, cRSE="XYZ_RGB", fp16_mode=0,
                 window_ordered=False):
        super().__init__()
        self.window_ordered = window_ordered      # as in Swin3DEncoder; the logits come back in input order
        self.stem_layer = StemConv(in_channels, channels[0])
        self.layers = nn.ModuleList([
            Stage(channels[i], depths[i], num_heads[i], window_sizes[i], quant_size,
                  out_channels=channels[i + 1] if i < num_layers - 1 else None,
                  down_stride=first_down_stride if i == 0 else 2, downsample=i < num_layers - 1,
                  cRSE=cRSE, fp16_mode=fp16_mode)
            for i in range(num_layers)])
        self.upsamples = nn.ModuleList([
            Upsample(channels[i], channels[i - 1], num_heads[i - 1], window_sizes[i - 1], quant_size,
                     attn="attn" in upsample, up_k=up_k, cRSE=cRSE, fp16_mode=fp16_mode)
            for i in range(num_layers - 1, 0, -1)])
        self.classifier = nn.Sequential(nn.Linear(channels[0], channels[0]), nn.BatchNorm1d(channels[0]),
                                        nn.ReLU(inplace=True), nn.Linear(channels[0], num_classes))
        self.num_classes = num_classes
        for m in self.modules():
            if isinstance(m, nn.Linear):
                nn.init.trunc_normal_(m.weight, std=0.02)
                if m.bias is not None:
                    nn.init.zeros_(m.bias)

    def forward(self, voxels, signals):
        """-> logits [N, num_classes] on the input voxels."""
        order = None
        if self.window_ordered:
            voxels, signals, order, neighbours, plans = plan_stages_window_ordered(voxels, signals, self.layers)
        else:
            neighbours, plans = plan_stages(voxels.coords, voxels.stride, signals, self.layers)
        voxels = self.stem_layer(voxels, neighbours)
        levels = []
        for layer, plan in zip(self.layers, plans):
            here, voxels_next, signals_next = layer(voxels, signals, plan)
            levels.append((here, signals))
            voxels, signals = voxels_next, signals_next
        voxels, signals = levels.pop()
        for level, upsample in zip(range(len(levels) - 1, -1, -1), self.upsamples):
            voxels_up, signals_up = levels.pop()
            # the decoder level works on the encoder level's voxels with the same window size: same window index
            voxels = upsample(voxels, signals, voxels_up, signals_up, plans[level])
            signals = signals_up
        logits = self.classifier(voxels.feats.float())
        if order is None:
            return logits
        back = torch.empty_like(logits)
        back[order] = logits          # row p of the window order is input row order[p]
        return back

    def load_pretrained_model(self, ckpt, skip_first_conv=True, verbose=True, strict_encoder=True):
        """Load the entries of a checkpoint that fit (Swin3D/models/Swin3D.py:173-183); the file is read
        with a loader that executes nothing from it.  The reference loads with strict=False and says nothing
        about stages that got no weights; here, with strict_encoder, a checkpoint that leaves any parameter
        of the encoder stages (`layers.*`) without a value raises instead of leaving it at random."""
        import os
        if not os.path.isfile(ckpt):
            if verbose:
                print("=> no weight found at '{}'".format(ckpt))
            return []
        checkpoint = torch.load(ckpt, map_location="cpu", weights_only=True)
        weights = checkpoint["state_dict"] if "state_dict" in checkpoint else checkpoint
        matched = load_state_with_same_shape(self, weights, skip_first_conv=skip_first_conv, verbose=verbose)
        left = unmatched_encoder_parameters(self, matched)
        if strict_encoder and left:
            raise RuntimeError(f"checkpoint '{ckpt}' has no fitting value for {len(left)} encoder entries: "
                               + ", ".join(left[:8]) + (" ..." if len(left) > 8 else ""))
        self.load_state_dict(matched, strict=False)
        if verbose:
            print("=> loaded weight '{}'".format(ckpt))
        return sorted(matched)


SWIN3D_S = dict(depths=[2, 4, 9, 4, 4], channels=[48, 96, 192, 384, 384], num_heads=[6, 6, 12, 24, 24],
                window_sizes=[5, 7, 7, 7, 7], quant_size=4)
SWIN3D_L = dict(depths=[2, 4, 9, 4, 4], channels=[80, 160, 320, 640, 640], num_heads=[10, 10, 20, 40, 40],
                window_sizes=[5, 7, 7, 7, 7], quant_size=4)
