"""Window index of the sparse window attention (host side of s3d_window_index).

Mirrors BasicLayer.get_window_mapping / get_index01 / get_shifted_sp
(Swin3D/modules/swin3d_layers.py:740-838) and sparse_self_attention (:76-150) without
MinkowskiEngine: one HIP call sorts the voxels into windows and emits the segment
offsets.  Window order is ascending (batch, wx, wy, wz); the reference's order is
whatever MinkowskiEngine's pooling emits and attention does not depend on it.
"""
from dataclasses import dataclass

import torch

from . import _lib


# s3d_window_index_grid (counting sort over the window lattice) where it applies; False: always the sort of all voxels
USE_GRID_PATH = True


@dataclass
class WindowIndex:
    n2n: torch.Tensor       # int32 [N]  window-sorted position -> original row
    w_w_id: torch.Tensor    # int32 [N]  local id lx*ws^2 + ly*ws + lz per sorted position
    w_sizes: torch.Tensor   # int32 [W]  voxels per window
    w2n: torch.Tensor       # int32 [W]  exclusive prefix sum of w_sizes
    num_windows: int        # W
    num_pairs: int          # M = sum w_sizes^2
    max_window_voxels: int
    window_size: int

    def local_xyz(self):
        """int32 [N,3] voxel position inside its window, window-sorted order."""
        ws = self.window_size
        wid = self.w_w_id
        return torch.stack([wid // (ws * ws), (wid // ws) % ws, wid % ws], dim=-1)

    def inverse(self):
        """int64 [N] original row -> window-sorted position."""
        inv = torch.empty(self.n2n.numel(), dtype=torch.int64, device=self.n2n.device)
        inv[self.n2n.long()] = torch.arange(self.n2n.numel(), device=self.n2n.device)
        return inv


def build_window_indices(coords, stride, window_size, shifts):
    """One WindowIndex per entry of `shifts` (voxels: 0, or window_size // 2 for the shifted window set; an entry
    may also be a pair (window size, shift) for a set with a window size of its own) for coords int32 [N,4]
    (batch,x,y,z) on the GPU.  All index builds are enqueued before the host reads the window counts back, so
    the call synchronises once however many sets it is given."""
    if not coords.is_cuda:
        raise RuntimeError("coords must be a CUDA (HIP) tensor")
    if coords.dim() != 2 or coords.shape[1] != 4:
        raise ValueError(f"coords must be [N,4] (batch,x,y,z), got {tuple(coords.shape)}")
    dev = coords.device
    coords = coords.to(torch.int32).contiguous()
    n = coords.shape[0]
    sets = [s if isinstance(s, (tuple, list)) else (window_size, s) for s in shifts]
    counts = torch.empty((len(sets), 4), dtype=torch.int64, device=dev)
    lib = _lib.lib()
    outputs = []

    def enqueue(i, window, shift, grid):
        fn, size_fn = ((lib.s3d_window_index_grid, lib.s3d_window_index_grid_workspace_bytes) if grid else
                       (lib.s3d_window_index, lib.s3d_window_index_workspace_bytes))
        ws_bytes = size_fn(n)
        n2n, wwid, w_sizes, w2n = (torch.empty(n, dtype=torch.int32, device=dev) for _ in range(4))
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        status = fn(coords.data_ptr(), n, int(stride), int(window), int(shift), n2n.data_ptr(), wwid.data_ptr(),
                    w_sizes.data_ptr(), w2n.data_ptr(), counts[i].data_ptr(), workspace.data_ptr(), ws_bytes,
                    torch.cuda.current_stream(dev).cuda_stream)
        _lib.check(status, fn.__name__)
        return n2n, wwid, w_sizes, w2n

    with torch.cuda.device(dev):
        # the counting sort over the window lattice first; a set whose lattice is too large for it (bit 1 of its
        # status word) is built again by the sort of all voxels, at the price of a second wait
        for i, (window, shift) in enumerate(sets):
            outputs.append(enqueue(i, window, shift, grid=USE_GRID_PATH))
        host_counts = counts.tolist()
        redo = [i for i, c in enumerate(host_counts) if c[3] & 2]
        if redo:
            for i in redo:
                outputs[i] = enqueue(i, sets[i][0], sets[i][1], grid=False)
            host_counts = counts.tolist()
    result = []
    for (n2n, wwid, w_sizes, w2n), (num_w, num_m, max_w, err), (window, _) in zip(outputs, host_counts, sets):
        if err & 1:
            raise ValueError("coords outside the supported range (batch 0..4095, window coordinate "
                             "-8192..8191)")
        sizes = w_sizes[:num_w]
        sizes._s3d_pairs = (sizes._version, int(num_m))   # ... and by its backward (the size of the pair store)
        result.append(WindowIndex(n2n, wwid, sizes, w2n[:num_w], int(num_w), int(num_m), int(max_w), int(window)))
    return result


def build_window_index(coords, stride, window_size, shift=0):
    """coords int32 [N,4] (batch,x,y,z) CUDA tensor -> WindowIndex.

    `shift` is in voxels (0, or window_size // 2 for the shifted window set).
    Synchronises once to read the window count back.
    """
    return build_window_indices(coords, stride, window_size, [shift])[0]


def window_signals(index, local_xyz, colors, num_signals=None, xyz_scale=1.0, other_scale=1.0):
    """fp32 [N, 3 + num_signals] signal matrix of the attention op in window-sorted order, one kernel:
    ((window-local voxel + local_xyz) * xyz_scale, colors[:, :num_signals] * other_scale), rows gathered through
    index.n2n.  Scales 1 give the reference's n_coords (swin3d_layers.py:800-804); quant_size and 2 * quant_size
    give the scaled signals WindowAttention.forward hands to the operator (:513-536)."""
    frac = local_xyz.to(torch.float32).contiguous()
    colors = colors.to(torch.float32)
    if colors.dim() != 2 or (colors.shape[1] > 0 and colors.stride(1) != 1):
        colors = colors.contiguous()
    if num_signals is None:
        num_signals = colors.shape[1]
    if num_signals > colors.shape[1]:
        raise ValueError(f"{num_signals} signal columns asked for, colors has {colors.shape[1]}")
    n = index.n2n.numel()
    if frac.shape != (n, 3) or colors.shape[0] != n:
        raise ValueError(f"local_xyz must be [{n},3] and colors [{n},*], got {tuple(frac.shape)} and "
                         f"{tuple(colors.shape)}")
    out = torch.empty((n, 3 + num_signals), dtype=torch.float32, device=frac.device)
    with torch.cuda.device(frac.device):
        status = _lib.lib().s3d_window_signals(
            index.w_w_id.data_ptr(), index.n2n.data_ptr(), frac.data_ptr(),
            colors.data_ptr() if num_signals > 0 else None, colors.stride(0) if num_signals > 0 else 0,
            int(num_signals), int(index.window_size), float(xyz_scale), float(other_scale), out.data_ptr(), n,
            torch.cuda.current_stream(frac.device).cuda_stream)
    _lib.check(status, "s3d_window_signals")
    return out


def sparse_self_attention(w_w_id, w_sizes, protocol="v1"):
    """O(pairs) pair index of the windows: x_offset / y_offset [M] (sorted positions of the
    query / key of every pair, query-major inside a window) and, for protocol "v2", also
    (m2w_indices [M], w_sizes, w2n_indices [W], w2m_indices [W]).  The fused attention op
    does not read these arrays; they exist for callers that want the reference's layout."""
    del w_w_id  # the pair index depends on the window sizes only
    sizes = w_sizes.long()
    sq = sizes * sizes
    w2n = torch.cumsum(sizes, 0) - sizes
    w2m = torch.cumsum(sq, 0) - sq
    windows = torch.arange(sizes.numel(), device=sizes.device)
    m2w = torch.repeat_interleave(windows, sq)
    within = torch.arange(m2w.numel(), device=sizes.device) - w2m[m2w]
    n_w = sizes[m2w]
    x_offset = w2n[m2w] + torch.div(within, n_w, rounding_mode="floor")
    y_offset = w2n[m2w] + within % n_w
    if protocol == "v1":
        return x_offset, y_offset
    if protocol == "v2":
        return x_offset, y_offset, m2w, w_sizes, w2n, w2m
    raise ValueError(f"unknown protocol {protocol!r}")


def get_index01(coords, stride, window_size, local_xyz, colors, shift=0, materialize_pairs=False):
    """Arguments of the attention op for one window set, in the reference's tuple order
    (x_offset, y_offset, m2w_indices, w_sizes, w2n_indices, n2n_indices, w2m_indices, n_coords).

    local_xyz [N,3] fractional position of the point inside its voxel, colors [N,0|3|6] the
    other signals, both in original row order.  n_coords = (window-local voxel + fraction,
    signals) in window-sorted order, fp32.  The four O(pairs) entries are None unless
    materialize_pairs is set.
    """
    index = build_window_index(coords, stride, window_size, shift)
    return index_arguments(index, local_xyz, colors, materialize_pairs)


def index_arguments(index, local_xyz, colors, materialize_pairs=False):
    """The argument tuple of get_index01 for an index that is already built."""
    n_coords = window_signals(index, local_xyz, colors)
    x_offset = y_offset = m2w = w2m = None
    if materialize_pairs:
        x_offset, y_offset, m2w, _, _, w2m = sparse_self_attention(index.w_w_id, index.w_sizes, "v2")
    return (x_offset, y_offset, m2w, index.w_sizes, index.w2n, index.n2n, w2m, n_coords)
