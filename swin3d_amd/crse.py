"""Argument preparation of the window-attention op (contextual relative signal encoding).

Host-side mirror of the table/coordinate conventions of WindowAttention
(Swin3D/modules/swin3d_layers.py:431-467 table shapes, :511-541 per-call prep):
  * one table per signal axis, axes ordered x, y, z, r, g, b, nx, ny, nz;
  * xyz tables have 2 * window_size * quant_size rows, colour and normal tables
    2 * 2 * (2 * quant_size) rows (signals span [-1, 1], finer quantisation);
  * each table is stored [row][head][channel]; the op receives the per-axis
    element counts rows * H * D (the reference calls them `table_offsets`);
  * the per-voxel signals are scaled by quant_size (xyz) and 2 * quant_size
    (colour, normal) before the op subtracts and truncates them.
"""
import torch

CRSE_MODES = ("XYZ", "XYZ_RGB", "XYZ_RGB_NORM")


def crse_num_axes(cRSE):
    if cRSE not in CRSE_MODES:
        raise ValueError(f"cRSE must be one of {CRSE_MODES}, got {cRSE!r}")
    return 3 * (1 + ("RGB" in cRSE) + ("NORM" in cRSE))


def crse_table_rows(window_size, quant_size, cRSE="XYZ_RGB"):
    """Rows of each per-axis table, in axis order."""
    crse_num_axes(cRSE)
    rows = [2 * window_size * quant_size] * 3
    signal_rows = 2 * 2 * (2 * quant_size)
    if "RGB" in cRSE:
        rows += [signal_rows] * 3
    if "NORM" in cRSE:
        rows += [signal_rows] * 3
    return rows


def crse_table_sizes(window_size, quant_size, num_heads, head_dim, cRSE="XYZ_RGB"):
    """Per-axis element counts rows * H * D (what the op takes as `table_offsets`)."""
    return [r * num_heads * head_dim for r in crse_table_rows(window_size, quant_size, cRSE)]


def scale_crse_coords(n_coords, quant_size, cRSE="XYZ_RGB"):
    """n_coords [N, 3|6|9] (window-local xyz, rgb, normal) -> scaled fp32 signals of the op."""
    nd = crse_num_axes(cRSE)
    if n_coords.shape[1] < nd:
        raise ValueError(f"cRSE={cRSE} needs {nd} signal columns, got {n_coords.shape[1]}")
    scale = torch.empty(nd, dtype=torch.float32, device=n_coords.device)
    scale[:3] = quant_size
    scale[3:] = 2 * quant_size
    return (n_coords[:, :nd].to(torch.float32) * scale).contiguous()
