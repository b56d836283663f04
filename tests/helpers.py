"""Shared builders of small attention / KNN problems for the tests (numpy only)."""
import numpy as np

from swin3d_amd import crse, synth


class AttnCase:
    """All arguments of the attention op as numpy arrays (float32 unless stated)."""

    def __init__(self, coords, stride, ws, quant, heads, dim, cRSE, index, n_coords, q, k, v,
                 tables, table_sizes):
        self.coords, self.stride, self.ws, self.quant = coords, stride, ws, quant
        self.H, self.D, self.cRSE = heads, dim, cRSE
        self.index = index                      # dict from oracle.window_index
        self.n_coords = n_coords                # [N,nd] fp32, sorted order, quant-scaled
        self.q, self.k, self.v = q, k, v
        self.tq, self.tk, self.tv = tables
        self.table_sizes = np.asarray(table_sizes, np.int32)

    @property
    def N(self):
        return self.q.shape[0]

    def oracle_args(self):
        i = self.index
        return (self.q, self.k, self.v, self.tq, self.tk, self.tv, self.table_sizes,
                i["w_sizes"], i["w2n"], i["n2n"], self.n_coords)

    def axis_tables(self, flat):
        """flat table -> list of [rows_n,H,D] arrays (one per axis)."""
        out, off = [], 0
        for size in self.table_sizes.tolist():
            out.append(np.asarray(flat[off:off + size]).reshape(-1, self.H, self.D))
            off += size
        return out


def n_coords_from_scene(oracle, coords, frac, sig, stride, ws, quant, cRSE, shift=0):
    """window index + the op's scaled fp32 signal matrix, following
    swin3d_layers.py:800-804 (w_w_xyz + local_xyz, cat colours) and :513-536 (quant scaling)."""
    index = oracle.window_index(coords, stride, ws, shift)
    wid = index["w_w_id"]
    lxyz = np.stack([wid // ws // ws, wid // ws % ws, wid % ws], axis=1).astype(np.float32)
    n2n = index["n2n"]
    xyz = (lxyz + frac[n2n].astype(np.float32)).astype(np.float32)
    cols = [(xyz * np.float32(quant)).astype(np.float32)]
    if sig.shape[1]:
        cols.append((sig[n2n].astype(np.float32) * np.float32(2 * quant)).astype(np.float32))
    return index, np.ascontiguousarray(np.concatenate(cols, axis=1), np.float32)


def make_attn_case(oracle, seed=0, n=120, ws=3, quant=2, heads=2, dim=8, cRSE="XYZ_RGB_NORM",
                   recipe="sharp", stride=1, extent=(4, 4, 2), batches=1, shift=0,
                   signal_range=(-1.0, 1.0)):
    from conftest import random_scene
    rng = np.random.default_rng(seed)
    coords = random_scene(rng, n, extent=extent, batches=batches, stride=stride)
    frac = rng.random((n, 3)).astype(np.float32)
    nsig = crse.crse_num_axes(cRSE) - 3
    sig = rng.uniform(signal_range[0], signal_range[1], size=(n, nsig)).astype(np.float32)
    index, n_coords = n_coords_from_scene(oracle, coords, frac, sig, stride, ws, quant, cRSE, shift)
    sizes = crse.crse_table_sizes(ws, quant, heads, dim, cRSE)
    q, k, v, tables = synth.layer_inputs(n, heads * dim, heads, int(sum(sizes)), seed=seed, recipe=recipe)
    return AttnCase(coords, stride, ws, quant, heads, dim, cRSE, index, n_coords, q, k, v, tables, sizes)


def scene_attn_case(oracle, scene, ws, quant, heads, dim, cRSE, recipe="layer", seed=0, stride=1,
                    shift=0):
    """AttnCase for a synthetic room (swin3d_amd.synth.Scene)."""
    sig = synth.signals(scene, cRSE)
    index, n_coords = n_coords_from_scene(oracle, scene.coords, scene.frac, sig, stride, ws, quant,
                                          cRSE, shift)
    sizes = crse.crse_table_sizes(ws, quant, heads, dim, cRSE)
    q, k, v, tables = synth.layer_inputs(scene.coords.shape[0], heads * dim, heads, int(sum(sizes)),
                                         seed=seed, recipe=recipe)
    return AttnCase(scene.coords, stride, ws, quant, heads, dim, cRSE, index, n_coords, q, k, v,
                    tables, sizes)


def to_half_and_back(case):
    """Round every floating input of the op to fp16 (what the fp16 kernel sees), keep fp32 storage."""
    h = lambda a: a.astype(np.float16).astype(np.float32)
    case.q, case.k, case.v = h(case.q), h(case.k), h(case.v)
    case.tq, case.tk, case.tv = h(case.tq), h(case.tk), h(case.tv)
    return case


def downsampled_stage_case(oracle, scene, levels, ws, quant, heads, dim, cRSE="XYZ_RGB_NORM", shift=0,
                           recipe="sharp", seed=0):
    """AttnCase of an encoder stage below the first: `scene` grid-downsampled by 2, `levels` times (tensor
    stride 2^levels), the kept point's position inside its coarse voxel as the fractional signal."""
    stride = 1
    for _ in range(levels):
        scene, _ = synth.grid_downsample(scene, 2 * stride)
        stride *= 2
    frac = ((scene.xyz - scene.coords[:, 1:]) / np.float32(stride)).astype(np.float32)
    frac = np.clip(frac, 0.0, np.float32(1.0 - 2.0 ** -24))
    sig = synth.signals(scene, cRSE)
    index, n_coords = n_coords_from_scene(oracle, scene.coords, frac, sig, stride, ws, quant, cRSE, shift)
    sizes = crse.crse_table_sizes(ws, quant, heads, dim, cRSE)
    n = scene.coords.shape[0]
    q, k, v, tables = synth.layer_inputs(n, heads * dim, heads, int(sum(sizes)), seed=seed, recipe=recipe)
    return AttnCase(scene.coords, stride, ws, quant, heads, dim, cRSE, index, n_coords, q, k, v, tables, sizes)
