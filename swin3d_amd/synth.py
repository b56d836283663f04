"""Deterministic synthetic rooms and layer inputs for the benchmark and the parity tests.

A room is a box (floor + 4 walls) with axis-aligned boxes standing on the floor.
Points are sampled area-uniformly on every face, voxelised at `voxel` metres, the
first point of every voxel is kept (its fractional position and the normal of its
face travel with it), colours are uniform random, and the scene is cropped along
x to the requested voxel count.  numpy's PCG64 with a fixed seed makes every
machine generate the same scene.
"""
from dataclasses import dataclass

import numpy as np


@dataclass
class Scene:
    coords: np.ndarray     # int32 [N,4] (batch, x, y, z) voxel coordinates, sorted by (x,y,z)
    frac: np.ndarray       # float32 [N,3] position of the kept point inside its voxel, [0,1)
    rgb: np.ndarray        # float32 [N,3]
    normal: np.ndarray     # float32 [N,3] unit normal of the generating face
    xyz: np.ndarray        # float32 [N,3] point position in voxel units (coords + frac)


def _faces(size, n_boxes, rng):
    """list of (origin[3], edge_u[3], edge_v[3], normal[3]) rectangles in metres."""
    lx, ly, lz = size
    faces = [
        ((0, 0, 0), (lx, 0, 0), (0, ly, 0), (0, 0, 1)),       # floor
        ((0, 0, 0), (0, ly, 0), (0, 0, lz), (1, 0, 0)),       # wall x = 0
        ((lx, 0, 0), (0, ly, 0), (0, 0, lz), (-1, 0, 0)),     # wall x = lx
        ((0, 0, 0), (lx, 0, 0), (0, 0, lz), (0, 1, 0)),       # wall y = 0
        ((0, ly, 0), (lx, 0, 0), (0, 0, lz), (0, -1, 0)),     # wall y = ly
    ]
    for _ in range(n_boxes):
        ex, ey, ez = rng.uniform(0.3, 1.5, size=3)
        ez = min(ez, lz)
        ox = rng.uniform(0.0, lx - ex)
        oy = rng.uniform(0.0, ly - ey)
        faces += [
            ((ox, oy, ez), (ex, 0, 0), (0, ey, 0), (0, 0, 1)),          # top
            ((ox, oy, 0), (0, ey, 0), (0, 0, ez), (-1, 0, 0)),          # x low
            ((ox + ex, oy, 0), (0, ey, 0), (0, 0, ez), (1, 0, 0)),      # x high
            ((ox, oy, 0), (ex, 0, 0), (0, 0, ez), (0, -1, 0)),          # y low
            ((ox, oy + ey, 0), (ex, 0, 0), (0, 0, ez), (0, 1, 0)),      # y high
        ]
    return faces


def make_room(size=(10.0, 8.0, 3.0), n_boxes=30, target_voxels=200_000, seed=0, voxel=0.02,
              points_per_cell=4.0, batch=0, rgb_range=(0.0, 1.0)):
    """Synthetic room cropped to the largest voxel count <= target_voxels."""
    rng = np.random.default_rng(seed)
    pts, nrm = [], []
    density = points_per_cell / (voxel * voxel)
    for origin, eu, ev, normal in _faces(size, n_boxes, rng):
        origin, eu, ev = (np.asarray(a, np.float64) for a in (origin, eu, ev))
        area = np.linalg.norm(eu) * np.linalg.norm(ev)
        count = int(np.ceil(area * density))
        uv = rng.random((count, 2))
        pts.append(origin + uv[:, :1] * eu + uv[:, 1:] * ev)
        nrm.append(np.broadcast_to(np.asarray(normal, np.float32), (count, 3)))
    pts = np.concatenate(pts) / voxel          # voxel units
    nrm = np.concatenate(nrm)
    pts = np.clip(pts, 0.0, None)
    vox = np.floor(pts).astype(np.int64)
    # first point of every voxel
    key = (vox[:, 0] * 1_000_000 + vox[:, 1]) * 1_000_000 + vox[:, 2]
    _, first = np.unique(key, return_index=True)      # sorted by (x,y,z)
    vox, pts, nrm = vox[first], pts[first], nrm[first]
    # crop along x at voxel granularity
    if vox.shape[0] > target_voxels:
        xs = vox[:, 0]                                  # ascending
        cut = xs[target_voxels]                         # voxels with x < cut number <= target
        keep = int(np.searchsorted(xs, cut, side="left"))
        if keep == 0:
            keep = target_voxels
        vox, pts, nrm = vox[:keep], pts[:keep], nrm[:keep]
    n = vox.shape[0]
    frac = (pts - vox).astype(np.float32)
    frac = np.minimum(frac, np.float32(1.0 - 2.0 ** -24))
    rgb = rng.uniform(rgb_range[0], rgb_range[1], size=(n, 3)).astype(np.float32)
    coords = np.concatenate([np.full((n, 1), batch, np.int64), vox], axis=1).astype(np.int32)
    xyz = vox.astype(np.float32) + frac
    return Scene(coords, frac, rgb, np.ascontiguousarray(nrm, np.float32), xyz)


def concat_scenes(scenes):
    """Stack scenes into one batch (batch column = position in the list)."""
    parts = []
    for b, s in enumerate(scenes):
        c = s.coords.copy()
        c[:, 0] = b
        parts.append(c)
    return Scene(np.concatenate(parts), np.concatenate([s.frac for s in scenes]),
                 np.concatenate([s.rgb for s in scenes]), np.concatenate([s.normal for s in scenes]),
                 np.concatenate([s.xyz for s in scenes]))


def grid_downsample(scene, factor=2):
    """Keep the first voxel (sorted order) of every factor^3 cell; coordinates stay in
    fine-voxel units (tensor stride grows by `factor`)."""
    cell = scene.coords[:, 1:] // factor
    key = ((scene.coords[:, 0].astype(np.int64) * 100_000 + cell[:, 0]) * 100_000 + cell[:, 1]) * 100_000 + cell[:, 2]
    _, first = np.unique(key, return_index=True)
    first.sort()
    coords = scene.coords[first].copy()
    coords[:, 1:] = cell[first] * factor
    return Scene(coords, scene.frac[first], scene.rgb[first], scene.normal[first], scene.xyz[first]), first


def signals(scene, cRSE):
    """[N, 0|3|6] colour (+ normal) signal columns selected by the cRSE mode."""
    cols = []
    if "RGB" in cRSE:
        cols.append(scene.rgb)
    if "NORM" in cRSE:
        cols.append(scene.normal)
    if not cols:
        return np.zeros((scene.coords.shape[0], 0), np.float32)
    return np.concatenate(cols, axis=1).astype(np.float32)


def layer_inputs(n, channels, heads, table_len, seed=0, recipe="layer", dtype=np.float32):
    """q, k, v [N,H,D] and the three flat tables.

    recipe "layer": feats ~ N(0,1), qkv = feats @ W^T with W ~ N(0, 0.02), q scaled by
    D^-0.5, tables ~ N(0, 0.02) (what a freshly initialised WindowAttention produces).
    recipe "sharp": q, k, v ~ N(0,1), tables ~ N(0, 0.5): peaky softmax with dominant
    table terms, for parity tests.
    """
    rng = np.random.default_rng(seed + 1000)
    d = channels // heads
    if recipe == "layer":
        feats = rng.standard_normal((n, channels), dtype=np.float32)
        w = (rng.standard_normal((3 * channels, channels), dtype=np.float32) * np.float32(0.02))
        qkv = (feats @ w.T).reshape(n, 3, heads, d)
        q = qkv[:, 0] * np.float32(d ** -0.5)
        k, v = qkv[:, 1], qkv[:, 2]
        tables = [rng.standard_normal(table_len, dtype=np.float32) * np.float32(0.02) for _ in range(3)]
    elif recipe == "sharp":
        q, k, v = (rng.standard_normal((n, heads, d), dtype=np.float32) for _ in range(3))
        tables = [rng.standard_normal(table_len, dtype=np.float32) * np.float32(0.5) for _ in range(3)]
    else:
        raise ValueError(recipe)
    q, k, v = (np.ascontiguousarray(x).astype(dtype) for x in (q, k, v))
    tables = [t.astype(dtype) for t in tables]
    return q, k, v, tables


def encoder_inputs(scene):
    """Model inputs of a Scene in the reference's conventions (Swin3D/models/Swin3D.py:117-129):
    features [N,9] = (rgb, normal, point position inside the voxel), all in [-1,1]-ish ranges, and
    coordinate signals [N,10] = (batch, xyz in voxel units, rgb in [-1,1], normal)."""
    rgb = scene.rgb * np.float32(2.0) - np.float32(1.0)
    feats = np.concatenate([rgb, scene.normal, scene.frac - np.float32(0.5)], axis=1).astype(np.float32)
    signals = np.concatenate([scene.coords[:, :1].astype(np.float32), scene.xyz, rgb, scene.normal],
                             axis=1).astype(np.float32)
    return feats, signals
