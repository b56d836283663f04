"""Writes the committed fixtures of this directory.

The reference ships no tests, golden vectors or fixtures for this path, so these vectors come from
the brute-force numpy statements in oracle/numpy_ref.py (python dict grouping, per-axis 3-D tables,
explicit softmax, full distance matrices), not from the C oracle and not from the HIP library: both
of those are CHECKED against the files written here (tests/test_golden.py).

    python tests/golden/make_golden.py          # rewrites the three .npz files (deterministic)
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import numpy_ref            # noqa: E402
from swin3d_amd import crse             # noqa: E402


def _distinct_voxels(rng, n, extent, batches=1, stride=1, low=0):
    cells = set()
    while len(cells) < n:
        b = int(rng.integers(batches))
        xyz = tuple(int(v) * stride for v in (rng.integers(low, extent[0]), rng.integers(low, extent[1]),
                                              rng.integers(low, extent[2])))
        cells.add((b,) + xyz)
    return np.asarray(sorted(cells), np.int32)


def _half_exact(a):
    return np.asarray(a, np.float32).astype(np.float16).astype(np.float32)


def attention_fixture():
    """~200 voxels, window 5, quant 4, all nine cRSE axes, H=2, D=8; every floating-point input is
    exactly representable in fp16, so that the same expected output serves fp32 and fp16 runs."""
    rng = np.random.default_rng(2024)
    ws, quant, heads, dim, mode = 5, 4, 2, 8, "XYZ_RGB_NORM"
    coords = _distinct_voxels(rng, 200, (11, 9, 4))
    n = coords.shape[0]
    frac = rng.random((n, 3)).astype(np.float32)
    sig = rng.uniform(-1.0, 1.0, size=(n, 6)).astype(np.float32)
    index = numpy_ref.window_index_bruteforce(coords, 1, ws, 0)
    n2n, wid = index["n2n"], index["w_w_id"]
    # signal matrix of the operator: position inside the window (cell + fraction) times quant, colour and
    # normal times 2*quant (Swin3D/modules/swin3d_layers.py:800-804 and :513-536), sorted order
    cell = np.stack([wid // ws // ws, wid // ws % ws, wid % ws], axis=1).astype(np.float32)
    xyz = (cell + frac[n2n]).astype(np.float32)
    n_coords = np.concatenate([(xyz * np.float32(quant)).astype(np.float32),
                               (sig[n2n] * np.float32(2 * quant)).astype(np.float32)], axis=1)
    n_coords = np.ascontiguousarray(n_coords, np.float32)
    sizes = np.asarray(crse.crse_table_sizes(ws, quant, heads, dim, mode), np.int32)
    q = _half_exact(rng.standard_normal((n, heads, dim)))
    k = _half_exact(rng.standard_normal((n, heads, dim)))
    v = _half_exact(rng.standard_normal((n, heads, dim)) * 0.4)
    tq, tk = (_half_exact(rng.standard_normal(int(sizes.sum())) * 0.5) for _ in range(2))
    tv = _half_exact(rng.standard_normal(int(sizes.sum())) * 0.1)

    def axes(flat):
        out, off = [], 0
        for s in sizes.tolist():
            out.append(flat[off:off + s].reshape(-1, heads, dim))
            off += s
        return out

    out = numpy_ref.attn_fwd_bruteforce(q, k, v, axes(tq), axes(tk), axes(tv), n_coords, n2n, index["w_sizes"])
    np.savez_compressed(os.path.join(HERE, "attn_small.npz"), coords=coords, ws=ws, quant=quant, heads=heads,
                        dim=dim, table_sizes=sizes, q=q, k=k, v=v, tq=tq, tk=tk, tv=tv, n_coords=n_coords,
                        n2n=n2n.astype(np.int32), w_sizes=index["w_sizes"].astype(np.int32),
                        w2n=index["w2n"].astype(np.int32), out=out)


def window_index_fixture():
    """negative coordinates, two batches, tensor stride 2, window 3, shifted by one voxel."""
    rng = np.random.default_rng(2025)
    coords = _distinct_voxels(rng, 400, (9, 8, 7), batches=2, stride=2, low=-6)
    coords = coords[rng.permutation(coords.shape[0])]
    idx = numpy_ref.window_index_bruteforce(coords, 2, 3, 1)
    np.savez_compressed(os.path.join(HERE, "window_index_small.npz"), coords=coords, stride=2, ws=3, shift=1,
                        n2n=idx["n2n"].astype(np.int32), w_w_id=idx["w_w_id"].astype(np.int32),
                        w_sizes=idx["w_sizes"].astype(np.int32), w2n=idx["w2n"].astype(np.int32),
                        W=idx["W"], M=idx["M"])


def knn_fixture():
    """two segments (one with fewer sources than K), lattice sources so that ties occur, K=5."""
    rng = np.random.default_rng(2026)
    lattice = rng.integers(0, 6, size=(260, 3)).astype(np.float32)
    few = rng.random((3, 3)).astype(np.float32) * 4
    src = np.concatenate([lattice, few])
    qry = np.concatenate([rng.integers(0, 6, size=(60, 3)).astype(np.float32) + np.float32(0.5),
                          rng.random((40, 3)).astype(np.float32) * 6,
                          rng.random((7, 3)).astype(np.float32) * 4])
    src_offset = np.asarray([260, 263], np.int32)
    query_offset = np.asarray([100, 107], np.int32)
    idx, d2 = numpy_ref.knn_bruteforce(5, src, qry, src_offset, query_offset)
    np.savez_compressed(os.path.join(HERE, "knn_small.npz"), k=5, src=src, qry=qry, src_offset=src_offset,
                        query_offset=query_offset, idx=idx, d2=d2)


if __name__ == "__main__":
    attention_fixture()
    window_index_fixture()
    knn_fixture()
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
