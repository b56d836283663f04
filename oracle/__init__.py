"""ctypes bindings of the CPU oracle (oracle/s3d_oracle.c) over numpy arrays.

TEST INFRASTRUCTURE ONLY.  Importable from tests/, from the smoke test and from
the CPU-baseline leg of the benchmark; the product package never imports it.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

KNN_PAD_DIST2 = np.float32(2147483648.0)


def build(force=False):
    """Compile oracle/s3d_oracle.c with gcc (see oracle/Makefile)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE, "CC=gcc"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        for name in (
            "s3d_oracle_window_index",
            "s3d_oracle_pair_index",
            "s3d_oracle_crse_rows",
            "s3d_oracle_attn_fwd_f64",
            "s3d_oracle_attn_fwd_f32",
            "s3d_oracle_attn_bwd_f64",
            "s3d_oracle_knn",
            "s3d_oracle_knn_heap",
            "s3d_oracle_knn_interpolate",
            "s3d_oracle_max_threads",
        ):
            getattr(_lib, name).restype = ctypes.c_int
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def max_threads():
    return int(lib().s3d_oracle_max_threads())


def window_index(coords, stride, window_size, shift=0):
    """coords [N,4] int32 (batch,x,y,z) -> dict(n2n, w_w_id, w_sizes, w2n, W, M)."""
    coords = _c(coords, np.int32)
    n = coords.shape[0]
    n2n = np.empty(n, np.int32)
    wwid = np.empty(n, np.int32)
    w_sizes = np.empty(max(n, 1), np.int32)
    w2n = np.empty(max(n, 1), np.int32)
    counts = np.zeros(2, np.int64)
    rc = lib().s3d_oracle_window_index(
        _p(coords), ctypes.c_int64(n), ctypes.c_int32(stride), ctypes.c_int32(window_size),
        ctypes.c_int32(shift), _p(n2n), _p(wwid), _p(w_sizes), _p(w2n), _p(counts))
    if rc != 0:
        raise ValueError(f"s3d_oracle_window_index failed: {rc}")
    w = int(counts[0])
    return dict(n2n=n2n, w_w_id=wwid, w_sizes=w_sizes[:w].copy(), w2n=w2n[:w].copy(),
                W=w, M=int(counts[1]))


def pair_index(w_sizes):
    """-> (w2m[W], m2w[M], x_offset[M], y_offset[M]) as int64."""
    w_sizes = _c(w_sizes, np.int32)
    nw = w_sizes.shape[0]
    m = int((w_sizes.astype(np.int64) ** 2).sum())
    w2m = np.empty(nw, np.int64)
    m2w = np.empty(m, np.int64)
    xo = np.empty(m, np.int64)
    yo = np.empty(m, np.int64)
    lib().s3d_oracle_pair_index(_p(w_sizes), ctypes.c_int64(nw), _p(w2m), _p(m2w), _p(xo), _p(yo))
    return w2m, m2w, xo, yo


def crse_rows(n_coords, table_sizes, hd, i, j):
    n_coords = _c(n_coords, np.float32)
    table_sizes = _c(table_sizes, np.int32)
    nd = table_sizes.shape[0]
    rows = np.empty(nd, np.int32)
    edges = lib().s3d_oracle_crse_rows(_p(n_coords), ctypes.c_int32(nd), _p(table_sizes),
                                       ctypes.c_int32(hd), ctypes.c_int64(i), ctypes.c_int64(j),
                                       _p(rows))
    return rows, int(edges)


def attn_fwd(q, k, v, tq, tk, tv, table_sizes, w_sizes, w2n, n2n, n_coords, acc="f64",
             num_threads=None, return_stats=False):
    """Attention forward on float arrays (fp16 callers widen first).

    Returns out [N,H,D] (float64 for acc='f64', float32 for 'f32'); with
    return_stats also (max [N,H], sum [N,H], edge_pairs).
    """
    q, k, v = (_c(x, np.float32) for x in (q, k, v))
    tq, tk, tv = (_c(x, np.float32).reshape(-1) for x in (tq, tk, tv))
    table_sizes = _c(table_sizes, np.int32)
    w_sizes, w2n, n2n = (_c(x, np.int32) for x in (w_sizes, w2n, n2n))
    n_coords = _c(n_coords, np.float32)
    n, h, d = q.shape
    nd = table_sizes.shape[0]
    assert n_coords.shape == (n, nd), (n_coords.shape, n, nd)
    assert tq.shape[0] == int(table_sizes.sum()) == tk.shape[0] == tv.shape[0]
    assert int(w_sizes.sum()) == n and n2n.shape[0] == n
    dt = np.float64 if acc == "f64" else np.float32
    fn = lib().s3d_oracle_attn_fwd_f64 if acc == "f64" else lib().s3d_oracle_attn_fwd_f32
    out = np.zeros((n, h, d), dt)
    omax = np.zeros((n, h), dt)
    osum = np.zeros((n, h), dt)
    edges = np.zeros(1, np.int64)
    if num_threads is None:
        num_threads = max_threads()
    rc = fn(_p(q), _p(k), _p(v), _p(tq), _p(tk), _p(tv), _p(table_sizes), ctypes.c_int32(nd),
            _p(w_sizes), _p(w2n), _p(n2n), _p(n_coords), _p(out), _p(omax), _p(osum),
            ctypes.c_int64(n), ctypes.c_int32(h), ctypes.c_int32(d),
            ctypes.c_int64(w_sizes.shape[0]), _p(edges), ctypes.c_int32(num_threads))
    if rc != 0:
        raise ValueError(f"s3d_oracle_attn_fwd failed: {rc}")
    if return_stats:
        return out, omax, osum, int(edges[0])
    return out


def attn_bwd(q, k, v, tq, tk, tv, table_sizes, w_sizes, w2n, n2n, n_coords, dout):
    """Attention backward in float64 -> (dq, dk, dv [N,H,D], dtq, dtk, dtv [table_len])."""
    q, k, v, dout = (_c(x, np.float32) for x in (q, k, v, dout))
    tq, tk, tv = (_c(x, np.float32).reshape(-1) for x in (tq, tk, tv))
    table_sizes = _c(table_sizes, np.int32)
    w_sizes, w2n, n2n = (_c(x, np.int32) for x in (w_sizes, w2n, n2n))
    n_coords = _c(n_coords, np.float32)
    n, h, d = q.shape
    nd = table_sizes.shape[0]
    assert dout.shape == q.shape and n_coords.shape == (n, nd)
    assert tq.shape[0] == int(table_sizes.sum()) == tk.shape[0] == tv.shape[0]
    assert int(w_sizes.sum()) == n and n2n.shape[0] == n
    dq, dk, dv = (np.zeros((n, h, d), np.float64) for _ in range(3))
    dtq, dtk, dtv = (np.zeros(tq.shape[0], np.float64) for _ in range(3))
    rc = lib().s3d_oracle_attn_bwd_f64(
        _p(q), _p(k), _p(v), _p(tq), _p(tk), _p(tv), _p(table_sizes), ctypes.c_int32(nd), _p(w_sizes),
        _p(w2n), _p(n2n), _p(n_coords), _p(dout), _p(dq), _p(dk), _p(dv), _p(dtq), _p(dtk), _p(dtv),
        ctypes.c_int64(n), ctypes.c_int32(h), ctypes.c_int32(d), ctypes.c_int64(w_sizes.shape[0]))
    if rc != 0:
        raise ValueError(f"s3d_oracle_attn_bwd failed: {rc}")
    return dq, dk, dv, dtq, dtk, dtv


def knn(k, src_xyz, query_xyz, src_offset, query_offset, heap_order=False, num_threads=None):
    """-> (idx int32 [Nq,K], squared distances fp32 [Nq,K])."""
    src_xyz = _c(src_xyz, np.float32)
    query_xyz = _c(query_xyz, np.float32)
    src_offset = _c(src_offset, np.int32)
    query_offset = _c(query_offset, np.int32)
    nq = query_xyz.shape[0]
    idx = np.empty((nq, k), np.int32)
    d2 = np.empty((nq, k), np.float32)
    if num_threads is None:
        num_threads = max_threads()
    args = [ctypes.c_int32(k), _p(src_xyz), ctypes.c_int64(src_xyz.shape[0]), _p(query_xyz),
            ctypes.c_int64(nq), _p(src_offset), _p(query_offset),
            ctypes.c_int32(src_offset.shape[0]), _p(idx), _p(d2)]
    if heap_order:
        rc = lib().s3d_oracle_knn_heap(*args)
    else:
        rc = lib().s3d_oracle_knn(*args, ctypes.c_int32(num_threads))
    if rc != 0:
        raise ValueError(f"s3d_oracle_knn failed: {rc}")
    return idx, d2


def knn_interpolate(idx, dist2, src_feat):
    """Inverse-distance interpolation from KNN results -> float64 [Nq,C]."""
    idx = _c(idx, np.int32)
    dist2 = _c(dist2, np.float32)
    src_feat = _c(src_feat, np.float32)
    nq, k = idx.shape
    out = np.zeros((nq, src_feat.shape[1]), np.float64)
    rc = lib().s3d_oracle_knn_interpolate(_p(idx), _p(dist2), ctypes.c_int32(k), ctypes.c_int64(nq), _p(src_feat),
                                          ctypes.c_int32(src_feat.shape[1]), _p(out))
    if rc != 0:
        raise ValueError(f"s3d_oracle_knn_interpolate failed: {rc}")
    return out
