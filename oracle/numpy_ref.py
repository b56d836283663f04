"""Brute-force numpy/python statements of the hot path for TINY inputs.

TEST INFRASTRUCTURE ONLY.  A second, independent statement of the same math as
oracle/s3d_oracle.c, written with different data structures on purpose (python
dict grouping, per-axis 3-D table arrays indexed [row][h][c], explicit
softmax), so that a slip in one statement shows up as a disagreement.

Reference text followed:
  window grouping   Swin3D/modules/swin3d_layers.py:713-787
  pair enumeration  Swin3D/modules/swin3d_layers.py:139-140, attn_utils.cuh:379-380
  cRSE rows         Swin3D/src/attn/attn_utils.cuh:437-453
  attention         Swin3D/src/attn/self_attn_aio_fwd.cu:16-52, 111-188; attn_coff.py:184
  knn               Swin3D/src/knn/knn_cuda_kernel.cu:139-204 (canonical order)
"""
import numpy as np


def window_index_bruteforce(coords, stride, ws, shift=0):
    """dict grouping by (b, x // (ws*stride), ...) then sort by local id."""
    coords = np.asarray(coords, dtype=np.int64)
    groups = {}
    for row, (b, x, y, z) in enumerate(coords.tolist()):
        c = [x + shift * stride, y + shift * stride, z + shift * stride]
        win = tuple(ci // (ws * stride) for ci in c)  # python // floors toward -inf
        loc = [(ci // stride) % ws for ci in c]
        local = loc[0] * ws * ws + loc[1] * ws + loc[2]
        groups.setdefault((b,) + win, []).append((local, row))
    n2n, wwid, w_sizes = [], [], []
    for key in sorted(groups):
        members = sorted(groups[key])
        w_sizes.append(len(members))
        for local, row in members:
            n2n.append(row)
            wwid.append(local)
    w_sizes = np.asarray(w_sizes, np.int64)
    w2n = np.concatenate([[0], np.cumsum(w_sizes)[:-1]]) if len(w_sizes) else np.zeros(0, np.int64)
    return dict(n2n=np.asarray(n2n, np.int64), w_w_id=np.asarray(wwid, np.int64),
                w_sizes=w_sizes, w2n=w2n.astype(np.int64), W=len(w_sizes),
                M=int((w_sizes ** 2).sum()))


def pair_index_python_statement(w_sizes):
    """Vectorised statement of the reference's python pair index (cumsum form)."""
    w_sizes = np.asarray(w_sizes, np.int64)
    sq = w_sizes ** 2
    w2n = np.concatenate([[0], np.cumsum(w_sizes)[:-1]])
    w2m = np.concatenate([[0], np.cumsum(sq)[:-1]])
    m_total = int(sq.sum())
    flag = np.zeros(m_total, np.int64)
    off = np.zeros(m_total, np.int64)
    flag[w2m[1:]] = 1
    off[w2m[1:]] = sq[:-1]
    m2w = np.cumsum(flag)
    m2w_off = np.cumsum(off)
    m_off = np.arange(m_total) - m2w_off
    sizes = w_sizes[m2w]
    y = w2n[m2w] + m_off % sizes
    x = w2n[m2w] + m_off // sizes
    return w2m, m2w, x, y


def crse_row(ci, cj, rows_n):
    """One row index with every step rounded to fp32, upper edge folded to rows_n-1."""
    rel = np.float32(np.float32(ci) - np.float32(cj))
    rel = np.float32(rel + np.float32(rows_n // 2))
    hi = np.float32(np.float64(rows_n) - 1e-10)
    rel = min(max(np.float32(0.0), rel), hi)
    return min(int(rel), rows_n - 1)


def attn_fwd_bruteforce(q, k, v, tq_axes, tk_axes, tv_axes, n_coords, n2n, w_sizes):
    """q,k,v [N,H,D]; t*_axes: list (one per axis) of [rows_n,H,D]; n_coords [N,nd]
    in sorted order; returns out [N,H,D] float64."""
    q, k, v = (np.asarray(x, np.float64) for x in (q, k, v))
    n, h, d = q.shape
    nd = len(tq_axes)
    out = np.zeros((n, h, d))
    start = 0
    for n_w in [int(x) for x in w_sizes]:
        pos = list(range(start, start + n_w))
        start += n_w
        for i in pos:
            t_q = np.zeros((n_w, h, d))
            t_k = np.zeros((n_w, h, d))
            t_v = np.zeros((n_w, h, d))
            for jj, j in enumerate(pos):
                for ax in range(nd):
                    r = crse_row(n_coords[i, ax], n_coords[j, ax], tq_axes[ax].shape[0])
                    t_q[jj] += np.asarray(tq_axes[ax][r], np.float64)
                    t_k[jj] += np.asarray(tk_axes[ax][r], np.float64)
                    t_v[jj] += np.asarray(tv_axes[ax][r], np.float64)
            qi = q[n2n[i]]  # [H,D]
            kj = k[[n2n[j] for j in pos]]  # [n_w,H,D]
            vj = v[[n2n[j] for j in pos]]
            logits = (qi[None] * kj + qi[None] * t_q + kj * t_k).sum(-1)  # [n_w,H]
            logits = logits - logits.max(0, keepdims=True)
            p = np.exp(logits)
            p = p / p.sum(0, keepdims=True)
            out[n2n[i]] = (p[:, :, None] * (vj + t_v)).sum(0)
    return out


def knn_bruteforce(kk, src, qry, src_offset, query_offset):
    """full fp32 distance matrix per segment, lexsort by (dist, idx)."""
    src = np.asarray(src, np.float32)
    qry = np.asarray(qry, np.float32)
    nq = qry.shape[0]
    idx = np.full((nq, kk), -1, np.int32)
    d2 = np.full((nq, kk), 2147483648.0, np.float32)
    s_prev = q_prev = 0
    for b in range(len(src_offset)):
        s_end, q_end = int(src_offset[b]), int(query_offset[b])
        s = src[s_prev:s_end]
        for g in range(q_prev, q_end):
            if s.shape[0]:
                dx = (s[:, 0] - qry[g, 0]).astype(np.float32)
                dy = (s[:, 1] - qry[g, 1]).astype(np.float32)
                dz = (s[:, 2] - qry[g, 2]).astype(np.float32)
                dist = ((dx * dx).astype(np.float32) + (dy * dy).astype(np.float32)).astype(np.float32)
                dist = (dist + (dz * dz).astype(np.float32)).astype(np.float32)
                order = np.lexsort((np.arange(s.shape[0]), dist))[:kk]
                idx[g, :len(order)] = order + s_prev
                d2[g, :len(order)] = dist[order]
        s_prev, q_prev = s_end, q_end
    return idx, d2
