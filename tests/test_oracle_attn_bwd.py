"""Pins of the attention-backward oracle (CPU): automatic differentiation of an independent dense
torch statement of the forward, and central differences of the forward oracle."""
import numpy as np
import pytest
import torch

from oracle import numpy_ref
from helpers import make_attn_case


def _torch_forward(case, q, k, v, tq, tk, tv):
    """Dense float64 statement of the operator with torch ops only (autograd differentiates it):
    per window, gather the table rows of every pair (rows from the numpy quantiser), form the
    logits, softmax over the keys, weight value + value-table rows."""
    h, d = case.H, case.D
    sizes = case.table_sizes.tolist()
    offs = np.concatenate([[0], np.cumsum(sizes)])
    out = torch.zeros_like(q)
    n2n = case.index["n2n"]
    start = 0
    for n_w in case.index["w_sizes"].tolist():
        pos = np.arange(start, start + n_w)
        start += n_w
        rows_v = torch.from_numpy(n2n[pos].astype(np.int64))
        qw, kw, vw = q[rows_v], k[rows_v], v[rows_v]                      # [n_w,H,D]
        bq = torch.zeros((n_w, n_w, h, d), dtype=torch.float64)
        bk, bv = torch.zeros_like(bq), torch.zeros_like(bq)
        for ax, size in enumerate(sizes):
            rows_n = size // (h * d)
            r = np.array([[numpy_ref.crse_row(case.n_coords[i, ax], case.n_coords[j, ax], rows_n)
                           for j in pos] for i in pos], np.int64)
            r = torch.from_numpy(r)
            sl = slice(int(offs[ax]), int(offs[ax + 1]))
            bq = bq + tq[sl].reshape(rows_n, h, d)[r]
            bk = bk + tk[sl].reshape(rows_n, h, d)[r]
            bv = bv + tv[sl].reshape(rows_n, h, d)[r]
        logits = (qw[:, None] * kw[None] + qw[:, None] * bq + kw[None] * bk).sum(-1)   # [i,j,H]
        p = torch.softmax(logits, dim=1)
        out = out.index_add(0, rows_v, (p[..., None] * (vw[None] + bv)).sum(1))
    return out


@pytest.mark.parametrize("cRSE,heads,dim", [("XYZ", 2, 4), ("XYZ_RGB_NORM", 2, 8), ("XYZ_RGB", 3, 4)])
def test_backward_matches_autograd(oracle_lib, cRSE, heads, dim):
    case = make_attn_case(oracle_lib, seed=51, n=70, ws=3, quant=2, heads=heads, dim=dim, cRSE=cRSE)
    rng = np.random.default_rng(52)
    dout = rng.standard_normal(case.q.shape).astype(np.float32)
    t = lambda a: torch.from_numpy(np.asarray(a, np.float64)).requires_grad_(True)
    leaves = [t(a) for a in (case.q, case.k, case.v, case.tq, case.tk, case.tv)]
    out = _torch_forward(case, *leaves)
    np.testing.assert_allclose(out.detach().numpy(), oracle_lib.attn_fwd(*case.oracle_args()), rtol=1e-11,
                               atol=1e-12)
    grads = torch.autograd.grad(out, leaves, torch.from_numpy(dout.astype(np.float64)))
    got = oracle_lib.attn_bwd(*case.oracle_args(), dout)
    for name, g, ref in zip(("dq", "dk", "dv", "dtq", "dtk", "dtv"), got, grads):
        ref = ref.numpy()
        np.testing.assert_allclose(g, ref.reshape(g.shape), rtol=1e-9, atol=1e-11 * max(1.0, np.abs(ref).max()),
                                   err_msg=name)


def test_backward_matches_central_differences(oracle_lib):
    """<grad, direction> against (f(x + e d) - f(x - e d)) / 2e contracted with dout; inputs and
    directions are multiples of 2^-10 and e = 2^-8, so x +- e d is exact in fp32."""
    case = make_attn_case(oracle_lib, seed=53, n=60, ws=3, quant=2, heads=2, dim=8)
    snap = lambda a, s=1024.0: (np.round(np.asarray(a, np.float64) * s) / s).astype(np.float32)
    for name in ("q", "k", "v", "tq", "tk", "tv"):
        setattr(case, name, snap(getattr(case, name)))
    rng = np.random.default_rng(54)
    dout = rng.standard_normal(case.q.shape).astype(np.float32)
    grads = dict(zip(("q", "k", "v", "tq", "tk", "tv"), oracle_lib.attn_bwd(*case.oracle_args(), dout)))
    eps = 2.0 ** -8
    for name in ("q", "k", "v", "tq", "tk", "tv"):
        base = getattr(case, name).copy()
        direction = snap(rng.integers(-4, 5, size=base.shape) / 4.0)
        setattr(case, name, (base + np.float32(eps) * direction).astype(np.float32))
        plus = oracle_lib.attn_fwd(*case.oracle_args())
        setattr(case, name, (base - np.float32(eps) * direction).astype(np.float32))
        minus = oracle_lib.attn_fwd(*case.oracle_args())
        setattr(case, name, base)
        numeric = ((plus - minus) / (2 * eps) * dout).sum()
        analytic = (grads[name].reshape(base.shape) * direction).sum()
        assert abs(numeric - analytic) <= 2e-3 * max(1.0, abs(analytic)), (name, numeric, analytic)


def test_backward_closed_forms(oracle_lib):
    """q = k = 0 and zero query/key tables: uniform weights, so dv_j = mean over the window's queries of
    dout_i, and dq = dk = 0 only if dout is orthogonal to the value spread; checked: dv and the row sums."""
    case = make_attn_case(oracle_lib, seed=55, n=50, ws=3, quant=2, heads=2, dim=4, cRSE="XYZ")
    case.q[:] = 0
    case.k[:] = 0
    case.tq[:] = 0
    case.tk[:] = 0
    rng = np.random.default_rng(56)
    dout = rng.standard_normal(case.q.shape).astype(np.float32)
    dq, dk, dv, dtq, dtk, dtv = oracle_lib.attn_bwd(*case.oracle_args(), dout)
    n2n, start = case.index["n2n"], 0
    for n_w in case.index["w_sizes"].tolist():
        rows = n2n[start:start + n_w]
        start += n_w
        expect = dout[rows].astype(np.float64).sum(0) / n_w
        np.testing.assert_allclose(dv[rows], np.broadcast_to(expect, dv[rows].shape), rtol=1e-12, atol=1e-13)
    # every pair adds dout_i / n_w to one row of every axis table: the table gradient sums to nd * sum(dout)
    # per (head, channel)
    h, d = case.H, case.D
    per_hc = dtv.reshape(-1, h, d).sum(0)
    np.testing.assert_allclose(per_hc, 3 * dout.astype(np.float64).sum(0), rtol=1e-10, atol=1e-10)
    # softmax rows sum to one: the logit gradients of a row sum to zero, hence sum_j dk-part from q = 0 ...
    # with q = 0 and Tk = 0, dk = coff_grad * 0 = 0 exactly
    assert np.abs(dk).max() == 0.0
