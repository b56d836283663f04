"""Rows that are in window-sorted order already (`n2n` = NULL / None): the instantiations of the sweep kernel that
read q, k, v and write out without the row map - the gather of Swin3D/src/attn/attn_utils.cuh:391-409 removed.
q, k, v are permuted into window order on the host, the op is called without a row map through every entry point
that takes one (Python surface; C ABI building its own work list, on a plan, and without a workspace), and the
result, put back into voxel order, is compared with the float64 oracle and bit for bit with the call that uses the
row map (same work list, same arithmetic per query: the bits must not depend on where a row lives)."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import AttnCase, n_coords_from_scene, to_half_and_back
from swin3d_amd import crse, synth

pytestmark = pytest.mark.gpu


def _scene(rng, ws):
    """Two batch elements: a block of well-filled windows (more than 64 voxels each, up to ~250 at window 7) next
    to a sparse region of small windows, rows in random order."""
    dense = np.stack(np.meshgrid(np.arange(3 * ws), np.arange(2 * ws), np.arange(ws), indexing="ij"), -1).reshape(-1, 3)
    dense = dense[rng.random(dense.shape[0]) < 0.72]
    sparse = np.stack(np.meshgrid(np.arange(4 * ws), np.arange(4 * ws), np.arange(2 * ws), indexing="ij"), -1).reshape(-1, 3)
    sparse = sparse[rng.random(sparse.shape[0]) < 0.12] + np.array([5 * ws, 0, 0])
    rows = []
    for b, part in enumerate((np.concatenate([dense, sparse]), sparse[: sparse.shape[0] // 2] - np.array([ws, 3, 0]))):
        rows.append(np.concatenate([np.full((part.shape[0], 1), b, np.int64), part], 1))
    coords = np.concatenate(rows).astype(np.int32)
    order = rng.permutation(coords.shape[0])
    order = order[np.argsort(coords[order, 0], kind="stable")]      # batches stay contiguous
    return coords[order]


def _case(oracle_lib, seed, heads, dim, ws, cRSE, fp16):
    rng = np.random.default_rng(seed)
    coords = _scene(rng, ws)
    n = coords.shape[0]
    quant = 4
    frac = rng.random((n, 3)).astype(np.float32)
    sig = rng.uniform(-1, 1, (n, crse.crse_num_axes(cRSE) - 3)).astype(np.float32)
    index, n_coords = n_coords_from_scene(oracle_lib, coords, frac, sig, 1, ws, quant, cRSE)
    sizes = crse.crse_table_sizes(ws, quant, heads, dim, cRSE)
    q, k, v, tables = synth.layer_inputs(n, heads * dim, heads, int(sum(sizes)), seed=seed, recipe="sharp")
    case = AttnCase(coords, 1, ws, quant, heads, dim, cRSE, index, n_coords, q, k, v, tables, sizes)
    if fp16:
        case.v *= np.float32(0.4)       # keeps the fp16 rounding of the output itself below the tolerance
        case.tv *= np.float32(0.2)
        to_half_and_back(case)
    return case


def _c_abi_sorted(hip_lib, x, sizes, code, how):
    """One call with a NULL row map through the C ABI -> (out, max, sum) in window-sorted row order."""
    from swin3d_amd import _lib
    n, h, d = x["q"].shape
    w = x["w_sizes"].numel()
    c_sizes = (ctypes.c_int32 * len(sizes))(*sizes)
    stream = torch.cuda.current_stream().cuda_stream
    dtype = x["q"].dtype
    out = torch.full((n, h, d), float("nan"), dtype=dtype, device="cuda")
    omax = torch.full((n, h), float("nan"), dtype=torch.float32, device="cuda")
    osum = torch.full((n, h), float("nan"), dtype=torch.float32, device="cuda")
    head = [x["q"].data_ptr(), x["k"].data_ptr(), x["v"].data_ptr(), x["tq"].data_ptr(), x["tk"].data_ptr(),
            x["tv"].data_ptr(), c_sizes, len(sizes), x["tq"].numel(), x["w_sizes"].data_ptr(), x["w2n"].data_ptr(),
            None, x["n_coords"].data_ptr(), out.data_ptr(), omax.data_ptr(), osum.data_ptr(), n, h, d, w]
    if how == "noalloc":
        _lib.check(hip_lib.s3d_attn_fwd_noalloc(*head, 0, code, stream), "s3d_attn_fwd_noalloc")
    elif how == "planned":
        nbytes = hip_lib.s3d_attn_plan_bytes(h, n, w)
        plan = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        _lib.check(hip_lib.s3d_attn_plan(c_sizes, len(sizes), x["tq"].numel(), x["w_sizes"].data_ptr(),
                                         x["w2n"].data_ptr(), n, h, d, w, code, plan.data_ptr(), nbytes, stream),
                   "s3d_attn_plan")
        for _ in range(2):      # a plan serves call after call
            _lib.check(hip_lib.s3d_attn_fwd(*head, 0, code, _lib.S3D_ATTN_PLANNED, plan.data_ptr(), nbytes, stream),
                       "s3d_attn_fwd (planned)")
    else:
        nbytes = hip_lib.s3d_attn_fwd_workspace_bytes(h, n, w)
        workspace = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        _lib.check(hip_lib.s3d_attn_fwd(*head, 0, code, 0, workspace.data_ptr(), nbytes, stream), "s3d_attn_fwd")
    torch.cuda.synchronize()
    return out, omax, osum


# heads chosen so that the wavefronts carry one, two and three heads (fp16 head_dim 8: H = 5, 4, 6; fp16 head_dim
# 16 and fp32 head_dim 8: pairs at even H), every head_dim, three signal sets
SHAPES = [
    (torch.float16, 5, 8, 5, "XYZ_RGB_NORM"), (torch.float16, 4, 8, 5, "XYZ_RGB"), (torch.float16, 6, 8, 5, "XYZ_RGB_NORM"),
    (torch.float16, 6, 16, 7, "XYZ_RGB_NORM"), (torch.float16, 5, 16, 7, "XYZ"), (torch.float16, 2, 32, 7, "XYZ_RGB_NORM"),
    (torch.float32, 4, 8, 5, "XYZ_RGB_NORM"), (torch.float32, 5, 8, 7, "XYZ_RGB"), (torch.float32, 4, 16, 7, "XYZ_RGB_NORM"),
    (torch.float32, 2, 32, 5, "XYZ"),
]


@pytest.mark.parametrize("dtype,heads,dim,ws,cRSE", SHAPES)
def test_rows_in_window_order_need_no_row_map(oracle_lib, hip_lib, dtype, heads, dim, ws, cRSE):
    import swin3d_amd
    from swin3d_amd import _lib
    from gpu_helpers import assert_attn_close
    case = _case(oracle_lib, 700 + heads * dim + ws, heads, dim, ws, cRSE, dtype == torch.float16)
    i = case.index
    assert int(i["w_sizes"].max()) > 64 and int(i["w_sizes"].min()) < 32
    ref, rmax, rsum, _ = oracle_lib.attn_fwd(*case.oracle_args(), return_stats=True)
    dev = torch.device("cuda")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    n2n = t(i["n2n"]).long()
    x = dict(tq=t(case.tq).to(dtype), tk=t(case.tk).to(dtype), tv=t(case.tv).to(dtype),
             w_sizes=t(i["w_sizes"]).int(), w2n=t(i["w2n"]).int(), n_coords=t(case.n_coords).float().contiguous())
    rows = {name: t(getattr(case, name)).to(dtype) for name in "qkv"}
    sizes = [int(s) for s in case.table_sizes]
    # the call with the row map, on rows in voxel order
    mapped = swin3d_amd.window_attention_forward(rows["q"], rows["k"], rows["v"], x["tq"], x["tk"], x["tv"], sizes,
                                                 x["w_sizes"], x["w2n"], n2n.int(), x["n_coords"], return_stats=True)
    assert_attn_close(mapped[0].double().cpu().numpy(), ref, dtype)
    # the same rows gathered into window order: sorted position p holds row n2n[p]
    for name in "qkv":
        x[name] = rows[name][n2n].contiguous()
    code = _lib.S3D_DTYPE_F16 if dtype == torch.float16 else _lib.S3D_DTYPE_F32
    results = {"python": swin3d_amd.window_attention_forward(x["q"], x["k"], x["v"], x["tq"], x["tk"], x["tv"], sizes,
                                                             x["w_sizes"], x["w2n"], None, x["n_coords"],
                                                             return_stats=True)}
    for how in ("own list", "planned", "noalloc"):
        results[how] = _c_abi_sorted(hip_lib, x, sizes, code, how)
    torch.cuda.synchronize()
    for how, (out_s, max_s, sum_s) in results.items():
        out = torch.empty_like(out_s)
        omax, osum = torch.empty_like(max_s), torch.empty_like(sum_s)
        out[n2n], omax[n2n], osum[n2n] = out_s, max_s, sum_s          # back to voxel order
        assert torch.isfinite(out).all(), how
        assert_attn_close(out.double().cpu().numpy(), ref, dtype)
        stat_tol = 2e-3 if dtype == torch.float16 else 1e-4
        assert np.abs(omax.double().cpu().numpy() - rmax).max() <= stat_tol * max(1.0, np.abs(rmax).max()), how
        assert np.abs(osum.double().cpu().numpy() / rsum - 1.0).max() <= 5 * stat_tol, how
        assert torch.equal(out, mapped[0]) and torch.equal(omax, mapped[1]) and torch.equal(osum, mapped[2]), how


BWD_SHAPES = [(torch.float16, 6, 8, 5, "XYZ_RGB_NORM", None), (torch.float32, 4, 8, 5, "XYZ_RGB", None),
              (torch.float16, 4, 16, 7, "XYZ_RGB_NORM", None), (torch.float32, 3, 16, 7, "XYZ", 0),
              (torch.float16, 6, 8, 5, "XYZ_RGB_NORM", 0), (torch.float32, 2, 32, 5, "XYZ", None)]


@pytest.mark.parametrize("dtype,heads,dim,ws,cRSE,pairs", BWD_SHAPES)
def test_backward_on_rows_in_window_order(oracle_lib, hip_lib, dtype, heads, dim, ws, cRSE, pairs):
    """s3d_attn_bwd with a NULL row map (the library reads the identity map that it writes into its workspace): all
    six gradients against the float64 oracle, dq / dk / dv bit for bit those of the call with the row map on rows in
    voxel order.  pairs None: the pair sweeps and their store; 0: the fused sweeps; head_dim 32: the general form."""
    import swin3d_amd
    case = _case(oracle_lib, 900 + heads * dim + ws, heads, dim, ws, cRSE, dtype == torch.float16)
    rng = np.random.default_rng(5)
    dout = rng.standard_normal(case.q.shape).astype(np.float32)
    if dtype == torch.float16:
        dout = dout.astype(np.float16).astype(np.float32)
    ref = [np.asarray(r, np.float64) for r in oracle_lib.attn_bwd(*case.oracle_args(), dout)]
    dev = torch.device("cuda")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    i = case.index
    n2n = t(i["n2n"]).long()
    tabs = [t(a).to(dtype) for a in (case.tq, case.tk, case.tv)]
    tail = (t(case.table_sizes), t(i["w_sizes"]), t(i["w2n"]))
    n_coords = t(case.n_coords)
    rows = [t(a).to(dtype) for a in (case.q, case.k, case.v)]
    d_out = t(dout).to(dtype)

    def grads(feats, row_map, dout_rows):
        args = (*feats, *tabs, *tail, row_map, n_coords)
        out, omax, osum = swin3d_amd.window_attention_forward(*args, return_stats=True)
        return swin3d_amd.window_attention_backward(*args, out, omax, osum, dout_rows, pairs=pairs)

    mapped = grads(rows, n2n.int(), d_out)
    ordered = grads([r[n2n].contiguous() for r in rows], None, d_out[n2n].contiguous())
    torch.cuda.synchronize()
    rel = 2e-5 if dtype == torch.float32 else 3e-3
    scale_rows = max(np.abs(r).max() for r in ref[:3])
    scale_tabs = max(np.abs(r).max() for r in ref[3:])
    for which, (g_sorted, g_mapped, r) in enumerate(zip(ordered, mapped, ref)):
        if which < 3:
            g = torch.empty_like(g_sorted)
            g[n2n] = g_sorted                                        # back to voxel order
            if dim != 32:        # the general form adds dk, dv with atomics: not the same bits from call to call
                assert torch.equal(g, g_mapped), which
            scale = scale_rows
        else:
            g, scale = g_sorted, scale_tabs
        got = g.double().cpu().numpy().reshape(r.shape)
        assert np.isfinite(got).all(), which
        assert np.abs(got - r).max() <= rel * scale, (which, np.abs(got - r).max(), scale)
