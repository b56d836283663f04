"""Pins oracle.attn_fwd (CPU): numpy brute force with 4-D indexed tables, softmax(QK^T)V
special case against torch, closed forms, invariances, quantiser edges."""
import numpy as np
import pytest
import torch

from oracle import numpy_ref
from helpers import make_attn_case
from swin3d_amd import crse


@pytest.mark.parametrize("cRSE", ["XYZ", "XYZ_RGB", "XYZ_RGB_NORM"])
@pytest.mark.parametrize("heads,dim", [(2, 8), (3, 4)])
def test_matches_numpy_bruteforce(oracle_lib, cRSE, heads, dim):
    case = make_attn_case(oracle_lib, seed=11, n=90, ws=3, quant=2, heads=heads, dim=dim, cRSE=cRSE)
    got = oracle_lib.attn_fwd(*case.oracle_args())
    ref = numpy_ref.attn_fwd_bruteforce(case.q, case.k, case.v, case.axis_tables(case.tq),
                                        case.axis_tables(case.tk), case.axis_tables(case.tv),
                                        case.n_coords, case.index["n2n"], case.index["w_sizes"])
    np.testing.assert_allclose(got, ref, rtol=1e-12, atol=1e-13)


def test_f32_variant_close_to_f64(oracle_lib):
    case = make_attn_case(oracle_lib, seed=12, n=150, ws=4, quant=2, heads=2, dim=8)
    a = oracle_lib.attn_fwd(*case.oracle_args(), acc="f64")
    b = oracle_lib.attn_fwd(*case.oracle_args(), acc="f32", num_threads=2)
    np.testing.assert_allclose(b, a, rtol=2e-4, atol=2e-5)


def test_zero_tables_equal_block_diagonal_sdpa(oracle_lib):
    """All tables zero => softmax(q k^T) v inside every window (scale 1: q is pre-scaled)."""
    case = make_attn_case(oracle_lib, seed=13, n=200, ws=4, quant=2, heads=4, dim=8)
    case.tq[:] = 0
    case.tk[:] = 0
    case.tv[:] = 0
    got = oracle_lib.attn_fwd(*case.oracle_args())
    n2n, w2n, w_sizes = (case.index[key] for key in ("n2n", "w2n", "w_sizes"))
    window_of = np.empty(case.N, np.int64)
    for w, (s, c) in enumerate(zip(w2n, w_sizes)):
        window_of[n2n[s:s + c]] = w
    mask = torch.from_numpy(window_of[:, None] == window_of[None, :])
    q, k, v = (torch.from_numpy(x).double().permute(1, 0, 2) for x in (case.q, case.k, case.v))
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask, scale=1.0)
    np.testing.assert_allclose(got, ref.permute(1, 0, 2).numpy(), rtol=1e-10, atol=1e-12)


def test_zero_qk_gives_mean_of_values_plus_table(oracle_lib):
    case = make_attn_case(oracle_lib, seed=14, n=60, ws=3, quant=2, heads=2, dim=8, cRSE="XYZ_RGB")
    case.q[:] = 0
    case.k[:] = 0
    got = oracle_lib.attn_fwd(*case.oracle_args())
    tv = case.axis_tables(case.tv)
    n2n, w2n, w_sizes = (case.index[key] for key in ("n2n", "w2n", "w_sizes"))
    for s, c in zip(w2n, w_sizes):
        for i in range(s, s + c):
            acc = np.zeros((case.H, case.D))
            for j in range(s, s + c):
                acc += case.v[n2n[j]]
                for ax in range(len(tv)):
                    acc += tv[ax].astype(np.float64)[numpy_ref.crse_row(case.n_coords[i, ax], case.n_coords[j, ax], tv[ax].shape[0])]
            np.testing.assert_allclose(got[n2n[i]], acc / c, rtol=1e-10, atol=1e-12)


def test_single_voxel_window_closed_form(oracle_lib):
    """One voxel per window: out = v + sum_n table_v[n][rows_n/2] (rel = 0 lands on the middle row)."""
    ws, quant, heads, dim = 5, 4, 2, 8
    coords = np.array([[0, 0, 0, 0], [0, 50, 0, 0], [1, 3, 3, 3]], np.int32)
    case = make_attn_case(oracle_lib, seed=15, n=3, ws=ws, quant=quant, heads=heads, dim=dim)
    from helpers import n_coords_from_scene
    frac = np.random.default_rng(1).random((3, 3)).astype(np.float32)
    sig = np.random.default_rng(2).uniform(-1, 1, (3, 6)).astype(np.float32)
    case.index, case.n_coords = n_coords_from_scene(oracle_lib, coords, frac, sig, 1, ws, quant, case.cRSE)
    assert case.index["W"] == 3
    got = oracle_lib.attn_fwd(*case.oracle_args())
    tv = case.axis_tables(case.tv)
    expect = case.v.astype(np.float64) + sum(t[t.shape[0] // 2].astype(np.float64) for t in tv)[None]
    np.testing.assert_allclose(got, expect, rtol=1e-12)


def test_constant_value_passes_through(oracle_lib):
    case = make_attn_case(oracle_lib, seed=16, n=80, ws=3, quant=2, heads=2, dim=8)
    case.tv[:] = 0
    case.v[:] = 0.75
    got = oracle_lib.attn_fwd(*case.oracle_args())
    np.testing.assert_allclose(got, 0.75, rtol=1e-12)


def test_head_independence_and_row_permutation(oracle_lib):
    case = make_attn_case(oracle_lib, seed=17, n=100, ws=3, quant=2, heads=3, dim=8)
    base = oracle_lib.attn_fwd(*case.oracle_args())
    # changing head 2 leaves heads 0, 1 untouched
    q2 = case.q.copy()
    q2[:, 2] += 1.0
    args = list(case.oracle_args())
    args[0] = q2
    moved = oracle_lib.attn_fwd(*args)
    np.testing.assert_array_equal(moved[:, :2], base[:, :2])
    assert np.abs(moved[:, 2] - base[:, 2]).max() > 1e-3
    # permuting the voxel rows (and n2n with them) permutes the output rows
    perm = np.random.default_rng(0).permutation(case.N)
    inv = np.argsort(perm)
    args = list(case.oracle_args())
    args[0], args[1], args[2] = case.q[perm], case.k[perm], case.v[perm]
    args[9] = inv[case.index["n2n"]].astype(np.int32)
    permuted = oracle_lib.attn_fwd(*args)
    np.testing.assert_array_equal(permuted, base[perm])


def test_translation_by_whole_windows_is_invariant(oracle_lib):
    from helpers import n_coords_from_scene
    case = make_attn_case(oracle_lib, seed=18, n=100, ws=3, quant=2, heads=2, dim=8, cRSE="XYZ")
    base = oracle_lib.attn_fwd(*case.oracle_args())
    rng = np.random.default_rng(18)
    # regenerate the same scene moved by two windows: identical index and n_coords
    from conftest import random_scene
    coords = random_scene(rng, 100, extent=(4, 4, 2))
    frac = rng.random((100, 3)).astype(np.float32)
    np.testing.assert_array_equal(coords, case.coords)
    moved = coords.copy()
    moved[:, 1:] += 2 * case.ws
    index, n_coords = n_coords_from_scene(oracle_lib, moved, frac, np.zeros((100, 0), np.float32), 1,
                                          case.ws, case.quant, "XYZ")
    np.testing.assert_array_equal(n_coords, case.n_coords)
    case.index, case.n_coords = index, n_coords
    np.testing.assert_array_equal(oracle_lib.attn_fwd(*case.oracle_args()), base)


def test_stats_are_max_and_sum_of_logits(oracle_lib):
    case = make_attn_case(oracle_lib, seed=19, n=40, ws=3, quant=2, heads=2, dim=8, cRSE="XYZ")
    out, mx, sm, _ = oracle_lib.attn_fwd(*case.oracle_args(), return_stats=True)
    tq, tk = case.axis_tables(case.tq), case.axis_tables(case.tk)
    n2n, w2n, w_sizes = (case.index[key] for key in ("n2n", "w2n", "w_sizes"))
    s, c = w2n[0], w_sizes[0]
    i = s
    logits = np.zeros((c, case.H))
    for jj, j in enumerate(range(s, s + c)):
        bq = sum(t[numpy_ref.crse_row(case.n_coords[i, a], case.n_coords[j, a], t.shape[0])].astype(np.float64) for a, t in enumerate(tq))
        bk = sum(t[numpy_ref.crse_row(case.n_coords[i, a], case.n_coords[j, a], t.shape[0])].astype(np.float64) for a, t in enumerate(tk))
        qi, kj = case.q[n2n[i]].astype(np.float64), case.k[n2n[j]].astype(np.float64)
        logits[jj] = (qi * kj + qi * bq + kj * bk).sum(-1)
    np.testing.assert_allclose(mx[n2n[i]], logits.max(0), rtol=1e-12)
    np.testing.assert_allclose(sm[n2n[i]], np.exp(logits - logits.max(0)).sum(0), rtol=1e-12)


# ---- quantiser (attn_utils.cuh:444-450) ------------------------------------------------------

def _row(oracle_lib, ci, cj, rows, hd=16):
    n_coords = np.array([[ci], [cj]], np.float32)
    got, edges = oracle_lib.crse_rows(n_coords, np.array([rows * hd], np.int32), hd, 0, 1)
    return int(got[0]), edges


def test_quantiser_known_values(oracle_lib):
    rows = 40  # ws 5, quant 4
    assert _row(oracle_lib, 0.0, 0.0, rows) == (20, 0)                 # rel 0 -> middle row
    assert _row(oracle_lib, 3.0, 1.0, rows) == (22, 0)                 # integer difference
    assert _row(oracle_lib, 1.0, 3.0, rows) == (18, 0)
    assert _row(oracle_lib, 1.0, 1.5, rows) == (19, 0)                 # -0.5 + 20 = 19.5 -> 19 (floor)
    assert _row(oracle_lib, 1.5, 1.0, rows) == (20, 0)                 # +0.5 -> 20
    assert _row(oracle_lib, 0.0, 19.999, rows) == (0, 0)               # just above 0
    assert _row(oracle_lib, 0.0, 25.0, rows) == (0, 0)                 # below 0: clamped
    assert _row(oracle_lib, 19.5, 0.0, rows) == (39, 0)                # 39.5 -> last row
    below = np.nextafter(np.float32(20.0), np.float32(0.0))
    assert _row(oracle_lib, below, 0.0, rows)[1] in (0, 1)             # rounding decides; never OOB
    assert _row(oracle_lib, 20.0, 0.0, rows) == (39, 1)                # rel == rows: folded + counted
    assert _row(oracle_lib, 100.0, 0.0, rows) == (39, 1)
    # odd row count: rows // 2 is an integer division (attn_utils.cuh:448)
    assert _row(oracle_lib, 0.0, 0.0, 33) == (16, 0)


def test_quantiser_is_fp32(oracle_lib):
    """A difference that only rounds to the integer in fp32 must land on the fp32 answer."""
    ci = np.float32(16.0) + np.float32(2.0 ** -20)      # representable
    cj = np.float32(2.0 ** -21)                         # exact difference 16 + 2^-21: rounds to 16
    rel32 = np.float32(np.float32(ci - cj) + np.float32(20))
    row, _ = _row(oracle_lib, ci, cj, 40)
    assert row == int(rel32) == numpy_ref.crse_row(ci, cj, 40)
    # sum just below an integer in exact arithmetic but equal to it after fp32 rounding
    ci, cj = np.float32(5.0), np.float32(2.0 ** -22)
    exact = float(ci) - float(cj) + 20.0
    assert int(np.floor(exact)) == 24
    assert _row(oracle_lib, ci, cj, 40)[0] == 25 == numpy_ref.crse_row(ci, cj, 40)


def test_edge_counter_counts_pair_axes(oracle_lib):
    # two voxels in one window whose normals are opposite on one axis: scaled difference = +-16 = rows/2
    ws, quant, heads, dim = 5, 4, 1, 8
    sizes = crse.crse_table_sizes(ws, quant, heads, dim, "XYZ_RGB_NORM")
    n_coords = np.zeros((2, 9), np.float32)
    n_coords[0, 6], n_coords[1, 6] = 8.0, -8.0           # nx = +1 / -1 times 2*quant
    rng = np.random.default_rng(0)
    q, k, v = (rng.standard_normal((2, heads, dim)).astype(np.float32) for _ in range(3))
    t = [rng.standard_normal(sum(sizes)).astype(np.float32) for _ in range(3)]
    out, _, _, edges = oracle_lib.attn_fwd(q, k, v, *t, sizes, np.array([2], np.int32),
                                           np.array([0], np.int32), np.array([0, 1], np.int32),
                                           n_coords, return_stats=True)
    assert edges == 1                                    # only the (0 -> 1) direction hits rel == rows
    assert np.isfinite(out).all()
