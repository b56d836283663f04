"""Pins oracle.window_index / pair_index (CPU): brute force, invariants, shift property,
and both reference statements of the pair decode (swin3d_layers.py:139-140,
attn_utils.cuh:379-380)."""
import numpy as np
import pytest

from oracle import numpy_ref
from conftest import random_scene


@pytest.mark.parametrize("ws,stride,shift", [(5, 1, 0), (5, 1, 2), (7, 2, 3), (3, 4, 1), (2, 1, 0)])
@pytest.mark.parametrize("seed", [0, 1])
def test_matches_dict_grouping(oracle_lib, ws, stride, shift, seed):
    rng = np.random.default_rng(seed)
    coords = random_scene(rng, 400, batches=3, stride=stride)
    got = oracle_lib.window_index(coords, stride, ws, shift)
    ref = numpy_ref.window_index_bruteforce(coords, stride, ws, shift)
    assert got["W"] == ref["W"] and got["M"] == ref["M"]
    for key in ("n2n", "w_w_id", "w_sizes", "w2n"):
        np.testing.assert_array_equal(got[key], ref[key], err_msg=key)


def test_invariants(oracle_lib):
    rng = np.random.default_rng(3)
    ws, stride = 5, 2
    coords = random_scene(rng, 3000, extent=(40, 30, 10), batches=2, stride=stride)
    r = oracle_lib.window_index(coords, stride, ws, 0)
    n = coords.shape[0]
    assert sorted(r["n2n"].tolist()) == list(range(n))                    # permutation
    assert r["w_sizes"].sum() == n and (r["w_sizes"] > 0).all()
    np.testing.assert_array_equal(r["w2n"], np.cumsum(r["w_sizes"]) - r["w_sizes"])
    assert r["M"] == int((r["w_sizes"].astype(np.int64) ** 2).sum())
    sc = coords[r["n2n"]]
    win = np.concatenate([sc[:, :1], np.floor_divide(sc[:, 1:], ws * stride)], axis=1)
    starts = r["w2n"]
    keys = [tuple(win[s]) for s in starts]
    assert keys == sorted(keys) and len(set(keys)) == len(keys)             # strictly increasing
    for s, c in zip(starts, r["w_sizes"]):
        assert (win[s:s + c] == win[s]).all()                              # one window per segment
        assert (np.diff(r["w_w_id"][s:s + c]) > 0).all()                   # local ids increasing
    loc = np.floor_divide(sc[:, 1:], stride) % ws
    np.testing.assert_array_equal(r["w_w_id"], (loc[:, 0] * ws + loc[:, 1]) * ws + loc[:, 2])


def test_negative_coordinates_floor(oracle_lib):
    # voxel -1 belongs to window -1 (floor), local id ws-1: not to window 0
    coords = np.array([[0, -1, 0, 0], [0, 0, 0, 0], [0, -5, 0, 0], [0, -6, 0, 0]], np.int32)
    r = oracle_lib.window_index(coords, 1, 5, 0)
    assert r["W"] == 3
    np.testing.assert_array_equal(r["w_sizes"], [1, 2, 1])
    np.testing.assert_array_equal(r["n2n"], [3, 2, 0, 1])                 # windows -2, -1, -1, 0
    np.testing.assert_array_equal(r["w_w_id"], [4 * 25, 0, 4 * 25, 0])


def test_translation_by_one_window_keeps_index(oracle_lib):
    rng = np.random.default_rng(5)
    ws, stride = 5, 2
    coords = random_scene(rng, 500, stride=stride)
    moved = coords.copy()
    moved[:, 1:] += ws * stride
    a = oracle_lib.window_index(coords, stride, ws, 2)
    b = oracle_lib.window_index(moved, stride, ws, 2)
    for key in ("n2n", "w_w_id", "w_sizes", "w2n"):
        np.testing.assert_array_equal(a[key], b[key])


def test_shift_equals_moved_coordinates(oracle_lib):
    # get_shifted_sp adds shift*stride to every coordinate before the window split
    rng = np.random.default_rng(6)
    ws, stride, shift = 7, 2, 3
    coords = random_scene(rng, 500, stride=stride)
    moved = coords.copy()
    moved[:, 1:] += shift * stride
    a = oracle_lib.window_index(coords, stride, ws, shift)
    b = oracle_lib.window_index(moved, stride, ws, 0)
    for key in ("n2n", "w_w_id", "w_sizes", "w2n"):
        np.testing.assert_array_equal(a[key], b[key])


def test_duplicate_coordinates_keep_row_order(oracle_lib):
    coords = np.array([[0, 1, 1, 1], [0, 0, 0, 0], [0, 1, 1, 1], [0, 1, 1, 1]], np.int32)
    r = oracle_lib.window_index(coords, 1, 5, 0)
    np.testing.assert_array_equal(r["n2n"], [1, 0, 2, 3])


def test_empty_and_single(oracle_lib):
    r = oracle_lib.window_index(np.zeros((0, 4), np.int32), 1, 5, 0)
    assert r["W"] == 0 and r["M"] == 0 and r["n2n"].shape == (0,)
    r = oracle_lib.window_index(np.array([[2, 7, 8, 9]], np.int32), 1, 5, 0)
    assert r["W"] == 1 and r["M"] == 1 and r["w_w_id"][0] == (2 * 5 + 3) * 5 + 4


def test_pair_index_matches_both_reference_statements(oracle_lib):
    rng = np.random.default_rng(7)
    w_sizes = rng.integers(1, 9, size=40).astype(np.int32)
    w2m, m2w, xo, yo = oracle_lib.pair_index(w_sizes)
    # python statement (cumsum / scatter form)
    p_w2m, p_m2w, p_x, p_y = numpy_ref.pair_index_python_statement(w_sizes)
    np.testing.assert_array_equal(w2m, p_w2m)
    np.testing.assert_array_equal(m2w, p_m2w)
    np.testing.assert_array_equal(xo, p_x)
    np.testing.assert_array_equal(yo, p_y)
    # kernel statement: w = m2w[m]; off = m - w2m[w]; q = w2n[w] + off / n_w; k = w2n[w] + off % n_w
    w2n = np.cumsum(w_sizes) - w_sizes
    for m in range(0, len(m2w), 7):
        w = m2w[m]
        off = m - w2m[w]
        assert xo[m] == w2n[w] + off // w_sizes[w]
        assert yo[m] == w2n[w] + off % w_sizes[w]
    # every (query, key) pair of a window appears exactly once
    assert len(set(zip(xo.tolist(), yo.tolist()))) == len(xo) == int((w_sizes.astype(int) ** 2).sum())
