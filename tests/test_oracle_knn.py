"""Pins oracle.knn (CPU): numpy lexsort brute force, scipy cKDTree, constructed ties,
batch segments, short segments; documents where the reference's heap order differs."""
import numpy as np
import pytest
from scipy.spatial import cKDTree

from oracle import numpy_ref


def _cloud(rng, n, scale=20.0):
    return (rng.random((n, 3)) * scale).astype(np.float32)


@pytest.mark.parametrize("k", [1, 3, 16])
def test_matches_lexsort_bruteforce(oracle_lib, k):
    rng = np.random.default_rng(k)
    src, qry = _cloud(rng, 300), _cloud(rng, 90)
    so, qo = np.array([120, 300], np.int32), np.array([40, 90], np.int32)
    idx, d2 = oracle_lib.knn(k, src, qry, so, qo)
    ridx, rd2 = numpy_ref.knn_bruteforce(k, src, qry, so, qo)
    np.testing.assert_array_equal(idx, ridx)
    np.testing.assert_array_equal(d2, rd2)          # bit-exact fp32 distances


def test_matches_ckdtree_on_tie_free_input(oracle_lib):
    rng = np.random.default_rng(21)
    src, qry = _cloud(rng, 2000), _cloud(rng, 400)
    so, qo = np.array([2000], np.int32), np.array([400], np.int32)
    idx, d2 = oracle_lib.knn(8, src, qry, so, qo)
    dist, tidx = cKDTree(src.astype(np.float64)).query(qry.astype(np.float64), k=8)
    np.testing.assert_array_equal(idx, tidx.astype(np.int32))
    np.testing.assert_allclose(np.sqrt(d2), dist, rtol=1e-5)
    assert (np.diff(d2, axis=1) >= 0).all()


def test_ties_go_to_the_lower_row(oracle_lib):
    # integer lattice: many exactly equal distances
    g = np.arange(-2, 3, dtype=np.float32)
    src = np.stack(np.meshgrid(g, g, g, indexing="ij"), -1).reshape(-1, 3)
    qry = np.zeros((1, 3), np.float32)
    so, qo = np.array([src.shape[0]], np.int32), np.array([1], np.int32)
    idx, d2 = oracle_lib.knn(5, src, qry, so, qo)
    d_all = (src ** 2).sum(1)
    expect = np.lexsort((np.arange(src.shape[0]), d_all))[:5]
    np.testing.assert_array_equal(idx[0], expect)
    np.testing.assert_array_equal(d2[0], [0, 1, 1, 1, 1])
    # the six distance-1 points have rows 37 < 57 < 61 < 63 < 67 < 87: the lowest four are kept
    assert idx[0, 1:].tolist() == sorted(np.flatnonzero(d_all == 1).tolist())[:4]


def test_heap_order_differs_only_on_ties(oracle_lib):
    rng = np.random.default_rng(23)
    src, qry = _cloud(rng, 500), _cloud(rng, 60)
    so, qo = np.array([500], np.int32), np.array([60], np.int32)
    a = oracle_lib.knn(16, src, qry, so, qo)
    b = oracle_lib.knn(16, src, qry, so, qo, heap_order=True)
    np.testing.assert_array_equal(a[0], b[0])        # tie-free: identical
    np.testing.assert_array_equal(a[1], b[1])
    # the documented tie case d = [1,1,1,0,1], K = 3: canonical {3,0,1}, heap order keeps {3,1,2}
    src = np.array([[1, 0, 0], [0, 1, 0], [0, 0, 1], [0, 0, 0], [-1, 0, 0]], np.float32)
    qry = np.zeros((1, 3), np.float32)
    so, qo = np.array([5], np.int32), np.array([1], np.int32)
    assert oracle_lib.knn(3, src, qry, so, qo)[0][0].tolist() == [3, 0, 1]
    assert sorted(oracle_lib.knn(3, src, qry, so, qo, heap_order=True)[0][0].tolist()) == [1, 2, 3]


def test_segments_and_padding(oracle_lib):
    rng = np.random.default_rng(24)
    src, qry = _cloud(rng, 12), _cloud(rng, 9)
    so = np.array([2, 2, 12], np.int32)     # segment 1 is empty, segment 0 has 2 < K sources
    qo = np.array([3, 6, 9], np.int32)
    idx, d2 = oracle_lib.knn(4, src, qry, so, qo)
    assert set(idx[:3, :2].ravel().tolist()) <= {0, 1} and (idx[:3, 2:] == -1).all()
    assert (d2[:3, 2:] == np.float32(2147483648.0)).all()
    assert (idx[3:6] == -1).all()
    assert ((idx[6:] >= 2) & (idx[6:] < 12)).all()
    ridx, rd2 = numpy_ref.knn_bruteforce(4, src, qry, so, qo)
    np.testing.assert_array_equal(idx, ridx)
    np.testing.assert_array_equal(d2, rd2)


def test_distance_expression_is_unfused_fp32(oracle_lib):
    # dx*dx + dy*dy with a fused multiply-add differs from the individually rounded form here
    src = np.array([[1.0000001, 3.0000002, 0.3]], np.float32)
    qry = np.array([[0.1, 0.2, 0.7]], np.float32)
    one = np.array([1], np.int32)
    _, d2 = oracle_lib.knn(1, src, qry, one, one)
    dx, dy, dz = (np.float32(src[0, a] - qry[0, a]) for a in range(3))
    expect = np.float32(np.float32(np.float32(dx * dx) + np.float32(dy * dy)) + np.float32(dz * dz))
    assert d2[0, 0] == expect


def test_interpolate_closed_forms(oracle_lib):
    """Pins of the inverse-distance interpolation: hand-computed weights, a constant field, a query on
    top of a source, padded slots."""
    # two neighbours at distances 1 and 3: weights (1/1, 1/3) / (4/3) = 0.75, 0.25
    idx = np.array([[0, 1]], np.int32)
    d2 = np.array([[1.0, 9.0]], np.float32)
    feat = np.array([[8.0, -4.0], [0.0, 4.0]], np.float32)
    np.testing.assert_allclose(oracle_lib.knn_interpolate(idx, d2, feat), [[6.0, -2.0]], rtol=1e-7)
    # three neighbours at distances 1, 2, 4: weights 4/7, 2/7, 1/7
    idx = np.array([[2, 0, 1]], np.int32)
    d2 = np.array([[1.0, 4.0, 16.0]], np.float32)
    feat = np.array([[7.0], [14.0], [21.0]], np.float32)       # rows 2, 0, 1 -> 21, 7, 14
    np.testing.assert_allclose(oracle_lib.knn_interpolate(idx, d2, feat), [[(4 * 21 + 2 * 7 + 14) / 7.0]], rtol=1e-7)
    # constant field stays constant; a query on a source returns that source (weight 1e8 against ~1)
    rng = np.random.default_rng(27)
    src, qry = _cloud(rng, 200), _cloud(rng, 50)
    qry[:10] = src[:10]
    one_s, one_q = np.array([200], np.int32), np.array([50], np.int32)
    idx, d2 = oracle_lib.knn(3, src, qry, one_s, one_q)
    const = np.full((200, 5), 3.25, np.float32)
    np.testing.assert_allclose(oracle_lib.knn_interpolate(idx, d2, const), 3.25, rtol=1e-12)
    feat = rng.standard_normal((200, 5)).astype(np.float32)
    out = oracle_lib.knn_interpolate(idx, d2, feat)
    np.testing.assert_allclose(out[:10], feat[:10], rtol=0, atol=1e-6)
    # result lies in the convex hull of the neighbours' features
    lo, hi = feat[idx].min(1), feat[idx].max(1)
    assert (out >= lo - 1e-9).all() and (out <= hi + 1e-9).all()
    # padded slots (segment with fewer sources than K) carry no weight
    idx = np.array([[1, -1, -1]], np.int32)
    d2 = np.array([[4.0, 2147483648.0, 2147483648.0]], np.float32)
    np.testing.assert_allclose(oracle_lib.knn_interpolate(idx, d2, feat), feat[1:2], rtol=1e-12)
