"""GPU parity of the grid-bucketed KNN (bit-exact indices and fp32 squared distances)."""
import numpy as np
import pytest
import torch

from swin3d_amd import synth

pytestmark = pytest.mark.gpu


def _run(k, src, qry, so, qo, cell=0.0):
    import swin3d_amd
    c = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    idx, d2 = swin3d_amd.knn_query(k, c(src), c(qry), c(so), c(qo), cell_size=cell)
    torch.cuda.synchronize()
    return idx.cpu().numpy(), d2.cpu().numpy()


def _compare(oracle_lib, k, src, qry, so, qo, cell=0.0):
    ridx, rd2 = oracle_lib.knn(k, src, qry, so, qo)
    idx, d2 = _run(k, src, qry, so, qo, cell)
    np.testing.assert_array_equal(idx, ridx)
    np.testing.assert_array_equal(d2, rd2)


@pytest.mark.parametrize("k", [1, 3, 5, 16, 33, 64])
@pytest.mark.parametrize("cell", [0.0, 0.7, 5.0, 1000.0])
def test_random_clouds(oracle_lib, hip_lib, k, cell):
    rng = np.random.default_rng(k)
    src = (rng.random((4000, 3)) * [30, 20, 5]).astype(np.float32)
    qry = (rng.random((1500, 3)) * [34, 24, 9] - 2).astype(np.float32)     # some queries outside the box
    so, qo = np.array([1500, 4000], np.int32), np.array([700, 1500], np.int32)
    _compare(oracle_lib, k, src, qry, so, qo, cell)


def test_lattice_ties_go_to_lower_row(oracle_lib, hip_lib):
    g = np.arange(0, 12, dtype=np.float32)
    src = np.stack(np.meshgrid(g, g, g, indexing="ij"), -1).reshape(-1, 3)
    rng = np.random.default_rng(5)
    src = src[rng.permutation(src.shape[0])]
    qry = np.concatenate([src[:200], src[:200] + np.float32(0.5)])          # on and between lattice points
    one = lambda n: np.array([n], np.int32)
    for k in (3, 7, 16):
        for cell in (0.0, 1.0, 2.5):
            _compare(oracle_lib, k, src, qry, one(src.shape[0]), one(qry.shape[0]), cell)


def test_short_empty_and_unassigned_segments(oracle_lib, hip_lib):
    rng = np.random.default_rng(6)
    src = rng.random((50, 3)).astype(np.float32) * 10
    qry = rng.random((30, 3)).astype(np.float32) * 10
    so = np.array([2, 2, 40], np.int32)       # 2 sources, none, 38; rows 40..49 belong to no segment
    qo = np.array([10, 20, 25], np.int32)     # queries 25..29 belong to no segment
    ridx, rd2 = oracle_lib.knn(4, src, qry, so, qo)
    idx, d2 = _run(4, src, qry, so, qo)
    np.testing.assert_array_equal(idx, ridx)
    np.testing.assert_array_equal(d2, rd2)
    assert (idx[10:20] == -1).all() and (idx[25:] == -1).all() and (idx[:10, 2:] == -1).all()
    assert (d2[25:] == np.float32(2147483648.0)).all()


def test_identical_points_and_degenerate_extent(oracle_lib, hip_lib):
    src = np.zeros((100, 3), np.float32)
    src[:, 0] = np.repeat(np.arange(10, dtype=np.float32), 10)             # a line with 10-fold duplicates
    qry = np.array([[4.2, 0, 0], [100, 100, 100], [-3, 0, 0]], np.float32)
    one = lambda n: np.array([n], np.int32)
    _compare(oracle_lib, 16, src, qry, one(100), one(3))
    _compare(oracle_lib, 16, np.zeros((40, 3), np.float32), qry, one(40), one(3))   # all sources identical


def test_autograd_function_returns_euclidean_distance(oracle_lib, hip_lib):
    import swin3d_amd
    rng = np.random.default_rng(7)
    src = (rng.random((500, 3)) * 10).astype(np.float32)
    qry = (rng.random((100, 3)) * 10).astype(np.float32)
    so, qo = torch.tensor([500], dtype=torch.int32).cuda(), torch.tensor([100], dtype=torch.int32).cuda()
    idx, dist = swin3d_amd.KNN.apply(3, torch.from_numpy(src).cuda(), torch.from_numpy(qry).cuda(), so, qo)
    ridx, rd2 = oracle_lib.knn(3, src, qry, so.cpu().numpy(), qo.cpu().numpy())
    assert idx.dtype == torch.int32 and dist.dtype == torch.float32
    np.testing.assert_array_equal(idx.cpu().numpy(), ridx)
    np.testing.assert_array_equal(dist.cpu().numpy(), np.sqrt(rd2))


def _knn_scene():
    scene = synth.make_room((10, 8, 3), 30, 200_000, seed=0)
    coarse, _ = synth.grid_downsample(scene, 2)
    centres = (coarse.coords[:, 1:].astype(np.float32) + np.float32(1.0))[:50_000]   # (cell + 0.5) * 2
    return scene.xyz, np.ascontiguousarray(centres)


@pytest.mark.parametrize("direction", ["down", "up"])
def test_headline_sizes(oracle_lib, hip_lib, direction):
    """Config 4: 200k sources / 50k cell-centre queries, K=16, and the reverse with K=3.
    Whole output: every row is compared bit for bit with the brute-force oracle (10^10 candidate distances, about a
    second on the host threads), on top of the ordering and self-consistency properties."""
    fine, centres = _knn_scene()
    src, qry, k = (fine, centres, 16) if direction == "down" else (centres, fine, 3)
    one = lambda n: np.array([n], np.int32)
    idx, d2 = _run(k, src, qry, one(src.shape[0]), one(qry.shape[0]))
    assert (idx >= 0).all() and (idx < src.shape[0]).all()
    assert (np.diff(d2, axis=1) >= 0).all()
    tie = np.diff(d2, axis=1) == 0
    assert (np.diff(idx, axis=1)[tie] > 0).all()                          # equal distance: ascending row
    d = src[idx] - qry[:, None, :]
    recomputed = ((d[..., 0] * d[..., 0]).astype(np.float32) + (d[..., 1] * d[..., 1]).astype(np.float32)).astype(np.float32)
    recomputed = (recomputed + (d[..., 2] * d[..., 2]).astype(np.float32)).astype(np.float32)
    np.testing.assert_array_equal(d2, recomputed)
    ridx, rd2 = oracle_lib.knn(k, src, qry, one(src.shape[0]), one(qry.shape[0]))
    np.testing.assert_array_equal(idx, ridx)
    np.testing.assert_array_equal(d2, rd2)


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("channels", [48, 7])
def test_interpolate_matches_oracle(oracle_lib, hip_lib, half, channels):
    """Fused inverse-distance interpolation (K=3) against the oracle: fp32 within 1e-5 of the largest
    neighbour feature, fp16 within 2e-3 absolute; two segments, one with fewer sources than K."""
    import swin3d_amd
    rng = np.random.default_rng(41)
    src = (rng.random((403, 3)) * 8).astype(np.float32)
    qry = (rng.random((900, 3)) * 8).astype(np.float32)
    qry[:20] = src[:20]                                     # queries on top of sources
    so, qo = np.array([401, 403], np.int32), np.array([850, 900], np.int32)
    feat = rng.standard_normal((403, channels)).astype(np.float32)
    if half:
        feat = feat.astype(np.float16).astype(np.float32)
    t = lambda a: torch.from_numpy(a).cuda()
    idx, d2 = swin3d_amd.knn_query(3, t(src), t(qry), t(so), t(qo))
    ridx, rd2 = oracle_lib.knn(3, src, qry, so, qo)
    np.testing.assert_array_equal(idx.cpu().numpy(), ridx)
    assert (ridx[850:, 2] == -1).all()
    ref = oracle_lib.knn_interpolate(ridx, rd2, feat)
    f = t(feat).half() if half else t(feat)
    got = swin3d_amd.knn_interpolate(idx, d2, f)
    torch.cuda.synchronize()
    assert got.dtype == f.dtype
    tol = 2e-3 if half else 1e-5 * np.abs(feat).max()
    assert np.abs(got.double().cpu().numpy() - ref).max() <= tol


def test_interpolate_autograd(oracle_lib, hip_lib):
    """Gradient w.r.t. the source features = transposed weights applied to the output gradient."""
    import swin3d_amd
    rng = np.random.default_rng(42)
    src = (rng.random((300, 3)) * 6).astype(np.float32)
    qry = (rng.random((700, 3)) * 6).astype(np.float32)
    one = lambda n: torch.tensor([n], dtype=torch.int32).cuda()
    t = lambda a: torch.from_numpy(a).cuda()
    idx, d2 = swin3d_amd.knn_query(3, t(src), t(qry), one(300), one(700))
    feat = t(rng.standard_normal((300, 16)).astype(np.float32)).requires_grad_(True)
    dout = rng.standard_normal((700, 16)).astype(np.float32)
    out = swin3d_amd.KNNInterpolate.apply(idx, d2, feat)
    out.backward(t(dout))
    # linear map: <out, dout> = <feat, grad> for the oracle's weights
    basis = np.eye(300, dtype=np.float32)
    weights = oracle_lib.knn_interpolate(idx.cpu().numpy(), d2.cpu().numpy(), basis)     # [700,300]
    ref = weights.T @ dout.astype(np.float64)
    np.testing.assert_allclose(feat.grad.double().cpu().numpy(), ref, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("channels", [160, 37])
def test_max_pool_over_neighbours_matches_gather_and_max(hip_lib, dtype, channels):
    """s3d_knn_max_pool against the tensor statement (clamped gather to [Nq,K,C], max over K): bit-exact, with
    padded slots (segments with fewer than K sources) in the index."""
    from swin3d_amd.sparse_dl.knn import knn_max_pool, knn_query
    rng = np.random.default_rng(12)
    src = torch.from_numpy(rng.uniform(0, 10, (3000, 3)).astype(np.float32)).cuda()
    qry = torch.from_numpy(rng.uniform(0, 10, (700, 3)).astype(np.float32)).cuda()
    so = torch.tensor([2990, 3000], dtype=torch.int32).cuda()      # second segment: 10 sources for K = 16
    qo = torch.tensor([600, 700], dtype=torch.int32).cuda()
    idx, _ = knn_query(16, src, qry, so, qo)
    assert int((idx < 0).sum()) == 100 * 6
    feat = torch.from_numpy(rng.standard_normal((3000, channels)).astype(np.float32)).cuda().to(dtype)
    ref = feat[idx.view(-1).long().clamp(min=0)].view(700, 16, channels).amax(dim=1)
    assert torch.equal(knn_max_pool(idx, feat), ref)
