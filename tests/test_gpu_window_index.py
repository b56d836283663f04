"""GPU parity of the window sort / segment offsets (bit-exact against the CPU oracle)."""
import numpy as np
import pytest
import torch

from conftest import random_scene
from swin3d_amd import synth

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["grid", "sort"], autouse=True)
def index_path(request, monkeypatch):
    """Every test of this file runs on both builders: s3d_window_index_grid (counting sort over the window
    lattice, the default where it applies) and s3d_window_index (sort of all voxels)."""
    from swin3d_amd import window_index
    monkeypatch.setattr(window_index, "USE_GRID_PATH", request.param == "grid")
    return request.param


def _run(coords, stride, ws, shift):
    import swin3d_amd
    index = swin3d_amd.build_window_index(torch.from_numpy(coords).cuda(), stride, ws, shift)
    torch.cuda.synchronize()
    return index


def _compare(oracle_lib, coords, stride, ws, shift):
    ref = oracle_lib.window_index(coords, stride, ws, shift)
    got = _run(coords, stride, ws, shift)
    assert got.num_windows == ref["W"] and got.num_pairs == ref["M"]
    assert got.max_window_voxels == (int(ref["w_sizes"].max()) if ref["W"] else 0)
    np.testing.assert_array_equal(got.n2n.cpu().numpy(), ref["n2n"])
    np.testing.assert_array_equal(got.w_w_id.cpu().numpy(), ref["w_w_id"])
    np.testing.assert_array_equal(got.w_sizes.cpu().numpy(), ref["w_sizes"])
    np.testing.assert_array_equal(got.w2n.cpu().numpy(), ref["w2n"])
    return got


@pytest.mark.parametrize("ws,stride,shift", [(5, 1, 0), (5, 1, 2), (7, 2, 3), (7, 4, 0), (3, 8, 1), (10, 1, 5)])
@pytest.mark.parametrize("seed", [0, 1])
def test_random_scenes(oracle_lib, hip_lib, ws, stride, shift, seed):
    rng = np.random.default_rng(seed)
    coords = random_scene(rng, 5000, extent=(40, 40, 12), batches=3, stride=stride)
    _compare(oracle_lib, coords, stride, ws, shift)


def test_duplicates_keep_row_order(oracle_lib, hip_lib):
    rng = np.random.default_rng(2)
    coords = random_scene(rng, 3000, extent=(6, 6, 3), duplicates=True)
    assert len({tuple(r) for r in coords.tolist()}) < coords.shape[0]
    _compare(oracle_lib, coords, 1, 5, 0)


def test_empty_single_and_one_window(oracle_lib, hip_lib):
    _compare(oracle_lib, np.zeros((0, 4), np.int32), 1, 5, 0)
    _compare(oracle_lib, np.array([[3, -7, 8, 9]], np.int32), 1, 5, 2)
    g = np.stack(np.meshgrid(np.arange(5), np.arange(5), np.arange(5), indexing="ij"), -1).reshape(-1, 3)
    coords = np.concatenate([np.zeros((125, 1), np.int64), g], 1).astype(np.int32)[::-1].copy()
    got = _compare(oracle_lib, coords, 1, 5, 0)
    assert got.num_windows == 1 and got.num_pairs == 125 * 125


def test_out_of_range_coordinates_are_reported(hip_lib):
    import swin3d_amd
    coords = torch.tensor([[0, 0, 0, 0], [0, 5 * 9000, 0, 0]], dtype=torch.int32).cuda()
    with pytest.raises(ValueError, match="range"):
        swin3d_amd.build_window_index(coords, 1, 5, 0)
    with pytest.raises(ValueError):
        swin3d_amd.build_window_index(coords, 1, 11, 0)        # window size beyond the key layout


@pytest.mark.parametrize("shift", [0, 2])
def test_headline_room(oracle_lib, hip_lib, shift):
    scene = synth.make_room((10, 8, 3), 30, 200_000, seed=0)
    rng = np.random.default_rng(0)
    coords = scene.coords[rng.permutation(scene.coords.shape[0])]     # arbitrary input order
    got = _compare(oracle_lib, coords, 1, 5, shift)
    assert got.inverse()[got.n2n.long()].tolist()[:100] == list(range(100))


def test_get_index01_matches_reference_formulas(oracle_lib, hip_lib):
    """n_coords = window-local voxel + fraction, signals appended, all gathered by n2n
    (swin3d_layers.py:800-804); pair arrays on request."""
    import swin3d_amd
    from helpers import n_coords_from_scene
    rng = np.random.default_rng(4)
    coords = random_scene(rng, 2000, extent=(15, 15, 6), batches=2)
    frac = rng.random((2000, 3)).astype(np.float32)
    sig = rng.uniform(-1, 1, (2000, 6)).astype(np.float32)
    args = swin3d_amd.get_index01(torch.from_numpy(coords).cuda(), 1, 5, torch.from_numpy(frac).cuda(),
                                  torch.from_numpy(sig).cuda(), shift=2, materialize_pairs=True)
    x_off, y_off, m2w, w_sizes, w2n, n2n, w2m, n_coords = args
    index, scaled = n_coords_from_scene(oracle_lib, coords, frac, sig, 1, 5, 4, "XYZ_RGB_NORM", shift=2)
    np.testing.assert_array_equal(n2n.cpu().numpy(), index["n2n"])
    got_scaled = swin3d_amd.scale_crse_coords(n_coords, 4, "XYZ_RGB_NORM").cpu().numpy()
    np.testing.assert_array_equal(got_scaled, scaled)                 # bit-exact fp32
    o_w2m, o_m2w, o_x, o_y = oracle_lib.pair_index(index["w_sizes"])
    np.testing.assert_array_equal(x_off.cpu().numpy(), o_x)
    np.testing.assert_array_equal(y_off.cpu().numpy(), o_y)
    np.testing.assert_array_equal(m2w.cpu().numpy(), o_m2w)
    np.testing.assert_array_equal(w2m.cpu().numpy(), o_w2m)


@pytest.mark.parametrize("num_signals", [0, 3, 6])
def test_window_signals_match_the_tensor_statement(hip_lib, num_signals):
    """The fused signal-matrix kernel against the reference's tensor statements (window-local voxel + fraction,
    other signals appended, gathered into sorted order; then the quantiser scales): bit-exact, with the signals
    given as a strided column slice as the encoder does."""
    import swin3d_amd
    rng = np.random.default_rng(7)
    ws, quant = 7, 4
    coords = torch.from_numpy(random_scene(rng, 6000, extent=(30, 30, 10), batches=2, stride=2)).cuda()
    table = torch.from_numpy(rng.uniform(-1, 1, (6000, 10)).astype(np.float32)).cuda()
    frac, colors = table[:, 1:4].contiguous(), table[:, 4:4 + num_signals]
    index = swin3d_amd.build_window_index(coords, 2, ws, 3)
    order = index.n2n.long()
    ref = torch.cat([index.local_xyz().float() + frac[order], colors[order]], 1)
    got = swin3d_amd.window_signals(index, frac, colors)
    assert torch.equal(got, ref)
    scale = torch.tensor([quant] * 3 + [2 * quant] * num_signals, dtype=torch.float32, device="cuda")
    got = swin3d_amd.window_signals(index, frac, table[:, 4:], num_signals, quant, 2 * quant)
    assert torch.equal(got, ref * scale)


def test_several_window_sets_in_one_call(oracle_lib, hip_lib):
    """build_window_indices enqueues all sets before its one host wait; each equals its single build."""
    import swin3d_amd
    rng = np.random.default_rng(8)
    coords = random_scene(rng, 4000, extent=(30, 30, 10), batches=2, stride=1)
    sets = swin3d_amd.build_window_indices(torch.from_numpy(coords).cuda(), 1, 5, (0, 2))
    for got, shift in zip(sets, (0, 2)):
        ref = oracle_lib.window_index(coords, 1, 5, shift)
        assert got.num_windows == ref["W"] and got.num_pairs == ref["M"]
        np.testing.assert_array_equal(got.n2n.cpu().numpy(), ref["n2n"])
        np.testing.assert_array_equal(got.w_sizes.cpu().numpy(), ref["w_sizes"])
        np.testing.assert_array_equal(got.w2n.cpu().numpy(), ref["w2n"])


def test_lattice_too_large_falls_back_to_the_sort(oracle_lib, hip_lib, index_path):
    """Voxels spread so far apart that the bounding lattice of their windows has more cells than the grid path
    takes: s3d_window_index_grid reports it (status bit 1, nothing written) and the wrapper builds the set with the
    sort; the result is the oracle's either way."""
    import ctypes
    rng = np.random.default_rng(9)
    coords = np.concatenate([np.zeros((3000, 1), np.int64), rng.integers(-30000, 30000, size=(3000, 3))], 1).astype(np.int32)
    coords = np.unique(coords, axis=0)
    _compare(oracle_lib, coords, 1, 5, 2)
    if index_path == "grid":
        n = coords.shape[0]
        c = torch.from_numpy(coords).cuda()
        outs = [torch.full((n,), -7, dtype=torch.int32, device="cuda") for _ in range(4)]
        counts = torch.zeros(4, dtype=torch.int64, device="cuda")
        ws_bytes = hip_lib.s3d_window_index_grid_workspace_bytes(n)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
        status = hip_lib.s3d_window_index_grid(c.data_ptr(), n, 1, 5, 2, *(o.data_ptr() for o in outs), counts.data_ptr(),
                                               ws.data_ptr(), ws_bytes, torch.cuda.current_stream().cuda_stream)
        assert status == 0
        torch.cuda.synchronize()
        assert int(counts[3]) & 2
        assert all(bool((o == -7).all()) for o in outs)
