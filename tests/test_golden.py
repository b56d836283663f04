"""The committed fixtures of tests/golden/ (brute-force numpy vectors, see make_golden.py) against
the C oracle (CPU) and against the HIP library through its Python surface (GPU)."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    with np.load(os.path.join(GOLDEN, name), allow_pickle=False) as f:
        return {k: f[k] for k in f.files}


def test_oracle_attention_matches_fixture(oracle_lib):
    g = _load("attn_small.npz")
    got = oracle_lib.attn_fwd(g["q"], g["k"], g["v"], g["tq"], g["tk"], g["tv"], g["table_sizes"],
                              g["w_sizes"], g["w2n"], g["n2n"], g["n_coords"])
    np.testing.assert_allclose(got, g["out"], rtol=1e-12, atol=1e-13)


def test_oracle_window_index_matches_fixture(oracle_lib):
    g = _load("window_index_small.npz")
    idx = oracle_lib.window_index(g["coords"], int(g["stride"]), int(g["ws"]), int(g["shift"]))
    for key in ("n2n", "w_w_id", "w_sizes", "w2n"):
        np.testing.assert_array_equal(idx[key], g[key])
    assert idx["W"] == int(g["W"]) and idx["M"] == int(g["M"])


def test_oracle_knn_matches_fixture(oracle_lib):
    g = _load("knn_small.npz")
    idx, d2 = oracle_lib.knn(int(g["k"]), g["src"], g["qry"], g["src_offset"], g["query_offset"])
    np.testing.assert_array_equal(idx, g["idx"])
    np.testing.assert_array_equal(d2, g["d2"])


@pytest.mark.gpu
@pytest.mark.parametrize("half", [False, True])
def test_hip_attention_matches_fixture(hip_lib, half):
    import torch
    import swin3d_amd
    from gpu_helpers import assert_attn_close
    g = _load("attn_small.npz")
    dev = torch.device("cuda")
    dtype = torch.float16 if half else torch.float32
    f = lambda a: torch.from_numpy(a).to(dev).to(dtype)       # inputs are fp16-exact
    t = lambda a: torch.from_numpy(a).to(dev)
    out = swin3d_amd.window_attention_forward(
        f(g["q"]), f(g["k"]), f(g["v"]), f(g["tq"]), f(g["tk"]), f(g["tv"]), t(g["table_sizes"]),
        t(g["w_sizes"]), t(g["w2n"]), t(g["n2n"]), t(g["n_coords"]))
    torch.cuda.synchronize()
    assert_attn_close(out.double().cpu().numpy(), g["out"], dtype)


@pytest.mark.gpu
def test_hip_window_index_matches_fixture(hip_lib):
    import torch
    import swin3d_amd
    g = _load("window_index_small.npz")
    idx = swin3d_amd.build_window_index(torch.from_numpy(g["coords"]).cuda(), int(g["stride"]), int(g["ws"]),
                                        int(g["shift"]))
    assert idx.num_windows == int(g["W"]) and idx.num_pairs == int(g["M"])
    np.testing.assert_array_equal(idx.n2n.cpu().numpy(), g["n2n"])
    np.testing.assert_array_equal(idx.w_w_id.cpu().numpy(), g["w_w_id"])
    np.testing.assert_array_equal(idx.w_sizes.cpu().numpy(), g["w_sizes"])
    np.testing.assert_array_equal(idx.w2n.cpu().numpy(), g["w2n"])


@pytest.mark.gpu
def test_hip_knn_matches_fixture(hip_lib):
    import torch
    import swin3d_amd
    g = _load("knn_small.npz")
    t = lambda a: torch.from_numpy(a).cuda()
    idx, d2 = swin3d_amd.knn_query(int(g["k"]), t(g["src"]), t(g["qry"]), t(g["src_offset"]), t(g["query_offset"]))
    np.testing.assert_array_equal(idx.cpu().numpy(), g["idx"])
    np.testing.assert_array_equal(d2.cpu().numpy(), g["d2"])
