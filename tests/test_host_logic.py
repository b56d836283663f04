"""Host-side mirror of the reference interface (runs without a GPU)."""
import numpy as np
import pytest
import torch

import swin3d_amd
from swin3d_amd import crse
from swin3d_amd.sparse_dl.attn import attn_coff
from swin3d_amd.sparse_dl.knn import KNN


def test_enum_wire_values_match_the_reference():
    # enum.auto() order of Swin3D/sparse_dl/attn/attn_coff.py:20-40
    assert [e.value for e in attn_coff.PosEmb] == [1, 2, 3] and attn_coff.PosEmb.SEPARATE.value == 3
    assert attn_coff.TableDims.D0.value == 3
    assert attn_coff.IndexMode.DIRECT.value == 1 and attn_coff.IndexMode.INDIRECT.value == 2
    assert [e.name for e in attn_coff.PrecisionMode] == ["HALF_ALL", "HALF_FORWARD", "HALF_NONE"]


def test_table_sizes_follow_window_attention():
    # Swin3D-S stage 1: ws 5, quant 4, 6 heads x 8 -> xyz rows 40, colour / normal rows 32
    assert crse.crse_table_rows(5, 4, "XYZ_RGB_NORM") == [40] * 3 + [32] * 6
    assert crse.crse_table_sizes(5, 4, 6, 8, "XYZ_RGB_NORM") == [1920] * 3 + [1536] * 6
    assert crse.crse_table_sizes(5, 4, 6, 8, "XYZ_RGB") == [1920] * 3 + [1536] * 3
    assert crse.crse_table_sizes(7, 4, 6, 16, "XYZ_RGB_NORM") == [5376] * 3 + [3072] * 6
    assert sum(crse.crse_table_sizes(5, 4, 6, 8, "XYZ_RGB_NORM")) == 14976
    with pytest.raises(ValueError):
        crse.crse_table_rows(5, 4, "RGB")


def test_scale_crse_coords():
    n_coords = torch.arange(18, dtype=torch.float32).reshape(2, 9) / 7
    got = crse.scale_crse_coords(n_coords, 4, "XYZ_RGB_NORM")
    expect = torch.cat([n_coords[:, :3] * 4, n_coords[:, 3:6] * 8, n_coords[:, 6:9] * 8], 1)
    assert torch.equal(got, expect)
    assert crse.scale_crse_coords(n_coords, 4, "XYZ").shape == (2, 3)
    with pytest.raises(ValueError):
        crse.scale_crse_coords(n_coords[:, :4], 4, "XYZ_RGB")


@pytest.mark.parametrize("autocast", [False, True])
@pytest.mark.parametrize("precision", list(attn_coff.PrecisionMode))
def test_compute_dtype_policy(autocast, precision, monkeypatch):
    # attn_coff.py:172-175: autocast dtype iff autocast is on and precision != HALF_NONE.
    # torch disables CUDA autocast on a machine without a GPU, so the two queries are patched.
    monkeypatch.setattr(torch, "is_autocast_enabled", lambda *a: autocast)
    monkeypatch.setattr(torch, "get_autocast_dtype", lambda dev: torch.float16)
    got = attn_coff._compute_dtype(precision)
    expect = torch.float16 if autocast and precision != attn_coff.PrecisionMode.HALF_NONE else torch.float32
    assert got == expect


def test_cpu_tensors_are_rejected_not_emulated():
    q = torch.zeros(4, 2, 8)
    sizes = torch.tensor([16 * 4] * 3, dtype=torch.int32)
    t = torch.zeros(16 * 4 * 3)
    idx = [None, torch.tensor([4]), None, torch.tensor([0]), torch.arange(4), torch.zeros(4, 3)]
    with pytest.raises(RuntimeError, match="CUDA"):
        swin3d_amd.SelfAttnAIOFunction.apply(q, q, q, t, t, t, sizes, idx, swin3d_amd.PosEmb.SEPARATE,
                                             swin3d_amd.TableDims.D0, swin3d_amd.IndexMode.INDIRECT,
                                             swin3d_amd.PrecisionMode.HALF_NONE)
    with pytest.raises(RuntimeError, match="CUDA"):
        KNN.apply(3, torch.zeros(5, 3), torch.zeros(2, 3), torch.tensor([5]), torch.tensor([2]))
    with pytest.raises(RuntimeError, match="CUDA"):
        swin3d_amd.build_window_index(torch.zeros(3, 4, dtype=torch.int32), 1, 5)


def test_unsupported_modes_raise():
    q = torch.zeros(4, 2, 8)
    args = [q, q, q, q, q, q, None, [None] * 6]
    with pytest.raises(NotImplementedError):
        swin3d_amd.SelfAttnAIOFunction.apply(*args, swin3d_amd.PosEmb.SEPARATE, swin3d_amd.TableDims.WHCD,
                                             swin3d_amd.IndexMode.INDIRECT, swin3d_amd.PrecisionMode.HALF_NONE)
    with pytest.raises(NotImplementedError):
        swin3d_amd.SelfAttnAIOFunction.apply(*args, swin3d_amd.PosEmb.SEPARATE, swin3d_amd.TableDims.D0,
                                             swin3d_amd.IndexMode.DIRECT, swin3d_amd.PrecisionMode.HALF_NONE)
    with pytest.raises(NotImplementedError):
        swin3d_amd.SelfAttnAIOFunction.apply(*args, swin3d_amd.PosEmb.LINEAR, swin3d_amd.TableDims.D0,
                                             swin3d_amd.IndexMode.INDIRECT, swin3d_amd.PrecisionMode.HALF_NONE)


def test_pair_index_matches_oracle(oracle_lib):
    w_sizes = torch.tensor([3, 1, 4, 2], dtype=torch.int32)
    x, y, m2w, ws, w2n, w2m = swin3d_amd.sparse_self_attention(None, w_sizes, "v2")
    o_w2m, o_m2w, o_x, o_y = oracle_lib.pair_index(w_sizes.numpy())
    np.testing.assert_array_equal(x.numpy(), o_x)
    np.testing.assert_array_equal(y.numpy(), o_y)
    np.testing.assert_array_equal(m2w.numpy(), o_m2w)
    np.testing.assert_array_equal(w2m.numpy(), o_w2m)
    np.testing.assert_array_equal(w2n.numpy(), [0, 3, 4, 8])
    assert len(swin3d_amd.sparse_self_attention(None, w_sizes)) == 2


def test_synthetic_room_is_deterministic_and_dense():
    from swin3d_amd import synth
    a = synth.make_room((6, 5, 3), 8, 20000, seed=0)
    b = synth.make_room((6, 5, 3), 8, 20000, seed=0)
    assert a.coords.shape == (20000, 4) or a.coords.shape[0] <= 20000
    np.testing.assert_array_equal(a.coords, b.coords)
    np.testing.assert_array_equal(a.frac, b.frac)
    assert len({tuple(r) for r in a.coords.tolist()}) == a.coords.shape[0]      # distinct voxels
    assert ((a.frac >= 0) & (a.frac < 1)).all()
    assert np.allclose(np.linalg.norm(a.normal, axis=1), 1.0)
    order = np.lexsort((a.coords[:, 3], a.coords[:, 2], a.coords[:, 1]))
    np.testing.assert_array_equal(order, np.arange(a.coords.shape[0]))          # sorted by (x,y,z)
