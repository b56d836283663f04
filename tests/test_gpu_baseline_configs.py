"""Whole-output GPU parity of the attention forward at the shapes of the baseline's configurations: the stage-1
layer on the 200k-voxel room, the deeper stages of Swin3D-S, every stage of Swin3D-L (10 / 20 / 40 heads) on a
batch of two 300k-voxel rooms, regular and shifted windows; and the Swin3D-L encoder end to end.  The float64 oracle covers every output element (no sampling)."""
import numpy as np
import pytest
import torch

from helpers import downsampled_stage_case, scene_attn_case, to_half_and_back
from swin3d_amd import synth

pytestmark = pytest.mark.gpu


def _sharp16(case):
    # keeps the fp16 rounding of the output itself below the 2e-3 tolerance (values in [-2, 2])
    case.v *= np.float32(0.4)
    case.tv *= np.float32(0.2)
    return case


def _whole_output_parity(oracle_lib, case):
    from gpu_helpers import run_attention, assert_attn_close
    to_half_and_back(case)
    ref, rmax, rsum, _ = oracle_lib.attn_fwd(*case.oracle_args(), return_stats=True)
    got, gmax, gsum = run_attention(case, torch.float16, return_stats=True)
    assert_attn_close(got, ref, torch.float16)
    assert np.isfinite(gmax).all() and (gsum >= 1.0 - 1e-6).all()
    # the statistics the backward reads: the largest logit and the sum of exp(logit - max) of every (voxel, head)
    assert np.abs(gmax - rmax).max() <= 2e-3 * max(1.0, np.abs(rmax).max())
    assert np.abs(gsum / rsum - 1.0).max() <= 1e-2


@pytest.fixture(scope="module")
def headline_room():
    return synth.make_room((10, 8, 3), 30, 200_000, seed=0)


@pytest.fixture(scope="module")
def two_rooms():
    return synth.concat_scenes([synth.make_room((10, 8, 3), 30, 300_000, seed=s) for s in (0, 1)])


@pytest.mark.parametrize("recipe", ["layer", "sharp"])
def test_stage1_headline_whole_output(oracle_lib, hip_lib, headline_room, recipe):
    """Config 2: 200k voxels, C=48, 6 heads, window 5, nine axes, fp16."""
    case = scene_attn_case(oracle_lib, headline_room, 5, 4, 6, 8, "XYZ_RGB_NORM", recipe=recipe)
    if recipe == "sharp":
        _sharp16(case)
    _whole_output_parity(oracle_lib, case)


@pytest.mark.parametrize("shifted", [False, True])
@pytest.mark.parametrize("stage,heads,levels", [(2, 6, 1), (3, 12, 2), (4, 24, 3), (5, 24, 4)])
def test_swin3d_s_deeper_stages_whole_output(oracle_lib, hip_lib, headline_room, stage, heads, levels, shifted):
    """Config 3: window 7, head_dim 16, the room grid-downsampled by 2 per stage."""
    case = downsampled_stage_case(oracle_lib, headline_room, levels, 7, 4, heads, 16, shift=3 if shifted else 0,
                                  seed=stage)
    _whole_output_parity(oracle_lib, _sharp16(case))


@pytest.mark.parametrize("shifted", [False, True])
@pytest.mark.parametrize("stage,heads,dim,ws", [(1, 10, 8, 5), (2, 10, 16, 7), (3, 20, 16, 7), (4, 40, 16, 7),
                                                (5, 40, 16, 7)])
def test_swin3d_l_stages_whole_output(oracle_lib, hip_lib, two_rooms, stage, heads, dim, ws, shifted):
    """Config 5: the attention layers of Swin3D-L, channels [80,160,320,640,640], heads [10,10,20,40,40]."""
    case = downsampled_stage_case(oracle_lib, two_rooms, stage - 1, ws, 4, heads, dim, shift=ws // 2 if shifted else 0,
                                  seed=10 + stage)
    _whole_output_parity(oracle_lib, _sharp16(case))


def test_swin3d_l_encoder_forward(hip_lib, two_rooms, monkeypatch):
    """Config 5 end to end: Swin3DEncoder(**SWIN3D_L) under fp16 autocast on ~600k voxels; the fused inference
    path against the network whose levels are kept in window order (the regular blocks then run without a row
    map), and against the path that uses torch's own LayerNorm and residual adds."""
    from swin3d_amd import encoder
    feats, signals = synth.encoder_inputs(two_rooms)
    dev = torch.device("cuda")
    vox = encoder.SparseVoxels(torch.from_numpy(two_rooms.coords).to(dev), torch.from_numpy(feats).to(dev), 1)
    sig = torch.from_numpy(signals).to(dev)
    torch.manual_seed(0)
    model = encoder.Swin3DEncoder(**encoder.SWIN3D_L, in_channels=9, cRSE="XYZ_RGB_NORM", fp16_mode=2).to(dev).eval()
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
        outs = [o.feats.float().cpu() for o in model(vox, sig)]
        coords = [o.coords.cpu() for o in model(vox, sig)]
        model.window_ordered = True
        ordered = model(vox, sig)
        model.window_ordered = False
        # rows of the window-ordered levels back in the order of the plain ones (same voxel sets, sorted by key)
        outs_ordered = []
        for o, c in zip(ordered, coords):
            back = torch.argsort(torch.argsort(encoder.pack_coords(c.to(dev))))
            outs_ordered.append(o.feats[torch.argsort(encoder.pack_coords(o.coords))][back].float().cpu())
        monkeypatch.setattr(encoder, "_fused_norm_applies", lambda feats: False)
        outs_torch = [o.feats.float().cpu() for o in model(vox, sig)]
    assert [o.shape[1] for o in outs] == [80, 160, 320, 640, 640]
    assert coords[0].shape[0] == two_rooms.coords.shape[0]
    for stage, (a, b, c) in enumerate(zip(outs, outs_ordered, outs_torch)):
        assert torch.isfinite(a).all()
        scale = max(1.0, float(c.abs().max()))
        # fp16 attention and fp16 GEMM inputs along 2 .. 23 blocks: agreement to fp16 resolution of O(1) features
        assert float((a - b).abs().max()) < 2e-2 * scale, stage
        assert float((a - c).abs().max()) < 2e-2 * scale, stage
