"""Residual add fused with LayerNorm (s3d_add_layernorm) against torch's fp32 LayerNorm of the same sum."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("channels", [48, 80, 96, 160, 320, 640, 1024])
@pytest.mark.parametrize("res_dtype", [None, torch.float16, torch.float32])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
def test_add_layernorm_matches_torch(hip_lib, channels, res_dtype, out_dtype):
    from swin3d_amd.fused_norm import add_layernorm
    torch.manual_seed(channels)
    dev = torch.device("cuda")
    n = 1037                                   # not a multiple of the rows a workgroup covers
    x = (torch.randn(n, channels, device=dev) * 3 + 0.7).float()
    res = None if res_dtype is None else torch.randn(n, channels, device=dev).to(res_dtype)
    norm = torch.nn.LayerNorm(channels).to(dev)
    with torch.no_grad():
        norm.weight.uniform_(0.5, 1.5)
        norm.bias.uniform_(-0.5, 0.5)
        summed, y = add_layernorm(x, res, norm, out_dtype=out_dtype)
        want_sum = x if res is None else x + res.float()
        want = norm(want_sum)
    torch.cuda.synchronize()
    assert y.dtype == out_dtype and y.shape == x.shape
    assert torch.equal(summed, want_sum)       # one fp32 addition per element: bit-exact
    # fp32: summation order differs from torch's; fp16: one rounding of values of magnitude <= ~6 (ulp 4e-3)
    tol = 2e-5 if out_dtype == torch.float32 else 4e-3
    assert (y.float() - want).abs().max().item() <= tol


def test_inplace_and_empty(hip_lib):
    from swin3d_amd.fused_norm import add_layernorm
    dev = torch.device("cuda")
    norm = torch.nn.LayerNorm(64).to(dev)
    x = torch.randn(300, 64, device=dev)
    res = torch.randn(300, 64, device=dev).half()
    want = x + res.float()
    with torch.no_grad():
        summed, y = add_layernorm(x, res, norm, inplace=True)
    assert summed.data_ptr() == x.data_ptr() and torch.equal(x, want)
    with torch.no_grad():
        s0, y0 = add_layernorm(torch.empty(0, 64, device=dev), None, norm)
    assert y0.shape == (0, 64)
    with pytest.raises(ValueError):
        add_layernorm(x.half(), None, norm)
    with pytest.raises(ValueError):
        add_layernorm(torch.randn(10, 66, device=dev), None, torch.nn.LayerNorm(66).to(dev))


def test_swin_block_fused_path_matches_torch_path(hip_lib):
    """The block's inference path under fp16 autocast (fused add + LayerNorm kernels) against the same block with
    autograd enabled (torch kernels): same weights, same inputs."""
    import numpy as np
    from swin3d_amd import encoder, synth
    from swin3d_amd.window_index import get_index01
    dev = torch.device("cuda")
    scene = synth.make_room((3.0, 3.0, 2.0), 4, 6000, seed=3)
    coords = torch.from_numpy(scene.coords).to(dev)
    args = get_index01(coords, 1, 5, torch.from_numpy(scene.frac).to(dev),
                       torch.from_numpy(synth.signals(scene, "XYZ_RGB")).to(dev))
    torch.manual_seed(0)
    block = encoder.SwinBlock(48, 6, 5, 4, cRSE="XYZ_RGB", fp16_mode=2).to(dev).eval()
    feats = torch.randn(coords.shape[0], 48, device=dev)
    with torch.autocast("cuda", dtype=torch.float16):
        with torch.no_grad():
            fused = block(feats, args)
        plain = block(feats, args)             # grad mode on: torch LayerNorm and adds
    torch.cuda.synchronize()
    assert fused.dtype == torch.float32
    assert (fused - plain.detach()).abs().max().item() <= 2e-2 * plain.detach().abs().max().item()


def test_stage_with_downsample_fused_path_matches_torch_path(hip_lib):
    """A whole stage (two blocks + KNN downsample) on the inference path, where the last block's MLP output is
    added inside the downsample's LayerNorm kernel, against the same stage with autograd enabled (torch adds and
    LayerNorms); the caller's input features stay untouched."""
    from swin3d_amd import encoder, synth
    dev = torch.device("cuda")
    scene = synth.make_room((3.0, 3.0, 2.0), 4, 6000, seed=5)
    coords = torch.from_numpy(scene.coords).to(dev)
    signals = torch.from_numpy(synth.encoder_inputs(scene)[1][:, :7].copy()).to(dev)      # batch, xyz, rgb
    torch.manual_seed(1)
    stage = encoder.Stage(48, 2, 6, 5, 4, out_channels=96, cRSE="XYZ_RGB", fp16_mode=2).to(dev).eval()
    feats = torch.randn(coords.shape[0], 48, device=dev)
    kept = feats.clone()
    voxels = encoder.SparseVoxels(coords, feats, 1)
    with torch.autocast("cuda", dtype=torch.float16):
        with torch.no_grad():
            plan = stage.plan(coords, 1, signals)
            fine_f, down_f, sig_f = stage(voxels, signals, plan)
        fine_p, down_p, sig_p = stage(voxels, signals, plan)          # grad mode on: torch kernels
    torch.cuda.synchronize()
    assert torch.equal(feats, kept)
    assert torch.equal(down_f.coords, down_p.coords) and torch.equal(sig_f, sig_p)
    for fused, plain in ((fine_f.feats, fine_p.feats.detach()), (down_f.feats, down_p.feats.detach())):
        assert fused.dtype == torch.float32 and fused.shape == plain.shape
        assert (fused - plain).abs().max().item() <= 2e-2 * plain.abs().max().item()
