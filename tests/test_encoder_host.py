"""Torch-only substrate of the encoder (runs on the CPU): sparse convolution against a dense
conv3d, coordinate pooling and the representative pick against brute force."""
import numpy as np
import pytest
import torch

from conftest import random_scene
from swin3d_amd import encoder


def test_sparse_conv_matches_dense_conv3d():
    rng = np.random.default_rng(0)
    coords = torch.from_numpy(random_scene(rng, 300, extent=(4, 4, 3), batches=2))
    cin, cout = 5, 7
    feats = torch.randn(300, cin, dtype=torch.float64)
    weight = torch.randn(27, cin, cout, dtype=torch.float64)
    got = encoder.sparse_conv3x3x3(encoder.SparseVoxels(coords, feats, 1), weight)
    # dense volume [B, Cin, X, Y, Z] with the same voxels, zero elsewhere
    lo = coords[:, 1:].min(0).values
    size = (coords[:, 1:].max(0).values - lo + 1).tolist()
    dense = torch.zeros(2, cin, *size, dtype=torch.float64)
    c = coords.long()
    dense[c[:, 0], :, c[:, 1] - lo[0], c[:, 2] - lo[1], c[:, 3] - lo[2]] = feats
    w = weight.reshape(3, 3, 3, cin, cout).permute(4, 3, 0, 1, 2)      # [Cout, Cin, kx, ky, kz]
    ref = torch.nn.functional.conv3d(dense, w, padding=1)
    ref = ref[c[:, 0], :, c[:, 1] - lo[0], c[:, 2] - lo[1], c[:, 3] - lo[2]]
    torch.testing.assert_close(got, ref)


def test_sparse_conv_respects_tensor_stride():
    coords = torch.tensor([[0, 0, 0, 0], [0, 2, 0, 0], [0, 1, 0, 0]], dtype=torch.int32)   # stride 2 lattice + a stray
    feats = torch.eye(3, dtype=torch.float64)
    weight = torch.zeros(27, 3, 1, dtype=torch.float64)
    weight[(2 * 3 + 1) * 3 + 1] = 1.0            # offset (+1, 0, 0) in units of the stride
    out = encoder.sparse_conv3x3x3(encoder.SparseVoxels(coords, feats, 2), weight)
    # voxel (0,0,0) sees voxel (2,0,0) (row 1); nothing else has a +stride neighbour
    assert out[:, 0].tolist() == [1.0, 0.0, 0.0]


def test_pool_coordinates_and_representatives():
    rng = np.random.default_rng(1)
    coords_np = random_scene(rng, 500, extent=(6, 6, 3), batches=2, stride=2)
    coords = torch.from_numpy(coords_np)
    coarse, cell_of_row = encoder.pool_coordinates(coords, 2, 2)
    cells = {}
    for row, (b, x, y, z) in enumerate(coords_np.tolist()):
        cells.setdefault((b, x // 4 * 4, y // 4 * 4, z // 4 * 4), []).append(row)
    keys = sorted(cells)
    assert coarse.tolist() == [list(k) for k in keys]                      # sorted by (b, x, y, z)
    assert [keys[c] for c in cell_of_row.tolist()] == [(b, x // 4 * 4, y // 4 * 4, z // 4 * 4) for b, x, y, z in coords_np.tolist()]
    signals = torch.from_numpy(rng.random((500, 10)).astype(np.float32))
    signals[:, 0] = coords[:, 0].float()
    signals[10] = signals[11]                                               # a tie inside one cell is possible
    pick = encoder.pick_cell_representatives(signals, cell_of_row, coarse.shape[0])
    sig = signals.numpy().astype(np.float64)
    for ci, key in enumerate(keys):
        rows = cells[key]
        mean = signals[rows].float().mean(0).numpy()
        d = np.sqrt(((signals[rows].float().numpy() - mean) ** 2).sum(1))
        best = [r for r, dd in zip(rows, d) if np.isclose(dd, d.min(), rtol=1e-6, atol=1e-7)]
        assert int(pick[ci]) in best and int(pick[ci]) in rows


def test_segment_offsets():
    batch = torch.tensor([0, 0, 0, 1, 1, 3], dtype=torch.int32)
    assert encoder.segment_offsets(batch).tolist() == [3, 5, 5, 6]
    assert encoder.segment_offsets(batch).dtype == torch.int32


def test_pack_coords_is_order_preserving():
    coords = torch.tensor([[0, -5, 3, 2], [0, -5, 3, 3], [0, 4, -100000, 0], [1, -200000, 0, 0], [63, 0, 0, 0]])
    keys = encoder.pack_coords(coords)
    assert (keys[1:] > keys[:-1]).all()


def test_load_state_with_same_shape_filters_like_the_reference(tmp_path):
    """Key filtering of Swin3D/models/Swin3D.py:12-40: `module.` prefix stripped, decoder / classifier /
    (optionally) stem entries dropped, wrong shapes dropped; then load_pretrained_model on a file."""
    from swin3d_amd import encoder
    torch.manual_seed(0)
    cfg = dict(depths=[1, 1], channels=[16, 32], num_heads=[2, 2], window_sizes=[5, 7], quant_size=4, num_layers=2)
    model = encoder.Swin3DUNet(**cfg, in_channels=6, cRSE="XYZ_RGB", num_classes=5)
    donor = encoder.Swin3DUNet(**cfg, in_channels=6, cRSE="XYZ_RGB", num_classes=5)
    state = {"module." + k: v.clone() + 1.0 for k, v in donor.state_dict().items() if v.dtype.is_floating_point}
    bad = "module.layers.0.blocks.0.attn.proj.weight"
    state[bad] = torch.zeros(3, 3)                                  # wrong shape
    state["module.not_in_model.weight"] = torch.zeros(2)            # unknown name
    kept = encoder.load_state_with_same_shape(model, state, skip_first_conv=True, verbose=False)
    assert kept and all(not k.startswith("module.") for k in kept)
    assert not any("upsamples" in k or "classifier" in k or "stem_layer" in k for k in kept)
    assert "layers.0.blocks.0.attn.proj.weight" not in kept and "not_in_model.weight" not in kept
    assert "layers.0.blocks.0.attn.qkv.weight" in kept
    kept_with_stem = encoder.load_state_with_same_shape(model, state, skip_first_conv=False, verbose=False)
    assert any("stem_layer" in k for k in kept_with_stem)
    path = tmp_path / "ckpt.pth"
    torch.save({"state_dict": state}, path)
    before = model.state_dict()["layers.0.blocks.0.attn.qkv.weight"].clone()
    with pytest.raises(RuntimeError, match="attn.proj.weight"):      # the wrong-shaped entry leaves a stage parameter unset
        model.load_pretrained_model(str(path), verbose=False)
    loaded = model.load_pretrained_model(str(path), verbose=False, strict_encoder=False)
    after = model.state_dict()["layers.0.blocks.0.attn.qkv.weight"]
    assert "layers.0.blocks.0.attn.qkv.weight" in loaded
    assert torch.equal(after, donor.state_dict()["layers.0.blocks.0.attn.qkv.weight"] + 1.0) and not torch.equal(after, before)
    assert model.load_pretrained_model(str(tmp_path / "missing.pth"), verbose=False) == []


def _reference_named_state(channels, heads, windows, quant, in_channels, num_classes):
    """State-dict names and shapes of the reference's Swin3DUNet(stem_transformer=True, cRSE="XYZ_RGB", depths of 1,
    knn_down=True), written out by hand from its sources: MinkConvBNRelu.conv_layers = Sequential(MinkowskiConvolution
    [`kernel`, (27, in, out)], MinkowskiBatchNorm [`bn`]) (Swin3D/modules/mink_layers.py:62-74); BasicLayer.blocks /
    .downsample (swin3d_layers.py:679-711); SwinTransformerBlock.norm1 / attn / norm2 / mlp (:597-617);
    Mlp.fc1 / fc2 (:165-167); WindowAttention tables (3, 2*ws*quant | 2*2*2*quant, H, D), qkv, proj (:433-475);
    GridKNNDownsample.norm / linear without bias (:288-289); Upsample.linear1 / linear2 = Sequential(LayerNorm, Linear),
    .block (:340-349); classifier = Sequential(Linear, BatchNorm1d, ReLU, Linear) (Swin3D/models/Swin3D.py:107-112)."""
    shapes = {}

    def norm(prefix, c):
        shapes[prefix + ".weight"] = (c,)
        shapes[prefix + ".bias"] = (c,)

    def linear(prefix, cin, cout, bias=True):
        shapes[prefix + ".weight"] = (cout, cin)
        if bias:
            shapes[prefix + ".bias"] = (cout,)

    def batchnorm(prefix, c):
        norm(prefix, c)
        shapes[prefix + ".running_mean"] = (c,)
        shapes[prefix + ".running_var"] = (c,)
        shapes[prefix + ".num_batches_tracked"] = ()

    def block(prefix, c, h, ws):
        norm(prefix + ".norm1", c)
        for kind in ("query", "key", "value"):
            shapes[f"{prefix}.attn.{kind}_xyz_table"] = (3, 2 * ws * quant, h, c // h)
            shapes[f"{prefix}.attn.{kind}_rgb_table"] = (3, 2 * 2 * 2 * quant, h, c // h)
        linear(prefix + ".attn.qkv", c, 3 * c)
        linear(prefix + ".attn.proj", c, c)
        norm(prefix + ".norm2", c)
        linear(prefix + ".mlp.fc1", c, 4 * c)
        linear(prefix + ".mlp.fc2", 4 * c, c)

    shapes["stem_layer.conv_layers.0.kernel"] = (27, in_channels, channels[0])
    batchnorm("stem_layer.conv_layers.1.bn", channels[0])
    for i, (c, h, ws) in enumerate(zip(channels, heads, windows)):
        block(f"layers.{i}.blocks.0", c, h, ws)
        if i + 1 < len(channels):
            norm(f"layers.{i}.downsample.norm", c)
            linear(f"layers.{i}.downsample.linear", c, channels[i + 1], bias=False)
    for u, i in enumerate(range(len(channels) - 1, 0, -1)):
        cin, cout = channels[i], channels[i - 1]
        norm(f"upsamples.{u}.linear1.0", cout)
        linear(f"upsamples.{u}.linear1.1", cout, cout)
        norm(f"upsamples.{u}.linear2.0", cin)
        linear(f"upsamples.{u}.linear2.1", cin, cout)
        block(f"upsamples.{u}.block.blocks.0", cout, heads[i - 1], windows[i - 1])
    linear("classifier.0", channels[0], channels[0])
    batchnorm("classifier.1", channels[0])
    linear("classifier.3", channels[0], num_classes)
    return shapes


def test_state_dict_names_are_the_reference_checkpoints(tmp_path):
    """A checkpoint with the reference's key names (written from the reference's sources, not from this model's
    state_dict) fills every parameter of the model: same names, same shapes, nothing left over on either side.
    load_pretrained_model refuses a checkpoint that leaves encoder stages without weights."""
    from swin3d_amd import encoder
    channels, heads, windows, quant = [16, 32], [2, 2], [5, 7], 4
    model = encoder.Swin3DUNet(depths=[1, 1], channels=channels, num_heads=heads, window_sizes=windows, quant_size=quant,
                               num_layers=2, in_channels=6, cRSE="XYZ_RGB", num_classes=5, upsample="linear_attn")
    shapes = _reference_named_state(channels, heads, windows, quant, 6, 5)
    own = {k: tuple(v.shape) for k, v in model.state_dict().items()}
    assert own == shapes
    g = torch.Generator().manual_seed(3)
    state = {"module." + k: (torch.randn(shape, generator=g) if k.split(".")[-1] != "num_batches_tracked"
                             else torch.tensor(7)) for k, shape in shapes.items()}
    path = tmp_path / "reference_named.pth"
    torch.save({"state_dict": state}, path)
    loaded = model.load_pretrained_model(str(path), skip_first_conv=False, verbose=False)
    assert sorted(loaded) == sorted(k for k in shapes if "upsamples" not in k and "classifier" not in k)
    after = model.state_dict()
    for k in loaded:
        assert torch.equal(after[k], state["module." + k]), k
    assert encoder.unmatched_encoder_parameters(model, loaded) == []
    # the MLP and the stem were the silent losses of differently named modules
    assert "layers.1.blocks.0.mlp.fc2.weight" in loaded and "stem_layer.conv_layers.0.kernel" in loaded
    # a checkpoint whose MLPs have other names leaves encoder parameters at random: refused
    renamed = {k.replace(".mlp.fc1.", ".mlp.0.").replace(".mlp.fc2.", ".mlp.2."): v for k, v in state.items()}
    torch.save({"state_dict": renamed}, tmp_path / "renamed.pth")
    with pytest.raises(RuntimeError, match="mlp.fc1"):
        model.load_pretrained_model(str(tmp_path / "renamed.pth"), verbose=False)
    assert model.load_pretrained_model(str(tmp_path / "renamed.pth"), verbose=False, strict_encoder=False)
