"""End-to-end encoder forward on the HIP operators (GPU)."""
import numpy as np
import pytest
import torch

from swin3d_amd import encoder, synth
from swin3d_amd.sparse_dl.attn import attn_coff

pytestmark = pytest.mark.gpu


def _inputs(target=12000, batches=2):
    scenes = [synth.make_room((4.0, 3.0, 2.5), 4, target, seed=s) for s in range(batches)]
    scene = synth.concat_scenes(scenes)
    feats, signals = synth.encoder_inputs(scene)
    dev = torch.device("cuda")
    vox = encoder.SparseVoxels(torch.from_numpy(scene.coords).to(dev), torch.from_numpy(feats).to(dev), 1)
    return vox, torch.from_numpy(signals).to(dev)


def _small_model(fp16_mode):
    torch.manual_seed(0)
    cfg = dict(depths=[2, 2, 2], channels=[48, 96, 192], num_heads=[6, 6, 12], window_sizes=[5, 7, 7],
               quant_size=4, num_layers=3)
    return encoder.Swin3DEncoder(**cfg, in_channels=9, cRSE="XYZ_RGB_NORM", fp16_mode=fp16_mode).cuda().eval()


def test_encoder_forward_fp16(hip_lib):
    """fp16 inference; the blocks of a stage share one work list per window set (kept on the index tensors), and a
    pass in which every attention call builds its own list gives the same bits."""
    vox, signals = _inputs()
    model = _small_model(fp16_mode=2)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
        outs = model(vox, signals)
        attn_coff.REUSE_PLANS = False
        try:
            outs_own_lists = model(vox, signals)
        finally:
            attn_coff.REUSE_PLANS = True
    torch.cuda.synchronize()
    assert [o.feats.shape[1] for o in outs] == [48, 96, 192]
    assert [o.stride for o in outs] == [1, 2, 4]
    assert outs[0].coords.shape[0] == vox.coords.shape[0]
    assert outs[1].coords.shape[0] < outs[0].coords.shape[0] and outs[2].coords.shape[0] < outs[1].coords.shape[0]
    for a, b in zip(outs, outs_own_lists):
        assert torch.isfinite(a.feats).all()
        assert torch.equal(a.coords, b.coords)
        assert torch.equal(a.feats, b.feats)
    # batches stay contiguous and ascending at every level, coordinates sit on the level's lattice
    for o in outs:
        bcol = o.coords[:, 0]
        assert (bcol[1:] >= bcol[:-1]).all()
        assert (o.coords[:, 1:] % o.stride == 0).all()


def test_window_ordered_levels_equal_input_ordered_levels(hip_lib):
    """The encoder keeps every level's voxels in the order of the level's regular windows (window_ordered): same voxel sets and the same features as with the levels in input / cell order, the regular window
    index of every level is the identity, and the UNet's logits come back in input order."""
    from swin3d_amd import build_window_index
    vox, signals = _inputs()
    ordered, plain = _small_model(fp16_mode=2), _small_model(fp16_mode=2)     # same seed: same weights
    ordered.window_ordered, plain.window_ordered = True, False
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
        outs_o, outs_p = ordered(vox, signals), plain(vox, signals)
    torch.cuda.synchronize()
    assert plain.last_input_order is None
    assert torch.equal(outs_o[0].coords, vox.coords[ordered.last_input_order])
    for level, (a, b) in enumerate(zip(outs_o, outs_p)):
        ka, kb = encoder.pack_coords(a.coords), encoder.pack_coords(b.coords)
        ia, ib = torch.argsort(ka), torch.argsort(kb)
        assert torch.equal(ka[ia], kb[ib]), level
        scale = max(1.0, float(b.feats.abs().max()))
        assert float((a.feats[ia] - b.feats[ib]).abs().max()) < 2e-3 * scale, level
        index = build_window_index(a.coords, a.stride, ordered.layers[level].window_size, 0)
        assert torch.equal(index.n2n.long(), torch.arange(a.coords.shape[0], device="cuda")), level
        assert not torch.equal(build_window_index(b.coords, b.stride, ordered.layers[level].window_size, 0).n2n.long(),
                               torch.arange(b.coords.shape[0], device="cuda"))
    # the regular blocks of such levels get no row map at all (the kernels then read the rows in place); the
    # shifted blocks keep theirs
    _, _, _, _, plans = encoder.plan_stages_window_ordered(vox, signals, ordered.layers)
    for level, (args, _) in enumerate(plans):
        assert args[0][5] is None and args[1][5] is not None, level
    _, plans = encoder.plan_stages(vox.coords, vox.stride, signals, plain.layers)
    assert all(a[5] is not None for args, _ in plans for a in args)
    unet_o, unet_p = _small_unet(fp16_mode=2), _small_unet(fp16_mode=2)
    unet_o.eval(), unet_p.eval()
    unet_o.window_ordered, unet_p.window_ordered = True, False
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
        lo, lp = unet_o(vox, signals), unet_p(vox, signals)
    assert lo.shape == lp.shape
    assert float((lo - lp).abs().max()) < 2e-3 * max(1.0, float(lp.abs().max()))


def test_window_ordered_levels_train_like_input_ordered_levels(hip_lib):
    """fp32 forward and backward (the attention backward gets no row map for the regular blocks either): logits and
    parameter gradients of the window-ordered network equal those of the input-ordered one to fp32 rounding."""
    vox, signals = _inputs(target=4000, batches=2)
    nets = _small_unet(fp16_mode=0), _small_unet(fp16_mode=0)       # same seed: same weights
    nets[0].window_ordered, nets[1].window_ordered = True, False
    labels = (vox.coords[:, 3] // 8 % 13).long()
    logits = []
    for net in nets:
        out = net(vox, signals)
        torch.nn.functional.cross_entropy(out, labels).backward()
        logits.append(out.detach())
    assert float((logits[0] - logits[1]).abs().max()) < 1e-4 * max(1.0, float(logits[1].abs().max()))
    for name in ("layers.0.blocks.0.attn.query_xyz_table", "layers.0.blocks.0.attn.value_norm_table",
                 "layers.1.blocks.0.attn.qkv.weight", "layers.2.blocks.0.attn.key_rgb_table", "stem_layer.conv_layers.0.kernel"):
        ga, gb = (dict(net.named_parameters())[name].grad for net in nets)
        assert ga is not None and float(gb.abs().max()) > 0, name
        assert float((ga - gb).abs().max()) < 1e-3 * float(gb.abs().max()), name


def test_knn_downsample_matches_oracle_neighbours(oracle_lib, hip_lib):
    vox, signals = _inputs(target=6000, batches=2)
    torch.manual_seed(1)
    down = encoder.GridKNNDownsample(9, 16).cuda().eval()
    with torch.no_grad():
        coarse, coarse_signals = down(vox, signals)
    src = signals[:, 1:4].contiguous().cpu().numpy()
    qry = coarse_signals[:, 1:4].contiguous().cpu().numpy()
    so = encoder.segment_offsets(vox.coords[:, 0]).cpu().numpy()
    qo = encoder.segment_offsets(coarse.coords[:, 0]).cpu().numpy()
    idx, _ = oracle_lib.knn(16, src, qry, so, qo)
    with torch.no_grad():
        grouped = vox.feats[torch.from_numpy(idx).long().cuda().view(-1)].view(-1, 16, 9)
        ref = down.linear(down.norm(grouped)).amax(dim=1)
    torch.testing.assert_close(coarse.feats, ref.float(), rtol=1e-5, atol=1e-6)
    # the representative of a cell is one of the cell's own points
    cell = torch.div(coarse_signals[:, 1:4], 2, rounding_mode="floor") * 2
    assert torch.equal(cell.int(), coarse.coords[:, 1:])


def _small_unet(fp16_mode, upsample="linear_attn"):
    torch.manual_seed(0)
    cfg = dict(depths=[1, 1, 1], channels=[48, 96, 192], num_heads=[6, 6, 12], window_sizes=[5, 7, 7],
               quant_size=4, num_layers=3)
    return encoder.Swin3DUNet(**cfg, in_channels=9, cRSE="XYZ_RGB_NORM", fp16_mode=fp16_mode, num_classes=13,
                              upsample=upsample).cuda()


def test_unet_forward_and_training_step(hip_lib):
    """Swin3DUNet: logits on the input voxels; one optimisation step in fp32 (attention backward through
    s3d_attn_bwd, interpolation backward) lowers the loss on a fixed batch."""
    vox, signals = _inputs(target=5000, batches=2)
    model = _small_unet(fp16_mode=0)
    labels = (vox.coords[:, 3] // 8 % 13).long()           # height bands: learnable from the features
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    losses = []
    for _ in range(3):
        opt.zero_grad()
        logits = model(vox, signals)
        assert logits.shape == (vox.coords.shape[0], 13) and torch.isfinite(logits).all()
        loss = torch.nn.functional.cross_entropy(logits, labels)
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    table = model.layers[0].blocks[0].attn.query_xyz_table
    assert table.grad is not None and torch.isfinite(table.grad).all() and float(table.grad.abs().max()) > 0
    qkv = model.layers[1].blocks[0].attn.qkv.weight
    assert qkv.grad is not None and float(qkv.grad.abs().max()) > 0
    assert losses[-1] < losses[0], losses


def test_unet_forward_fp16(hip_lib):
    vox, signals = _inputs(target=5000, batches=1)
    model = _small_unet(fp16_mode=2, upsample="linear").eval()
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
        logits = model(vox, signals)
    assert logits.shape == (vox.coords.shape[0], 13) and torch.isfinite(logits).all()


def test_window_attention_module_argument_prep(oracle_lib, hip_lib):
    """WindowAttention (fp32) against a float64 statement of the reference's argument prep
    (Swin3D/modules/swin3d_layers.py:502-541: q, k, v = split(Linear(feats)), q *= D^-0.5, tables = cat of the
    flattened (3, rows, H, D) parameters in the order xyz, rgb, norm, signals scaled by quant / 2*quant) fed to
    the attention oracle, then the output projection.  Forward and the gradients of a linear loss."""
    from swin3d_amd import crse
    vox, signals = _inputs(target=2500, batches=1)
    torch.manual_seed(3)
    ws, quant, dim, heads = 5, 4, 48, 6
    attn = encoder.WindowAttention(dim, ws, quant, heads, cRSE="XYZ_RGB_NORM", fp16_mode=0).cuda()
    for kind in ("query", "key", "value"):
        for name in ("xyz", "rgb", "norm"):
            torch.nn.init.normal_(getattr(attn, f"{kind}_{name}_table"), std=0.3)
    n = vox.coords.shape[0]
    feats = torch.randn(n, dim, device="cuda", requires_grad=True)
    local = (signals[:, 1:4].float() - vox.coords[:, 1:].float())
    args = encoder.get_index01(vox.coords, 1, ws, local, signals[:, 4:].float(), shift=0)
    out = attn(feats, args)
    grad_out = torch.randn_like(out)
    out.backward(grad_out)
    torch.cuda.synchronize()

    # float64 statement on the host
    f64 = lambda t: t.detach().double().cpu().numpy()
    x = f64(feats)
    qkv = x @ f64(attn.qkv.weight).T + f64(attn.qkv.bias)
    d = dim // heads
    q = (qkv[:, :dim] * d ** -0.5).reshape(n, heads, d)
    k = qkv[:, dim:2 * dim].reshape(n, heads, d)
    v = qkv[:, 2 * dim:].reshape(n, heads, d)
    flat = lambda kind: np.concatenate([f64(getattr(attn, f"{kind}_{nm}_table")).reshape(-1) for nm in ("xyz", "rgb", "norm")])
    sizes = crse.crse_table_sizes(ws, quant, heads, d, "XYZ_RGB_NORM")
    _, _, _, w_sizes, w2n, n2n, _, n_coords = args
    scale = np.array([quant] * 3 + [2 * quant] * 6, np.float32)
    n_crse = (n_coords.cpu().numpy().astype(np.float32) * scale).astype(np.float32)
    idx = [t.cpu().numpy() for t in (w_sizes, w2n, n2n)]
    to32 = lambda a: a.astype(np.float32)
    # the oracle takes fp32 inputs: feed it the fp32 roundings the module itself produces
    o = oracle_lib.attn_fwd(to32(q), to32(k), to32(v), to32(flat("query")), to32(flat("key")), to32(flat("value")),
                            sizes, *idx, n_crse)
    ref = o.reshape(n, dim) @ f64(attn.proj.weight).T + f64(attn.proj.bias)
    np.testing.assert_allclose(f64(out), ref, rtol=2e-4, atol=2e-5 * np.abs(ref).max())

    # gradients: d out / d attention output = grad_out @ W_proj; the oracle backward gives dq, dk, dv and the tables
    dattn = (f64(grad_out) @ f64(attn.proj.weight)).reshape(n, heads, d)
    dq, dk, dv, dtq, dtk, dtv = oracle_lib.attn_bwd(to32(q), to32(k), to32(v), to32(flat("query")), to32(flat("key")),
                                                    to32(flat("value")), sizes, *idx, n_crse, to32(dattn))
    dqkv = np.concatenate([dq.reshape(n, dim) * d ** -0.5, dk.reshape(n, dim), dv.reshape(n, dim)], axis=1)
    ref_dfeats = dqkv @ f64(attn.qkv.weight)
    np.testing.assert_allclose(f64(feats.grad), ref_dfeats, rtol=1e-3, atol=1e-4 * np.abs(ref_dfeats).max())
    rows_xyz = sizes[0] // dim
    got_xyz = f64(attn.key_xyz_table.grad).reshape(-1)
    np.testing.assert_allclose(got_xyz, dtk[: 3 * rows_xyz * dim], rtol=1e-3, atol=1e-4 * np.abs(dtk).max())
    got_norm = f64(attn.value_norm_table.grad).reshape(-1)
    np.testing.assert_allclose(got_norm, dtv[-got_norm.size:], rtol=1e-3, atol=1e-4 * np.abs(dtv).max())


@pytest.mark.parametrize("stride,factor", [(1, 2), (2, 2), (4, 3)])
def test_cell_pooling_on_the_gpu_matches_the_host_statement(hip_lib, stride, factor):
    """On the GPU the coarse cells come from the window sort (a cell is a window of `factor` voxels); the host
    statement is unique + scatter.  Same cells in the same order, same cell of every row; segment offsets with
    the batch count given (no host wait) equal the bincount statement."""
    from conftest import random_scene
    rng = np.random.default_rng(9)
    coords = torch.from_numpy(random_scene(rng, 5000, extent=(20, 20, 8), batches=3, stride=stride))
    ref_coarse, ref_inverse = encoder.pool_coordinates(coords, stride, factor)
    got_coarse, got_inverse = encoder.pool_coordinates(coords.cuda(), stride, factor)
    assert torch.equal(got_coarse.cpu(), ref_coarse) and torch.equal(got_inverse.cpu(), ref_inverse)
    column = got_coarse[:, 0]
    assert torch.equal(encoder.segment_offsets(column, 3), encoder.segment_offsets(column))
    assert torch.equal(encoder.segment_offsets(column, 5).cpu()[3:], torch.full((2,), column.numel(), dtype=torch.int32))


@pytest.mark.parametrize("stride", [1, 2])
def test_stem_neighbour_rows_on_the_gpu_match_the_host_statement(hip_lib, stride):
    """s3d_key_neighbours (binary search of key + offset in the sorted keys) against the tensor statement that
    runs on the host: same row, or N, for each of the 27 offsets of every voxel; negative coordinates included."""
    from conftest import random_scene
    rng = np.random.default_rng(10)
    coords = torch.from_numpy(random_scene(rng, 6000, extent=(14, 14, 6), batches=2, stride=stride))
    ref = encoder.conv3x3x3_neighbours(coords, stride)
    got = encoder.conv3x3x3_neighbours(coords.cuda(), stride)
    assert torch.equal(got.cpu(), ref)
    assert int((ref < coords.shape[0]).sum()) > 27 * 100          # the scene is dense enough to have neighbours


def test_cell_representatives_on_the_gpu_match_the_host_statement(hip_lib):
    """s3d_cell_representatives against the host statement (scatter sums, mean, distances, scatter minimum) on
    signals that are multiples of 1/64, for which every sum is exact whatever its order: same coarse voxels, same
    representative rows, ties to the lower row."""
    from conftest import random_scene
    rng = np.random.default_rng(11)
    coords = torch.from_numpy(random_scene(rng, 5000, extent=(12, 12, 6), batches=2, stride=2))
    signals = torch.from_numpy((rng.integers(-64, 65, (5000, 10)) / 64.0).astype(np.float32))
    signals[:40] = signals[40:80]                      # duplicates: exact ties somewhere
    ref_coarse, ref_pick = encoder.pool_and_pick(coords, 2, 2, signals)
    got_coarse, got_pick = encoder.pool_and_pick(coords.cuda(), 2, 2, signals.cuda())
    assert torch.equal(got_coarse.cpu(), ref_coarse) and torch.equal(got_pick.cpu(), ref_pick)


def test_inference_copies_of_parameters_follow_training_updates(hip_lib):
    """The autocast-dtype copies that the layers keep for inference are renewed after any forward with autograd
    enabled, also when the update went through `param.data` (which leaves the version counter alone), and on
    request (drop_inference_copies)."""
    torch.manual_seed(3)
    layer = torch.nn.Linear(16, 8).cuda()
    x = torch.randn(5, 16, device="cuda")

    def infer():
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
            return encoder._linear(layer, x).float()

    first = infer()
    assert torch.equal(infer(), first) and hasattr(layer, "_s3d_cast")
    layer.weight.data.mul_(2.0)                 # version counter unchanged
    layer.bias.data.zero_()
    encoder._linear(layer, x).sum().backward()  # a training forward in between
    second = infer()
    expect = torch.nn.functional.linear(x.half(), layer.weight.half(), layer.bias.half()).float()
    assert torch.equal(second, expect) and not torch.equal(second, first)
    layer.weight.data.mul_(0.5)                 # no training forward: the copy is stale until it is dropped
    encoder.drop_inference_copies(layer)
    third = infer()
    assert torch.equal(third, torch.nn.functional.linear(x.half(), layer.weight.half(), layer.bias.half()).float())
