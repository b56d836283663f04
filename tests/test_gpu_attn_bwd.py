"""GPU parity of the window attention backward (HIP through the C ABI) against the float64 CPU oracle, on both
of its paths (with and without the window set's pair count).

Tolerance: |got - ref| <= rel * scale with rel = 2e-5 for fp32 and 3e-3 for fp16 (fp16: the forward output
o that enters dout.o, and dq / dk / dv themselves, are rounded to fp16); scale = largest |ref| over
(dq, dk, dv) for those three and over the three table gradients for those."""
import numpy as np
import pytest
import torch

from helpers import make_attn_case, scene_attn_case, to_half_and_back, n_coords_from_scene
from swin3d_amd import synth

pytestmark = pytest.mark.gpu

NAMES = ("dq", "dk", "dv", "dtable_q", "dtable_k", "dtable_v")


def _run(case, dout, dtype, pairs=None):
    import swin3d_amd
    dev = torch.device("cuda")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    f = lambda a: t(a).to(dtype)
    i = case.index
    args = (f(case.q), f(case.k), f(case.v), f(case.tq), f(case.tk), f(case.tv), t(case.table_sizes),
            t(i["w_sizes"]), t(i["w2n"]), t(i["n2n"]), t(case.n_coords))
    out, omax, osum = swin3d_amd.window_attention_forward(*args, return_stats=True)
    grads = swin3d_amd.window_attention_backward(*args, out, omax, osum, f(dout), pairs=pairs)
    torch.cuda.synchronize()
    return [g.double().cpu().numpy() for g in grads]


def _assert_close(got, ref, dtype):
    """The scale of a tolerance is the largest |ref| of the GROUP a tensor belongs to (dq, dk, dv / the three
    table gradients): dq and dk are sums of P (dP - dout.o) terms that cancel (exactly, for a single-voxel
    window), so their rounding error is set by the size of the terms, which dv shares, not by the result."""
    rel = 2e-5 if dtype == torch.float32 else 3e-3
    ref = [np.asarray(r, np.float64).reshape(g.shape) for g, r in zip(got, ref)]
    scales = [max(np.abs(r).max() for r in ref[:3])] * 3 + [max(np.abs(r).max() for r in ref[3:])] * 3
    for name, g, r, scale in zip(NAMES, got, ref, scales):
        assert np.isfinite(g).all(), name
        err = np.abs(g - r).max()
        assert err <= rel * max(scale, 1e-30), f"{name}: max err {err:.3e}, scale {scale:.3e}"


def _half_rounding(wide, scale):
    """Bound on |fp16(x') - x| where x' is x with its fp32 sum reordered: half an fp16 unit in the last place of x
    (2^-11 |x|, 2^-25 for subnormals) plus the reordering (2e-6 of the largest element)."""
    return wide.abs() * (2.0 ** -11 * 1.001) + 2.0 ** -25 + 2e-6 * scale


def _check(oracle_lib, case, dtype, seed=0, dout_scale=1.0):
    if dtype == torch.float16:
        to_half_and_back(case)
    rng = np.random.default_rng(seed + 900)
    dout = (rng.standard_normal(case.q.shape) * dout_scale).astype(np.float32)
    if dtype == torch.float16:
        dout = dout.astype(np.float16).astype(np.float32)
    ref = oracle_lib.attn_bwd(*case.oracle_args(), dout)
    # both ways through s3d_attn_bwd: the pair sweeps with their store of dL and P (the pair count from w_sizes),
    # and the fused sweeps that run when the caller gives no pair count
    _assert_close(_run(case, dout, dtype), ref, dtype)
    _assert_close(_run(case, dout, dtype, pairs=0), ref, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("cRSE", ["XYZ", "XYZ_RGB", "XYZ_RGB_NORM"])
@pytest.mark.parametrize("heads,dim,ws", [(6, 8, 5), (3, 16, 7)])
def test_random_scenes(oracle_lib, hip_lib, dtype, cRSE, heads, dim, ws):
    case = make_attn_case(oracle_lib, seed=61, n=900, ws=ws, quant=4, heads=heads, dim=dim, cRSE=cRSE,
                          extent=(10, 10, 3) if ws == 5 else (12, 12, 4))
    if dtype == torch.float16:
        case.v *= np.float32(0.4)
        case.tv *= np.float32(0.2)
    _check(oracle_lib, case, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_room_layer_recipe(oracle_lib, hip_lib, dtype):
    """A small synthetic room with the freshly-initialised-layer recipe (near-uniform softmax); tiny
    gradient scale on purpose: the fixed-point histograms are scaled per step, not by a constant."""
    scene = synth.make_room((3.0, 2.0, 1.5), 3, 4000, seed=3)
    case = scene_attn_case(oracle_lib, scene, 5, 4, 6, 8, "XYZ_RGB_NORM", recipe="layer")
    _check(oracle_lib, case, dtype, dout_scale=1e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_dense_windows_up_to_343_voxels(oracle_lib, hip_lib, dtype):
    ws, quant, heads, dim = 7, 4, 2, 16
    g = np.stack(np.meshgrid(np.arange(14), np.arange(7), np.arange(7), indexing="ij"), -1).reshape(-1, 3)
    coords = np.concatenate([np.zeros((g.shape[0], 1), np.int64), g], 1).astype(np.int32)
    rng = np.random.default_rng(63)
    coords = coords[rng.permutation(coords.shape[0])]
    frac = rng.random((coords.shape[0], 3)).astype(np.float32)
    sig = rng.uniform(-1, 1, (coords.shape[0], 6)).astype(np.float32)
    case = make_attn_case(oracle_lib, seed=63, n=coords.shape[0], ws=ws, quant=quant, heads=heads, dim=dim,
                          extent=(12, 12, 6))
    case.coords = coords
    case.index, case.n_coords = n_coords_from_scene(oracle_lib, coords, frac, sig, 1, ws, quant, case.cRSE)
    if dtype == torch.float16:
        case.v *= np.float32(0.4)
        case.tv *= np.float32(0.2)
    _check(oracle_lib, case, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("heads,dim", [(2, 8), (2, 16)])
def test_window_sizes_at_the_kernel_boundaries(oracle_lib, hip_lib, dtype, heads, dim):
    """Windows of exactly 1, 16, 31..33, 63..65, 127..129, 192 and 193 voxels: where the sweeps change their lane
    mapping and start splitting a window into chunks of 64 owned elements."""
    from test_gpu_attn import boundary_size_case
    case = boundary_size_case(oracle_lib, heads, dim, seed=71)
    if dtype == torch.float16:
        case.v *= np.float32(0.4)
        case.tv *= np.float32(0.2)
    _check(oracle_lib, case, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("ws,quant,heads,dim,cRSE", [
    (3, 4, 4, 8, "XYZ_RGB_NORM"),     # small tables
    (4, 8, 3, 8, "XYZ_RGB_NORM"),     # quant 8: 576 table rows per head, nine 64-row register blocks
    (8, 4, 2, 16, "XYZ"),             # window 8, head_dim 16, three axes
    (4, 4, 2, 16, "XYZ_RGB"),         # six axes
])
def test_other_window_and_quant_sizes(oracle_lib, hip_lib, dtype, ws, quant, heads, dim, cRSE):
    case = make_attn_case(oracle_lib, seed=70 + ws, n=600, ws=ws, quant=quant, heads=heads, dim=dim, cRSE=cRSE,
                          extent=(8, 8, 3))
    if dtype == torch.float16:
        case.v *= np.float32(0.4)
        case.tv *= np.float32(0.2)
    _check(oracle_lib, case, dtype)


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes(oracle_lib, hip_lib, seed):
    """Randomly drawn shapes: head counts that do and do not divide the grid of workgroups evenly, both
    head_dims (VALU and MFMA table-gradient updates), 3 / 6 / 9 axes, sparse to dense windows (every size class of
    the unit list), several batch elements, strides and window shifts; fp32 on even seeds, fp16 on odd ones."""
    rng = np.random.default_rng(2000 + seed)
    ws = int(rng.choice([3, 5, 7]))
    heads = int(rng.choice([1, 2, 3, 5, 6, 7]))
    dim = int(rng.choice([8, 16]))
    cRSE = str(rng.choice(["XYZ", "XYZ_RGB", "XYZ_RGB_NORM"]))
    stride = int(rng.choice([1, 2, 4]))
    shift = int(rng.choice([0, ws // 2]))
    batches = int(rng.integers(1, 4))
    half = tuple(int(v) for v in rng.integers(3, 8, size=3))         # half extent of the box in voxels
    capacity = batches * 8 * half[0] * half[1] * half[2]
    n = int(capacity * rng.uniform(0.05, 0.75))
    case = make_attn_case(oracle_lib, seed=2000 + seed, n=n, ws=ws, quant=4, heads=heads, dim=dim, cRSE=cRSE,
                          extent=half, batches=batches, stride=stride, shift=shift, recipe="layer")
    _check(oracle_lib, case, torch.float32 if seed % 2 == 0 else torch.float16, seed=seed)


@pytest.mark.parametrize("heads,dim,ws,cRSE", [(6, 8, 5, "XYZ_RGB_NORM"), (3, 16, 7, "XYZ_RGB_NORM"), (2, 16, 7, "XYZ"),
                                               (4, 8, 3, "XYZ_RGB"), (20, 16, 7, "XYZ_RGB_NORM")])
def test_fp32_arithmetic_on_fp16_rows(oracle_lib, hip_lib, heads, dim, ws, cRSE):
    """fp16 features beside fp32 tables (the backward of an fp16 forward computed in fp32, PrecisionMode.HALF_FORWARD,
    Swin3D/sparse_dl/attn/attn_coff.py:206-215): dq, dk, dv are the fp32 call's on fp32 copies of the features,
    rounded to fp16 - the same arithmetic, so they agree to that rounding (half an fp16 unit in the last place) plus
    the reordering of an fp32 sum (the two kernel instantiations may pack the windows differently); the table
    gradients agree with that call's as two calls of one form do.  Without a pair count the operator makes the copies
    itself."""
    import swin3d_amd
    case = make_attn_case(oracle_lib, seed=91, n=1500 if ws < 7 else 2500, ws=ws, quant=4, heads=heads, dim=dim, cRSE=cRSE,
                          extent=(10, 10, 3) if ws < 7 else (14, 14, 5))
    case.v *= np.float32(0.4)
    case.tv *= np.float32(0.2)
    for name in ("q", "k", "v"):                       # fp16 features, fp32 tables
        setattr(case, name, getattr(case, name).astype(np.float16).astype(np.float32))
    dev = torch.device("cuda")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    i = case.index
    feats16 = [t(x).half() for x in (case.q, case.k, case.v)]
    tables = [t(x) for x in (case.tq, case.tk, case.tv)]
    idx = (t(case.table_sizes), t(i["w_sizes"]), t(i["w2n"]), t(i["n2n"]), t(case.n_coords))
    # the forward as HALF_FORWARD runs it: fp16 everywhere
    out, omax, osum = swin3d_amd.window_attention_forward(*feats16, *[x.half() for x in tables], *idx, return_stats=True)
    dout = torch.from_numpy(np.random.default_rng(92).standard_normal(case.q.shape).astype(np.float32)).to(dev).half()
    wide = swin3d_amd.window_attention_backward(*[x.float() for x in feats16], *tables, *idx, out.float(), omax, osum,
                                                dout.float())
    mixed = swin3d_amd.window_attention_backward(*feats16, *tables, *idx, out, omax, osum, dout)
    fused = swin3d_amd.window_attention_backward(*feats16, *tables, *idx, out, omax, osum, dout, pairs=0)
    torch.cuda.synchronize()
    row_scale = max(float(w.abs().max()) for w in wide[:3])
    for name, g, w, f in zip(NAMES[:3], mixed, wide, fused):
        assert g.dtype == torch.float16 and f.dtype == torch.float16, name
        assert bool(((g.float() - w).abs() <= _half_rounding(w, row_scale)).all()), name
        # the fused form is another algorithm: the fp32 tolerance of this file on top
        assert bool(((f.float() - w).abs() <= _half_rounding(w, row_scale) + 2e-5 * row_scale).all()), name
    scale = max(float(w.abs().max()) for w in wide[3:])
    for name, g, w, f in zip(NAMES[3:], mixed[3:], wide[3:], fused[3:]):
        assert g.dtype == torch.float32, name
        assert float((g - w).abs().max()) <= 1e-5 * scale, name
        assert float((f - w).abs().max()) <= 2e-5 * scale, name
    # against the oracle, which gets what the kernels got: the fp16 output of the fp16 forward enters dout . o
    ref = oracle_lib.attn_bwd(*case.oracle_args(), dout.float().cpu().numpy())
    got = [g.double().cpu().numpy() for g in mixed]
    _assert_close(got, ref, torch.float16)


def test_fp16_rows_without_a_pair_count_are_refused_by_the_library(hip_lib):
    """dtype S3D_DTYPE_F32_F16_ROWS exists in the pair form only: the C entry point says so instead of reading fp16
    rows as fp32."""
    import ctypes
    from swin3d_amd import _lib, crse
    dev = torch.device("cuda")
    n, heads, dim = 64, 2, 8
    sizes = crse.crse_table_sizes(5, 4, heads, dim, "XYZ")
    table_len = int(sum(sizes))
    rows = torch.zeros((n, heads, dim), dtype=torch.float16, device=dev)
    table = torch.zeros(table_len, device=dev)
    stats = torch.ones((n, heads), device=dev)
    ints = torch.zeros(n, dtype=torch.int32, device=dev)
    coords = torch.zeros((n, 3), device=dev)
    lib = _lib.lib()
    ws_bytes = lib.s3d_attn_bwd_workspace_bytes(heads, dim, 3, table_len, n, 1, 0)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    c_sizes = (ctypes.c_int32 * 3)(*sizes)
    p = lambda x: x.data_ptr()
    status = lib.s3d_attn_bwd(p(rows), p(rows), p(rows), p(table), p(table), p(table), c_sizes, 3, table_len, p(ints),
                              p(ints), p(ints), p(coords), p(rows), p(stats), p(stats), p(rows), p(rows), p(rows), p(rows),
                              p(table), p(table), p(table), n, heads, dim, 1, 0, _lib.S3D_DTYPE_F32_F16_ROWS, p(ws),
                              ws_bytes, None)
    assert status == -4 and b"pair count" in lib.s3d_last_error_string()


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("ws,quant,heads,dim,cRSE", [
    (5, 4, 3, 32, "XYZ_RGB_NORM"),    # head_dim 32
    (7, 4, 2, 32, "XYZ"),
    (7, 8, 2, 8, "XYZ"),              # 112 rows per axis: more than the register blocks of the table-gradient kernels
    (10, 4, 2, 16, "XYZ"),            # window 10: 80 rows on each of the three position axes
])
def test_general_form(oracle_lib, hip_lib, dtype, ws, quant, heads, dim, cRSE):
    """head_dim 32 and tables of more than 64 rows per axis on average run in the library's general form (global
    atomic adds, as the reference works); the pair count is ignored there."""
    from swin3d_amd.sparse_dl.attn import attn_coff
    case = make_attn_case(oracle_lib, seed=400 + ws + dim, n=800, ws=ws, quant=quant, heads=heads, dim=dim, cRSE=cRSE,
                          extent=(10, 10, 4))
    rows = int(sum(case.table_sizes)) // (heads * dim)
    assert dim == 32 or rows > attn_coff.BWD_MAX_ROWS_PER_AXIS * len(case.table_sizes)
    if dtype == torch.float16:
        case.v *= np.float32(0.4)
        case.tv *= np.float32(0.2)
    _check(oracle_lib, case, dtype)


def test_general_form_on_fp16_rows_with_fp32_tables(oracle_lib, hip_lib):
    """The general form under PrecisionMode.HALF_FORWARD: fp16 tensors, fp32 tables, against the fp32 call on copies."""
    import swin3d_amd
    case = make_attn_case(oracle_lib, seed=433, n=800, ws=5, quant=4, heads=3, dim=32, cRSE="XYZ_RGB_NORM",
                          extent=(10, 10, 4))
    case.v *= np.float32(0.4)
    case.tv *= np.float32(0.2)
    dev = torch.device("cuda")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    i = case.index
    feats16 = [t(x).half() for x in (case.q, case.k, case.v)]
    tables = [t(x) for x in (case.tq, case.tk, case.tv)]
    idx = (t(case.table_sizes), t(i["w_sizes"]), t(i["w2n"]), t(i["n2n"]), t(case.n_coords))
    out, omax, osum = swin3d_amd.window_attention_forward(*feats16, *[x.half() for x in tables], *idx, return_stats=True)
    dout = torch.from_numpy(np.random.default_rng(434).standard_normal(case.q.shape).astype(np.float32)).to(dev).half()
    wide = swin3d_amd.window_attention_backward(*[x.float() for x in feats16], *tables, *idx, out.float(), omax, osum,
                                                dout.float())
    mixed = swin3d_amd.window_attention_backward(*feats16, *tables, *idx, out, omax, osum, dout)
    torch.cuda.synchronize()
    row_scale = max(float(w.abs().max()) for w in wide[:3])
    for name, g, w in zip(NAMES[:3], mixed, wide):
        assert g.dtype == torch.float16, name
        assert bool(((g.float() - w).abs() <= _half_rounding(w, row_scale) + 2e-5 * row_scale).all()), name
    scale = max(float(w.abs().max()) for w in wide[3:])
    for name, g, w in zip(NAMES[3:], mixed[3:], wide[3:]):
        assert g.dtype == torch.float32 and float((g - w).abs().max()) <= 2e-5 * scale, name


def test_single_voxel_windows(oracle_lib, hip_lib):
    coords = np.array([[0, 0, 0, 0], [0, 50, 0, 0], [0, 51, 0, 0], [1, 3, 3, 3]], np.int32)
    case = make_attn_case(oracle_lib, seed=64, n=4, ws=5, quant=4, heads=1, dim=8, cRSE="XYZ")
    frac = np.random.default_rng(3).random((4, 3)).astype(np.float32)
    case.index, case.n_coords = n_coords_from_scene(oracle_lib, coords, frac, np.zeros((4, 0), np.float32),
                                                    1, 5, 4, "XYZ")
    _check(oracle_lib, case, torch.float32)


def test_empty_input(hip_lib):
    import swin3d_amd
    from swin3d_amd import crse
    dev = torch.device("cuda")
    q = torch.zeros((0, 6, 8), device=dev)
    t = torch.zeros(14976, device=dev)
    sizes = crse.crse_table_sizes(5, 4, 6, 8, "XYZ_RGB_NORM")
    e = torch.zeros(0, dtype=torch.int32, device=dev)
    s = torch.zeros((0, 6), device=dev)
    grads = swin3d_amd.window_attention_backward(q, q, q, t, t, t, sizes, e, e, e, torch.zeros((0, 9), device=dev),
                                                 q, s, s, q)
    assert grads[0].shape == (0, 6, 8) and float(grads[3].abs().max()) == 0.0


@pytest.mark.parametrize("precision_name", ["HALF_NONE", "HALF_ALL"])
def test_autograd_function(oracle_lib, hip_lib, precision_name):
    """loss.backward() through SelfAttnAIOFunction with the reference's argument list (fp32 leaves; fp16 features
    from a layer under autocast with HALF_FORWARD: test_autograd_half_forward_on_fp16_features)."""
    from swin3d_amd.sparse_dl.attn.attn_coff import (SelfAttnAIOFunction, PosEmb, TableDims, IndexMode,
                                                     PrecisionMode)
    case = make_attn_case(oracle_lib, seed=65, n=500, ws=5, quant=4, heads=6, dim=8, extent=(8, 8, 3))
    half = precision_name == "HALF_ALL"
    if half:
        case.v *= np.float32(0.4)
        case.tv *= np.float32(0.2)
        to_half_and_back(case)
    dev = torch.device("cuda")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    leaves = [t(a).requires_grad_(True) for a in (case.q, case.k, case.v, case.tq, case.tk, case.tv)]
    i = case.index
    indices = [None, t(i["w_sizes"]).long(), None, t(i["w2n"]).long(), t(i["n2n"]).long(), t(case.n_coords)]
    rng = np.random.default_rng(66)
    dout = rng.standard_normal(case.q.shape).astype(np.float32)
    if half:
        dout = dout.astype(np.float16).astype(np.float32)
    with torch.autocast("cuda", dtype=torch.float16, enabled=half):
        out = SelfAttnAIOFunction.apply(*leaves, case.table_sizes.tolist(), indices, PosEmb.SEPARATE,
                                        TableDims.D0, IndexMode.INDIRECT, getattr(PrecisionMode, precision_name))
    assert out.dtype == (torch.float16 if half else torch.float32)
    out.backward(t(dout).to(out.dtype))
    torch.cuda.synchronize()
    ref = oracle_lib.attn_bwd(*case.oracle_args(), dout)
    got = [leaf.grad.double().cpu().numpy() for leaf in leaves]
    assert all(leaf.grad.dtype == torch.float32 for leaf in leaves)
    _assert_close(got, ref, torch.float16 if half else torch.float32)


def test_autograd_half_forward_on_fp16_features(oracle_lib, hip_lib):
    """HALF_FORWARD as a layer under autocast uses it: q, k, v arrive in fp16 (the output of an autocast linear
    layer), the tables are fp32 parameters; the forward runs in fp16 and the backward in fp32 on the fp16 tensors.
    The feature gradients come back in fp16 and equal those of fp32 leaves holding the same values (the reference's
    own way through this mode: copies cast up, gradients cast down) to the rounding to fp16."""
    from swin3d_amd.sparse_dl.attn.attn_coff import (SelfAttnAIOFunction, PosEmb, TableDims, IndexMode,
                                                     PrecisionMode)
    case = make_attn_case(oracle_lib, seed=67, n=1500, ws=5, quant=4, heads=6, dim=8, extent=(9, 9, 3))
    case.v *= np.float32(0.4)
    case.tv *= np.float32(0.2)
    dev = torch.device("cuda")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    i = case.index
    indices = [None, t(i["w_sizes"]).long(), None, t(i["w2n"]).long(), t(i["n2n"]).long(), t(case.n_coords)]
    dout = t(np.random.default_rng(68).standard_normal(case.q.shape).astype(np.float32)).half()

    def grads_of(feat_dtype):
        feats = [t(a).half().to(feat_dtype).requires_grad_(True) for a in (case.q, case.k, case.v)]
        tables = [t(a).requires_grad_(True) for a in (case.tq, case.tk, case.tv)]
        with torch.autocast("cuda", dtype=torch.float16):
            out = SelfAttnAIOFunction.apply(*feats, *tables, case.table_sizes.tolist(), indices, PosEmb.SEPARATE,
                                            TableDims.D0, IndexMode.INDIRECT, PrecisionMode.HALF_FORWARD)
        assert out.dtype == torch.float16
        out.backward(dout)
        torch.cuda.synchronize()
        return [x.grad for x in feats + tables]

    half, wide = grads_of(torch.float16), grads_of(torch.float32)
    row_scale = max(float(w.abs().max()) for w in wide[:3])
    for name, h, w in zip(NAMES[:3], half, wide):
        assert h.dtype == torch.float16 and w.dtype == torch.float32, name
        assert bool(((h.float() - w).abs() <= _half_rounding(w, row_scale)).all()), name
    scale = max(float(w.abs().max()) for w in wide[3:])
    for name, h, w in zip(NAMES[3:], half[3:], wide[3:]):
        assert h.dtype == torch.float32 and float((h - w).abs().max()) <= 1e-5 * scale, name


def test_headline_size_properties(hip_lib):
    """Swin3D-S stage-1 size (200k voxels, fp16): closed forms that hold for any input.
    Softmax rows sum to one, hence per window and head  sum_j dv_j = sum_i dout_i,  and for every axis
    sum_rows dTv[axis][row][h][c] = sum_i dout_i[h][c];  logit gradients of a row sum to zero, hence
    sum_rows dTq[axis][row][h][c] = sum_i q_i[h][c] * 0 ... checked through linearity in dout instead:
    bwd(2 * dout) = 2 * bwd(dout) exactly in the deterministic outputs."""
    import swin3d_amd
    from swin3d_amd import crse
    dev = torch.device("cuda")
    scene = synth.make_room((10.0, 8.0, 3.0), 30, 200_000, seed=0)
    heads, dim, ws, quant, mode = 6, 8, 5, 4, "XYZ_RGB_NORM"
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    n = scene.coords.shape[0]
    args = swin3d_amd.get_index01(t(scene.coords), 1, ws, t(scene.frac), t(synth.signals(scene, mode)))
    _, _, _, w_sizes, w2n, n2n, _, n_coords = args
    n_crse = crse.scale_crse_coords(n_coords, quant, mode)
    sizes = crse.crse_table_sizes(ws, quant, heads, dim, mode)
    q, k, v, tables = synth.layer_inputs(n, heads * dim, heads, int(sum(sizes)), seed=0, dtype=np.float16)
    dout = np.random.default_rng(5).standard_normal((n, heads, dim)).astype(np.float16)
    a = (t(q), t(k), t(v), t(tables[0]), t(tables[1]), t(tables[2]), sizes, w_sizes, w2n, n2n, n_crse)
    out, omax, osum = swin3d_amd.window_attention_forward(*a, return_stats=True)
    g1 = swin3d_amd.window_attention_backward(*a, out, omax, osum, t(dout))
    g2 = swin3d_amd.window_attention_backward(*a, out, omax, osum, t(dout) * 2)
    torch.cuda.synchronize()
    assert all(torch.isfinite(g).all() for g in g1)
    for x, y in zip(g1[:3], g2[:3]):
        # a power of two commutes with every rounding involved except the one to fp16 subnormals
        # (spacing 2^-24) of the stored result
        assert float((x.float() * 2 - y.float()).abs().max()) <= 2.0 ** -23
    # sum over the keys of a window of dv = sum over its queries of dout
    win = torch.repeat_interleave(torch.arange(w_sizes.numel(), device=dev), w_sizes.long())
    rows = n2n.long()
    dv_w = torch.zeros((w_sizes.numel(), heads, dim), device=dev).index_add_(0, win, g1[2][rows].float())
    do_w = torch.zeros_like(dv_w).index_add_(0, win, t(dout)[rows].float())
    assert float((dv_w - do_w).abs().max()) <= 3e-3 * float(do_w.abs().max())
    total = t(dout).float().sum(0)            # [H,D]
    off = 0
    for size in sizes:
        block = g1[5][off:off + size].reshape(-1, heads, dim).sum(0)
        off += size
        assert float((block - total).abs().max()) <= 1e-3 * float(t(dout).float().abs().sum(0).max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_repeated_calls(oracle_lib, hip_lib, dtype):
    """dq, dk, dv have one owner per element and come out bit-identical on every call.  The table gradients are sums
    of per-wavefront partial sums, and which units a wavefront draws from the work queues varies between calls: they
    agree to fp32 rounding (1e-5 of the largest element here; 1e-6 is typical), not bit for bit."""
    import swin3d_amd
    case = make_attn_case(oracle_lib, seed=77, n=20000, ws=5, quant=4, heads=6, dim=8, extent=(24, 24, 8), recipe="layer")
    dev = torch.device("cuda")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    i = case.index
    feats = [t(x).to(dtype) for x in (case.q, case.k, case.v, case.tq, case.tk, case.tv)]
    idx = [t(i["w_sizes"]).int(), t(i["w2n"]).int(), t(i["n2n"]).int(), t(case.n_coords)]
    sizes = [int(x) for x in case.table_sizes]
    out, mx, sm = swin3d_amd.window_attention_forward(*feats, sizes, *idx, return_stats=True)
    dout = torch.randn_like(out)
    first = swin3d_amd.window_attention_backward(*feats, sizes, *idx, out, mx, sm, dout)
    for _ in range(3):
        again = swin3d_amd.window_attention_backward(*feats, sizes, *idx, out, mx, sm, dout)
        torch.cuda.synchronize()
        for a, b in zip(first[:3], again[:3]):
            assert torch.equal(a, b)
        for a, b in zip(first[3:], again[3:]):
            assert float((a - b).abs().max()) <= 1e-5 * float(a.abs().max())


def test_pair_count_larger_than_needed(oracle_lib, hip_lib):
    """pairs is a capacity: a store larger than the window set's sum of squares gives the same gradients."""
    import swin3d_amd
    case = make_attn_case(oracle_lib, seed=78, n=3000, ws=5, quant=4, heads=6, dim=8, extent=(16, 16, 8), recipe="layer")
    dev = torch.device("cuda")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    i = case.index
    feats = [t(x).half() for x in (case.q, case.k, case.v, case.tq, case.tk, case.tv)]
    idx = [t(i["w_sizes"]).int(), t(i["w2n"]).int(), t(i["n2n"]).int(), t(case.n_coords)]
    sizes = [int(x) for x in case.table_sizes]
    out, mx, sm = swin3d_amd.window_attention_forward(*feats, sizes, *idx, return_stats=True)
    dout = torch.randn_like(out)
    m = int((idx[0].long() ** 2).sum())
    exact = swin3d_amd.window_attention_backward(*feats, sizes, *idx, out, mx, sm, dout, pairs=m)
    roomy = swin3d_amd.window_attention_backward(*feats, sizes, *idx, out, mx, sm, dout, pairs=m + 12345)
    for a, b in zip(exact[:3], roomy[:3]):
        assert torch.equal(a, b)
    for a, b in zip(exact[3:], roomy[3:]):
        assert float((a - b).abs().max()) <= 1e-5 * float(a.abs().max())


@pytest.mark.parametrize("heads,dim", [(10, 16), (20, 16), (40, 16), (40, 8)])
def test_head_counts_of_the_large_model(oracle_lib, hip_lib, heads, dim):
    """Swin3D-L runs 10, 20 and 40 heads of 16 channels (many head groups: the sweeps' workgroups then take the
    head groups in turn instead of in whole sets per XCD)."""
    case = make_attn_case(oracle_lib, seed=300 + heads, n=700, ws=7, quant=4, heads=heads, dim=dim, extent=(12, 12, 6),
                          recipe="layer")
    _check(oracle_lib, case, torch.float16, seed=heads)


def test_pair_count_too_small_is_loud(oracle_lib, hip_lib):
    """A pair count below the window set's sum of squares cannot hold every window's records: no fault, and the
    gradients that are incomplete come out as NaN (all three table gradients, the rows of the skipped windows)."""
    import swin3d_amd
    case = make_attn_case(oracle_lib, seed=79, n=3000, ws=5, quant=4, heads=6, dim=8, extent=(16, 16, 8), recipe="layer")
    dev = torch.device("cuda")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    i = case.index
    feats = [t(x).half() for x in (case.q, case.k, case.v, case.tq, case.tk, case.tv)]
    idx = [t(i["w_sizes"]).int(), t(i["w2n"]).int(), t(i["n2n"]).int(), t(case.n_coords)]
    sizes = [int(x) for x in case.table_sizes]
    out, mx, sm = swin3d_amd.window_attention_forward(*feats, sizes, *idx, return_stats=True)
    dout = torch.randn_like(out)
    m = int((idx[0].long() ** 2).sum())
    full = swin3d_amd.window_attention_backward(*feats, sizes, *idx, out, mx, sm, dout, pairs=m)
    short = swin3d_amd.window_attention_backward(*feats, sizes, *idx, out, mx, sm, dout, pairs=m // 2)
    torch.cuda.synchronize()
    for g in short[3:]:
        assert torch.isnan(g).all()
    for g, ref in zip(short[:3], full[:3]):
        bad = torch.isnan(g.float()).any(dim=2).any(dim=1)
        assert bad.any() and not bad.all()
        assert torch.equal(g[~bad], ref[~bad])      # the windows inside the store are complete
