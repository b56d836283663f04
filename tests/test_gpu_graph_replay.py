"""The forward that allocates nothing (s3d_attn_fwd_noalloc), the planned forward and the backward under HIP graph capture: the
launches are recorded once and replayed on changed inputs, with the program's own eager work and synchronisations
between the replays; every replay must give the bits of the eager call on the same inputs.  (The work list's
queue counters are put back to zero by the sweep kernel itself, so a replay needs no clearing node.)"""
import ctypes

import numpy as np
import pytest
import torch

from helpers import make_attn_case

pytestmark = pytest.mark.gpu


def _inputs(oracle_lib, seed):
    case = make_attn_case(oracle_lib, seed=seed, n=5000, ws=5, quant=4, heads=6, dim=8, extent=(26, 26, 8), recipe="layer")
    dev = torch.device("cuda")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    i = case.index
    x = dict(q=t(case.q).half(), k=t(case.k).half(), v=t(case.v).half(), tq=t(case.tq).half(), tk=t(case.tk).half(),
             tv=t(case.tv).half(), w_sizes=t(i["w_sizes"]).int(), w2n=t(i["w2n"]).int(), n2n=t(i["n2n"]).int(),
             n_coords=t(case.n_coords).float().contiguous())
    return case, x


@pytest.mark.parametrize("entry", ["noalloc", "planned"])
def test_replays_equal_eager_calls(oracle_lib, hip_lib, entry):
    from swin3d_amd import _lib
    case, x = _inputs(oracle_lib, 101)
    n, h, d = x["q"].shape
    w = x["w_sizes"].numel()
    sizes = [int(s) for s in case.table_sizes]
    c_sizes = (ctypes.c_int32 * len(sizes))(*sizes)
    out = torch.zeros_like(x["q"])
    plan = torch.empty(hip_lib.s3d_attn_plan_bytes(h, n, w), dtype=torch.uint8, device="cuda")
    side = torch.cuda.Stream()      # default priority

    def launch(stream):
        head = [x["q"].data_ptr(), x["k"].data_ptr(), x["v"].data_ptr(), x["tq"].data_ptr(), x["tk"].data_ptr(),
                x["tv"].data_ptr(), c_sizes, len(sizes), x["tq"].numel(), x["w_sizes"].data_ptr(), x["w2n"].data_ptr(),
                x["n2n"].data_ptr(), x["n_coords"].data_ptr(), out.data_ptr(), None, None, n, h, d, w]
        if entry == "noalloc":
            status = hip_lib.s3d_attn_fwd_noalloc(*head, 0, _lib.S3D_DTYPE_F16, stream)
        else:
            status = hip_lib.s3d_attn_fwd(*head, 0, _lib.S3D_DTYPE_F16, _lib.S3D_ATTN_PLANNED, plan.data_ptr(),
                                          plan.numel(), stream)
        _lib.check(status, entry)

    if entry == "planned":
        _lib.check(hip_lib.s3d_attn_plan(c_sizes, len(sizes), x["tq"].numel(), x["w_sizes"].data_ptr(), x["w2n"].data_ptr(),
                                         n, h, d, w, _lib.S3D_DTYPE_F16, plan.data_ptr(), plan.numel(),
                                         torch.cuda.current_stream().cuda_stream), "s3d_attn_plan")
    # one eager call before the capture: the first call on a device looks up the scratch array's address and the
    # first call of a shape raises the kernel's dynamic-LDS limit; the calls after it enqueue kernels only
    launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        graph.capture_begin()
        launch(side.cuda_stream)
        graph.capture_end()
    torch.cuda.synchronize()
    rng = torch.Generator(device="cuda").manual_seed(7)
    for _ in range(3):
        # new contents in the recorded buffers, eager work between the replays
        x["q"].copy_(torch.randn(x["q"].shape, generator=rng, device="cuda").half() * 0.1)
        x["v"].copy_(torch.randn(x["v"].shape, generator=rng, device="cuda").half())
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = out.clone()
        out.fill_(float("nan"))
        launch(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert torch.isfinite(replayed).all()
        assert torch.equal(replayed, out)


def test_backward_replays_equal_eager_calls(oracle_lib, hip_lib):
    """s3d_attn_bwd with its pair store under graph capture: the whole call - list builds, pair sweeps,
    table-gradient kernels, reductions - is kernels on the caller's stream and clears what it needs itself."""
    from swin3d_amd import _lib
    import swin3d_amd
    case, x = _inputs(oracle_lib, 102)
    n, h, d = x["q"].shape
    w = x["w_sizes"].numel()
    sizes = [int(s) for s in case.table_sizes]
    c_sizes = (ctypes.c_int32 * len(sizes))(*sizes)
    table_len = x["tq"].numel()
    pairs = int((x["w_sizes"].long() ** 2).sum())
    out, omax, osum = swin3d_amd.window_attention_forward(x["q"], x["k"], x["v"], x["tq"], x["tk"], x["tv"], sizes,
                                                          x["w_sizes"], x["w2n"], x["n2n"], x["n_coords"],
                                                          return_stats=True)
    dout = torch.randn_like(out)
    grads = [torch.empty_like(x["q"]) for _ in range(3)] + [torch.empty(table_len, dtype=torch.float32, device="cuda")
                                                           for _ in range(3)]
    nbytes = hip_lib.s3d_attn_bwd_workspace_bytes(h, d, len(sizes), table_len, n, w, pairs)
    workspace = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    side = torch.cuda.Stream()      # default priority

    def launch(stream):
        status = hip_lib.s3d_attn_bwd(
            x["q"].data_ptr(), x["k"].data_ptr(), x["v"].data_ptr(), x["tq"].data_ptr(), x["tk"].data_ptr(),
            x["tv"].data_ptr(), c_sizes, len(sizes), table_len, x["w_sizes"].data_ptr(), x["w2n"].data_ptr(),
            x["n2n"].data_ptr(), x["n_coords"].data_ptr(), out.data_ptr(), omax.data_ptr(), osum.data_ptr(),
            dout.data_ptr(), *(g.data_ptr() for g in grads), n, h, d, w, pairs, _lib.S3D_DTYPE_F16,
            workspace.data_ptr(), nbytes, stream)
        _lib.check(status, "s3d_attn_bwd")

    launch(torch.cuda.current_stream().cuda_stream)          # eager warm-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        graph.capture_begin()
        launch(side.cuda_stream)
        graph.capture_end()
    torch.cuda.synchronize()
    rng = torch.Generator(device="cuda").manual_seed(8)
    for _ in range(3):
        dout.copy_(torch.randn(dout.shape, generator=rng, device="cuda").half())
        for g in grads:
            g.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = [g.clone() for g in grads]
        for g in grads:
            g.fill_(float("nan"))
        launch(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        for a, b in zip(replayed[:3], grads[:3]):
            assert torch.isfinite(a).all() and torch.equal(a, b)
        for a, b in zip(replayed[3:], grads[3:]):
            assert torch.isfinite(a).all()
            assert float((a - b).abs().max()) <= 1e-5 * float(b.abs().max())
