"""s3d_attn_fwd_noalloc, the forward that takes no workspace and allocates nothing: called through the C ABI and
compared with s3d_attn_fwd (sweep kernel) on the same inputs, on two calls in a row, the second with a smaller
input (both calls use the one scratch array of the GPU, which keeps the first call's contents)."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import make_attn_case

pytestmark = pytest.mark.gpu


def _device_case(oracle_lib, seed, n, heads, dim, ws, dtype, extent):
    case = make_attn_case(oracle_lib, seed=seed, n=n, ws=ws, quant=4, heads=heads, dim=dim, extent=extent,
                          recipe="layer")
    dev = torch.device("cuda")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    f = lambda a: t(a).to(dtype)
    i = case.index
    tensors = dict(q=f(case.q), k=f(case.k), v=f(case.v), tq=f(case.tq), tk=f(case.tk), tv=f(case.tv),
                   w_sizes=t(i["w_sizes"]).int(), w2n=t(i["w2n"]).int(), n2n=t(i["n2n"]).int(),
                   n_coords=t(case.n_coords).float().contiguous())
    return case, tensors


def _call_both(hip_lib, case, x, dtype):
    from swin3d_amd import _lib
    n, h, d = x["q"].shape
    w = x["w_sizes"].numel()
    sizes = [int(s) for s in case.table_sizes]
    c_sizes = (ctypes.c_int32 * len(sizes))(*sizes)
    code = _lib.S3D_DTYPE_F16 if dtype == torch.float16 else _lib.S3D_DTYPE_F32
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for which in ("workspace", "noalloc"):
        out = torch.full((n, h, d), float("nan"), dtype=dtype, device="cuda")
        omax = torch.full((n, h), float("nan"), dtype=torch.float32, device="cuda")
        osum = torch.full((n, h), float("nan"), dtype=torch.float32, device="cuda")
        head = [x["q"].data_ptr(), x["k"].data_ptr(), x["v"].data_ptr(), x["tq"].data_ptr(), x["tk"].data_ptr(),
                x["tv"].data_ptr(), c_sizes, len(sizes), x["tq"].numel(), x["w_sizes"].data_ptr(), x["w2n"].data_ptr(),
                x["n2n"].data_ptr(), x["n_coords"].data_ptr(), out.data_ptr(), omax.data_ptr(), osum.data_ptr(),
                n, h, d, w]
        if which == "workspace":
            ws_bytes = hip_lib.s3d_attn_fwd_workspace_bytes(h, n, w)
            workspace = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
            status = hip_lib.s3d_attn_fwd(*head, 0, code, 0, workspace.data_ptr(), ws_bytes, stream)
            _lib.check(status, "s3d_attn_fwd")
        else:
            # one call first: the code object, the scratch array's address and the kernel's LDS limit are set up
            # by the first call on a device (and of a shape); the measured call comes after it
            _lib.check(hip_lib.s3d_attn_fwd_noalloc(*head, 0, code, stream), "s3d_attn_fwd_noalloc")
            torch.cuda.synchronize()
            out.fill_(float("nan")), omax.fill_(float("nan")), osum.fill_(float("nan"))
            torch.cuda.synchronize()
            before = torch.cuda.memory_allocated()          # torch's caching allocator
            free_before = torch.cuda.mem_get_info()[0]      # the device's free bytes (hipMemGetInfo): sees any hipMalloc
            status = hip_lib.s3d_attn_fwd_noalloc(*head, 0, code, stream)
            _lib.check(status, "s3d_attn_fwd_noalloc")
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated() == before
            assert torch.cuda.mem_get_info()[0] == free_before
        torch.cuda.synchronize()
        outs.append((out, omax, osum))
    return outs


@pytest.mark.parametrize("dtype,heads,dim,ws", [(torch.float16, 6, 8, 5), (torch.float32, 4, 16, 7)])
def test_noalloc_forward_equals_workspace_forward_on_two_calls(oracle_lib, hip_lib, dtype, heads, dim, ws):
    from gpu_helpers import assert_attn_close
    for seed, n, extent in ((61, 6000, (30, 30, 10)), (62, 700, (12, 12, 6))):     # the second input is smaller
        case, x = _device_case(oracle_lib, seed, n, heads, dim, ws, dtype, extent)
        (ref, rmax, rsum), (got, gmax, gsum) = _call_both(hip_lib, case, x, dtype)
        assert torch.isfinite(ref).all() and torch.isfinite(got).all()
        # same kernels on the same work list: identical, and in any case within the operator's tolerance
        assert_attn_close(got.double().cpu().numpy(), ref.double().cpu().numpy(), dtype)
        assert torch.equal(got, ref) and torch.equal(gmax, rmax) and torch.equal(gsum, rsum)


def test_noalloc_forward_rejects_inputs_beyond_its_scratch(hip_lib):
    """More windows than the built-in work list holds: a clear error before anything is launched."""
    from swin3d_amd import _lib
    # the pointers below are placeholders, so the call must not get as far as a launch: sizes that no built-in
    # scratch of any plausible size holds (one voxel per window, 24 bytes of work list per window: 26 GB)
    n = w = 1 << 30
    sizes = [40 * 48] * 3
    c_sizes = (ctypes.c_int32 * 3)(*sizes)
    assert hip_lib.s3d_attn_fwd_workspace_bytes(6, n, w) > (1 << 34)
    one = torch.zeros(16, dtype=torch.float16, device="cuda")
    p = one.data_ptr()
    status = hip_lib.s3d_attn_fwd_noalloc(p, p, p, p, p, p, c_sizes, 3, sum(sizes), p, p, p, p, p, None, None,
                                          n, 6, 8, w, 0, _lib.S3D_DTYPE_F16, torch.cuda.current_stream().cuda_stream)
    assert status == -5      # S3D_ERR_WORKSPACE
    assert b"scratch" in hip_lib.s3d_last_error_string()
