"""Helpers of the GPU parity tests: move a numpy AttnCase to the device and call the op
through the Python surface (ctypes -> C ABI -> HIP)."""
import numpy as np
import torch

import swin3d_amd


def run_attention(case, dtype=torch.float32, return_stats=False, device="cuda", device_sizes=False):
    """-> numpy float64 output [N,H,D] of swin3d_amd.window_attention_forward.  device_sizes: the per-axis table
    sizes go in as a CUDA tensor (the sweep kernel reads them, the host never does) instead of a host list."""
    dev = torch.device(device)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    i = case.index
    res = swin3d_amd.window_attention_forward(
        t(case.q).to(dtype), t(case.k).to(dtype), t(case.v).to(dtype),
        t(case.tq).to(dtype), t(case.tk).to(dtype), t(case.tv).to(dtype),
        t(case.table_sizes) if device_sizes else [int(x) for x in case.table_sizes], t(i["w_sizes"]), t(i["w2n"]), t(i["n2n"]), t(case.n_coords),
        return_stats=return_stats)
    torch.cuda.synchronize()
    if return_stats:
        return tuple(r.double().cpu().numpy() for r in res)
    return res.double().cpu().numpy()


def assert_attn_close(got, ref, dtype):
    """fp32: |a-b| <= 1e-5 * scale, scale = max(largest |ref| over the D channels of the same
    (voxel, head), 1e-2 * max|ref|): 1e-5 relative to the head vector the element belongs to.
    An element-wise relative bound is not attainable in fp32: a channel that cancels to ~0 still
    carries the rounding of logits of magnitude ~10 (one fp32 ulp there is 1e-6, and an absolute
    logit error is a relative error of the softmax weight).  fp16: |a-b| <= 2e-3 absolute."""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    assert np.isfinite(got).all()
    err = np.abs(got - ref)
    if dtype == torch.float32:
        row_scale = np.abs(ref).max(axis=-1, keepdims=True)
        tol = 1e-5 * np.maximum(row_scale, 1e-2 * np.abs(ref).max()) * np.ones_like(ref)
    else:
        tol = np.full_like(ref, 2e-3)
    worst = np.unravel_index(np.argmax(err - tol), err.shape)
    assert (err <= tol).all(), (f"max err {err.max():.3e} (tol there {tol[worst]:.3e}) at {worst}: "
                                f"got {got[worst]:.6f} ref {ref[worst]:.6f}")


def elementwise_bound_failures(got, ref):
    """Elements outside the purely element-wise fp32 bound |a-b| <= 1e-5 * max(|b|, 1e-2 * max|ref|)
    -> (count, elements, largest |a-b| / bound)."""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    bound = 1e-5 * np.maximum(np.abs(ref), 1e-2 * np.abs(ref).max())
    ratio = np.abs(got - ref) / bound
    return int((ratio > 1.0).sum()), int(ref.size), float(ratio.max())
