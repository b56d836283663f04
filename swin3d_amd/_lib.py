"""ctypes loader of libswin3d_amd.so (the C-ABI HIP library declared in include/swin3d_amd.h).

There is no fallback: if the shared library is missing or a call fails, a
RuntimeError is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libswin3d_amd.so")

S3D_DTYPE_F32 = 0
S3D_DTYPE_F16 = 1
S3D_DTYPE_F32_F16_ROWS = 2     # s3d_attn_bwd only: fp32 tables beside fp16 rows
KNN_KMAX = 64
S3D_ATTN_PLANNED = 4
S3D_ATTN_SIZES_ON_DEVICE = 8

_lib = None

_vp = ctypes.c_void_p
_i32 = ctypes.c_int32
_i64 = ctypes.c_int64

# name -> (restype, argtypes); mirrors include/swin3d_amd.h
SIGNATURES = {
    "s3d_version": (ctypes.c_int, []),
    "s3d_last_error_string": (ctypes.c_char_p, []),
    "s3d_attn_fwd_workspace_bytes": (ctypes.c_size_t, [_i32, _i64, _i64]),
    "s3d_attn_fwd": (ctypes.c_int, [_vp] * 7 + [_i32, _i64] + [_vp] * 7 +
                     [_i64, _i32, _i32, _i64, _i64, _i32, _i32, _vp, ctypes.c_size_t, _vp]),
    "s3d_attn_plan_bytes": (ctypes.c_size_t, [_i32, _i64, _i64]),
    "s3d_attn_plan": (ctypes.c_int, [_vp, _i32, _i64, _vp, _vp, _i64, _i32, _i32, _i64, _i32, _vp, ctypes.c_size_t, _vp]),
    "s3d_attn_fwd_noalloc": (ctypes.c_int, [_vp] * 7 + [_i32, _i64] + [_vp] * 7 +
                             [_i64, _i32, _i32, _i64, _i64, _i32, _vp]),
    "s3d_attn_bwd_workspace_bytes": (ctypes.c_size_t, [_i32, _i32, _i32, _i64, _i64, _i64, _i64]),
    # q k v tq tk tv sizes | nd len | w_sizes w2n n2n coords out max sum dout dq dk dv dtq dtk dtv | N H D W pairs dtype | ws bytes stream
    "s3d_attn_bwd": (ctypes.c_int, [_vp] * 7 + [_i32, _i64] + [_vp] * 14 +
                     [_i64, _i32, _i32, _i64, _i64, _i32, _vp, ctypes.c_size_t, _vp]),
    "s3d_window_index_workspace_bytes": (ctypes.c_size_t, [_i64]),
    "s3d_window_index": (ctypes.c_int, [_vp, _i64, _i32, _i32, _i32] + [_vp] * 6 + [ctypes.c_size_t, _vp]),
    "s3d_window_index_grid_workspace_bytes": (ctypes.c_size_t, [_i64]),
    "s3d_window_index_grid": (ctypes.c_int, [_vp, _i64, _i32, _i32, _i32] + [_vp] * 6 + [ctypes.c_size_t, _vp]),
    "s3d_cell_representatives": (ctypes.c_int, [_vp, _vp, _vp, _i64, _vp, _i64, _i32, _vp, _vp]),
    "s3d_key_neighbours": (ctypes.c_int, [_vp, _vp, _i64, _vp, _i32, _vp, _vp]),
    "s3d_window_signals": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i64, _i32, _i32, ctypes.c_float, ctypes.c_float, _vp,
                                          _i64, _vp]),
    "s3d_knn_workspace_bytes": (ctypes.c_size_t, [_i64, _i64, _i32]),
    "s3d_knn": (ctypes.c_int, [_i32, _vp, _i64, _vp, _i64, _vp, _vp, _i32, _vp, _vp, ctypes.c_float,
                               _vp, ctypes.c_size_t, _vp]),
    "s3d_knn_interpolate": (ctypes.c_int, [_vp, _vp, _i32, _i64, _vp, _i64, _i32, _i32, _vp, _vp]),
    "s3d_knn_max_pool": (ctypes.c_int, [_vp, _i32, _i64, _vp, _i64, _i32, _i32, _vp, _vp]),
    "s3d_add_layernorm": (ctypes.c_int, [_vp, _vp, _i32, _vp, _vp, ctypes.c_float, _vp, _vp, _i32, _i64, _i32, _vp]),
}


def lib():
    """The loaded library; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m swin3d_amd.build` "
                "(hipcc --offload-arch=gfx950); swin3d_amd has no CPU or PyTorch fallback")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(status, what):
    if status != 0:
        msg = lib().s3d_last_error_string().decode("utf-8", "replace")
        kind = ValueError if status < 0 else RuntimeError
        raise kind(f"{what} failed with status {status}: {msg}")
