"""The C-ABI library loads and exports every symbol include/swin3d_amd.h declares
(no device calls: runs without a GPU)."""
import ctypes
import os
import re

from conftest import ROOT


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "swin3d_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(s3d_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared_symbols()
    for must in ("s3d_add_layernorm", "s3d_attn_fwd", "s3d_attn_bwd", "s3d_attn_bwd_workspace_bytes", "s3d_knn_interpolate", "s3d_knn_max_pool", "s3d_attn_plan", "s3d_attn_fwd_noalloc", "s3d_attn_fwd_workspace_bytes", "s3d_window_index", "s3d_window_index_workspace_bytes", "s3d_window_signals", "s3d_key_neighbours", "s3d_cell_representatives", "s3d_knn",
                 "s3d_knn_workspace_bytes", "s3d_last_error_string", "s3d_version"):
        assert must in names


def test_library_exports_every_declared_symbol(hip_lib):
    for name in _declared_symbols():
        assert hasattr(hip_lib, name), f"{name} is declared in the header but not exported"


def test_python_signatures_cover_the_header(hip_lib):
    from swin3d_amd import _lib
    assert sorted(_lib.SIGNATURES) == _declared_symbols()


def test_python_constants_equal_the_header():
    """The codes that the ctypes layer passes are the header's #defines."""
    from swin3d_amd import _lib
    text = open(os.path.join(ROOT, "include", "swin3d_amd.h")).read()
    defines = {name: int(value, 0) for name, value in re.findall(r"^#define (S3D_[A-Z0-9_]+) \(?(-?(?:0x)?[0-9a-fA-F]+)\)?\s*(?:/\*.*)?$",
                                                              text, flags=re.M)}
    for name in ("S3D_DTYPE_F32", "S3D_DTYPE_F16", "S3D_DTYPE_F32_F16_ROWS", "S3D_ATTN_PLANNED",
                 "S3D_ATTN_SIZES_ON_DEVICE"):
        assert defines[name] == getattr(_lib, name), name
    assert defines["S3D_KNN_KMAX"] == _lib.KNN_KMAX


def test_version_and_error_string(hip_lib):
    assert hip_lib.s3d_version() >= 200
    assert isinstance(hip_lib.s3d_last_error_string(), bytes)


def test_argument_errors_are_reported_without_a_device(hip_lib):
    from swin3d_amd import _lib
    # K out of range is rejected before anything touches the GPU
    status = hip_lib.s3d_knn(0, None, 0, None, 0, None, None, 1, None, None, 0.0, None, 0, None)
    assert status < 0
    assert b"K=0" in hip_lib.s3d_last_error_string()
    status = hip_lib.s3d_attn_fwd(*([None] * 7), 9, 0, *([None] * 7), 10, 6, 8, 1, 0, 1, 0, None, 0, None)
    assert status < 0 and b"table_len" in hip_lib.s3d_last_error_string()
    try:
        _lib.check(status, "s3d_attn_fwd")
    except ValueError as e:
        assert "s3d_attn_fwd failed" in str(e)
    else:
        raise AssertionError("check() must raise on a negative status")


def test_more_argument_errors_without_a_device(hip_lib):
    """Rejected before any launch: a row stride the kernels cannot read, the backward's table-row limit and
    missing workspace, the interpolation's K and dtype."""
    import ctypes
    from swin3d_amd import crse
    sizes = crse.crse_table_sizes(5, 4, 6, 8, "XYZ_RGB_NORM")
    c_sizes = (ctypes.c_int32 * 9)(*sizes)
    total = sum(sizes)
    st = hip_lib.s3d_attn_fwd(*([None] * 6), c_sizes, 9, total, *([None] * 7), 10, 6, 8, 1, 50, 1, 0, None, 0, None)
    assert st < 0 and b"qkv_row_stride" in hip_lib.s3d_last_error_string()
    # flag bits that name no behaviour of the call (1 and 2 selected a kernel in earlier versions of the library)
    st = hip_lib.s3d_attn_fwd(*([None] * 6), c_sizes, 9, total, *([None] * 7), 10, 6, 8, 1, 0, 1, 2, None, 0, None)
    assert st < 0 and b"flag" in hip_lib.s3d_last_error_string()
    # backward: workspace missing
    st = hip_lib.s3d_attn_bwd(*([None] * 6), c_sizes, 9, total, *([None] * 14), 10, 6, 8, 1, 0, 1, None, 0, None)
    assert st < 0 and (b"gradient pointer" in hip_lib.s3d_last_error_string()
                       or b"workspace" in hip_lib.s3d_last_error_string())
    # backward: a head_dim that no form covers
    small = crse.crse_table_sizes(5, 4, 6, 24, "XYZ_RGB_NORM")
    c_small = (ctypes.c_int32 * 9)(*small)
    st = hip_lib.s3d_attn_bwd(*([None] * 6), c_small, 9, sum(small), *([None] * 14), 10, 6, 24, 1, 0, 1, None, 0, None)
    assert st < 0 and b"head_dim 24" in hip_lib.s3d_last_error_string()
    table_len = sum(crse.crse_table_sizes(5, 4, 6, 8, "XYZ_RGB_NORM"))
    assert hip_lib.s3d_attn_bwd_workspace_bytes(6, 8, 9, table_len, 1000, 40, 0) >= 4 * (40 + 6) + 4 * 6000
    assert (hip_lib.s3d_attn_bwd_workspace_bytes(6, 8, 9, table_len, 1000, 40, 30000) >=
            hip_lib.s3d_attn_bwd_workspace_bytes(6, 8, 9, table_len, 1000, 40, 0) + 12 * 6 * 30000)
    # the general form (head_dim 32; more table rows per head than the register blocks cover, window 10 at quant 8):
    # fp32 accumulators of dk and dv, no pair store
    big = sum(crse.crse_table_sizes(10, 8, 6, 8, "XYZ_RGB_NORM"))
    for dim, length in ((32, table_len * 4), (8, big)):
        need = hip_lib.s3d_attn_bwd_workspace_bytes(6, dim, 9, length, 1000, 40, 30000)
        assert 2 * 4 * 1000 * 6 * dim + 4 * 6000 <= need <= 2 * 4 * 1000 * 6 * dim + 4 * 6000 + (1 << 20)
    st = hip_lib.s3d_knn_interpolate(None, None, 0, 10, None, 10, 8, 0, None, None)
    assert st < 0 and b"K=0" in hip_lib.s3d_last_error_string()
    st = hip_lib.s3d_knn_interpolate(None, None, 3, 10, None, 10, 8, 7, None, None)
    assert st < 0 and b"dtype" in hip_lib.s3d_last_error_string()
    assert hip_lib.s3d_knn_interpolate(None, None, 3, 0, None, 10, 8, 0, None, None) == 0   # nothing to do
    st = hip_lib.s3d_add_layernorm(None, None, 0, None, None, 1e-5, None, None, 1, 10, 66, None)
    assert st < 0 and b"multiple of 4" in hip_lib.s3d_last_error_string()
    st = hip_lib.s3d_add_layernorm(None, None, 0, None, None, 1e-5, None, None, 5, 10, 64, None)
    assert st < 0 and b"y_dtype" in hip_lib.s3d_last_error_string()
    assert hip_lib.s3d_add_layernorm(None, None, 0, None, None, 1e-5, None, None, 1, 0, 64, None) == 0


def test_work_list_size_depends_on_the_window_set_only(hip_lib):
    """The forward's workspace is its work list: counters per head, a record per unit of at least 8 queries, 24
    bytes per window and the list builder's notes; the plan buffer is the same thing."""
    for heads, n, w in ((6, 199_327, 7_554), (40, 2_713, 40), (10, 595_677, 22_000), (1, 0, 0)):
        need = hip_lib.s3d_attn_fwd_workspace_bytes(heads, n, w)
        assert need == hip_lib.s3d_attn_plan_bytes(heads, n, w)
        assert 2 * n + 24 * w <= need <= 2 * n + 24 * w + 2048 * heads + (1 << 19)
    assert hip_lib.s3d_attn_fwd_workspace_bytes(0, 10, 1) == 0 and hip_lib.s3d_attn_fwd_workspace_bytes(6, -1, 1) == 0


def test_window_signals_rejects_bad_arguments(hip_lib):
    """Argument checks run before anything touches the GPU."""
    import ctypes
    f = ctypes.c_float
    assert hip_lib.s3d_window_signals(None, None, None, None, 0, 0, 5, f(1), f(1), None, 0, None) == 0     # N = 0
    assert hip_lib.s3d_window_signals(None, None, None, None, 0, 0, 5, f(1), f(1), None, 4, None) < 0      # null pointers
    assert hip_lib.s3d_window_signals(None, None, None, None, 2, 6, 5, f(1), f(1), None, 4, None) < 0      # stride < columns
    assert hip_lib.s3d_window_signals(None, None, None, None, 0, 0, 11, f(1), f(1), None, 4, None) < 0     # window > 10
    assert b"s3d_window_signals" in hip_lib.s3d_last_error_string()
