// Entry points of the windowed self-attention forward: argument checks, work list, launch.
#include "attn_kernels.h"

#include <mutex>

namespace s3d {
namespace {

int fill_axes(AttnArgs &a, const int32_t *table_sizes, int nd, int64_t table_len)
{
    const int64_t hd = static_cast<int64_t>(a.H) * a.D;
    int64_t total = 0;
    int base = 0;
    for (int n = 0; n < nd; ++n) {
        const int64_t size = table_sizes[n];
        if (size <= 0 || size % hd != 0)
            return fail(S3D_ERR_BAD_SHAPE, "s3d_attn_fwd: table_sizes[%d] = %lld is not a positive "
                        "multiple of H*D = %lld", n, (long long)size, (long long)hd);
        total += size;
        a.rows[n] = static_cast<int32_t>(size / hd);
        a.base[n] = base;
        base += a.rows[n];
    }
    for (int n = nd; n < kMaxAxes; ++n) a.rows[n] = a.base[n] = 0;
    if (total != table_len)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_attn_fwd: sum(table_sizes) = %lld differs from table_len = %lld",
                    (long long)total, (long long)table_len);
    a.total_rows = base;
    return S3D_OK;
}

int check_shape(int64_t N, int64_t W, int32_t H, int32_t D, int32_t nd, int64_t table_len)
{
    if (N < 0 || W < 0 || H < 1 || D < 1 || nd < 1 || table_len < 1)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_attn_fwd: bad sizes N=%lld W=%lld H=%d D=%d nd=%d table_len=%lld",
                    (long long)N, (long long)W, H, D, nd, (long long)table_len);
    if (nd != 3 && nd != 6 && nd != 9)
        return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd: %d cRSE axes (3, 6 or 9)", nd);
    if (D != 8 && D != 16 && D != 32)
        return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd: head_dim %d (8, 16 or 32)", D);
    if (W > 0x7fffffffLL || N > 0x7fffffffLL || H > 65535)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_attn_fwd: N, W must fit 31 bits and H 16 bits");
    if (table_len / (static_cast<int64_t>(H) * D) > 65536)
        return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd: more than 65536 table rows per head");
    return S3D_OK;
}

}  // namespace
}  // namespace s3d

extern "C" __attribute__((visibility("default"))) size_t s3d_attn_fwd_workspace_bytes(int32_t H, int64_t N, int64_t W)
{
    if (H < 1 || N < 0 || W < 0) return 0;
    return s3d::attn_sweep_workspace_bytes(H, W, N);
}

namespace s3d {
namespace {

// Argument checks shared by the two forward entry points; fills `a` (everything but the workspace).
// *empty is set when there is nothing to compute.
int prepare_attn_args(const char *who, AttnArgs &a, bool *empty, const void *q, const void *k, const void *v,
                      const void *table_q, const void *table_k, const void *table_v, const int32_t *table_sizes,
                      int32_t nd, int64_t table_len, const int32_t *w_sizes, const int32_t *w2n, const int32_t *n2n,
                      const float *n_coords, void *out, float *out_max, float *out_sum, int64_t N, int32_t H,
                      int32_t D, int64_t W, int64_t qkv_row_stride, int32_t dtype, bool sizes_on_device = false)
{
    *empty = true;
    if (int rc = check_shape(N, W, H, D, nd, table_len)) return rc;
    if (dtype != S3D_DTYPE_F32 && dtype != S3D_DTYPE_F16)
        return fail(S3D_ERR_BAD_DTYPE, "%s: dtype %d (0 = fp32, 1 = fp16)", who, dtype);
    if (!table_sizes) return fail(S3D_ERR_NULL_POINTER, "%s: table_sizes (host) is null", who);
    // rows of q, k, v are read with 16-byte loads: the stride must keep them aligned
    if (qkv_row_stride != 0 && (qkv_row_stride < static_cast<int64_t>(H) * D || qkv_row_stride % 8 != 0))
        return fail(S3D_ERR_BAD_SHAPE, "%s: qkv_row_stride = %lld (0, or a multiple of 8 that is >= H*D = %d)", who,
                    (long long)qkv_row_stride, H * D);
    a.H = H;
    a.D = D;
    a.nd = nd;
    a.N = N;
    a.W = W;
    if (sizes_on_device) {
        // the per-axis sizes stay on the device: the host knows the rows of all axes together and nothing more
        const int64_t hd = static_cast<int64_t>(H) * D;
        if (table_len % hd != 0 || table_len / hd < nd)
            return fail(S3D_ERR_BAD_SHAPE, "%s: table_len = %lld is not a multiple of H*D = %lld with a row per axis", who,
                        (long long)table_len, (long long)hd);
        for (int n = 0; n < kMaxAxes; ++n) a.rows[n] = a.base[n] = 0;
        a.total_rows = static_cast<int32_t>(table_len / hd);
        a.sizes_dev = table_sizes;
    } else if (int rc = fill_axes(a, table_sizes, nd, table_len)) {
        return rc;
    }
    if (N == 0 || W == 0) return S3D_OK;
    if (!q || !k || !v || !table_q || !table_k || !table_v || !w_sizes || !w2n || !n_coords || !out)
        return fail(S3D_ERR_NULL_POINTER, "%s: null device pointer", who);
    a.q = q;
    a.k = k;
    a.v = v;
    a.row_stride = qkv_row_stride == 0 ? static_cast<int64_t>(H) * D : qkv_row_stride;
    a.table_q = table_q;
    a.table_k = table_k;
    a.table_v = table_v;
    a.w_sizes = w_sizes;
    a.w2n = w2n;
    a.n2n = n2n;
    a.n_coords = n_coords;
    a.out = out;
    a.out_max = out_max;
    a.out_sum = out_sum;
    *empty = false;
    return S3D_OK;
}

// Scratch of s3d_attn_fwd_noalloc: the sweep kernel's work list (queue counters, unit and window records, the
// list builder's notes) in a device array that lives as long as the process, one copy per GPU.  In host code
// the array's name is only a handle for hipGetSymbolAddress; kernels and copies get the address it returns.
constexpr size_t kScratchBytes = size_t(8) << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
void *scratch_address[kMaxDevices];   // per device; looked up on the first call there
std::mutex scratch_mutex;

int scratch_of_current_device(void **address)
{
    int device = -1;
    S3D_HIP_CHECK(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices)
        return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd_noalloc: device %d (at most %d devices)", device, kMaxDevices);
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_address[device]) {
        void *p = nullptr;
        S3D_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd_noalloc: no device address for the scratch array");
        scratch_address[device] = p;
    }
    *address = scratch_address[device];
    return S3D_OK;
}

}  // namespace
}  // namespace s3d

extern "C" __attribute__((visibility("default"))) int s3d_attn_fwd(
    const void *q, const void *k, const void *v, const void *table_q, const void *table_k,
    const void *table_v, const int32_t *table_sizes, int32_t nd, int64_t table_len,
    const int32_t *w_sizes, const int32_t *w2n, const int32_t *n2n, const float *n_coords, void *out,
    float *out_max, float *out_sum, int64_t N, int32_t H, int32_t D, int64_t W, int64_t qkv_row_stride,
    int32_t dtype, int32_t flags, void *workspace, size_t workspace_bytes, void *stream)
{
    using namespace s3d;
    AttnArgs a{};
    bool empty = true;
    if (flags & ~(S3D_ATTN_PLANNED | S3D_ATTN_SIZES_ON_DEVICE))
        return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd: unknown flag bits in %d", flags);
    const bool sizes_on_device = (flags & S3D_ATTN_SIZES_ON_DEVICE) != 0;
    if (int rc = prepare_attn_args("s3d_attn_fwd", a, &empty, q, k, v, table_q, table_k, table_v, table_sizes, nd,
                                   table_len, w_sizes, w2n, n2n, n_coords, out, out_max, out_sum, N, H, D, W,
                                   qkv_row_stride, dtype, sizes_on_device))
        return rc;
    if (empty) return S3D_OK;
    a.workspace = workspace;
    const size_t need = attn_sweep_workspace_bytes(H, W, N);
    if (!workspace || workspace_bytes < need)
        return fail(S3D_ERR_WORKSPACE, "s3d_attn_fwd: workspace %zu B < required %zu B",
                    workspace ? workspace_bytes : size_t(0), need);
    // with a plan the work list is in the workspace already
    return launch_attn_sweep(a, dtype, static_cast<hipStream_t>(stream),
                             (flags & S3D_ATTN_PLANNED) ? kAttnSweep : (kAttnBuildList | kAttnSweep));
}

extern "C" __attribute__((visibility("default"))) size_t s3d_attn_plan_bytes(int32_t H, int64_t N, int64_t W)
{
    if (H < 1 || N < 0 || W < 0) return 0;
    return s3d::attn_sweep_workspace_bytes(H, W, N);
}

extern "C" __attribute__((visibility("default"))) int s3d_attn_plan(
    const int32_t *table_sizes, int32_t nd, int64_t table_len, const int32_t *w_sizes, const int32_t *w2n,
    int64_t N, int32_t H, int32_t D, int64_t W, int32_t dtype, void *plan, size_t plan_bytes, void *stream)
{
    using namespace s3d;
    if (int rc = check_shape(N, W, H, D, nd, table_len)) return rc;
    if (dtype != S3D_DTYPE_F32 && dtype != S3D_DTYPE_F16)
        return fail(S3D_ERR_BAD_DTYPE, "s3d_attn_plan: dtype %d (0 = fp32, 1 = fp16)", dtype);
    AttnArgs a{};
    a.H = H;
    a.D = D;
    a.nd = nd;
    a.N = N;
    a.W = W;
    if (table_sizes) {
        if (int rc = fill_axes(a, table_sizes, nd, table_len)) return rc;
    } else {
        // the list depends on the tables through their total size only (how many workgroups share a CU)
        const int64_t hd = static_cast<int64_t>(H) * D;
        if (table_len % hd != 0) return fail(S3D_ERR_BAD_SHAPE, "s3d_attn_plan: table_len is not a multiple of H*D");
        a.total_rows = static_cast<int32_t>(table_len / hd);
    }
    if (N == 0 || W == 0) return S3D_OK;
    if (!w_sizes || !w2n) return fail(S3D_ERR_NULL_POINTER, "s3d_attn_plan: null device pointer");
    const size_t need = attn_sweep_workspace_bytes(H, W, N);
    if (!plan || plan_bytes < need)
        return fail(S3D_ERR_WORKSPACE, "s3d_attn_plan: plan buffer %zu B < required %zu B", plan ? plan_bytes : size_t(0), need);
    a.w_sizes = w_sizes;
    a.w2n = w2n;
    a.workspace = plan;
    return launch_attn_sweep(a, dtype, static_cast<hipStream_t>(stream), kAttnBuildList);
}

extern "C" __attribute__((visibility("default"))) int s3d_attn_fwd_noalloc(
    const void *q, const void *k, const void *v, const void *table_q, const void *table_k,
    const void *table_v, const int32_t *table_sizes, int32_t nd, int64_t table_len,
    const int32_t *w_sizes, const int32_t *w2n, const int32_t *n2n, const float *n_coords, void *out,
    float *out_max, float *out_sum, int64_t N, int32_t H, int32_t D, int64_t W, int64_t qkv_row_stride,
    int32_t dtype, void *stream)
{
    using namespace s3d;
    AttnArgs a{};
    bool empty = true;
    if (int rc = prepare_attn_args("s3d_attn_fwd_noalloc", a, &empty, q, k, v, table_q, table_k, table_v, table_sizes,
                                   nd, table_len, w_sizes, w2n, n2n, n_coords, out, out_max, out_sum, N, H, D, W,
                                   qkv_row_stride, dtype))
        return rc;
    if (empty) return S3D_OK;
    const size_t need = attn_sweep_workspace_bytes(H, W, N);
    if (need > kScratchBytes)
        return fail(S3D_ERR_WORKSPACE, "s3d_attn_fwd_noalloc: N = %lld voxels in W = %lld windows need %zu B of work "
                    "list, the built-in scratch holds %zu B; use s3d_attn_fwd with a workspace",
                    (long long)N, (long long)W, need, kScratchBytes);
    void *address = nullptr;
    if (int rc = scratch_of_current_device(&address)) return rc;
    a.workspace = address;
    // the list kernels write every word of the work list that the sweep kernel reads (the queue counters
    // included), so nothing of an earlier call's contents is used
    return launch_attn_sweep(a, dtype, static_cast<hipStream_t>(stream));
}
