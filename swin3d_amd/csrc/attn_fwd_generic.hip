// Sparse-voxel windowed self-attention forward with cRSE tables (gfx950): generic kernel.
//
// Covers every dtype / shape the library accepts (the MFMA kernel takes the fp16 cases).
// One workgroup owns one (window, head): it reads the window's q/k/v rows once,
// keeps the head's slice of the three relative-signal tables in LDS, runs an
// online softmax over the keys and writes each output row once.  There are no
// global atomics and no O(pairs) index arrays; the result is deterministic.
//
// Math (per window, sorted positions i, j, head h), following the reference
// kernels Swin3D/src/attn/self_attn_aio_fwd.cu:16-52 and :111-188:
//   row_n(i,j) = quantised (n_coords[i][n] - n_coords[j][n])   (attn_utils.cuh:437-453)
//   T*(i,j)[c] = sum_n table_*[n][row_n(i,j)][h][c]            (attn_utils.cuh:455-464)
//   L(i,j)     = sum_c q_i[c] k_j[c] + q_i[c] Tq(i,j)[c] + k_j[c] Tk(i,j)[c]
//   out_i[c]   = sum_j softmax_j(L(i,j)) (v_j[c] + Tv(i,j)[c])
#include "attn_kernels.h"

namespace s3d {
namespace {

constexpr int kThreads = 256;
constexpr int kQueryChunk = 64;   // queries per pass = lanes of one wave
constexpr int kKeyChunk = 64;     // keys staged in LDS per step
constexpr int kSlices = kThreads / kQueryChunk;  // key slices, one per wave

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(__half x) { return __half2float(x); }
__device__ __forceinline__ void from_float(float &dst, float x) { dst = x; }
__device__ __forceinline__ void from_float(__half &dst, float x) { dst = __float2half_rn(x); }

// Row of the axis table hit by a pair; fp32 arithmetic in the reference's
// operation order (subtract, add half the row count, clamp to [0, rows],
// truncate), with the upper edge folded onto the last row.
__device__ __forceinline__ int crse_row(float ci, float cj, int rows)
{
    float rel = ci - cj;
    rel = rel + static_cast<float>(rows / 2);
    rel = fminf(fmaxf(rel, 0.0f), static_cast<float>(rows));
    const int row = static_cast<int>(rel);
    return min(row, rows - 1);
}

template <int ND>
struct AxisRows {
    int rows[ND];
    int base[ND];
};

template <typename T, int D, int ND>
__global__ __launch_bounds__(kThreads) void attn_fwd_window_head_kernel(
    const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v,
    const T *__restrict__ table_q, const T *__restrict__ table_k, const T *__restrict__ table_v,
    AxisRows<ND> axes, int total_rows, const int32_t *__restrict__ w_sizes,
    const int32_t *__restrict__ w2n, const int32_t *__restrict__ n2n,
    const float *__restrict__ n_coords, T *__restrict__ out, float *__restrict__ out_max,
    float *__restrict__ out_sum, int H, int64_t row_stride)
{
    extern __shared__ float smem[];
    float *tab_q = smem;                         // [total_rows][D]
    float *tab_k = tab_q + total_rows * D;       // [total_rows][D]
    float *tab_v = tab_k + total_rows * D;       // [total_rows][D]
    float *key_s = tab_v + total_rows * D;       // [kKeyChunk][D]
    float *val_s = key_s + kKeyChunk * D;        // [kKeyChunk][D]
    float *crd_s = val_s + kKeyChunk * D;        // [kKeyChunk][ND]
    float *merge = crd_s + kKeyChunk * ND;       // [kSlices][kQueryChunk][D + 2]

    const int w = blockIdx.x;
    const int h = blockIdx.y;
    const int n_w = w_sizes[w];
    const int s0 = w2n[w];
    const int tid = threadIdx.x;
    const int lane_q = tid % kQueryChunk;
    const int slice = tid / kQueryChunk;
    const int HD = H * D;

    int rows_n[ND], base_n[ND];
#pragma unroll
    for (int n = 0; n < ND; ++n) {
        rows_n[n] = axes.rows[n];
        base_n[n] = axes.base[n];
    }

    for (int idx = tid; idx < total_rows * D; idx += kThreads) {
        const int r = idx / D, c = idx % D;
        const int64_t g = static_cast<int64_t>(r) * HD + h * D + c;
        tab_q[idx] = to_float(table_q[g]);
        tab_k[idx] = to_float(table_k[g]);
        tab_v[idx] = to_float(table_v[g]);
    }

    for (int q0 = 0; q0 < n_w; q0 += kQueryChunk) {
        const int i = q0 + lane_q;
        const bool valid_q = i < n_w;
        float qv[D], ci[ND], acc[D];
        float m = -INFINITY, l = 0.0f;
        int q_row = 0;
        if (valid_q) {
            q_row = n2n[s0 + i];
            const T *qp = q + static_cast<int64_t>(q_row) * row_stride + h * D;
#pragma unroll
            for (int c = 0; c < D; ++c) qv[c] = to_float(qp[c]);
#pragma unroll
            for (int n = 0; n < ND; ++n) ci[n] = n_coords[static_cast<int64_t>(s0 + i) * ND + n];
        } else {
#pragma unroll
            for (int c = 0; c < D; ++c) qv[c] = 0.0f;
#pragma unroll
            for (int n = 0; n < ND; ++n) ci[n] = 0.0f;
        }
#pragma unroll
        for (int c = 0; c < D; ++c) acc[c] = 0.0f;

        for (int k0 = 0; k0 < n_w; k0 += kKeyChunk) {
            const int kend = min(kKeyChunk, n_w - k0);
            __syncthreads();  // previous chunk (and the table staging) fully consumed / written
            for (int idx = tid; idx < kend * D; idx += kThreads) {
                const int jj = idx / D, c = idx % D;
                const int64_t g = static_cast<int64_t>(n2n[s0 + k0 + jj]) * row_stride + h * D + c;
                key_s[idx] = to_float(k[g]);
                val_s[idx] = to_float(v[g]);
            }
            for (int idx = tid; idx < kend * ND; idx += kThreads)
                crd_s[idx] = n_coords[static_cast<int64_t>(s0 + k0) * ND + idx];
            __syncthreads();

            for (int jj = slice; jj < kend; jj += kSlices) {
                float bq[D], bk[D], bv[D];
#pragma unroll
                for (int c = 0; c < D; ++c) bq[c] = bk[c] = bv[c] = 0.0f;
#pragma unroll
                for (int n = 0; n < ND; ++n) {
                    const int row = crse_row(ci[n], crd_s[jj * ND + n], rows_n[n]);
                    const int fr = min(base_n[n] + row, total_rows - 1) * D;
#pragma unroll
                    for (int c = 0; c < D; ++c) {
                        bq[c] += tab_q[fr + c];
                        bk[c] += tab_k[fr + c];
                        bv[c] += tab_v[fr + c];
                    }
                }
                float logit = 0.0f;
#pragma unroll
                for (int c = 0; c < D; ++c) {
                    const float kc = key_s[jj * D + c];
                    logit += qv[c] * kc + qv[c] * bq[c] + kc * bk[c];
                }
                const float m_new = fmaxf(m, logit);
                const float scale = __expf(m - m_new);
                const float p = __expf(logit - m_new);
                l = l * scale + p;
#pragma unroll
                for (int c = 0; c < D; ++c)
                    acc[c] = acc[c] * scale + p * (val_s[jj * D + c] + bv[c]);
                m = m_new;
            }
        }

        // merge the per-wave key slices of every query
        float *mine = merge + (slice * kQueryChunk + lane_q) * (D + 2);
        mine[0] = m;
        mine[1] = l;
#pragma unroll
        for (int c = 0; c < D; ++c) mine[2 + c] = acc[c];
        __syncthreads();
        if (slice == 0 && valid_q) {
            float mm = -INFINITY;
#pragma unroll
            for (int s = 0; s < kSlices; ++s)
                mm = fmaxf(mm, merge[(s * kQueryChunk + lane_q) * (D + 2)]);
            float ll = 0.0f, o[D];
#pragma unroll
            for (int c = 0; c < D; ++c) o[c] = 0.0f;
#pragma unroll
            for (int s = 0; s < kSlices; ++s) {
                const float *part = merge + (s * kQueryChunk + lane_q) * (D + 2);
                // a slice that saw no key has m = -inf, l = 0: its weight is exp(-inf) = 0
                const float wgt = (part[0] == -INFINITY) ? 0.0f : __expf(part[0] - mm);
                ll += part[1] * wgt;
#pragma unroll
                for (int c = 0; c < D; ++c) o[c] += part[2 + c] * wgt;
            }
            const float inv = 1.0f / ll;
            T *op = out + static_cast<int64_t>(q_row) * HD + h * D;
#pragma unroll
            for (int c = 0; c < D; ++c) from_float(op[c], o[c] * inv);
            if (out_max) out_max[static_cast<int64_t>(q_row) * H + h] = mm;
            if (out_sum) out_sum[static_cast<int64_t>(q_row) * H + h] = ll;
        }
        // the next pass rewrites `merge` only after its own __syncthreads() in the key loop
    }
}

template <int D, int ND>
size_t window_head_lds_bytes(int total_rows)
{
    return sizeof(float) * (static_cast<size_t>(3) * total_rows * D + 2 * kKeyChunk * D +
                            kKeyChunk * ND + kSlices * kQueryChunk * (D + 2));
}

template <typename T, int D, int ND>
int launch_window_head(const AttnArgs &a, hipStream_t stream)
{
    const size_t lds = window_head_lds_bytes<D, ND>(a.total_rows);
    if (lds > 160 * 1024)
        return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd: %d table rows x D=%d need %zu B of LDS (> 160 KiB)",
                    a.total_rows, D, lds);
    auto kernel = attn_fwd_window_head_kernel<T, D, ND>;
    S3D_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    AxisRows<ND> axes;
    for (int n = 0; n < ND; ++n) {
        axes.rows[n] = a.rows[n];
        axes.base[n] = a.base[n];
    }
    const dim3 grid(static_cast<unsigned>(a.W), static_cast<unsigned>(a.H));
    hipLaunchKernelGGL(kernel, grid, dim3(kThreads), lds, stream, static_cast<const T *>(a.q),
                       static_cast<const T *>(a.k), static_cast<const T *>(a.v),
                       static_cast<const T *>(a.table_q), static_cast<const T *>(a.table_k),
                       static_cast<const T *>(a.table_v), axes, a.total_rows, a.w_sizes, a.w2n, a.n2n,
                       a.n_coords, static_cast<T *>(a.out), a.out_max, a.out_sum, a.H, a.row_stride);
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}

template <typename T>
int dispatch_shape(const AttnArgs &a, hipStream_t stream)
{
#define S3D_CASE(DD, NN) \
    if (a.D == DD && a.nd == NN) return launch_window_head<T, DD, NN>(a, stream);
    S3D_CASE(8, 3) S3D_CASE(8, 6) S3D_CASE(8, 9)
    S3D_CASE(16, 3) S3D_CASE(16, 6) S3D_CASE(16, 9)
#undef S3D_CASE
    return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd: unsupported head_dim %d / cRSE axes %d "
                "(head_dim in {8,16}, axes in {3,6,9})", a.D, a.nd);
}

}  // namespace

int launch_attn_generic(const AttnArgs &a, int dtype, hipStream_t stream)
{
    switch (dtype) {
    case S3D_DTYPE_F32: return dispatch_shape<float>(a, stream);
    case S3D_DTYPE_F16: return dispatch_shape<__half>(a, stream);
    default: return fail(S3D_ERR_BAD_DTYPE, "s3d_attn_fwd: dtype %d (0 = fp32, 1 = fp16)", dtype);
    }
}

}  // namespace s3d
