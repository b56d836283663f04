// Sparse-voxel windowed self-attention forward with cRSE tables (gfx950): generic kernel.
//
// Covers every dtype / shape the library accepts with fp32 arithmetic on the vector ALU (the MFMA kernel
// takes the fp16 cases).  A workgroup serves one head for its whole life and keeps that head's slices of
// the three relative-signal tables in LDS (loaded once, not once per window).  A wavefront draws units from
// a per-head queue; a unit is one window and one chunk of 64 of its queries.  Lane = query: q_i, the running
// maximum, sum and output stay in the lane's registers while the window's keys stream through the
// wavefront one per step (two per step, in two 32-lane groups, when the window has at most 32 voxels), so
// there is no cross-lane reduction, no atomic and no O(pairs) index array; the result is deterministic.
//
// Math (per window, sorted positions i, j, head h), following the reference kernels
// Swin3D/src/attn/self_attn_aio_fwd.cu:16-52 and :111-188:
//   row_n(i,j) = quantised (n_coords[i][n] - n_coords[j][n])   (attn_utils.cuh:437-453)
//   T*(i,j)[c] = sum_n table_*[n][row_n(i,j)][h][c]            (attn_utils.cuh:455-464)
//   L(i,j)     = sum_c q_i[c] k_j[c] + q_i[c] Tq(i,j)[c] + k_j[c] Tk(i,j)[c]
//   out_i[c]   = sum_j softmax_j(L(i,j)) (v_j[c] + Tv(i,j)[c])
#include "attn_kernels.h"

#include <hip/hip_fp16.h>

namespace s3d {
namespace {

constexpr int kThreads = 256;
constexpr int kWavesPerGroup = kThreads / 64;
constexpr int kChunk = 64;   // queries per unit = lanes of a wavefront

template <int D> __device__ __forceinline__ void load_row(const float *p, float *dst)
{
#pragma unroll
    for (int c = 0; c < D; c += 4) {
        const float4 x = *reinterpret_cast<const float4 *>(p + c);
        dst[c] = x.x; dst[c + 1] = x.y; dst[c + 2] = x.z; dst[c + 3] = x.w;
    }
}
template <int D> __device__ __forceinline__ void load_row(const __half *p, float *dst)
{
#pragma unroll
    for (int c = 0; c < D; c += 8) {
        const uint4 x = *reinterpret_cast<const uint4 *>(p + c);
        const __half2 *hh = reinterpret_cast<const __half2 *>(&x);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float2 f = __half22float2(hh[e]);
            dst[c + 2 * e] = f.x;
            dst[c + 2 * e + 1] = f.y;
        }
    }
}
template <int D> __device__ __forceinline__ void store_row(float *p, const float *src)
{
#pragma unroll
    for (int c = 0; c < D; c += 4) *reinterpret_cast<float4 *>(p + c) = make_float4(src[c], src[c + 1], src[c + 2], src[c + 3]);
}
template <int D> __device__ __forceinline__ void store_row(__half *p, const float *src)
{
#pragma unroll
    for (int c = 0; c < D; c += 8) {
        uint4 x;
        __half2 *hh = reinterpret_cast<__half2 *>(&x);
#pragma unroll
        for (int e = 0; e < 4; ++e) hh[e] = __floats2half2_rn(src[c + 2 * e], src[c + 2 * e + 1]);
        *reinterpret_cast<uint4 *>(p + c) = x;
    }
}
__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(__half x) { return __half2float(x); }

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

// One (row, head) slice of D channels in registers.  fp32: D floats, products by FMA.  fp16: D/2 packed pairs
// kept as loaded; dot products with v_dot2_f32_f16 (exact fp16 products, fp32 accumulation), widening only
// where a sum of rows is needed.
template <typename T, int D> struct Slice;
template <int D> struct Slice<float, D> {
    float x[D];
    __device__ __forceinline__ void load(const float *p) { load_row<D>(p, x); }
    __device__ __forceinline__ float dot(const Slice &o, float acc) const
    {
#pragma unroll
        for (int c = 0; c < D; ++c) acc += x[c] * o.x[c];
        return acc;
    }
    __device__ __forceinline__ void add_to(float *sum, float) const
    {
#pragma unroll
        for (int c = 0; c < D; ++c) sum[c] += x[c];
    }
};
template <int D> struct Slice<__half, D> {
    half2_t x[D / 2];
    __device__ __forceinline__ void load(const __half *p)
    {
#pragma unroll
        for (int c = 0; c < D; c += 8) *reinterpret_cast<uint4 *>(&x[c / 2]) = *reinterpret_cast<const uint4 *>(p + c);
    }
    __device__ __forceinline__ float dot(const Slice &o, float acc) const
    {
#pragma unroll
        for (int e = 0; e < D / 2; ++e) acc = __builtin_amdgcn_fdot2(x[e], o.x[e], acc, false);
        return acc;
    }
    // sum += x, widened inside a mixed-precision FMA (x * one + sum, `one` opaque to the optimiser: a plain
    // add would be a conversion plus an add per element)
    __device__ __forceinline__ void add_to(float *sum, float one) const
    {
#pragma unroll
        for (int e = 0; e < D / 2; ++e) {
            sum[2 * e] = __builtin_fmaf(static_cast<float>(x[e][0]), one, sum[2 * e]);
            sum[2 * e + 1] = __builtin_fmaf(static_cast<float>(x[e][1]), one, sum[2 * e + 1]);
        }
    }
};

// Row of the axis table hit by a pair; fp32 arithmetic in the reference's operation order (subtract, add
// half the row count, clamp to [0, rows], truncate), with the upper edge folded onto the last row.
__device__ __forceinline__ int crse_row(float ci, float cj, int rows)
{
    float rel = ci - cj;
    rel = rel + static_cast<float>(rows / 2);
    rel = fminf(fmaxf(rel, 0.0f), static_cast<float>(rows));
    return min(static_cast<int>(rel), rows - 1);
}

// inclusive prefix of ceil(n_w / 64) over the windows (into a.items) and the per-head work counters
// (at the start of a.workspace); one workgroup
__global__ __launch_bounds__(1024) void generic_units_kernel(AttnArgs a)
{
    __shared__ int wave_total[16];
    int *unit_end = static_cast<int *>(a.items);
    int *counters = static_cast<int *>(a.workspace);
    const int W = static_cast<int>(a.W);
    const int per = (W + 1023) / 1024;
    const int begin = threadIdx.x * per, end = min(begin + per, W);
    int sum = 0;
    for (int w = begin; w < end; ++w) sum += (a.w_sizes[w] + kChunk - 1) / kChunk;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int incl = sum;
    for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(incl, off);
        if (lane >= off) incl += up;
    }
    if (lane == 63) wave_total[wave] = incl;
    __syncthreads();
    if (threadIdx.x < 16) {
        int v = wave_total[threadIdx.x];
        for (int off = 1; off < 16; off <<= 1) {
            const int up = __shfl_up(v, off);
            if (threadIdx.x >= off) v += up;
        }
        wave_total[threadIdx.x] = v;
    }
    __syncthreads();
    int run = incl + (wave > 0 ? wave_total[wave - 1] : 0) - sum;
    for (int w = begin; w < end; ++w) {
        run += (a.w_sizes[w] + kChunk - 1) / kChunk;
        unit_end[w] = run;
    }
    for (int t = threadIdx.x; t < a.H; t += 1024) counters[t] = 0;
}

// elements of T between table rows in LDS
template <typename T, int D> __host__ __device__ constexpr int table_row_stride()
{
    return D * sizeof(T) == 16 ? D : D + 16 / static_cast<int>(sizeof(T));
}

// workgroups per CU the register budget is set for (one wavefront of each on every SIMD)
template <typename T, int D> __host__ __device__ constexpr int groups_per_cu()
{
    return (D <= 8 ? 3 : 2) + (sizeof(T) == 2 ? 1 : 0);
}

template <typename T, int D, int ND>
__global__ __launch_bounds__(kThreads, (groups_per_cu<T, D>())) void attn_fwd_sweep_kernel(AttnArgs a)
{
    extern __shared__ float smem[];
    const int H = a.H;
    const int HD = H * D;
    const int h = blockIdx.x % H;
    // table slices of the head in the I/O type; rows longer than 16 bytes are padded by 16 bytes: with a 32- or
    // 64-byte row stride a wavefront's 16-byte gathers of different rows would fall on 4 or 2 of the eight
    // 4-bank groups
    constexpr int kRowStride = table_row_stride<T, D>();
    const int cells = a.total_rows * kRowStride;
    T *tab_q = reinterpret_cast<T *>(smem);
    T *tab_k = tab_q + cells;
    T *tab_v = tab_k + cells;
    {
        const T *gq = static_cast<const T *>(a.table_q);
        const T *gk = static_cast<const T *>(a.table_k);
        const T *gv = static_cast<const T *>(a.table_v);
        for (int t = threadIdx.x; t < a.total_rows * D; t += kThreads) {
            const int r = t / D, c = t - r * D;
            const int64_t g = static_cast<int64_t>(r) * HD + h * D + c;
            tab_q[r * kRowStride + c] = gq[g];
            tab_k[r * kRowStride + c] = gk[g];
            tab_v[r * kRowStride + c] = gv[g];
        }
    }
    __syncthreads();   // the only workgroup barrier

    const int lane = threadIdx.x & 63;
    float one = 1.0f;
    asm volatile("" : "+v"(one));
    const T *gq = static_cast<const T *>(a.q);
    const T *gk = static_cast<const T *>(a.k);
    const T *gv = static_cast<const T *>(a.v);
    const int *unit_end = static_cast<const int *>(a.items);
    const int total_units = __builtin_amdgcn_readfirstlane(unit_end[a.W - 1]);
    int *counter = static_cast<int *>(a.workspace) + h;

    for (;;) {
        int unit = 0;
        if (lane == 0) unit = atomicAdd(counter, 1);
        unit = __builtin_amdgcn_readfirstlane(unit);
        if (unit >= total_units) break;
        int lo = 0, hi = static_cast<int>(a.W) - 1;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (__builtin_amdgcn_readfirstlane(unit_end[mid]) > unit) hi = mid; else lo = mid + 1;
        }
        const int w = lo;
        const int n_w = __builtin_amdgcn_readfirstlane(a.w_sizes[w]);
        const int s0 = __builtin_amdgcn_readfirstlane(a.w2n[w]);
        const int chunk = unit - (w > 0 ? __builtin_amdgcn_readfirstlane(unit_end[w - 1]) : 0);
        // a window of at most 32 voxels streams two keys per step (lanes l and l + 32 own the same query)
        const int gs = n_w <= 32 ? 32 : 64;
        const int ng = 64 / gs;
        const int grp = lane / gs;
        const int own = chunk * kChunk + (lane - grp * gs);
        const bool own_valid = own < n_w;
        const int own_pos = s0 + min(own, n_w - 1);
        const int own_row = a.n2n[own_pos];

        Slice<T, D> qv;
        float ci[ND], acc[D];
        qv.load(gq + static_cast<int64_t>(own_row) * a.row_stride + h * D);
#pragma unroll
        for (int n = 0; n < ND; ++n) ci[n] = a.n_coords[static_cast<int64_t>(own_pos) * ND + n];
#pragma unroll
        for (int c = 0; c < D; ++c) acc[c] = 0.0f;
        float m = -INFINITY, l = 0.0f;

        const int steps = (n_w + ng - 1) / ng;
        int st_row_next = a.n2n[s0 + min(grp, n_w - 1)];
        for (int it = 0; it < steps; ++it) {
            const int st = it * ng + grp;
            const bool st_valid = st < n_w;
            const int st_pos = s0 + min(st, n_w - 1);
            const int st_row = st_row_next;
            if (it + 1 < steps) st_row_next = a.n2n[s0 + min(st + ng, n_w - 1)];
            Slice<T, D> kv, v_in;
            float vv[D], cj[ND];
            kv.load(gk + static_cast<int64_t>(st_row) * a.row_stride + h * D);
            v_in.load(gv + static_cast<int64_t>(st_row) * a.row_stride + h * D);
#pragma unroll
            for (int n = 0; n < ND; ++n) cj[n] = a.n_coords[static_cast<int64_t>(st_pos) * ND + n];
#pragma unroll
            for (int c = 0; c < D; ++c) vv[c] = 0.0f;
            v_in.add_to(vv, one);

            float logit = qv.dot(kv, 0.0f);
#pragma unroll
            for (int n = 0; n < ND; ++n) {
                const int off = (a.base[n] + crse_row(ci[n], cj[n], a.rows[n])) * kRowStride;
                Slice<T, D> tq_r, tk_r, tv_r;
                tq_r.load(tab_q + off);
                tk_r.load(tab_k + off);
                tv_r.load(tab_v + off);
                // short partial sums per axis, added to the logit as two terms: keeps the fp32 rounding of the
                // (up to 2*D*ND + D)-term logit at the level of a tree sum
                logit += qv.dot(tq_r, 0.0f) + kv.dot(tk_r, 0.0f);
                tv_r.add_to(vv, one);
            }
            if (st_valid) {
                const float m_new = fmaxf(m, logit);
                const float scale = __expf(m - m_new);   // exp(-inf) = 0 on the first key
                const float p = __expf(logit - m_new);
                l = l * scale + p;
#pragma unroll
                for (int c = 0; c < D; ++c) acc[c] = acc[c] * scale + p * vv[c];
                m = m_new;
            }
        }
        if (ng == 2) {
            // the two groups saw alternate keys of the same queries: merge their softmax states
            const float m_o = __shfl_xor(m, 32), l_o = __shfl_xor(l, 32);
            const float m_all = fmaxf(m, m_o);
            const float w_me = (m == -INFINITY) ? 0.0f : __expf(m - m_all);
            const float w_ot = (m_o == -INFINITY) ? 0.0f : __expf(m_o - m_all);
            l = l * w_me + l_o * w_ot;
#pragma unroll
            for (int c = 0; c < D; ++c) acc[c] = acc[c] * w_me + __shfl_xor(acc[c], 32) * w_ot;
            m = m_all;
        }
        if (own_valid && grp == 0) {
            const float inv = 1.0f / l;
#pragma unroll
            for (int c = 0; c < D; ++c) acc[c] *= inv;
            store_row<D>(static_cast<T *>(a.out) + static_cast<int64_t>(own_row) * HD + h * D, acc);
            if (a.out_max) a.out_max[static_cast<int64_t>(own_row) * H + h] = m;
            if (a.out_sum) a.out_sum[static_cast<int64_t>(own_row) * H + h] = l;
        }
    }
}

template <typename T, int D, int ND>
int launch_sweep(const AttnArgs &a, hipStream_t stream)
{
    const size_t lds = align_up(sizeof(T) * 3 * static_cast<size_t>(a.total_rows) * table_row_stride<T, D>(), 16);
    if (lds > 160 * 1024)
        return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd: %d table rows x D=%d need %zu B of LDS (> 160 KiB)",
                    a.total_rows, D, lds);
    auto kernel = attn_fwd_sweep_kernel<T, D, ND>;
    S3D_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    hipLaunchKernelGGL(generic_units_kernel, dim3(1), dim3(1024), 0, stream, a);
    S3D_HIP_CHECK(hipGetLastError());
    int device = 0, cus = 256;
    if (hipGetDevice(&device) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && v > 0) cus = v;
    }
    // a workgroup serves one head for its whole life: a multiple of H workgroups, as many per CU as
    // registers and LDS allow
    int per_cu = groups_per_cu<T, D>();
    while (per_cu > 1 && per_cu * lds > 160 * 1024) --per_cu;
    const int per_head = (per_cu * cus + a.H - 1) / a.H;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(per_head * a.H)), dim3(kThreads), lds, stream, a);
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}

template <typename T>
int dispatch_shape(const AttnArgs &a, hipStream_t stream)
{
#define S3D_CASE(DD, NN) \
    if (a.D == DD && a.nd == NN) return launch_sweep<T, DD, NN>(a, stream);
    S3D_CASE(8, 3) S3D_CASE(8, 6) S3D_CASE(8, 9)
    S3D_CASE(16, 3) S3D_CASE(16, 6) S3D_CASE(16, 9)
#undef S3D_CASE
    return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd: unsupported head_dim %d / cRSE axes %d "
                "(head_dim in {8,16}, axes in {3,6,9})", a.D, a.nd);
}

}  // namespace

size_t attn_generic_workspace_bytes(int H, int64_t W)
{
    // per-head work counters, then the prefix of 64-query chunks per window
    return align_up(sizeof(int32_t) * static_cast<size_t>(H), 256) +
           align_up(sizeof(int32_t) * static_cast<size_t>(W > 0 ? W : 1), 256);
}

int launch_attn_generic(const AttnArgs &a, int dtype, hipStream_t stream)
{
    switch (dtype) {
    case S3D_DTYPE_F32: return dispatch_shape<float>(a, stream);
    case S3D_DTYPE_F16: return dispatch_shape<__half>(a, stream);
    default: return fail(S3D_ERR_BAD_DTYPE, "s3d_attn_fwd: dtype %d (0 = fp32, 1 = fp16)", dtype);
    }
}

}  // namespace s3d
