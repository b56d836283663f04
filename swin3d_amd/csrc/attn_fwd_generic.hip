// Sparse-voxel windowed self-attention forward with cRSE tables (gfx950): sweep kernel.
//
// Covers every dtype / shape the library accepts on the vector ALU (fp32 arithmetic; fp16 inputs enter through
// packed dot products and mixed-precision FMAs with fp32 accumulation).  A workgroup serves one head for its
// whole life and keeps that head's slices of the three relative-signal tables in LDS (loaded once, not once per
// window).  A wavefront draws units from the head's work queues; a unit is 64 queries of a window against a
// block of at most 64 of its keys.  Lane = query: q_i, the running maximum, sum and output stay in the lane's
// registers while the keys stream through the wavefront one per step (two per step, in two 32-lane groups,
// when the window has at most 32 voxels), so there is no cross-lane reduction, no atomic on data and no
// O(pairs) index array; the result is deterministic.  Windows of more than 64 voxels leave one partial result
// per key block, combined by generic_merge_kernel.
//
// Math (per window, sorted positions i, j, head h), following the reference kernels
// Swin3D/src/attn/self_attn_aio_fwd.cu:16-52 and :111-188:
//   row_n(i,j) = quantised (n_coords[i][n] - n_coords[j][n])   (attn_utils.cuh:437-453)
//   T*(i,j)[c] = sum_n table_*[n][row_n(i,j)][h][c]            (attn_utils.cuh:455-464)
//   L(i,j)     = sum_c q_i[c] k_j[c] + q_i[c] Tq(i,j)[c] + k_j[c] Tk(i,j)[c]
//   out_i[c]   = sum_j softmax_j(L(i,j)) (v_j[c] + Tv(i,j)[c])
#include "attn_kernels.h"
#include "sweep_common.h"

namespace s3d {
namespace {

using namespace sweep;

constexpr int kThreads = 256;
constexpr int kChunk = 64;   // queries per unit = lanes of a wavefront
// key blocks a window of n voxels is split into (units stream at most kChunk keys), and their even size
__host__ __device__ inline int key_blocks(int n) { return (n + kChunk - 1) / kChunk; }
__host__ __device__ inline int key_block_size(int n) { const int b = key_blocks(n); return (n + b - 1) / b; }

// byte offsets inside the workspace: the queue counters, the unit count, the unit descriptors, the partial results
__host__ __device__ inline size_t ws_total_offset(int H) { return sizeof(int32_t) * static_cast<size_t>(H) * kQueues * kCounterStride; }
__host__ __device__ inline size_t ws_units_offset(int H) { return ws_total_offset(H) + 256; }
__host__ __device__ inline size_t ws_max_units(int64_t W, int64_t N, int max_blocks)
{
    return (static_cast<size_t>(W > 0 ? W : 1) + static_cast<size_t>(N > 0 ? N : 0) / kChunk) * max_blocks;
}
// list of the windows that are split along their keys (their count sits next to the unit count)
__host__ __device__ inline size_t ws_split_offset(int H, int64_t W, int64_t N, int max_blocks)
{
    return ws_units_offset(H) + (sizeof(int2) * ws_max_units(W, N, max_blocks) + 255) / 256 * 256;
}
__host__ __device__ inline size_t ws_partials_offset(int H, int64_t W, int64_t N, int max_blocks)
{
    return ws_split_offset(H, W, N, max_blocks) + (sizeof(int32_t) * static_cast<size_t>(W > 0 ? W : 1) + 255) / 256 * 256;
}

// Unit list of the launch: one descriptor (window, query chunk | key block << 16) per unit, the unit count,
// and the queue counters at zero; one workgroup.  A unit is 64 queries of a window against one block of at
// most 64 of its keys: the longest unit bounds the tail of the launch, so windows of more than 64 voxels are
// split along the keys as well and leave partial results that a second kernel combines.  Units of windows
// with more than 32 voxels (33 to 64 steps) come first, then the short ones (at most 16 steps), each class in
// window order: the launch ends on short units.  Windows beyond the caller's size bound get no units.
__global__ __launch_bounds__(1024) void generic_units_kernel(AttnArgs a)
{
    __shared__ int wave_long[16], wave_all[16];
    __shared__ int split_count;
    if (threadIdx.x == 0) split_count = 0;
    char *ws = static_cast<char *>(a.workspace);
    int *counters = reinterpret_cast<int *>(ws);
    int *total = reinterpret_cast<int *>(ws + ws_total_offset(a.H));
    int2 *units = reinterpret_cast<int2 *>(ws + ws_units_offset(a.H));
    int *split = reinterpret_cast<int *>(ws + ws_split_offset(a.H, a.W, a.N, a.max_key_tiles));
    const int W = static_cast<int>(a.W);
    const int per = (W + 1023) / 1024;
    const int begin = threadIdx.x * per, end = min(begin + per, W);
    auto units_of = [&](int n) {
        const int blocks = key_blocks(n);
        return blocks > a.max_key_tiles ? 0 : blocks * blocks;
    };
    // window sizes are fetched eight at a time with independent loads (a dependent load per window would make
    // this one-workgroup kernel a chain of memory round trips)
    constexpr int kBatch = 8;
    int sum_long = 0, sum_all = 0;
    for (int first = begin; first < end; first += kBatch) {
        int n[kBatch];
#pragma unroll
        for (int i = 0; i < kBatch; ++i) n[i] = first + i < end ? a.w_sizes[first + i] : 0;
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            sum_all += units_of(n[i]);
            if (n[i] > 32) sum_long += units_of(n[i]);
        }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int incl_long = sum_long, incl_all = sum_all;
    for (int off = 1; off < 64; off <<= 1) {
        const int up_long = __shfl_up(incl_long, off), up_all = __shfl_up(incl_all, off);
        if (lane >= off) { incl_long += up_long; incl_all += up_all; }
    }
    if (lane == 63) { wave_long[wave] = incl_long; wave_all[wave] = incl_all; }
    __syncthreads();
    if (threadIdx.x < 16) {
        int v_long = wave_long[threadIdx.x], v_all = wave_all[threadIdx.x];
        for (int off = 1; off < 16; off <<= 1) {
            const int up_long = __shfl_up(v_long, off), up_all = __shfl_up(v_all, off);
            if (static_cast<int>(threadIdx.x) >= off) { v_long += up_long; v_all += up_all; }
        }
        wave_long[threadIdx.x] = v_long;
        wave_all[threadIdx.x] = v_all;
    }
    __syncthreads();
    const int total_long = wave_long[15];
    const int before_long = incl_long + (wave > 0 ? wave_long[wave - 1] : 0) - sum_long;
    const int before_all = incl_all + (wave > 0 ? wave_all[wave - 1] : 0) - sum_all;
    int run_long = before_long;
    int run_short = total_long + (before_all - before_long);
    for (int first = begin; first < end; first += kBatch) {
        int sizes[kBatch];
#pragma unroll
        for (int i = 0; i < kBatch; ++i) sizes[i] = first + i < end ? a.w_sizes[first + i] : 0;
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            const int n = sizes[i], w = first + i;
            const int blocks = key_blocks(n);
            if (units_of(n) == 0) continue;
            int &run = n > 32 ? run_long : run_short;
            for (int c = 0; c < blocks; ++c)
                for (int kb = 0; kb < blocks; ++kb) units[run++] = make_int2(w, c | (kb << 16));
            if (blocks > 1) split[atomicAdd(&split_count, 1)] = w;   // any order: the merge treats windows independently
        }
    }
    __syncthreads();
    if (threadIdx.x == 1023) {
        total[0] = wave_all[15];
        total[1] = split_count;
    }
    for (int t = threadIdx.x; t < a.H * kQueues; t += 1024) counters[t * kCounterStride] = 0;
}

// Windows of more than 64 voxels: combine the per-key-block partial results (unnormalised output, running
// maximum, sum) of every (voxel, head).  Workgroups take the split windows of the launch in turn; one thread
// per (voxel of the window, head), voxel fastest.
template <typename T, int D>
__global__ __launch_bounds__(256) void generic_merge_kernel(AttnArgs a)
{
    const int H = a.H;
    const char *ws = static_cast<const char *>(a.workspace);
    const int count = reinterpret_cast<const int *>(ws + ws_total_offset(H))[1];
    const int *split = reinterpret_cast<const int *>(ws + ws_split_offset(H, a.W, a.N, a.max_key_tiles));
    const int64_t block_stride = static_cast<int64_t>(H) * a.N * (D + 2);
    for (int e = blockIdx.x; e < count; e += gridDim.x) {
        const int w = split[e];
        const int n_w = a.w_sizes[w], s0 = a.w2n[w];
        const int blocks = key_blocks(n_w);
        for (int t = threadIdx.x; t < n_w * H; t += blockDim.x) {
            const int h = t / n_w, pos = s0 + (t - h * n_w);
            const float *part = a.partials + (static_cast<int64_t>(h) * a.N + pos) * (D + 2);
            float m = -INFINITY;
            for (int kb = 0; kb < blocks; ++kb) m = fmaxf(m, part[kb * block_stride + D]);
            float l = 0.0f, o[D];
#pragma unroll
            for (int c = 0; c < D; ++c) o[c] = 0.0f;
            for (int kb = 0; kb < blocks; ++kb) {
                const float *pk = part + kb * block_stride;
                const float wgt = __expf(pk[D] - m);
                l += pk[D + 1] * wgt;
#pragma unroll
                for (int c = 0; c < D; ++c) o[c] += pk[c] * wgt;
            }
            const int row = a.n2n[pos];
            const float inv = 1.0f / l;
#pragma unroll
            for (int c = 0; c < D; ++c) o[c] *= inv;
            store_row<D>(static_cast<T *>(a.out) + (static_cast<int64_t>(row) * H + h) * D, o);
            if (a.out_max) a.out_max[static_cast<int64_t>(row) * H + h] = m;
            if (a.out_sum) a.out_sum[static_cast<int64_t>(row) * H + h] = l;
        }
    }
}

// workgroups per CU the register budget is set for (one wavefront of each on every SIMD)
template <typename T, int D> __host__ __device__ constexpr int groups_per_cu() { return sizeof(T) == 4 && D > 8 ? 3 : 4; }

// elements of T between table rows in LDS when a workgroup holds the slices of HP heads side by side
template <typename T, int D, int HP> __host__ __device__ constexpr int table_row_stride_heads()
{
    return HP * 3 * D + ((HP * 3 * D * static_cast<int>(sizeof(T)) / 4) % 8 == 0 ? 16 / static_cast<int>(sizeof(T)) : 0);
}

// HP: heads a wavefront carries through a unit (adjacent heads HP * g .. HP * g + HP - 1).  The cRSE rows and
// LDS addresses of a pair do not depend on the head, so two heads share that part of the work.
template <typename T, int D, int ND, int HP>
__global__ __launch_bounds__(kThreads, (HP == 1 ? groups_per_cu<T, D>() : 3)) void attn_fwd_sweep_kernel(AttnArgs a)
{
    // streamed keys per loop iteration: at head_dim 16 two interleaved chains hide the LDS round trips,
    // at head_dim 8 the extra registers cost more than they bring
    constexpr int kKeys = D <= 8 ? 1 : 2;
    extern __shared__ float smem[];
    const int H = a.H;
    const int HD = H * D;
    // workgroups go to the XCDs in turn: consecutive runs of eight serve one head group, so every XCD gets every head
    const int hg = (blockIdx.x / kQueues) % (H / HP);
    const int h = hg * HP;   // first head of the group
    // table slices of the heads in the I/O type, interleaved per row: [head][q-side | k-side | v-side]
    constexpr int kRowStride = table_row_stride_heads<T, D, HP>();
    T *tab = reinterpret_cast<T *>(smem);
    {
        const T *gq = static_cast<const T *>(a.table_q);
        const T *gk = static_cast<const T *>(a.table_k);
        const T *gv = static_cast<const T *>(a.table_v);
        // 16-byte pieces: a (row, head) slice of a table is D * sizeof(T) / 16 of them
        constexpr int kPieces = D * static_cast<int>(sizeof(T)) / 16;
        constexpr int kPerPiece = 16 / static_cast<int>(sizeof(T));
        for (int t = threadIdx.x; t < a.total_rows * HP * kPieces; t += kThreads) {
            const int r = t / (HP * kPieces), hp = t - r * (HP * kPieces);
            const int hh = hp / kPieces, c = (hp - hh * kPieces) * kPerPiece;
            const int64_t g = static_cast<int64_t>(r) * HD + (h + hh) * D + c;
            T *row = tab + r * kRowStride + hh * 3 * D + c;
            *reinterpret_cast<uint4 *>(row) = *reinterpret_cast<const uint4 *>(gq + g);
            *reinterpret_cast<uint4 *>(row + D) = *reinterpret_cast<const uint4 *>(gk + g);
            *reinterpret_cast<uint4 *>(row + 2 * D) = *reinterpret_cast<const uint4 *>(gv + g);
        }
    }
    __syncthreads();   // the only workgroup barrier

    const int lane = threadIdx.x & 63;
    const T *gq = static_cast<const T *>(a.q);
    const T *gk = static_cast<const T *>(a.k);
    const T *gv = static_cast<const T *>(a.v);
    const char *ws = static_cast<const char *>(a.workspace);
    const int2 *units = reinterpret_cast<const int2 *>(ws + ws_units_offset(H));
    const int total_units = __builtin_amdgcn_readfirstlane(*reinterpret_cast<const int *>(ws + ws_total_offset(H)));
    int *counters = static_cast<int *>(a.workspace) + hg * kQueues * kCounterStride;
    constexpr int kRowBytes = kRowStride * static_cast<int>(sizeof(T));
    constexpr uint32_t kHeadBytes = 3 * D * sizeof(T);   // one head's slices inside a row
    const uint32_t tab_addr = __builtin_amdgcn_readfirstlane(lds_address(tab));
    const uint32_t row_bytes = kRowBytes;
    float half_rows[ND], upper[ND];
    uint32_t base_off[ND];
#pragma unroll
    for (int n = 0; n < ND; ++n) {
        half_rows[n] = static_cast<float>(a.rows[n] / 2);
        upper[n] = crse_upper(a.rows[n]);
        // LDS byte address of the axis table's first row
        base_off[n] = __builtin_amdgcn_readfirstlane(tab_addr + a.base[n] * kRowBytes);
    }

    int queue = xcd_id() % kQueues;
    int tried = 0;       // queues found empty so far
    int drawn = 0;       // ticket of the next unit, drawn one unit ahead so that the atomic's round trip overlaps work
    if (lane == 0) drawn = atomicAdd(counters + queue * kCounterStride, 1);
    for (;;) {
        int unit = __builtin_amdgcn_readfirstlane(drawn) * kQueues + queue;
        while (unit >= total_units && ++tried < kQueues) {
            queue = (queue + 1) % kQueues;
            if (lane == 0) drawn = atomicAdd(counters + queue * kCounterStride, 1);
            unit = __builtin_amdgcn_readfirstlane(drawn) * kQueues + queue;
        }
        if (unit >= total_units) break;
        if (lane == 0) drawn = atomicAdd(counters + queue * kCounterStride, 1);
        const int2 desc = units[unit];
        const int w = __builtin_amdgcn_readfirstlane(desc.x);
        const int chunk = __builtin_amdgcn_readfirstlane(desc.y) & 0xffff;
        const int kb = __builtin_amdgcn_readfirstlane(desc.y) >> 16;
        const int n_w = __builtin_amdgcn_readfirstlane(a.w_sizes[w]);
        const int s0 = __builtin_amdgcn_readfirstlane(a.w2n[w]);
        // the unit's keys: block kb of the window's even split into blocks of at most 64
        const int blocks = key_blocks(n_w);
        const int k_begin = kb * key_block_size(n_w);
        const int n_k = min(key_block_size(n_w), n_w - k_begin);
        // a window of at most 32 voxels streams two keys per step (lanes l and l + 32 own the same query)
        const int gs = n_w <= 32 ? 32 : 64;
        const int ng = 64 / gs;
        const int grp = lane / gs;
        const int own = chunk * kChunk + (lane - grp * gs);
        const bool own_valid = own < n_w;
        const int own_pos = s0 + min(own, n_w - 1);
        const int own_row = a.n2n[own_pos];

        Slice<T, D> qv[HP];
        float ci[ND], acc[HP][D], m[HP], l[HP];
#pragma unroll
        for (int hh = 0; hh < HP; ++hh) {
            qv[hh].load(gq + static_cast<int64_t>(own_row) * a.row_stride + (h + hh) * D);
#pragma unroll
            for (int c = 0; c < D; ++c) acc[hh][c] = 0.0f;
            m[hh] = -INFINITY;
            l[hh] = 0.0f;
        }
#pragma unroll
        for (int n = 0; n < ND; ++n) ci[n] = a.n_coords[static_cast<int64_t>(own_pos) * ND + n];

        // kKeys streamed keys per iteration: their loads and dependent chains interleave, which hides the
        // LDS and cache round trips a single chain would wait out one after the other
        const int steps = (n_k + ng - 1) / ng;
        const int k0 = s0 + k_begin;
        int row_next[kKeys];
#pragma unroll
        for (int u = 0; u < kKeys; ++u) row_next[u] = a.n2n[k0 + min(u * ng + grp, n_k - 1)];
        for (int it = 0; it < steps; it += kKeys) {
            Slice<T, D> kv[kKeys][HP], v_in[kKeys][HP];
            float logit[kKeys][HP];
            uint32_t off[kKeys][ND];
            bool valid[kKeys];
#pragma unroll
            for (int u = 0; u < kKeys; ++u) {
                const int st = (it + u) * ng + grp;
                valid[u] = st < n_k;
                const int st_pos = k0 + min(st, n_k - 1);
                const int st_row = row_next[u];
                row_next[u] = a.n2n[k0 + min(st + kKeys * ng, n_k - 1)];
#pragma unroll
                for (int hh = 0; hh < HP; ++hh) {
                    kv[u][hh].load(gk + static_cast<int64_t>(st_row) * a.row_stride + (h + hh) * D);
                    v_in[u][hh].load(gv + static_cast<int64_t>(st_row) * a.row_stride + (h + hh) * D);
                }
                float cj[ND];
#pragma unroll
                for (int n = 0; n < ND; ++n) cj[n] = a.n_coords[static_cast<int64_t>(st_pos) * ND + n];
#pragma unroll
                for (int n = 0; n < ND; ++n)
                    off[u][n] = mad_u24(static_cast<uint32_t>(crse_row(ci[n], cj[n], half_rows[n], upper[n])), row_bytes, base_off[n]);
            }
#pragma unroll
            for (int u = 0; u < kKeys; ++u) {
#pragma unroll
                for (int hh = 0; hh < HP; ++hh) logit[u][hh] = qv[hh].dot(kv[u][hh], 0.0f);
#pragma unroll
                for (int n = 0; n < ND; ++n) {
#pragma unroll
                    for (int hh = 0; hh < HP; ++hh) {
                        Slice<T, D> tq_r, tk_r;
                        tq_r.load_lds(off[u][n] + hh * kHeadBytes);
                        tk_r.load_lds(off[u][n] + hh * kHeadBytes + D * sizeof(T));
                        if (Slice<T, D>::kChainLogit) logit[u][hh] = kv[u][hh].dot(tk_r, qv[hh].dot(tq_r, logit[u][hh]));
                        else logit[u][hh] += kv[u][hh].dot(tk_r, qv[hh].dot(tq_r, 0.0f));
                    }
                }
            }
            if (valid[0]) {   // slot 0 is the lowest key of the iteration
#pragma unroll
                for (int hh = 0; hh < HP; ++hh) {
                    float m_new = fmaxf(m[hh], logit[0][hh]);
#pragma unroll
                    for (int u = 1; u < kKeys; ++u) {
                        logit[u][hh] = valid[u] ? logit[u][hh] : -INFINITY;
                        m_new = fmaxf(m_new, logit[u][hh]);
                    }
                    const float scale = __expf(m[hh] - m_new);   // exp(-inf) = 0 on the first key
                    l[hh] *= scale;
#pragma unroll
                    for (int c = 0; c < D; ++c) acc[hh][c] *= scale;
#pragma unroll
                    for (int u = 0; u < kKeys; ++u) {
                        const float p = __expf(logit[u][hh] - m_new);
                        l[hh] += p;
                        v_in[u][hh].fma_to(acc[hh], p);
#pragma unroll
                        for (int n = 0; n < ND; ++n) {
                            Slice<T, D> tv_r;
                            tv_r.load_lds(off[u][n] + hh * kHeadBytes + 2 * D * sizeof(T));
                            tv_r.fma_to(acc[hh], p);
                        }
                    }
                    m[hh] = m_new;
                }
            }
        }
#pragma unroll
        for (int hh = 0; hh < HP; ++hh) {
            if (ng == 2) {
                // the two groups saw alternate keys of the same queries: merge their softmax states
                const float m_o = __shfl_xor(m[hh], 32), l_o = __shfl_xor(l[hh], 32);
                const float m_all = fmaxf(m[hh], m_o);
                const float w_me = (m[hh] == -INFINITY) ? 0.0f : __expf(m[hh] - m_all);
                const float w_ot = (m_o == -INFINITY) ? 0.0f : __expf(m_o - m_all);
                l[hh] = l[hh] * w_me + l_o * w_ot;
#pragma unroll
                for (int c = 0; c < D; ++c) acc[hh][c] = acc[hh][c] * w_me + __shfl_xor(acc[hh][c], 32) * w_ot;
                m[hh] = m_all;
            }
            if (own_valid && grp == 0) {
                if (blocks == 1) {
                    const float inv = 1.0f / l[hh];
#pragma unroll
                    for (int c = 0; c < D; ++c) acc[hh][c] *= inv;
                    store_row<D>(static_cast<T *>(a.out) + static_cast<int64_t>(own_row) * HD + (h + hh) * D, acc[hh]);
                    if (a.out_max) a.out_max[static_cast<int64_t>(own_row) * H + h + hh] = m[hh];
                    if (a.out_sum) a.out_sum[static_cast<int64_t>(own_row) * H + h + hh] = l[hh];
                } else {
                    float *part = a.partials + ((static_cast<int64_t>(kb) * H + h + hh) * a.N + own_pos) * (D + 2);
#pragma unroll
                    for (int c = 0; c < D; ++c) part[c] = acc[hh][c];
                    part[D] = m[hh];
                    part[D + 1] = l[hh];
                }
            }
        }
    }
}

template <typename T, int D, int ND, int HP>
int launch_sweep_heads(const AttnArgs &a, hipStream_t stream)
{
    const size_t lds = align_up(sizeof(T) * static_cast<size_t>(a.total_rows) * table_row_stride_heads<T, D, HP>(), 16);
    if (lds > 160 * 1024)
        return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd: %d table rows x D=%d need %zu B of LDS (> 160 KiB)",
                    a.total_rows, D, lds);
    auto kernel = attn_fwd_sweep_kernel<T, D, ND, HP>;
    S3D_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    hipLaunchKernelGGL(generic_units_kernel, dim3(1), dim3(1024), 0, stream, a);
    S3D_HIP_CHECK(hipGetLastError());
    int device = 0, cus = 256;
    if (hipGetDevice(&device) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && v > 0) cus = v;
    }
    // a workgroup serves one head group for its whole life: as many workgroups per CU as registers and LDS allow,
    // in whole sets of (XCDs x head groups)
    int per_cu = HP == 1 ? groups_per_cu<T, D>() : 3;
    while (per_cu > 1 && per_cu * lds > 160 * 1024) --per_cu;
    const int set = kQueues * (a.H / HP);
    const int sets = per_cu * cus / set > 0 ? per_cu * cus / set : 1;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(sets * set)), dim3(kThreads), lds, stream, a);
    S3D_HIP_CHECK(hipGetLastError());
    if (a.max_key_tiles > 1) {
        const int64_t want = a.W < 1024 ? a.W : 1024;
        hipLaunchKernelGGL((generic_merge_kernel<T, D>), dim3(static_cast<unsigned>(want > 0 ? want : 1)), dim3(256),
                           0, stream, a);
        S3D_HIP_CHECK(hipGetLastError());
    }
    return S3D_OK;
}

template <typename T, int D, int ND>
int launch_sweep(const AttnArgs &a, hipStream_t stream)
{
    // two heads per wavefront where the registers allow it (head_dim 8, fp16) and the heads pair up
    if constexpr (D <= 8 && sizeof(T) == 2) {
        if (a.H % 2 == 0) return launch_sweep_heads<T, D, ND, 2>(a, stream);
    }
    return launch_sweep_heads<T, D, ND, 1>(a, stream);
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

int attn_generic_key_blocks(int max_window_voxels) { return key_blocks(max_window_voxels > 0 ? max_window_voxels : 1); }

size_t attn_generic_workspace_bytes(int H, int D, int64_t W, int64_t N, int max_window_voxels)
{
    // queue counters, the unit count, the unit descriptors, and one partial record per (key block, head,
    // voxel) when some window may be split along its keys
    const int blocks = attn_generic_key_blocks(max_window_voxels);
    const size_t partials = blocks <= 1 ? 0 : sizeof(float) * static_cast<size_t>(N) * blocks * H * (D + 2);
    return ws_partials_offset(H, W, N, blocks) + align_up(partials, 256);
}

float *attn_generic_partials(void *workspace, int H, int64_t W, int64_t N, int max_window_voxels)
{
    return reinterpret_cast<float *>(static_cast<char *>(workspace) +
                                     ws_partials_offset(H, W, N, attn_generic_key_blocks(max_window_voxels)));
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
