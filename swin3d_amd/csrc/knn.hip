// Grid-bucketed exact K nearest neighbours inside batch segments (gfx950).
//
// Replaces the brute-force kernel of Swin3D/src/knn/knn_cuda_kernel.cu:139-204
// (one thread streaming every source of the batch through a 64-slot heap).
// Sources are bucketed into a uniform grid (one counting sort); a small group of
// lanes per query walks cubic shells of cells around the query's cell and keeps
// the K best candidates, ordered by (squared distance, source row).  A shell
// walk stops once the K-th best distance is provably smaller than the distance
// to anything outside the visited cube, so the result is exact and independent
// of the visiting order: ties go to the lower source row.
//
// Distance arithmetic: d = src - query per axis, ((dx*dx) + (dy*dy)) + (dz*dz),
// every operation individually rounded to fp32 (no fused multiply-add).
#include "s3d_common.h"

#include <cstring>

#include <rocprim/rocprim.hpp>

namespace s3d {
namespace {

constexpr int kThreads = 256;
constexpr int kMaxBatch = 4096;
constexpr int kBboxBlocks = 128;   // workgroups of the bounding-box pass = partial boxes the count pass reduces

struct KnnPlan {
    // bounding box of all sources as order-preserving integer images of the floats
    int lo[3], hi[3];
    float origin[3];
    float cell, inv_cell, slack;
    int dim[3];
    int cells_per_batch;
    int src_end;  // sources at or beyond this row belong to no batch segment
};

struct Layout {
    size_t plan, partials, counts, starts, src_place, sorted, temp, temp_bytes, total;
    int64_t cells_cap;
};

int64_t cells_cap_for(int64_t Ns)
{
    int64_t cap = 4 * Ns;
    if (cap < 4096) cap = 4096;
    if (cap > (1LL << 24)) cap = 1LL << 24;
    return cap;
}

size_t scan_temp_bytes(int64_t n)
{
    size_t bytes = 0;
    int32_t *p = nullptr;
    (void)rocprim::exclusive_scan(nullptr, bytes, p, p, 0, static_cast<size_t>(n),
                                  rocprim::plus<int32_t>(), hipStream_t(0));
    return bytes;
}

Layout make_layout(int64_t Ns)
{
    Layout L{};
    L.cells_cap = cells_cap_for(Ns);
    const size_t ns = static_cast<size_t>(Ns > 0 ? Ns : 1);
    const size_t cells = static_cast<size_t>(L.cells_cap) + 1;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        const size_t at = off;
        off = align_up(off + bytes, 256);
        return at;
    };
    L.plan = take(sizeof(KnnPlan));
    L.partials = take(sizeof(int32_t) * 6 * kBboxBlocks);
    L.counts = take(cells * sizeof(int32_t));
    L.starts = take(cells * sizeof(int32_t));
    L.src_place = take(ns * sizeof(int2));
    L.sorted = take(ns * sizeof(float4));
    L.temp_bytes = scan_temp_bytes(static_cast<int64_t>(cells));
    L.temp = take(L.temp_bytes);
    L.total = off;
    return L;
}

// order-preserving map float -> int (so integer atomicMin/Max work on floats)
__device__ __forceinline__ int float_to_ordered(float f)
{
    const int i = __float_as_int(f);
    return i >= 0 ? i : i ^ 0x7fffffff;
}
__device__ __forceinline__ float ordered_to_float(int i)
{
    return __int_as_float(i >= 0 ? i : i ^ 0x7fffffff);
}

// Bounding box of the sources, one partial box per workgroup (no atomics, nothing to initialise), and the cell
// counters set to zero: a small grid-stride grid.
__global__ __launch_bounds__(kThreads) void knn_bbox_kernel(const float *__restrict__ src, int64_t Ns,
                                                            int32_t *__restrict__ partials,
                                                            int32_t *__restrict__ counts, int64_t cells)
{
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < cells;
         i += static_cast<int64_t>(gridDim.x) * kThreads)
        counts[i] = 0;
    int lo[3] = {0x7fffffff, 0x7fffffff, 0x7fffffff};
    int hi[3] = {static_cast<int>(0x80000000u), static_cast<int>(0x80000000u),
                 static_cast<int>(0x80000000u)};
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < Ns;
         i += static_cast<int64_t>(gridDim.x) * kThreads) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            const int o = float_to_ordered(src[i * 3 + a]);
            lo[a] = min(lo[a], o);
            hi[a] = max(hi[a], o);
        }
    }
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        for (int off = 32; off > 0; off >>= 1) {
            lo[a] = min(lo[a], __shfl_down(lo[a], off));
            hi[a] = max(hi[a], __shfl_down(hi[a], off));
        }
    }
    __shared__ int part[kThreads / 64][6];
    if ((threadIdx.x & 63) == 0) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            part[threadIdx.x >> 6][a] = lo[a];
            part[threadIdx.x >> 6][3 + a] = hi[a];
        }
    }
    __syncthreads();
    if (threadIdx.x < 6) {
        int v = part[0][threadIdx.x];
        for (int w = 1; w < kThreads / 64; ++w)
            v = threadIdx.x < 3 ? min(v, part[w][threadIdx.x]) : max(v, part[w][threadIdx.x]);
        partials[blockIdx.x * 6 + threadIdx.x] = v;
    }
}

// One thread: turn the bounding box (plan->lo / hi) into grid parameters that fit `cells_cap`.
__device__ void make_plan(KnnPlan *plan, const int32_t *__restrict__ src_offset, int B, int64_t Ns, int K,
                          float cell_hint, int64_t cells_cap)
{
    int src_end = src_offset[B - 1];
    if (src_end > Ns) src_end = static_cast<int>(Ns);
    if (src_end < 0) src_end = 0;
    plan->src_end = src_end;
    if (src_end == 0) {  // no candidate anywhere: the query kernel pads every slot
        for (int a = 0; a < 3; ++a) {
            plan->origin[a] = 0.0f;
            plan->dim[a] = 1;
        }
        plan->cell = plan->inv_cell = 1.0f;
        plan->slack = 0.0f;
        plan->cells_per_batch = 1;
        return;
    }
    float ext[3], max_abs = 0.0f;
    for (int a = 0; a < 3; ++a) {
        const float lo = ordered_to_float(plan->lo[a]);
        const float hi = ordered_to_float(plan->hi[a]);
        plan->origin[a] = lo;
        ext[a] = fmaxf(hi - lo, 0.0f);
        max_abs = fmaxf(max_abs, fmaxf(fabsf(lo), fabsf(hi)));
    }
    const int64_t per_batch_cap = cells_cap / B;  // B <= kMaxBatch <= cells_cap
    float cell = cell_hint;
    if (!(cell > 0.0f)) {
        // no hint: about K / 32 sources per cell if the sources filled their box (scans of surfaces fill a small part
        // of the box, so the occupied cells hold more and most cells of a shell are empty, which the query kernel
        // skips cheaply; measured at K = 16 on a room scan, 200k sources, 50k queries: divisor 8, 16, 24, 32, 48, 64
        // -> 0.109, 0.113, 0.107, 0.106, 0.105, 0.111 ms per call), and never more cells than the cell array has
        const float floor_ext = fmaxf(fmaxf(ext[0], ext[1]), ext[2]) * 1e-3f + 1e-12f;
        const float vol = fmaxf(ext[0], floor_ext) * fmaxf(ext[1], floor_ext) * fmaxf(ext[2], floor_ext);
        cell = cbrtf(vol / static_cast<float>(src_end > 0 ? src_end : 1) * static_cast<float>(K) * (1.0f / 32.0f));
        cell = fmaxf(cell, cbrtf(vol / static_cast<float>(per_batch_cap > 0 ? per_batch_cap : 1)));
    }
    if (!(cell > 1e-20f)) cell = 1.0f;
    int dim[3];
    for (int iter = 0; iter < 400; ++iter) {
        double total = 1.0;
        for (int a = 0; a < 3; ++a) {
            const float cells_f = floorf(ext[a] / cell) + 1.0f;
            dim[a] = cells_f < 2.0e9f ? static_cast<int>(cells_f) : 2000000000;
            total *= static_cast<double>(dim[a]);
        }
        if (total <= static_cast<double>(per_batch_cap)) break;
        cell *= iter < 40 ? 1.03f : 1.25f;
    }
    {
        double total = static_cast<double>(dim[0]) * dim[1] * dim[2];
        if (total > static_cast<double>(per_batch_cap)) {  // degenerate input: single cell
            dim[0] = dim[1] = dim[2] = 1;
            cell = fmaxf(fmaxf(ext[0], ext[1]), ext[2]) * 2.0f + 1.0f;
        }
    }
    plan->cell = cell;
    plan->inv_cell = 1.0f / cell;
    // sources within `slack` of a cell face may sit in either neighbour cell
    plan->slack = 1e-3f * cell + 8e-6f * max_abs;
    for (int a = 0; a < 3; ++a) plan->dim[a] = dim[a];
    plan->cells_per_batch = dim[0] * dim[1] * dim[2];
}

// the plan of a call without sources (the query kernel pads every slot)
__global__ void knn_plan_kernel(KnnPlan *plan, const int32_t *__restrict__ src_offset, int B,
                                int64_t Ns, int K, float cell_hint, int64_t cells_cap)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    make_plan(plan, src_offset, B, Ns, K, cell_hint, cells_cap);
}

__device__ __forceinline__ int cell_coord(float p, float origin, float inv_cell)
{
    const float t = floorf((p - origin) * inv_cell);
    // keep the conversion defined for far-away queries
    return static_cast<int>(fminf(fmaxf(t, -1.0e9f), 1.0e9f));
}

__device__ __forceinline__ int find_batch(const int32_t *__restrict__ offset, int B, int64_t g)
{
    int b = 0;
    for (; b < B; ++b)
        if (g < offset[b]) break;
    return b;  // == B: beyond the last segment
}

// Every workgroup first reduces the partial boxes and derives the grid from them (the same arithmetic in every
// workgroup; workgroup 0 leaves the plan for the kernels that follow), then its sources take their places: a
// source's cell and its slot there, drawn from the cell's counter.  Neighbouring lanes that fall into the same
// cell (sources usually arrive in lattice order) draw one run of slots with one atomic.
__global__ __launch_bounds__(kThreads) void knn_count_kernel(
    const float *__restrict__ src, int64_t Ns, const int32_t *__restrict__ src_offset, int B,
    const int32_t *__restrict__ partials, int boxes, int K, float cell_hint, int64_t cells_cap,
    KnnPlan *__restrict__ plan_out,
    int32_t *__restrict__ counts, int2 *__restrict__ src_place)
{
    __shared__ KnnPlan plan;
    __shared__ int part[kThreads / 64][6];
    {
        int v[6];
#pragma unroll
        for (int a = 0; a < 6; ++a) v[a] = a < 3 ? 0x7fffffff : static_cast<int>(0x80000000u);
        for (int t = threadIdx.x; t < boxes; t += kThreads)
#pragma unroll
            for (int a = 0; a < 6; ++a) v[a] = a < 3 ? min(v[a], partials[t * 6 + a]) : max(v[a], partials[t * 6 + a]);
#pragma unroll
        for (int a = 0; a < 6; ++a)
            for (int off = 32; off > 0; off >>= 1) {
                const int o = __shfl_down(v[a], off);
                v[a] = a < 3 ? min(v[a], o) : max(v[a], o);
            }
        if ((threadIdx.x & 63) == 0)
#pragma unroll
            for (int a = 0; a < 6; ++a) part[threadIdx.x >> 6][a] = v[a];
        __syncthreads();
        if (threadIdx.x == 0) {
            for (int a = 0; a < 6; ++a) {
                int r = part[0][a];
                for (int w = 1; w < kThreads / 64; ++w) r = a < 3 ? min(r, part[w][a]) : max(r, part[w][a]);
                if (a < 3) plan.lo[a] = r; else plan.hi[a - 3] = r;
            }
            make_plan(&plan, src_offset, B, Ns, K, cell_hint, cells_cap);
            if (blockIdx.x == 0) *plan_out = plan;
        }
        __syncthreads();
    }
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const int lane = threadIdx.x & 63;
    int cell = -2;                       // beyond the array
    if (i < Ns) {
        const int b = find_batch(src_offset, B, i);
        cell = -1;                       // in no batch segment
        if (b < B) {
            int c[3];
#pragma unroll
            for (int a = 0; a < 3; ++a) {
                c[a] = cell_coord(src[i * 3 + a], plan.origin[a], plan.inv_cell);
                c[a] = min(max(c[a], 0), plan.dim[a] - 1);
            }
            cell = b * plan.cells_per_batch + (c[2] * plan.dim[1] + c[1]) * plan.dim[0] + c[0];
        }
    }
    // runs of equal cells along the lanes: the first lane of a run draws the run's slots
    const int before = __shfl_up(cell, 1);
    const bool head = lane == 0 || before != cell;
    const unsigned long long heads = __ballot(head);
    const unsigned long long upto = heads & (lane == 63 ? ~0ull : ((2ull << lane) - 1));
    const int my_head = 63 - __clzll(static_cast<long long>(upto));
    const unsigned long long above = lane == 63 ? 0ull : heads & ~((2ull << lane) - 1);
    const int next = above ? __ffsll(static_cast<long long>(above)) - 1 : 64;
    int base = 0;
    if (head && cell >= 0) base = atomicAdd(&counts[cell], next - lane);
    base = __shfl(base, my_head);
    if (i < Ns) src_place[i] = make_int2(cell, base + (lane - my_head));
}

__global__ __launch_bounds__(kThreads) void knn_scatter_kernel(
    const float *__restrict__ src, int64_t Ns, const int2 *__restrict__ src_place,
    const int32_t *__restrict__ starts, float4 *__restrict__ sorted)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (i >= Ns) return;
    const int2 place = src_place[i];
    if (place.x < 0) return;
    sorted[starts[place.x] + place.y] = make_float4(src[i * 3], src[i * 3 + 1], src[i * 3 + 2],
                                                    __int_as_float(static_cast<int>(i)));
}

// ((dx*dx) + (dy*dy)) + (dz*dz) with d = src - query and every operation rounded to fp32 on
// its own: contraction into fused multiply-adds is switched off for this function (the
// compiler's default for device code is to fuse).
__device__ __forceinline__ float dist2_unfused(float sx, float sy, float sz, float qx, float qy,
                                               float qz)
{
#pragma clang fp contract(off)
    const float dx = sx - qx, dy = sy - qy, dz = sz - qz;
    const float xx = dx * dx, yy = dy * dy, zz = dz * dz;
    const float xy = xx + yy;
    return xy + zz;
}

__device__ __forceinline__ bool cand_less(float d, int i, float d2, int i2)
{
    return d < d2 || (d == d2 && i < i2);
}

// One query per group of G lanes (G = 4, 8, 16 or 64 >= K).  The group keeps its K best candidates
// as ONE sorted list spread over its lanes (lane t holds the t-th best), so an insertion is a
// compare plus a one-lane shift for the whole group instead of a K-long loop per thread, the
// sources of a cell run are loaded G at a time (coalesced), and a 50k-query call fills the
// chip with wavefronts instead of leaving it with a few hundred.
template <int G>
__global__ __launch_bounds__(kThreads) void knn_query_kernel(
    int K, const float *__restrict__ qry, int64_t Nq, const int32_t *__restrict__ query_offset,
    int B, const KnnPlan *__restrict__ plan_ptr, const int32_t *__restrict__ starts,
    const float4 *__restrict__ sorted, int32_t *__restrict__ ret_idx, float *__restrict__ ret_dist2)
{
    const int lane = threadIdx.x & 63;
    const int t = lane % G;                    // position in the group's sorted list
    const int group_shift = lane - t;          // first lane of the group inside the wavefront
    const int64_t g_raw = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) / G;
    const bool live = g_raw < Nq;              // groups past the last query idle along (no early
    const int64_t g = live ? g_raw : Nq - 1;   // exit: their lanes may share a wavefront with live ones)
    const KnnPlan plan = *plan_ptr;
    float bd = INFINITY;
    int bi = 0x7fffffff;
    const int b = find_batch(query_offset, B, g);
    if (b < B && plan.src_end > 0) {
        const float qx = qry[g * 3], qy = qry[g * 3 + 1], qz = qry[g * 3 + 2];
        const float qp[3] = {qx, qy, qz};
        int qc[3], r_first = 0, r_last = 0;
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            qc[a] = cell_coord(qp[a], plan.origin[a], plan.inv_cell);
            const int below = -qc[a], above = qc[a] - (plan.dim[a] - 1);
            r_first = max(r_first, max(below, above));          // first shell touching the grid
            r_last = max(r_last, max(qc[a], -above));           // shell that covers the whole grid
        }
        r_last = max(r_last, r_first);
        const int32_t *cell_base = starts + static_cast<int64_t>(b) * plan.cells_per_batch;
        for (int r = r_first; r <= r_last; ++r) {
            const int z0 = max(qc[2] - r, 0), z1 = min(qc[2] + r, plan.dim[2] - 1);
            const int y0 = max(qc[1] - r, 0), y1 = min(qc[1] + r, plan.dim[1] - 1);
            const int ny = y1 - y0 + 1;
            const int n_rows = (z1 - z0 + 1) * ny;   // <= 0 when the shell misses the grid in z or y
            // source ranges of row u of the shell: a face row spans the whole x range of the cube
            // (one contiguous run of cells), an interior row only its two end cells
            auto row_ranges = [&](int u, int &a0, int &a1, int &b0, int &b1) {
                const int z = z0 + u / ny, y = y0 + u % ny;
                const bool face = r == 0 || z == qc[2] - r || z == qc[2] + r || y == qc[1] - r ||
                                  y == qc[1] + r;
                const int32_t *row = cell_base + (z * plan.dim[1] + y) * plan.dim[0];
                const int xl = qc[0] - r, xh = qc[0] + r;
                a0 = a1 = b0 = b1 = 0;
                if (face) {
                    const int x0 = max(xl, 0), x1 = min(xh, plan.dim[0] - 1);
                    if (x0 <= x1) {
                        a0 = row[x0];
                        a1 = row[x1 + 1];
                    }
                } else {
                    if (xl >= 0 && xl < plan.dim[0]) {
                        a0 = row[xl];
                        a1 = row[xl + 1];
                    }
                    if (xh >= 0 && xh < plan.dim[0]) {
                        b0 = row[xh];
                        b1 = row[xh + 1];
                    }
                }
            };
            auto scan_sources = [&](int s_begin, int s_end) {
                for (int s0 = s_begin; s0 < s_end; s0 += G) {
                    const int s = s0 + t;
                    const bool have = s < s_end;
                    const float4 p = sorted[have ? s : s_begin];
                    const float cd = have ? dist2_unfused(p.x, p.y, p.z, qx, qy, qz) : INFINITY;
                    const int ci = have ? __float_as_int(p.w) : 0x7fffffff;
                    // candidates that beat the current K-th best of the group
                    const float kth_d = __shfl(bd, K - 1, G);
                    const int kth_i = __shfl(bi, K - 1, G);
                    unsigned long long pass = __ballot(cand_less(cd, ci, kth_d, kth_i));
                    pass = (pass >> group_shift) & (G == 64 ? ~0ULL : ((1ULL << G) - 1));
                    while (pass) {
                        const int c = __ffsll(static_cast<long long>(pass)) - 1;
                        pass &= pass - 1;
                        const float xd = __shfl(cd, c, G);
                        const int xi = __shfl(ci, c, G);
                        const float pd = __shfl_up(bd, 1, G);
                        const int pi = __shfl_up(bi, 1, G);
                        const bool before_prev = t > 0 && cand_less(xd, xi, pd, pi);
                        const bool before_this = cand_less(xd, xi, bd, bi);
                        const float nd = before_prev ? pd : (before_this ? xd : bd);
                        const int ni = before_prev ? pi : (before_this ? xi : bi);
                        bd = nd;
                        bi = ni;
                    }
                }
            };
            // The rows of the shell, G at a time: every lane of the group looks up the source ranges of one row (the
            // lookups of up to G rows run side by side instead of one after the other on all lanes), then the group
            // scans the rows that have sources - on surface scans most cells of a shell are empty.
            for (int u0 = 0; u0 < n_rows; u0 += G) {
                int ma0 = 0, ma1 = 0, mb0 = 0, mb1 = 0;
                if (u0 + t < n_rows) row_ranges(u0 + t, ma0, ma1, mb0, mb1);
                unsigned long long todo = __ballot(ma1 > ma0 || mb1 > mb0);
                todo = (todo >> group_shift) & (G == 64 ? ~0ULL : ((1ULL << G) - 1));
                while (todo) {
                    const int k = __ffsll(static_cast<long long>(todo)) - 1;
                    todo &= todo - 1;
                    scan_sources(__shfl(ma0, k, G), __shfl(ma1, k, G));
                    scan_sources(__shfl(mb0, k, G), __shfl(mb1, k, G));
                }
            }
            if (__shfl(bi, K - 1, G) != 0x7fffffff) {
                // everything outside the visited cube is at least `bound` away from the query
                float bound = INFINITY;
#pragma unroll
                for (int a = 0; a < 3; ++a) {
                    const float lo_face = plan.origin[a] + static_cast<float>(qc[a] - r) * plan.cell;
                    const float hi_face = plan.origin[a] + static_cast<float>(qc[a] + r + 1) * plan.cell;
                    bound = fminf(bound, fminf(qp[a] - lo_face, hi_face - qp[a]));
                }
                bound -= plan.slack;
                if (bound > 0.0f && __shfl(bd, K - 1, G) < bound * bound) break;
            }
        }
    }
    if (live && t < K) {
        const bool filled = bi != 0x7fffffff;
        ret_idx[g * K + t] = filled ? bi : -1;
        ret_dist2[g * K + t] = filled ? bd : S3D_KNN_PAD_DIST2;
    }
}

// Inverse-distance interpolation over the K nearest sources of every query
// (Swin3D/modules/swin3d_layers.py:53-73): weight_i = 1 / (sqrt(dist2_i) + 1e-8), normalised over the K
// neighbours, out = sum_i weight_i * src_feat[idx_i].  One thread per (query, group of VEC channels);
// padded neighbour slots (index -1) carry no weight.  fp32 accumulation, one rounding to the output type.
template <typename T, int VEC>
__global__ __launch_bounds__(kThreads) void knn_interpolate_kernel(const int32_t *__restrict__ idx,
                                                                   const float *__restrict__ dist2, int K,
                                                                   int64_t Nq, const T *__restrict__ feat, int C,
                                                                   T *__restrict__ out)
{
    const int groups = C / VEC;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= Nq * groups) return;
    const int64_t qi = t / groups;
    const int c0 = static_cast<int>(t - qi * groups) * VEC;
    float norm = 0.0f;
    for (int i = 0; i < K; ++i)
        if (idx[qi * K + i] >= 0) norm += 1.0f / (sqrtf(dist2[qi * K + i]) + 1e-8f);
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.0f;
    for (int i = 0; i < K; ++i) {
        const int row = idx[qi * K + i];
        if (row < 0) continue;
        const float w = (1.0f / (sqrtf(dist2[qi * K + i]) + 1e-8f)) / norm;
        T v[VEC];
        if constexpr (VEC == 4) {
            if constexpr (sizeof(T) == 4)
                *reinterpret_cast<float4 *>(v) = *reinterpret_cast<const float4 *>(feat + static_cast<int64_t>(row) * C + c0);
            else
                *reinterpret_cast<uint2 *>(v) = *reinterpret_cast<const uint2 *>(feat + static_cast<int64_t>(row) * C + c0);
        } else {
            v[0] = feat[static_cast<int64_t>(row) * C + c0];
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] += w * static_cast<float>(v[e]);
    }
    T o[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) o[e] = static_cast<T>(acc[e]);
    if constexpr (VEC == 4) {
        if constexpr (sizeof(T) == 4)
            *reinterpret_cast<float4 *>(out + qi * C + c0) = *reinterpret_cast<const float4 *>(o);
        else
            *reinterpret_cast<uint2 *>(out + qi * C + c0) = *reinterpret_cast<const uint2 *>(o);
    } else {
        out[qi * C + c0] = o[0];
    }
}

template <typename T>
int launch_interpolate(const int32_t *idx, const float *dist2, int K, int64_t Nq, const void *feat, int C, void *out,
                       hipStream_t s)
{
    const T *f = static_cast<const T *>(feat);
    T *o = static_cast<T *>(out);
    if (C % 4 == 0) {
        const int64_t threads = Nq * (C / 4);
        hipLaunchKernelGGL((knn_interpolate_kernel<T, 4>), dim3(static_cast<unsigned>(ceil_div(threads, kThreads))),
                           dim3(kThreads), 0, s, idx, dist2, K, Nq, f, C, o);
    } else {
        const int64_t threads = Nq * C;
        hipLaunchKernelGGL((knn_interpolate_kernel<T, 1>), dim3(static_cast<unsigned>(ceil_div(threads, kThreads))),
                           dim3(kThreads), 0, s, idx, dist2, K, Nq, f, C, o);
    }
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}

// Channel-wise maximum over the K nearest sources of every query (the max-pool of the KNN downsample,
// Swin3D/modules/swin3d_layers.py:292-312: gather [Nq,K,C], then max over K) without the gathered intermediate.
// One thread per (query, 16 bytes of channels).  A padded slot (row -1) reads row 0, as the clamped gather of
// the tensor statement does.
template <typename T, int VEC>
__global__ __launch_bounds__(kThreads) void knn_max_pool_kernel(const int32_t *__restrict__ idx, int K, int64_t Nq,
                                                                const T *__restrict__ feat, int C,
                                                                T *__restrict__ out)
{
    const int groups = C / VEC;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= Nq * groups) return;
    const int64_t qi = t / groups;
    const int c0 = static_cast<int>(t - qi * groups) * VEC;
    T best[VEC];
    for (int i = 0; i < K; ++i) {
        const int row = max(idx[qi * K + i], 0);
        T v[VEC];
        if constexpr (VEC * sizeof(T) == 16)
            *reinterpret_cast<uint4 *>(v) = *reinterpret_cast<const uint4 *>(feat + static_cast<int64_t>(row) * C + c0);
        else
            v[0] = feat[static_cast<int64_t>(row) * C + c0];
#pragma unroll
        for (int e = 0; e < VEC; ++e) best[e] = (i == 0 || v[e] > best[e]) ? v[e] : best[e];
    }
    if constexpr (VEC * sizeof(T) == 16)
        *reinterpret_cast<uint4 *>(out + qi * C + c0) = *reinterpret_cast<const uint4 *>(best);
    else
        out[qi * C + c0] = best[0];
}

template <typename T>
int launch_max_pool(const int32_t *idx, int K, int64_t Nq, const void *feat, int C, void *out, hipStream_t s)
{
    const T *f = static_cast<const T *>(feat);
    T *o = static_cast<T *>(out);
    constexpr int kVec = 16 / static_cast<int>(sizeof(T));
    if (C % kVec == 0 && reinterpret_cast<uintptr_t>(feat) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
        const int64_t threads = Nq * (C / kVec);
        hipLaunchKernelGGL((knn_max_pool_kernel<T, kVec>), dim3(static_cast<unsigned>(ceil_div(threads, kThreads))),
                           dim3(kThreads), 0, s, idx, K, Nq, f, C, o);
    } else {
        const int64_t threads = Nq * C;
        hipLaunchKernelGGL((knn_max_pool_kernel<T, 1>), dim3(static_cast<unsigned>(ceil_div(threads, kThreads))),
                           dim3(kThreads), 0, s, idx, K, Nq, f, C, o);
    }
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}

}  // namespace
}  // namespace s3d

extern "C" __attribute__((visibility("default"))) int s3d_knn_max_pool(const int32_t *idx, int32_t K, int64_t Nq,
                                                                        const void *src_feat, int64_t Ns, int32_t C,
                                                                        int32_t dtype, void *out, void *stream)
{
    using namespace s3d;
    if (K < 1 || K > S3D_KNN_KMAX) return fail(S3D_ERR_BAD_SHAPE, "s3d_knn_max_pool: K=%d outside 1..%d", K, S3D_KNN_KMAX);
    if (Nq < 0 || Ns < 0 || C < 1 || Nq * static_cast<int64_t>(C) > 0x3fffffffffLL || (Nq > 0 && Ns < 1))
        return fail(S3D_ERR_BAD_SHAPE, "s3d_knn_max_pool: Nq=%lld Ns=%lld C=%d out of range", (long long)Nq, (long long)Ns,
                    C);
    if (dtype != S3D_DTYPE_F32 && dtype != S3D_DTYPE_F16)
        return fail(S3D_ERR_BAD_DTYPE, "s3d_knn_max_pool: dtype %d (0 = fp32, 1 = fp16)", dtype);
    if (Nq == 0) return S3D_OK;
    if (!idx || !out || !src_feat) return fail(S3D_ERR_NULL_POINTER, "s3d_knn_max_pool: null device pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dtype == S3D_DTYPE_F16 ? launch_max_pool<_Float16>(idx, K, Nq, src_feat, C, out, s)
                                  : launch_max_pool<float>(idx, K, Nq, src_feat, C, out, s);
}

extern "C" __attribute__((visibility("default"))) size_t s3d_knn_workspace_bytes(int64_t Ns, int64_t Nq, int32_t B)
{
    (void)Nq;
    (void)B;
    return s3d::make_layout(Ns).total;
}

extern "C" __attribute__((visibility("default"))) int s3d_knn(int32_t K, const float *src_xyz, int64_t Ns, const float *query_xyz,
                       int64_t Nq, const int32_t *src_offset, const int32_t *query_offset, int32_t B,
                       int32_t *ret_idx, float *ret_dist2, float cell_size, void *workspace,
                       size_t workspace_bytes, void *stream)
{
    using namespace s3d;
    if (K < 1 || K > S3D_KNN_KMAX)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_knn: K=%d outside 1..%d", K, S3D_KNN_KMAX);
    if (Ns < 0 || Nq < 0 || Ns > 0x7fffffffLL || Nq > 0x3fffffffLL || B < 1 || B > kMaxBatch)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_knn: Ns=%lld Nq=%lld B=%d out of range", (long long)Ns,
                    (long long)Nq, B);
    if (Nq == 0) return S3D_OK;
    if (!query_xyz || !src_offset || !query_offset || !ret_idx || !ret_dist2 || !workspace ||
        (Ns > 0 && !src_xyz))
        return fail(S3D_ERR_NULL_POINTER, "s3d_knn: null device pointer");
    const Layout L = make_layout(Ns);
    if (workspace_bytes < L.total)
        return fail(S3D_ERR_WORKSPACE, "s3d_knn: workspace %zu B < required %zu B", workspace_bytes,
                    L.total);
    hipStream_t s = static_cast<hipStream_t>(stream);
    char *base = static_cast<char *>(workspace);
    KnnPlan *plan = reinterpret_cast<KnnPlan *>(base + L.plan);
    int32_t *counts = reinterpret_cast<int32_t *>(base + L.counts);
    int32_t *starts = reinterpret_cast<int32_t *>(base + L.starts);
    int2 *src_place = reinterpret_cast<int2 *>(base + L.src_place);
    int32_t *partials = reinterpret_cast<int32_t *>(base + L.partials);
    float4 *sorted = reinterpret_cast<float4 *>(base + L.sorted);
    void *temp = base + L.temp;
    size_t temp_bytes = L.temp_bytes;
    const int64_t cells = L.cells_cap + 1;

    if (Ns > 0) {
        // bounding box + zeroed counters, places (grid derived in every workgroup), scan, scatter
        const dim3 sgrid(static_cast<unsigned>(ceil_div(Ns, kThreads)));
        hipLaunchKernelGGL(knn_bbox_kernel, dim3(kBboxBlocks), dim3(kThreads), 0, s, src_xyz, Ns, partials, counts, cells);
        S3D_HIP_CHECK(hipGetLastError());
        hipLaunchKernelGGL(knn_count_kernel, sgrid, dim3(kThreads), 0, s, src_xyz, Ns, src_offset, B, partials,
                           kBboxBlocks, K, cell_size, L.cells_cap, plan, counts, src_place);
        S3D_HIP_CHECK(hipGetLastError());
        S3D_HIP_CHECK(rocprim::exclusive_scan(temp, temp_bytes, counts, starts, 0,
                                              static_cast<size_t>(cells), rocprim::plus<int32_t>(), s));
        hipLaunchKernelGGL(knn_scatter_kernel, sgrid, dim3(kThreads), 0, s, src_xyz, Ns, src_place, starts, sorted);
        S3D_HIP_CHECK(hipGetLastError());
    } else {
        hipLaunchKernelGGL(knn_plan_kernel, dim3(1), dim3(64), 0, s, plan, src_offset, B, Ns, K,
                           cell_size, L.cells_cap);
        S3D_HIP_CHECK(hipGetLastError());
    }
    // lanes per query: the smallest group that holds the K entries, one per lane (two entries per lane on half the
    // lanes measured 5 % slower at K = 16 and 5 % slower than eight lanes at K <= 8)
    const int G = K <= 4 ? 4 : K <= 8 ? 8 : K <= 16 ? 16 : 64;
    const dim3 qgrid(static_cast<unsigned>(ceil_div(Nq * G, kThreads)));
    if (G == 4)
        hipLaunchKernelGGL(knn_query_kernel<4>, qgrid, dim3(kThreads), 0, s, K, query_xyz, Nq, query_offset,
                           B, plan, starts, sorted, ret_idx, ret_dist2);
    else if (G == 8)
        hipLaunchKernelGGL(knn_query_kernel<8>, qgrid, dim3(kThreads), 0, s, K, query_xyz, Nq, query_offset,
                           B, plan, starts, sorted, ret_idx, ret_dist2);
    else if (G == 16)
        hipLaunchKernelGGL(knn_query_kernel<16>, qgrid, dim3(kThreads), 0, s, K, query_xyz, Nq, query_offset,
                           B, plan, starts, sorted, ret_idx, ret_dist2);
    else
        hipLaunchKernelGGL(knn_query_kernel<64>, qgrid, dim3(kThreads), 0, s, K, query_xyz, Nq, query_offset,
                           B, plan, starts, sorted, ret_idx, ret_dist2);
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}

extern "C" __attribute__((visibility("default"))) int s3d_knn_interpolate(
    const int32_t *idx, const float *dist2, int32_t K, int64_t Nq, const void *src_feat, int64_t Ns, int32_t C,
    int32_t dtype, void *out, void *stream)
{
    using namespace s3d;
    if (K < 1 || K > S3D_KNN_KMAX) return fail(S3D_ERR_BAD_SHAPE, "s3d_knn_interpolate: K=%d outside 1..%d", K, S3D_KNN_KMAX);
    if (Nq < 0 || Ns < 0 || C < 1 || Nq * static_cast<int64_t>(C) > 0x3fffffffffLL)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_knn_interpolate: Nq=%lld Ns=%lld C=%d out of range", (long long)Nq,
                    (long long)Ns, C);
    if (dtype != S3D_DTYPE_F32 && dtype != S3D_DTYPE_F16)
        return fail(S3D_ERR_BAD_DTYPE, "s3d_knn_interpolate: dtype %d (0 = fp32, 1 = fp16)", dtype);
    if (Nq == 0) return S3D_OK;
    if (!idx || !dist2 || !out || (Ns > 0 && !src_feat))
        return fail(S3D_ERR_NULL_POINTER, "s3d_knn_interpolate: null device pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dtype == S3D_DTYPE_F16 ? launch_interpolate<_Float16>(idx, dist2, K, Nq, src_feat, C, out, s)
                                  : launch_interpolate<float>(idx, dist2, K, Nq, src_feat, C, out, s);
}
