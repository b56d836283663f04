// Window sort + segment offsets for sparse-voxel window attention (gfx950).
//
// Replaces the MinkowskiEngine pooling / kernel_map / torch.sort pipeline of
// Swin3D/modules/swin3d_layers.py:713-787 and the w2n / w_sizes scans of
// :96-103.  Every voxel gets one 64-bit key
//     [ batch:12 | wx+8192:14 | wy+8192:14 | wz+8192:14 | local id:10 ]
// with w = floor((coord + shift*stride) / (window*stride)) and
// local id = (lx*window + ly)*window + lz; a stable radix sort of (key, row)
// yields the window-sorted order, a flag + scan pass yields the segments.
// Integer work only; HBM traffic is a handful of passes over 12 B per voxel.
#include "s3d_common.h"

#include <cstring>

#include <rocprim/rocprim.hpp>

namespace s3d {
namespace {

constexpr int kThreads = 256;
constexpr int kLocalBits = 10;
constexpr int kAxisBits = 14;
constexpr int kAxisBias = 1 << (kAxisBits - 1);  // 8192
constexpr int kBatchBits = 12;

struct Layout {
    size_t keys_in, keys_out, vals_in, flags, ranks, temp, temp_bytes, total;
};

size_t sort_temp_bytes(int64_t N)
{
    size_t bytes = 0;
    uint64_t *kn = nullptr;
    int32_t *vn = nullptr;
    (void)rocprim::radix_sort_pairs(nullptr, bytes, kn, kn, vn, vn, static_cast<size_t>(N), 0, 64,
                                    hipStream_t(0));
    return bytes;
}

size_t scan_temp_bytes(int64_t N)
{
    size_t bytes = 0;
    int32_t *p = nullptr;
    (void)rocprim::inclusive_scan(nullptr, bytes, p, p, static_cast<size_t>(N),
                                  rocprim::plus<int32_t>(), hipStream_t(0));
    return bytes;
}

Layout make_layout(int64_t N)
{
    Layout L{};
    const size_t n = static_cast<size_t>(N > 0 ? N : 1);
    size_t off = 0;
    auto take = [&](size_t bytes) {
        const size_t at = off;
        off = align_up(off + bytes, 256);
        return at;
    };
    L.keys_in = take(n * sizeof(uint64_t));
    L.keys_out = take(n * sizeof(uint64_t));
    L.vals_in = take(n * sizeof(int32_t));
    L.flags = take(n * sizeof(int32_t));
    L.ranks = take(n * sizeof(int32_t));
    const size_t a = sort_temp_bytes(static_cast<int64_t>(n));
    const size_t b = scan_temp_bytes(static_cast<int64_t>(n));
    L.temp_bytes = a > b ? a : b;
    L.temp = take(L.temp_bytes);
    L.total = off;
    return L;
}

__device__ __forceinline__ int floordiv(int a, int b)
{
    int q = a / b;
    if ((a % b != 0) && ((a < 0) != (b < 0))) --q;
    return q;
}

__global__ void init_counts_kernel(int64_t *counts)
{
    if (threadIdx.x < 4) counts[threadIdx.x] = 0;
}

__global__ __launch_bounds__(kThreads) void build_keys_kernel(
    const int32_t *__restrict__ coords, int64_t N, int stride, int window, int shift,
    uint64_t *__restrict__ keys, int32_t *__restrict__ vals, int64_t *__restrict__ counts)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (i >= N) return;
    const int4 c = reinterpret_cast<const int4 *>(coords)[i];
    const int span = window * stride;
    const int cc[3] = {c.y + shift * stride, c.z + shift * stride, c.w + shift * stride};
    int wv[3], lv[3];
    bool bad = c.x < 0 || c.x >= (1 << kBatchBits);
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        wv[a] = floordiv(cc[a], span);
        lv[a] = (cc[a] - wv[a] * span) / stride;  // numerator in [0, span)
        bad = bad || wv[a] < -kAxisBias || wv[a] >= kAxisBias;
        wv[a] = min(max(wv[a], -kAxisBias), kAxisBias - 1);
    }
    if (bad) atomicMax(reinterpret_cast<unsigned long long *>(counts + 3), 1ULL);
    const uint64_t b = static_cast<uint64_t>(min(max(c.x, 0), (1 << kBatchBits) - 1));
    const uint64_t local = static_cast<uint64_t>((lv[0] * window + lv[1]) * window + lv[2]);
    uint64_t key = b;
    key = (key << kAxisBits) | static_cast<uint64_t>(wv[0] + kAxisBias);
    key = (key << kAxisBits) | static_cast<uint64_t>(wv[1] + kAxisBias);
    key = (key << kAxisBits) | static_cast<uint64_t>(wv[2] + kAxisBias);
    key = (key << kLocalBits) | local;
    keys[i] = key;
    vals[i] = static_cast<int32_t>(i);
}

__global__ __launch_bounds__(kThreads) void flag_kernel(const uint64_t *__restrict__ keys, int64_t N,
                                                        int32_t *__restrict__ flags,
                                                        int32_t *__restrict__ w_w_id)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (i >= N) return;
    const uint64_t key = keys[i];
    const bool first = (i == 0) || ((keys[i - 1] >> kLocalBits) != (key >> kLocalBits));
    flags[i] = first ? 1 : 0;
    w_w_id[i] = static_cast<int32_t>(key & ((1u << kLocalBits) - 1));
}

__global__ __launch_bounds__(kThreads) void segment_start_kernel(
    const int32_t *__restrict__ flags, const int32_t *__restrict__ ranks, int64_t N,
    int32_t *__restrict__ w2n, int64_t *__restrict__ counts)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (i >= N) return;
    if (flags[i]) w2n[ranks[i] - 1] = static_cast<int32_t>(i);
    if (i == N - 1) counts[0] = ranks[i];
}

__global__ __launch_bounds__(kThreads) void segment_size_kernel(const int32_t *__restrict__ w2n,
                                                                int64_t N,
                                                                int32_t *__restrict__ w_sizes,
                                                                int64_t *__restrict__ counts)
{
    const int64_t w = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const int64_t W = counts[0];  // written by the previous kernel on the same stream
    long long size = 0;
    if (w < W) {
        const int32_t begin = w2n[w];
        const int32_t end = (w + 1 < W) ? w2n[w + 1] : static_cast<int32_t>(N);
        size = end - begin;
        w_sizes[w] = static_cast<int32_t>(size);
    }
    long long sq = size * size, mx = size;
    for (int off = 32; off > 0; off >>= 1) {
        sq += __shfl_down(sq, off);
        mx = max(mx, __shfl_down(mx, off));
    }
    if ((threadIdx.x & 63) == 0 && mx > 0) {
        atomicAdd(reinterpret_cast<unsigned long long *>(counts + 1), static_cast<unsigned long long>(sq));
        atomicMax(reinterpret_cast<unsigned long long *>(counts + 2), static_cast<unsigned long long>(mx));
    }
}

// ---- grid path: the same index without a sort of all voxels ----------------------------------------------
// When the windows of a scene fit a dense lattice of at most cells_cap cells (they do for room-sized scenes: the
// lattice is the bounding box of the window coordinates), a window is a lattice cell and the index is a counting
// sort: every voxel draws a slot in its cell, a scan over the cells gives every non-empty cell its rank (= window
// number, ascending (batch, wx, wy, wz) because the cell number is) and its first position, the voxels are placed
// there, and each window's few voxels are put in (local id, row) order by one wavefront.  Five launches of a few
// microseconds instead of a block sort and eight merge passes.
constexpr int kGridBoxes = 128;          // workgroups of the bounding-box pass
constexpr int kSlotBits = 20;            // a voxel's slot in its cell, below its local id in one word
constexpr int kBadRange = 1, kNoGrid = 2;   // counts[3]: coordinates out of range / lattice too large for the grid path

struct GridPlan {
    int lo[4], dim[4];   // batch, wx, wy, wz: lowest value and extent of the lattice
    int ok;              // the lattice fits
};

struct GridLayout {
    size_t plan, partials, cells, scan, place, keys, temp, temp_bytes, total;
    int64_t cells_cap;
};

int64_t grid_cells_cap(int64_t N)
{
    int64_t cap = 2 * N;    // the scan over the cells is the longest of the five launches: no more cells than pay
    if (cap < 4096) cap = 4096;
    if (cap > (1LL << 24)) cap = 1LL << 24;
    return cap;
}

// (non-empty << 32 | voxels) of a cell: one scan yields a cell's window number and its first position
struct CellWord {
    __host__ __device__ uint64_t operator()(int32_t count) const
    {
        return (count > 0 ? (1ULL << 32) : 0ULL) | static_cast<uint32_t>(count);
    }
};
typedef rocprim::transform_iterator<const int32_t *, CellWord, uint64_t> CellWordIterator;

size_t grid_scan_temp_bytes(int64_t n)
{
    size_t bytes = 0;
    const int32_t *p = nullptr;
    uint64_t *o = nullptr;
    (void)rocprim::exclusive_scan(nullptr, bytes, CellWordIterator(p, CellWord()), o, uint64_t(0), static_cast<size_t>(n),
                                  rocprim::plus<uint64_t>(), hipStream_t(0));
    return bytes;
}

GridLayout make_grid_layout(int64_t N)
{
    GridLayout L{};
    L.cells_cap = grid_cells_cap(N);
    const size_t n = static_cast<size_t>(N > 0 ? N : 1), cells = static_cast<size_t>(L.cells_cap) + 1;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        const size_t at = off;
        off = align_up(off + bytes, 256);
        return at;
    };
    L.plan = take(sizeof(GridPlan));
    L.partials = take(sizeof(int32_t) * 9 * kGridBoxes);
    L.cells = take(cells * sizeof(int32_t));
    L.scan = take(cells * sizeof(uint64_t));
    L.place = take(n * sizeof(int2));
    L.keys = take(n * sizeof(uint64_t));
    L.temp_bytes = grid_scan_temp_bytes(static_cast<int64_t>(cells));
    L.temp = take(L.temp_bytes);
    L.total = off;
    return L;
}

// window coordinates and local id of a voxel; false when they are outside the supported range
__device__ __forceinline__ bool window_of(const int4 c, int stride, int window, int shift, int *w, int *local)
{
    const int span = window * stride;
    const int cc[3] = {c.y + shift * stride, c.z + shift * stride, c.w + shift * stride};
    int lv[3];
    bool bad = c.x < 0 || c.x >= (1 << kBatchBits);
    w[0] = min(max(c.x, 0), (1 << kBatchBits) - 1);
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        const int wv = floordiv(cc[a], span);
        lv[a] = (cc[a] - wv * span) / stride;
        bad = bad || wv < -kAxisBias || wv >= kAxisBias;
        w[1 + a] = min(max(wv, -kAxisBias), kAxisBias - 1);
    }
    *local = (lv[0] * window + lv[1]) * window + lv[2];
    return !bad;
}

// partial bounding boxes of the window coordinates (one per workgroup, no atomics), the cell counters and the
// call's totals and status word at zero (the later launches only ever OR bits into the status word)
__global__ __launch_bounds__(kThreads) void grid_bbox_kernel(const int32_t *__restrict__ coords, int64_t N, int stride,
                                                             int window, int shift, int32_t *__restrict__ partials,
                                                             int32_t *__restrict__ cells, int64_t num_cells,
                                                             int64_t *__restrict__ counts)
{
    if (blockIdx.x == 0 && threadIdx.x < 4) counts[threadIdx.x] = 0;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < num_cells;
         i += static_cast<int64_t>(gridDim.x) * kThreads)
        cells[i] = 0;
    int lo[4], hi[4], bad = 0;
#pragma unroll
    for (int a = 0; a < 4; ++a) { lo[a] = 0x7fffffff; hi[a] = static_cast<int>(0x80000000u); }
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < N;
         i += static_cast<int64_t>(gridDim.x) * kThreads) {
        int w[4], local;
        if (!window_of(reinterpret_cast<const int4 *>(coords)[i], stride, window, shift, w, &local)) bad = 1;
#pragma unroll
        for (int a = 0; a < 4; ++a) { lo[a] = min(lo[a], w[a]); hi[a] = max(hi[a], w[a]); }
    }
    for (int off = 32; off > 0; off >>= 1) {
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            lo[a] = min(lo[a], __shfl_down(lo[a], off));
            hi[a] = max(hi[a], __shfl_down(hi[a], off));
        }
        bad |= __shfl_down(bad, off);
    }
    __shared__ int part[kThreads / 64][9];
    if ((threadIdx.x & 63) == 0) {
#pragma unroll
        for (int a = 0; a < 4; ++a) { part[threadIdx.x >> 6][a] = lo[a]; part[threadIdx.x >> 6][4 + a] = hi[a]; }
        part[threadIdx.x >> 6][8] = bad;
    }
    __syncthreads();
    if (threadIdx.x < 9) {
        int v = part[0][threadIdx.x];
        for (int wv = 1; wv < kThreads / 64; ++wv)
            v = threadIdx.x < 4 ? min(v, part[wv][threadIdx.x]) : max(v, part[wv][threadIdx.x]);   // the flag: max = or
        partials[blockIdx.x * 9 + threadIdx.x] = v;
    }
}

// Every workgroup reduces the partial boxes to the lattice (workgroup 0 records it and its bits of the status word);
// then every voxel draws a slot in its cell - neighbouring lanes of one cell with one atomic.  A cell that runs
// out of slot numbers (more than 2^kSlotBits voxels in one window: only with masses of equal coordinates) sets the
// "no grid" bit as well: the status word was zeroed by the launch before this one and every writer ORs into it, so
// no bit is lost whichever workgroup comes first, and the later launches of the call write nothing once it is set.
__global__ __launch_bounds__(kThreads) void grid_count_kernel(
    const int32_t *__restrict__ coords, int64_t N, int stride, int window, int shift,
    const int32_t *__restrict__ partials, int64_t cells_cap, GridPlan *__restrict__ plan_out,
    int32_t *__restrict__ cells, int2 *__restrict__ place, int64_t *__restrict__ counts)
{
    __shared__ GridPlan plan;
    __shared__ int part[kThreads / 64][9];
    {
        int v[9];
#pragma unroll
        for (int a = 0; a < 9; ++a) v[a] = a < 4 ? 0x7fffffff : static_cast<int>(0x80000000u);
        for (int t = threadIdx.x; t < kGridBoxes; t += kThreads)
#pragma unroll
            for (int a = 0; a < 9; ++a) v[a] = a < 4 ? min(v[a], partials[t * 9 + a]) : max(v[a], partials[t * 9 + a]);
#pragma unroll
        for (int a = 0; a < 9; ++a)
            for (int off = 32; off > 0; off >>= 1) {
                const int o = __shfl_down(v[a], off);
                v[a] = a < 4 ? min(v[a], o) : max(v[a], o);
            }
        if ((threadIdx.x & 63) == 0)
#pragma unroll
            for (int a = 0; a < 9; ++a) part[threadIdx.x >> 6][a] = v[a];
        __syncthreads();
        if (threadIdx.x == 0) {
            int r[9];
            for (int a = 0; a < 9; ++a) {
                r[a] = part[0][a];
                for (int wv = 1; wv < kThreads / 64; ++wv) r[a] = a < 4 ? min(r[a], part[wv][a]) : max(r[a], part[wv][a]);
            }
            double total = 1.0;
            for (int a = 0; a < 4; ++a) {
                plan.lo[a] = r[a];
                plan.dim[a] = r[4 + a] - r[a] + 1;
                total *= static_cast<double>(plan.dim[a]);
            }
            const bool bad = r[8] > 0;
            plan.ok = !bad && total <= static_cast<double>(cells_cap);
            if (blockIdx.x == 0) {
                *plan_out = plan;
                const unsigned long long bits = (bad ? kBadRange : 0) | (plan.ok ? 0 : kNoGrid);
                if (bits) atomicOr(reinterpret_cast<unsigned long long *>(counts + 3), bits);
            }
        }
        __syncthreads();
    }
    if (!plan.ok) return;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const int lane = threadIdx.x & 63;
    int cell = -1, local = 0;
    if (i < N) {
        int w[4];
        window_of(reinterpret_cast<const int4 *>(coords)[i], stride, window, shift, w, &local);
        cell = (((w[0] - plan.lo[0]) * plan.dim[1] + (w[1] - plan.lo[1])) * plan.dim[2] + (w[2] - plan.lo[2])) * plan.dim[3] +
               (w[3] - plan.lo[3]);
    }
    const int before = __shfl_up(cell, 1);
    const bool head = lane == 0 || before != cell;
    const unsigned long long heads = __ballot(head);
    const unsigned long long upto = heads & (lane == 63 ? ~0ull : ((2ull << lane) - 1));
    const int my_head = 63 - __clzll(static_cast<long long>(upto));
    const unsigned long long above = lane == 63 ? 0ull : heads & ~((2ull << lane) - 1);
    const int next = above ? __ffsll(static_cast<long long>(above)) - 1 : 64;
    int base = 0;
    if (head && cell >= 0) base = atomicAdd(&cells[cell], next - lane);
    base = __shfl(base, my_head);
    if (i < N) {
        const int slot = base + (lane - my_head);
        if (slot >= (1 << kSlotBits)) atomicOr(reinterpret_cast<unsigned long long *>(counts + 3), static_cast<unsigned long long>(kNoGrid));
        place[i] = make_int2(cell, (slot & ((1 << kSlotBits) - 1)) | (local << kSlotBits));
    }
}

// every voxel to its window's segment (slot order); the voxel in slot 0 also records the window
__global__ __launch_bounds__(kThreads) void grid_place_kernel(const int2 *__restrict__ place, int64_t N,
                                                              const GridPlan *__restrict__ plan,
                                                              const uint64_t *__restrict__ scan, int64_t cells_cap,
                                                              uint64_t *__restrict__ keys, int32_t *__restrict__ w2n,
                                                              int32_t *__restrict__ w_sizes, int64_t *__restrict__ counts)
{
    if (!plan->ok || (counts[3] & kNoGrid)) return;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (i == 0) counts[0] = static_cast<int64_t>(scan[cells_cap] >> 32);   // non-empty cells before the end = windows
    if (i >= N) return;
    const int2 p = place[i];
    const uint64_t here = scan[p.x];
    const int start = static_cast<int>(here & 0xffffffffu), slot = p.y & ((1 << kSlotBits) - 1);
    keys[start + slot] = (static_cast<uint64_t>(p.y >> kSlotBits) << 32) | static_cast<uint32_t>(i);
    if (slot == 0) {
        const int rank = static_cast<int>(here >> 32);
        w2n[rank] = start;
        w_sizes[rank] = static_cast<int>(scan[p.x + 1] & 0xffffffffu) - start;
    }
}

// One wavefront per window at a time: the window's voxels in (local id, row) order.  The rank of an element is
// the number of smaller ones, counted against every element of the window (a few dozen to a few hundred voxels).
// Also the totals: sum of squared sizes and the largest size, one pair of atomics per workgroup.
__global__ __launch_bounds__(kThreads) void grid_order_kernel(const GridPlan *__restrict__ plan,
                                                              const uint64_t *__restrict__ keys,
                                                              const int32_t *__restrict__ w2n,
                                                              const int32_t *__restrict__ w_sizes,
                                                              int32_t *__restrict__ n2n, int32_t *__restrict__ w_w_id,
                                                              int64_t *__restrict__ counts)
{
    if (!plan->ok || (counts[3] & kNoGrid)) return;
    constexpr int kOrderStage = 512;                       // keys of a window staged in LDS at a time, per wavefront
    constexpr int kTotalGroups = 32;
    __shared__ uint64_t stage_all[kThreads / 64][kOrderStage];
    uint64_t *stage = stage_all[threadIdx.x >> 6];
    const int lane = threadIdx.x & 63;
    const int W = static_cast<int>(counts[0]);
    const int waves = static_cast<int>(gridDim.x) * (kThreads / 64);
    for (int w = static_cast<int>(blockIdx.x) * (kThreads / 64) + (threadIdx.x >> 6); w < W; w += waves) {
        const int start = w2n[w], n = w_sizes[w];
        if (n <= 64) {
            // one element per lane, the others read lane by lane
            const uint64_t mine = lane < n ? keys[start + lane] : ~0ULL;
            int rank = 0;
            for (int j = 0; j < n; ++j) {
                const uint64_t other = (static_cast<uint64_t>(static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(mine >> 32), j))) << 32) |
                                       static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(mine), j));
                rank += other < mine;
            }
            if (lane < n) {
                n2n[start + rank] = static_cast<int32_t>(mine & 0xffffffffu);
                w_w_id[start + rank] = static_cast<int32_t>(mine >> 32);
            }
            continue;
        }
        // larger windows: the keys staged in LDS, every lane ranks its elements against all of them; a window
        // beyond the staging area (only with many voxels of equal coordinates) is staged piece by piece per chunk
        auto stage_keys = [&](int base, int m) {
            __builtin_amdgcn_wave_barrier();
            for (int t = lane; t < m; t += 64) stage[t] = keys[start + base + t];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        };
        const bool whole = n <= kOrderStage;
        if (whole) stage_keys(0, n);
        for (int first = 0; first < n; first += 64) {
            const int e = first + lane;
            const uint64_t mine = e < n ? (whole ? stage[e] : keys[start + e]) : ~0ULL;
            int rank = 0;
            for (int base = 0; base < n; base += kOrderStage) {
                const int m = min(kOrderStage, n - base);
                if (!whole) stage_keys(base, m);
#pragma unroll 4
                for (int j = 0; j < m; ++j) rank += stage[j] < mine;
            }
            if (e < n) {
                n2n[start + rank] = static_cast<int32_t>(mine & 0xffffffffu);
                w_w_id[start + rank] = static_cast<int32_t>(mine >> 32);
            }
        }
    }
    // the totals (sum of squared sizes, largest size): the first kTotalGroups workgroups share the windows, one pair
    // of atomics each
    if (blockIdx.x >= kTotalGroups) return;
    long long squares = 0, largest = 0;
    for (int w = static_cast<int>(blockIdx.x) * kThreads + threadIdx.x; w < W; w += kTotalGroups * kThreads) {
        const long long n = w_sizes[w];
        squares += n * n;
        largest = max(largest, n);
    }
    for (int off = 32; off > 0; off >>= 1) {
        squares += __shfl_down(squares, off);
        largest = max(largest, __shfl_down(largest, off));
    }
    __shared__ long long part[kThreads / 64][2];
    if (lane == 0) { part[threadIdx.x >> 6][0] = squares; part[threadIdx.x >> 6][1] = largest; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int wv = 1; wv < kThreads / 64; ++wv) { squares += part[wv][0]; largest = max(largest, part[wv][1]); }
        if (largest > 0) {
            atomicAdd(reinterpret_cast<unsigned long long *>(counts + 1), static_cast<unsigned long long>(squares));
            atomicMax(reinterpret_cast<unsigned long long *>(counts + 2), static_cast<unsigned long long>(largest));
        }
    }
}

// one thread per (sorted position, column); the add and the multiply stay separate roundings, as in the
// reference's tensor statement (sum, then scale)
__global__ __launch_bounds__(kThreads) void window_signals_kernel(
    const int32_t *__restrict__ w_w_id, const int32_t *__restrict__ n2n, const float *__restrict__ frac,
    const float *__restrict__ signals, int64_t signals_stride, int columns, int window, float xyz_scale,
    float other_scale, float *__restrict__ out, int64_t N)
{
#pragma clang fp contract(off)
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (t >= N * columns) return;
    const int64_t p = t / columns;
    const int c = static_cast<int>(t - p * columns);
    const int64_t row = n2n[p];
    float v;
    if (c < 3) {
        const int id = w_w_id[p];
        const int cell = c == 0 ? id / (window * window) : c == 1 ? (id / window) % window : id % window;
        v = (static_cast<float>(cell) + frac[row * 3 + c]) * xyz_scale;
    } else {
        v = signals[row * signals_stride + (c - 3)] * other_scale;
    }
    out[t] = v;
}

// one thread per (sorted voxel, offset): binary search of key + delta in the sorted keys
__global__ __launch_bounds__(kThreads) void key_neighbours_kernel(const int64_t *__restrict__ sorted_keys,
                                                                  const int64_t *__restrict__ order, int64_t N,
                                                                  const int64_t *__restrict__ deltas, int M,
                                                                  int64_t *__restrict__ out)
{
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (t >= N * M) return;
    const int64_t i = t / M;
    const int d = static_cast<int>(t - i * M);
    const int64_t key = sorted_keys[i] + deltas[d];
    int64_t lo = 0, hi = N;   // first position whose key is not below `key`
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (sorted_keys[mid] < key) lo = mid + 1;
        else hi = mid;
    }
    const bool found = lo < N && sorted_keys[lo] == key;
    out[order[i] * M + d] = found ? order[lo] : N;
}

// one thread per cell (= window of the sort): mean of the members' signal rows, then the member nearest to it
constexpr int kMaxCellSignals = 16;
__global__ __launch_bounds__(kThreads) void cell_representatives_kernel(
    const int32_t *__restrict__ n2n, const int32_t *__restrict__ w2n, const int32_t *__restrict__ w_sizes, int64_t W,
    const float *__restrict__ signals, int64_t signals_stride, int S, int64_t *__restrict__ out)
{
#pragma clang fp contract(off)
    const int64_t w = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (w >= W) return;
    const int begin = w2n[w], size = w_sizes[w];
    float mean[kMaxCellSignals];
#pragma unroll
    for (int c = 0; c < kMaxCellSignals; ++c) mean[c] = 0.0f;
    for (int p = begin; p < begin + size; ++p) {
        const float *row = signals + static_cast<int64_t>(n2n[p]) * signals_stride;
#pragma unroll
        for (int c = 0; c < kMaxCellSignals; ++c)
            if (c < S) mean[c] += row[c];
    }
#pragma unroll
    for (int c = 0; c < kMaxCellSignals; ++c) mean[c] /= static_cast<float>(size);
    float best = INFINITY;
    int best_row = 0x7fffffff;
    for (int p = begin; p < begin + size; ++p) {
        const int r = n2n[p];
        const float *row = signals + static_cast<int64_t>(r) * signals_stride;
        float sq = 0.0f;
#pragma unroll
        for (int c = 0; c < kMaxCellSignals; ++c) {
            if (c < S) {
                const float d = row[c] - mean[c];
                sq += d * d;
            }
        }
        const float dist = sqrtf(sq);
        if (dist < best || (dist == best && r < best_row)) {
            best = dist;
            best_row = r;
        }
    }
    out[w] = best_row;
}

}  // namespace
}  // namespace s3d

extern "C" __attribute__((visibility("default"))) int s3d_cell_representatives(
    const int32_t *n2n, const int32_t *w2n, const int32_t *w_sizes, int64_t W, const float *signals,
    int64_t signals_stride, int32_t num_signals, int64_t *out, void *stream)
{
    using namespace s3d;
    if (W < 0 || num_signals < 1 || num_signals > kMaxCellSignals || signals_stride < num_signals)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_cell_representatives: W=%lld num_signals=%d (1..%d) signals_stride=%lld",
                    (long long)W, num_signals, kMaxCellSignals, (long long)signals_stride);
    if (W == 0) return S3D_OK;
    if (!n2n || !w2n || !w_sizes || !signals || !out)
        return fail(S3D_ERR_NULL_POINTER, "s3d_cell_representatives: null device pointer");
    const dim3 grid(static_cast<unsigned>(ceil_div(W, kThreads)));
    hipLaunchKernelGGL(cell_representatives_kernel, grid, dim3(kThreads), 0, static_cast<hipStream_t>(stream), n2n, w2n,
                       w_sizes, W, signals, signals_stride, num_signals, out);
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}

extern "C" __attribute__((visibility("default"))) int s3d_key_neighbours(const int64_t *sorted_keys,
                                                                          const int64_t *order, int64_t N,
                                                                          const int64_t *deltas, int32_t M,
                                                                          int64_t *out, void *stream)
{
    using namespace s3d;
    if (N < 0 || M < 1 || M > 1024 || N * static_cast<int64_t>(M) > 0x3fffffffffLL)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_key_neighbours: N=%lld M=%d out of range", (long long)N, M);
    if (N == 0) return S3D_OK;
    if (!sorted_keys || !order || !deltas || !out)
        return fail(S3D_ERR_NULL_POINTER, "s3d_key_neighbours: null device pointer");
    const dim3 grid(static_cast<unsigned>(ceil_div(N * M, kThreads)));
    hipLaunchKernelGGL(key_neighbours_kernel, grid, dim3(kThreads), 0, static_cast<hipStream_t>(stream), sorted_keys,
                       order, N, deltas, M, out);
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}

extern "C" __attribute__((visibility("default"))) int s3d_window_signals(
    const int32_t *w_w_id, const int32_t *n2n, const float *frac, const float *signals, int64_t signals_stride,
    int32_t num_signals, int32_t window, float xyz_scale, float other_scale, float *out, int64_t N, void *stream)
{
    using namespace s3d;
    if (N < 0 || num_signals < 0 || window < 1 || window > 10 || (num_signals > 0 && signals_stride < num_signals))
        return fail(S3D_ERR_BAD_SHAPE, "s3d_window_signals: N=%lld num_signals=%d signals_stride=%lld window=%d",
                    (long long)N, num_signals, (long long)signals_stride, window);
    if (N == 0) return S3D_OK;
    if (!w_w_id || !n2n || !frac || !out || (num_signals > 0 && !signals))
        return fail(S3D_ERR_NULL_POINTER, "s3d_window_signals: null device pointer");
    const int columns = 3 + num_signals;
    const dim3 grid(static_cast<unsigned>(ceil_div(N * columns, kThreads)));
    hipLaunchKernelGGL(window_signals_kernel, grid, dim3(kThreads), 0, static_cast<hipStream_t>(stream), w_w_id, n2n,
                       frac, signals, signals_stride, columns, window, xyz_scale, other_scale, out, N);
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}

extern "C" __attribute__((visibility("default"))) size_t s3d_window_index_workspace_bytes(int64_t N)
{
    return s3d::make_layout(N).total;
}

extern "C" __attribute__((visibility("default"))) int s3d_window_index(const int32_t *coords, int64_t N, int32_t stride, int32_t window,
                                int32_t shift, int32_t *n2n, int32_t *w_w_id, int32_t *w_sizes,
                                int32_t *w2n, int64_t *counts, void *workspace,
                                size_t workspace_bytes, void *stream)
{
    using namespace s3d;
    if (N < 0 || N > 0x7fffffffLL)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_window_index: N=%lld out of range", (long long)N);
    if (stride < 1 || window < 1 || window > 10 || shift < 0 || shift >= window)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_window_index: stride=%d window=%d shift=%d (need stride>=1, "
                    "1<=window<=10, 0<=shift<window)", stride, window, shift);
    if (!counts) return fail(S3D_ERR_NULL_POINTER, "s3d_window_index: counts is null");
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(init_counts_kernel, dim3(1), dim3(64), 0, s, counts);
    S3D_HIP_CHECK(hipGetLastError());
    if (N == 0) return S3D_OK;
    if (!coords || !n2n || !w_w_id || !w_sizes || !w2n || !workspace)
        return fail(S3D_ERR_NULL_POINTER, "s3d_window_index: null device pointer");
    if (reinterpret_cast<uintptr_t>(coords) % 16 != 0)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_window_index: coords must be 16-byte aligned");
    const Layout L = make_layout(N);
    if (workspace_bytes < L.total)
        return fail(S3D_ERR_WORKSPACE, "s3d_window_index: workspace %zu B < required %zu B",
                    workspace_bytes, L.total);
    char *base = static_cast<char *>(workspace);
    uint64_t *keys_in = reinterpret_cast<uint64_t *>(base + L.keys_in);
    uint64_t *keys_out = reinterpret_cast<uint64_t *>(base + L.keys_out);
    int32_t *vals_in = reinterpret_cast<int32_t *>(base + L.vals_in);
    int32_t *flags = reinterpret_cast<int32_t *>(base + L.flags);
    int32_t *ranks = reinterpret_cast<int32_t *>(base + L.ranks);
    void *temp = base + L.temp;
    size_t temp_bytes = L.temp_bytes;

    const dim3 grid(static_cast<unsigned>(ceil_div(N, kThreads)));
    hipLaunchKernelGGL(build_keys_kernel, grid, dim3(kThreads), 0, s, coords, N, stride, window,
                       shift, keys_in, vals_in, counts);
    S3D_HIP_CHECK(hipGetLastError());
    S3D_HIP_CHECK(rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_out, vals_in, n2n,
                                            static_cast<size_t>(N), 0, 64, s));
    hipLaunchKernelGGL(flag_kernel, grid, dim3(kThreads), 0, s, keys_out, N, flags, w_w_id);
    S3D_HIP_CHECK(hipGetLastError());
    temp_bytes = L.temp_bytes;
    S3D_HIP_CHECK(rocprim::inclusive_scan(temp, temp_bytes, flags, ranks, static_cast<size_t>(N),
                                          rocprim::plus<int32_t>(), s));
    hipLaunchKernelGGL(segment_start_kernel, grid, dim3(kThreads), 0, s, flags, ranks, N, w2n, counts);
    S3D_HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL(segment_size_kernel, grid, dim3(kThreads), 0, s, w2n, N, w_sizes, counts);
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}

extern "C" __attribute__((visibility("default"))) size_t s3d_window_index_grid_workspace_bytes(int64_t N)
{
    return s3d::make_grid_layout(N).total;
}

extern "C" __attribute__((visibility("default"))) int s3d_window_index_grid(
    const int32_t *coords, int64_t N, int32_t stride, int32_t window, int32_t shift, int32_t *n2n, int32_t *w_w_id,
    int32_t *w_sizes, int32_t *w2n, int64_t *counts, void *workspace, size_t workspace_bytes, void *stream)
{
    using namespace s3d;
    if (N < 0 || N > 0x7fffffffLL)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_window_index_grid: N=%lld out of range", (long long)N);
    if (stride < 1 || window < 1 || window > 10 || shift < 0 || shift >= window)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_window_index_grid: stride=%d window=%d shift=%d (need stride>=1, "
                    "1<=window<=10, 0<=shift<window)", stride, window, shift);
    if (!counts) return fail(S3D_ERR_NULL_POINTER, "s3d_window_index_grid: counts is null");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (N == 0) {
        hipLaunchKernelGGL(init_counts_kernel, dim3(1), dim3(64), 0, s, counts);
        S3D_HIP_CHECK(hipGetLastError());
        return S3D_OK;
    }
    if (!coords || !n2n || !w_w_id || !w_sizes || !w2n || !workspace)
        return fail(S3D_ERR_NULL_POINTER, "s3d_window_index_grid: null device pointer");
    if (reinterpret_cast<uintptr_t>(coords) % 16 != 0)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_window_index_grid: coords must be 16-byte aligned");
    const GridLayout L = make_grid_layout(N);
    if (workspace_bytes < L.total)
        return fail(S3D_ERR_WORKSPACE, "s3d_window_index_grid: workspace %zu B < required %zu B", workspace_bytes, L.total);
    char *base = static_cast<char *>(workspace);
    GridPlan *plan = reinterpret_cast<GridPlan *>(base + L.plan);
    int32_t *partials = reinterpret_cast<int32_t *>(base + L.partials);
    int32_t *cells = reinterpret_cast<int32_t *>(base + L.cells);
    uint64_t *scan = reinterpret_cast<uint64_t *>(base + L.scan);
    int2 *place = reinterpret_cast<int2 *>(base + L.place);
    uint64_t *keys = reinterpret_cast<uint64_t *>(base + L.keys);
    size_t temp_bytes = L.temp_bytes;
    const int64_t num_cells = L.cells_cap + 1;
    const dim3 grid(static_cast<unsigned>(ceil_div(N, kThreads)));
    hipLaunchKernelGGL(grid_bbox_kernel, dim3(kGridBoxes), dim3(kThreads), 0, s, coords, N, stride, window, shift, partials,
                       cells, num_cells, counts);
    S3D_HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL(grid_count_kernel, grid, dim3(kThreads), 0, s, coords, N, stride, window, shift, partials,
                       L.cells_cap, plan, cells, place, counts);
    S3D_HIP_CHECK(hipGetLastError());
    S3D_HIP_CHECK(rocprim::exclusive_scan(base + L.temp, temp_bytes, CellWordIterator(cells, CellWord()), scan, uint64_t(0),
                                          static_cast<size_t>(num_cells), rocprim::plus<uint64_t>(), s));
    hipLaunchKernelGGL(grid_place_kernel, grid, dim3(kThreads), 0, s, place, N, plan, scan, L.cells_cap, keys, w2n, w_sizes,
                       counts);
    S3D_HIP_CHECK(hipGetLastError());
    // about one window per wavefront if the windows hold 16 voxels on average, more in turn otherwise
    int64_t order_blocks = ceil_div(N, 64);
    order_blocks = order_blocks < 32 ? 32 : (order_blocks > 4096 ? 4096 : order_blocks);
    hipLaunchKernelGGL(grid_order_kernel, dim3(static_cast<unsigned>(order_blocks)), dim3(kThreads), 0, s, plan, keys, w2n,
                       w_sizes, n2n, w_w_id, counts);
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}
