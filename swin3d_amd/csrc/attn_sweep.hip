// Sparse-voxel windowed self-attention with cRSE tables (gfx950): the sweep kernel of the forward and, on the same
// work list, the pair sweeps of the backward (dq; dk and dv - further down).
//
// Covers every dtype / shape the library accepts on the vector ALU (fp32 arithmetic; fp16 inputs enter through
// packed dot products and mixed-precision FMAs with fp32 accumulation).  A workgroup serves one to three heads
// for its whole life and keeps the slices of the three relative-signal tables in LDS (loaded once, not once
// per window).  Lane = one query against (a share of) the keys of its window: q_i, the running
// maximum, sum and output stay in the lane's registers while the lane streams its own window's keys, one per
// step, no atomic on data and no O(pairs) index array; the result is
// deterministic.  The slots of all windows, sorted by step count, are packed into units of 64 (the lanes of a
// wavefront carry queries of several small windows); wavefronts draw units from the head's work queues.
// A query of a window of more than the step target gets 2, 4 or 8 adjacent lanes that take alternate keys and merge
// their softmax states by shuffles at the end of the unit.
//
// Math (per window, sorted positions i, j, head h), following the reference kernels
// Swin3D/src/attn/self_attn_aio_fwd.cu:16-52 and :111-188:
//   row_n(i,j) = quantised (n_coords[i][n] - n_coords[j][n])   (attn_utils.cuh:437-453)
//   T*(i,j)[c] = sum_n table_*[n][row_n(i,j)][h][c]            (attn_utils.cuh:455-464)
//   L(i,j)     = sum_c q_i[c] k_j[c] + q_i[c] Tq(i,j)[c] + k_j[c] Tk(i,j)[c]
//   out_i[c]   = sum_j softmax_j(L(i,j)) (v_j[c] + Tv(i,j)[c])
#include "attn_kernels.h"
#include "sweep_common.h"

#include <mutex>
#include <vector>

namespace s3d {
namespace {

using namespace sweep;

constexpr int kChunk = 64;   // lanes of a wavefront = lanes of a unit
constexpr int kListThreads = 256, kListGroups = 32;   // the list builder's workgroups: size, and how many at most
constexpr float kSlack = 10.0f;   // how far a logit may exceed the softmax reference exponent before it moves
// A window of n voxels belongs to class g (0..kMaxSplit): each of its queries is served by 2^g adjacent lanes that
// take alternate keys, g the smallest value for which a lane streams at most `target` keys (the launch's step
// target: 64, or 32 / 16 in small launches that would otherwise not fill the chip).  Windows of more than
// target << kMaxSplit voxels stay in the last class and take more steps.
constexpr int kMaxSplit = 3;
constexpr int kClasses = kMaxSplit + 1;
constexpr int kMaxSteps = 64;                    // step counts that have a bin of their own; longer ones share the last
constexpr int kBins = kClasses * kMaxSteps;      // (class, steps), class 3 first, longest first inside a class
constexpr int kSections = kMaxSplit + 3;         // classes 3..1, then class 0 in units of 64, 32 and 16 queries
static_assert(kBins == kListThreads, "one thread per bin");
__host__ __device__ inline int window_class(int n, int target_shift)
{
    int g = 0;
    while (g < kMaxSplit && ((n + (1 << g) - 1) >> g) > (1 << target_shift)) ++g;
    return g;
}
__host__ __device__ inline int window_bin(int n, int g)
{
    const int steps = (n + (1 << g) - 1) >> g;
    return (kMaxSplit - g) * kMaxSteps + (kMaxSteps - (steps < kMaxSteps ? steps : kMaxSteps));
}
// The step target of a launch, as a shift.  The launch ends when its last wavefront does, so a unit must stay
// short against what a wavefront does in the whole launch: N^2 / W pairs at least, per head group, over the
// lanes of `waves` wavefronts that serve the group.  64 steps unless that leaves fewer than about six units per
// wavefront; not below 32 where the mean window has at most 32 voxels: a target of 16 would give the typical
// window two lanes per query, whose softmax states are merged at the end of the unit, where one lane per query
// serves it in 32 steps without a merge (-3.5 % on 26-voxel windows; on window-7 levels, 57 voxels a window and
// most pairs in windows of more than 64, the target of 32 measured +4 %: longer units, the same merges).
__host__ inline int target_shift_for(int64_t N, int64_t W, int waves)
{
    if (N <= 0 || W <= 0) return 6;
    const double lane_steps = static_cast<double>(N) * static_cast<double>(N) / static_cast<double>(W);
    const int least = N <= 32 * W ? 5 : 4;
    int shift = 6;
    while (shift > least && lane_steps / (64.0 * (1 << shift)) < 6.0 * (waves > 0 ? waves : 1)) --shift;
    return shift;
}

// byte offsets inside the workspace: the queue counters, the totals, one record per unit, the sorted window
// entries, the placement notes and per-workgroup bin totals of the list builder
__host__ __device__ inline size_t ws_round(size_t bytes) { return (bytes + 255) / 256 * 256; }
__host__ __device__ inline size_t ws_total_offset(int H) { return sizeof(int32_t) * static_cast<size_t>(H) * kQueues * kCounterStride; }
// after the totals (one cache line): one exit counter per queue index, each on a cache line of its own
__host__ __device__ inline size_t ws_units_offset(int H) { return ws_total_offset(H) + 256 * (1 + kQueues); }
// a unit holds at least 64 >> kMaxSplit = 8 queries, except the last one of each section
__host__ __device__ inline size_t ws_max_units(int64_t N)
{
    return static_cast<size_t>(N > 0 ? N : 0) / (kChunk >> kMaxSplit) + kSections + 1;
}
__host__ __device__ inline size_t ws_entries_offset(int H, int64_t N)
{
    return ws_units_offset(H) + ws_round(sizeof(int4) * ws_max_units(N));
}
__host__ __device__ inline size_t ws_place_offset(int H, int64_t W, int64_t N)
{
    return ws_entries_offset(H, N) + ws_round(sizeof(int4) * (static_cast<size_t>(W > 0 ? W : 0) + kChunk));
}
__host__ __device__ inline size_t ws_bins_offset(int H, int64_t W, int64_t N)
{
    return ws_place_offset(H, W, N) + ws_round(sizeof(int2) * static_cast<size_t>(W > 0 ? W : 1));
}
__host__ __device__ inline size_t ws_end_offset(int H, int64_t W, int64_t N)
{
    return ws_bins_offset(H, W, N) + ws_round(sizeof(unsigned long long) * kListGroups * (kListThreads / 64 + 1) * kBins);
}

// How the queries of class 0 (sorted by steps, longest first) are cut into units.  A unit is one pass of a
// wavefront: 64 queries, or 32 queries with two adjacent lanes each (alternate keys, half the steps), or 16
// queries with four lanes each (a quarter).  The launch ends when the last wavefront ends, so the last queries
// go into the finer units: about two 16-query units and one 32-query unit per wavefront of a head group
// (`waves`), everything before them into 64-query units.
struct UnitPlan {
    int units[3];   // units of 64, 32 and 16 queries, in this order along the queries
    __host__ __device__ int first_slot(int g) const { return g == 0 ? 0 : g == 1 ? units[0] * kChunk : units[0] * kChunk + units[1] * (kChunk / 2); }
    __host__ __device__ int first_unit(int g) const { return g == 0 ? 0 : g == 1 ? units[0] : units[0] + units[1]; }
};
__host__ __device__ inline UnitPlan plan_units(int total_slots, int waves)
{
    const int fine = 32 * (waves > 0 ? waves : 1);   // queries of each finer kind
    const int in_c = total_slots < fine ? total_slots : fine;
    const int in_b = total_slots - in_c < fine ? total_slots - in_c : fine;
    UnitPlan plan;
    plan.units[0] = (total_slots - in_c - in_b + kChunk - 1) / kChunk;
    const int left_b = total_slots - plan.units[0] * kChunk;            // may be negative by rounding
    const int take_b = left_b < 0 ? 0 : (left_b < in_b ? left_b : in_b);
    plan.units[1] = (take_b + kChunk / 2 - 1) / (kChunk / 2);
    const int left_c = total_slots - plan.units[0] * kChunk - plan.units[1] * (kChunk / 2);
    plan.units[2] = left_c <= 0 ? 0 : (left_c + kChunk / 4 - 1) / (kChunk / 4);
    return plan;
}

// Work list of the launch, built by two small kernels.  The windows are sorted by (class, steps), highest class and
// longest first - a counting sort over the kBins possible keys - and the queries of each class are numbered
// back to back in that order, [window][voxel], and cut into units: 64 >> g queries of class g, each on 2^g
// adjacent lanes.  A wavefront's lanes so carry queries of several windows when the windows are small, every
// lane of a unit runs (almost) the same number of steps, a query's keys never leave its wavefront (the lanes
// that share a query merge their softmax states by shuffles), and the launch ends on its shortest units.
//
// sweep_count_kernel: every wavefront takes a run of consecutive windows, 64 at a time.  A window's place in the
// bin of its (class, steps) - its rank there and the queries before it - follows the window numbers: the lanes
// of each bin present among the 64 are ranked by their lane numbers on top of the bin's running totals, which
// the wavefront keeps in registers (lane b % 64 holds bin b), and the wavefront leaves its bin totals.  No
// atomics: the list, and with it the cut of the queries into units and so every bit of the result, is the same
// on every run.
__global__ __launch_bounds__(kListThreads) void sweep_count_kernel(AttnArgs a)
{
    constexpr int kWaves = kListThreads / 64;
    const int lane = threadIdx.x & 63;
    const int table = static_cast<int>(blockIdx.x) * kWaves + static_cast<int>(threadIdx.x >> 6);
    const int tables = static_cast<int>(gridDim.x) * kWaves;
    char *ws = static_cast<char *>(a.workspace);
    int2 *place = reinterpret_cast<int2 *>(ws + ws_place_offset(a.H, a.W, a.N));
    unsigned long long *group_bins = reinterpret_cast<unsigned long long *>(ws + ws_bins_offset(a.H, a.W, a.N));
    const int W = static_cast<int>(a.W);
    const int per = (W + tables - 1) / tables;
    const int begin = min(table * per, W), end = min(begin + per, W);
    uint32_t held_c[kBins / 64], held_s[kBins / 64];   // bins lane, lane + 64, ...: windows and queries so far
#pragma unroll
    for (int j = 0; j < kBins / 64; ++j) held_c[j] = held_s[j] = 0;
    for (int w0 = begin; w0 < end; w0 += 64) {
        const int w = w0 + lane;
        const int n = w < end ? a.w_sizes[w] : 0;
        const int b = n > 0 ? window_bin(n, window_class(n, a.block_shift)) : -1;
        int2 got = make_int2(-1, 0);
        unsigned long long todo = __ballot(b >= 0);
        while (todo != 0) {
            const int leader = __ffsll(todo) - 1;
            const int cb = __builtin_amdgcn_readlane(b, leader), n_lead = __builtin_amdgcn_readlane(n, leader);
            const bool in = b == cb;
            const unsigned long long same = __ballot(in);
            const int below = __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(same >> 32),
                                                        __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(same), 0u));
            int before_n, all_n;
            if (__ballot(in && n != n_lead) == 0) {   // the usual case: a bin of class 0 is one window size
                before_n = below * n_lead;
                all_n = __popcll(same) * n_lead;
            } else {
                int incl = in ? n : 0;
                for (int off = 1; off < 64; off <<= 1) {
                    const int up = __shfl_up(incl, off);
                    if (lane >= off) incl += up;
                }
                before_n = incl - (in ? n : 0);
                all_n = __builtin_amdgcn_readlane(incl, 63);
            }
            uint32_t c = 0, q = 0;
#pragma unroll
            for (int j = 0; j < kBins / 64; ++j)
                if ((cb >> 6) == j) { c = held_c[j]; q = held_s[j]; }
            c = __builtin_amdgcn_readlane(c, cb & 63);
            q = __builtin_amdgcn_readlane(q, cb & 63);
            if (in) got = make_int2(static_cast<int>(c) + below, static_cast<int>(q) + before_n);
#pragma unroll
            for (int j = 0; j < kBins / 64; ++j)
                if ((cb >> 6) == j && lane == (cb & 63)) { held_c[j] += __popcll(same); held_s[j] += all_n; }
            todo &= ~same;
        }
        if (w < end) place[w] = got;
    }
    // the wavefront's totals, and the workgroup's (what the place kernel sums over the launch)
    __shared__ unsigned long long wave_bins[kWaves][kBins];
    unsigned long long *sum_bins = group_bins + static_cast<size_t>(kListGroups) * kWaves * kBins;
#pragma unroll
    for (int j = 0; j < kBins / 64; ++j) {
        const unsigned long long v = (static_cast<unsigned long long>(held_c[j]) << 32) | held_s[j];
        group_bins[static_cast<size_t>(table) * kBins + j * 64 + lane] = v;
        wave_bins[threadIdx.x >> 6][j * 64 + lane] = v;
    }
    __syncthreads();
    unsigned long long sum = 0;
#pragma unroll
    for (int v = 0; v < kWaves; ++v) sum += wave_bins[v][threadIdx.x];
    sum_bins[static_cast<size_t>(blockIdx.x) * kBins + threadIdx.x] = sum;
}

// sweep_place_kernel (same grid): bins in order, wavefronts in order inside a bin.  Writes one entry (first
// query of its class, voxels, first sorted position, class) per window in sorted order, one record per unit
// (the entry that holds its first query, lanes per query as a shift, first query, queries), the totals, and
// the queue counters at zero.
__global__ __launch_bounds__(kListThreads) void sweep_place_kernel(AttnArgs a)
{
    constexpr int kWaves = kListThreads / 64;
    __shared__ int bin_entry[kWaves][kBins], bin_slot[kWaves][kBins];
    __shared__ int wave_c[kWaves], wave_s[kWaves];
    __shared__ int class_base[kClasses + 1];       // queries before each class (index = kMaxSplit - g), and all
    __shared__ int total_entries_s;
    char *ws = static_cast<char *>(a.workspace);
    int *counters = reinterpret_cast<int *>(ws);
    int *total = reinterpret_cast<int *>(ws + ws_total_offset(a.H));
    int4 *unit_info = reinterpret_cast<int4 *>(ws + ws_units_offset(a.H));
    int4 *entries = reinterpret_cast<int4 *>(ws + ws_entries_offset(a.H, a.N));
    const int2 *place = reinterpret_cast<const int2 *>(ws + ws_place_offset(a.H, a.W, a.N));
    const unsigned long long *group_bins =
        reinterpret_cast<const unsigned long long *>(ws + ws_bins_offset(a.H, a.W, a.N));
    const int tables = static_cast<int>(gridDim.x) * kWaves, first_table = static_cast<int>(blockIdx.x) * kWaves;
    const unsigned long long *sum_bins = group_bins + static_cast<size_t>(kListGroups) * kWaves * kBins;
    // thread t holds bin t: the launch's total, and what the workgroups before this one put there; an exclusive
    // scan over the threads gives the bins their places (entries over all bins, queries restarting per class)
    {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        unsigned long long all = 0, before = 0;
#pragma unroll 8
        for (int g = 0; g < static_cast<int>(gridDim.x); ++g) {
            const unsigned long long v = sum_bins[static_cast<size_t>(g) * kBins + threadIdx.x];
            all += v;
            before += g < static_cast<int>(blockIdx.x) ? v : 0;
        }
        const int cnt = static_cast<int>(all >> 32), slots = static_cast<int>(all & 0xffffffffu);
        int incl_c = cnt, incl_s = slots;
        for (int off = 1; off < 64; off <<= 1) {
            const int up_c = __shfl_up(incl_c, off), up_s = __shfl_up(incl_s, off);
            if (lane >= off) { incl_c += up_c; incl_s += up_s; }
        }
        if (lane == 63) { wave_c[wave] = incl_c; wave_s[wave] = incl_s; }
        __syncthreads();
        int base_c = 0, base_s = 0;
        for (int v = 0; v < wave; ++v) { base_c += wave_c[v]; base_s += wave_s[v]; }
        static_assert(kMaxSteps == 64, "a class is the bins of one wavefront of the scan");
        // queries are numbered per class: the class's bins are this wavefront's, so drop the earlier wavefronts' sum
#pragma unroll
        for (int v = 0; v < kWaves; ++v) {
            bin_entry[v][threadIdx.x] = base_c + incl_c - cnt + static_cast<int>(before >> 32);
            bin_slot[v][threadIdx.x] = incl_s - slots + static_cast<int>(before & 0xffffffffu);
            before += group_bins[static_cast<size_t>(first_table + v) * kBins + threadIdx.x];
        }
        if (lane == 0) class_base[wave] = base_s;
        if (threadIdx.x == kListThreads - 1) { class_base[kClasses] = base_s + incl_s; total_entries_s = base_c + incl_c; }
    }
    __syncthreads();
    const int total_entries = total_entries_s;
    // sections: classes kMaxSplit..1 in units of 64 >> g queries, then class 0 in its three kinds of unit
    int sec_unit[kSections + 1], class_total[kClasses];
#pragma unroll
    for (int c = 0; c < kClasses; ++c) class_total[c] = class_base[c + 1] - class_base[c];
    const UnitPlan plan = plan_units(class_total[kMaxSplit], a.target_items);
    sec_unit[0] = 0;
#pragma unroll
    for (int c = 0; c < kMaxSplit; ++c) {
        const int per = kChunk >> (kMaxSplit - c);
        sec_unit[c + 1] = sec_unit[c] + (class_total[c] + per - 1) / per;
    }
#pragma unroll
    for (int k = 0; k < 3; ++k) sec_unit[kMaxSplit + k + 1] = sec_unit[kMaxSplit + k] + plan.units[k];
    const int W = static_cast<int>(a.W);
    const int my_wave = threadIdx.x >> 6;
    const int per_wave = (W + tables - 1) / tables;     // the count kernel's runs
    const int begin = min((first_table + my_wave) * per_wave, W), end = min(begin + per_wave, W);
    for (int w = begin + (threadIdx.x & 63); w < end; w += 64) {
        const int2 got = place[w];
        if (got.x < 0) continue;
        const int n = a.w_sizes[w];
        const int g = window_class(n, a.block_shift), b = window_bin(n, g);
        const int e = bin_entry[my_wave][b] + got.x;
        const int s = bin_slot[my_wave][b] + got.y;      // first query of the window inside its class
        entries[e] = make_int4(s, n, a.w2n[w], g);
        const int s_end = s + n;
        if (g > 0) {
            // the units whose first query is one of this window's
            const int size = kChunk >> g, c = kMaxSplit - g, all = class_total[c];
            for (int v = (s + size - 1) / size; v * size < s_end; ++v)
                unit_info[sec_unit[c] + v] = make_int4(e, g, v * size, min(size, all - v * size));
        } else {
            const int all = class_total[kMaxSplit];
#pragma unroll
            for (int k = 0; k < 3; ++k) {
                const int size = kChunk >> k, from = plan.first_slot(k), count = plan.units[k];
                int v = s <= from ? 0 : (s - from + size - 1) / size;
                for (; v < count && from + v * size < s_end; ++v)
                    unit_info[sec_unit[kMaxSplit + k] + v] = make_int4(e, k, from + v * size, min(size, all - (from + v * size)));
            }
        }
    }
    if (blockIdx.x == 0) {
        // a wavefront reads 64 entries from a unit's first one: pad the list with entries no query belongs to
        if (threadIdx.x < kChunk) entries[total_entries + threadIdx.x] = make_int4(0x7fffffff, 1, 0, -1);
        if (threadIdx.x == 0) {
            total[0] = sec_unit[kSections];
            total[1] = 0;   // exit counters of a sweep launch: cache lines that are complete, and one per line
        }
        if (threadIdx.x < kQueues) total[(1 + threadIdx.x) * kCounterStride] = 0;
        for (int t = threadIdx.x; t < a.H * kQueues; t += kListThreads) counters[t * kCounterStride] = 0;
    }
}

// Raises a kernel's dynamic-LDS limit to `bytes`.  The runtime keeps the limit per function and device, so it is
// set when a (function, device) pair first needs that much and not again: a call under stream capture then issues
// kernel launches only (one eager call per shape and device has to come before the capture).
inline int allow_dynamic_lds(const void *kernel, size_t bytes)
{
    struct Granted { const void *kernel; int device; size_t bytes; };
    static std::mutex mutex;
    static std::vector<Granted> granted;
    int device = 0;
    S3D_HIP_CHECK(hipGetDevice(&device));
    std::lock_guard<std::mutex> lock(mutex);
    for (Granted &g : granted) {
        if (g.kernel == kernel && g.device == device) {
            if (g.bytes >= bytes) return S3D_OK;
            S3D_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)));
            g.bytes = bytes;
            return S3D_OK;
        }
    }
    S3D_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)));
    granted.push_back({kernel, device, bytes});
    return S3D_OK;
}

inline int device_cus()
{
    int device = 0, v = 0;
    if (hipGetDevice(&device) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && v > 0)
        return v;
    return 256;
}

// Workgroup shapes.  A workgroup holds its heads' table slices once, so what fits a CU is set by registers and LDS:
//   one head per wavefront: four workgroups of four wavefronts per CU at head_dim 8 (one wavefront of each on every
//     SIMD), three at head_dim 16, two at head_dim 32 (an fp32 query, key, value and output row are 128 registers);
//   fp16, head_dim 8, two heads: four of four (128 registers without spills; the fourth wavefront per SIMD measured
//     -2 to -3 %); three heads: one workgroup of twelve wavefronts (168 registers, 45 KB of tables: -4 % against
//     three workgroups of four; sixteen-wavefront workgroups for the one- and two-head instances measured +-2 %);
//   fp32, head_dim 8, two heads: two workgroups of eight wavefronts (126 registers, 65 KB of tables each: four
//     wavefronts per SIMD; one workgroup of twelve measured 17 % slower than one head per wavefront, this -4 %);
//   fp16, head_dim 16, two heads: one workgroup of twelve wavefronts (75 KB of tables, three wavefronts per SIMD; two
//     workgroups of six measured 25 % slower than one of twelve);
//   fp32, head_dim 16: one workgroup of twelve wavefronts as well (75 KB of tables, 160 registers: -19 % against two
//     workgroups of four, which is all that LDS held); fp32, head_dim 32: one workgroup of eight (125 KB of tables).
template <typename T, int D, int HP> __host__ __device__ constexpr int group_threads()
{
    return sizeof(T) == 4 && D == 32 ? 512
           : HP == 3 ? 768
           : HP == 2 && sizeof(T) == 4 && D == 8 ? 512
           : (HP == 2 || sizeof(T) == 4) && D == 16 ? 768 : 256;
}
template <typename T, int D, int HP> __host__ __device__ constexpr int groups_per_cu()
{
    return sizeof(T) == 4 && D == 32 ? 1
           : group_threads<T, D, HP>() == 512 ? 2 : group_threads<T, D, HP>() == 768 ? 1
           : D > 16 ? 2 : D > 8 ? 3 : 4;
}

// elements of T between table rows in LDS when a workgroup holds the slices of HP heads side by side
template <typename T, int D, int HP> __host__ __device__ constexpr int table_row_stride_heads()
{
    return HP * 3 * D + ((HP * 3 * D * static_cast<int>(sizeof(T)) / 4) % 8 == 0 ? 16 / static_cast<int>(sizeof(T)) : 0);
}

// HP: heads a wavefront carries through a unit (adjacent heads HP * g .. HP * g + HP - 1).  The cRSE rows and
// LDS addresses of a pair do not depend on the head, so two or three heads share that part of the work.
// kSorted: q, k, v and out rows are in window-sorted order already (no n2n).
template <typename T, int D, int ND, int HP, bool kSorted>
__global__ __launch_bounds__((group_threads<T, D, HP>()), (groups_per_cu<T, D, HP>())) void attn_fwd_sweep_kernel(AttnArgs a)
{
    constexpr int kThreads = group_threads<T, D, HP>();
    // streamed keys per loop iteration: at head_dim 16 with one head two interleaved chains hide the LDS round trips;
    // with two heads the heads are the two chains
    constexpr int kKeys = D == 16 && HP == 1 ? 2 : 1;
    // lazy softmax reference (see the loop): -4 % for fp16; fp32 measured no gain (head_dim 8) or a loss (16)
    constexpr bool kLazy = sizeof(T) == 2;
    // 16-byte aligned like the table rows behind it, which are read 16 bytes at a time
    extern __shared__ __align__(16) float smem[];
    __shared__ __align__(16) int group_exit_counter[4];   // [0]: wavefronts of this workgroup that have left their loop
    int &group_exited = group_exit_counter[0];
    if (threadIdx.x == 0) group_exited = 0;
    const int H = a.H;
    const int HD = H * D;
    // workgroups go to the XCDs in turn: consecutive runs of eight serve one head group, so every XCD gets every head
    // (or, with many head groups, the head groups take the workgroups in turn: see the launch)
    const int hg = a.spread_groups ? blockIdx.x % (H / HP) : (blockIdx.x / kQueues) % (H / HP);
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
    const int4 *unit_info = reinterpret_cast<const int4 *>(ws + ws_units_offset(H));
    const int4 *entries = reinterpret_cast<const int4 *>(ws + ws_entries_offset(H, a.N));
    const int total_units = __builtin_amdgcn_readfirstlane(reinterpret_cast<const int *>(ws + ws_total_offset(H))[0]);
    int *counters = static_cast<int *>(a.workspace) + hg * kQueues * kCounterStride;
    constexpr int kRowBytes = kRowStride * static_cast<int>(sizeof(T));
    constexpr uint32_t kHeadBytes = 3 * D * sizeof(T);   // one head's slices inside a row
    const uint32_t tab_addr = __builtin_amdgcn_readfirstlane(lds_address(tab));
    const uint32_t row_bytes = kRowBytes;
    float half_rows[ND], upper[ND];
    uint32_t base_off[ND];
    {
        // rows of every axis table: kernel arguments, or (sizes_dev) read from the caller's device tensor of table
        // sizes, which the host has not seen - clipped so that every axis keeps a row inside the head's table
        int run = 0;
#pragma unroll
        for (int n = 0; n < ND; ++n) {
            int rows = a.rows[n], first = a.base[n];
            if (a.sizes_dev) {
                rows = __builtin_amdgcn_readfirstlane(a.sizes_dev[n]) / HD;
                rows = max(1, min(rows, a.total_rows - run - (ND - 1 - n)));
                first = run;
                run += rows;
            }
            half_rows[n] = static_cast<float>(rows / 2);
            upper[n] = crse_upper(rows);
            // LDS byte address of the axis table's first row
            base_off[n] = __builtin_amdgcn_readfirstlane(tab_addr + first * kRowBytes);
        }
    }

    int queue = xcd_id() % kQueues;
    int tried = 0;       // queues found empty so far
    int drawn = 0;       // ticket of the next unit
    if (lane == 0) drawn = atomicAdd(counters + queue * kCounterStride, 1);
    for (;;) {
        int unit = __builtin_amdgcn_readfirstlane(drawn) * kQueues + queue;
        while (unit >= total_units && ++tried < kQueues) {
            queue = (queue + 1) % kQueues;
            if (lane == 0) drawn = atomicAdd(counters + queue * kCounterStride, 1);
            unit = __builtin_amdgcn_readfirstlane(drawn) * kQueues + queue;
        }
        if (unit >= total_units) break;
        // The unit: 64 >> gshift queries (consecutive in the sorted numbering of their class), each on 2^gshift
        // adjacent lanes that take alternate keys.  The queries lie in at most 64 consecutive entries from the
        // unit's first one; each lane reads one entry and finds its own (the last entry of the class that starts at
        // or before its query) by a search across the lanes.
        const int4 info = unit_info[unit];
        const int first = __builtin_amdgcn_readfirstlane(info.x);
        const int gshift = __builtin_amdgcn_readfirstlane(info.y);
        const int queries = __builtin_amdgcn_readfirstlane(info.w);
        const int sub = lane & ((1 << gshift) - 1);
        const bool own_valid = (lane >> gshift) < queries;
        const int query = __builtin_amdgcn_readfirstlane(info.z) + min(lane >> gshift, queries - 1);   // lanes past the end repeat the last one
        const int4 seen = entries[first + lane];
        const int seen_from = seen.w == __builtin_amdgcn_readfirstlane(seen.w) ? seen.x : 0x7fffffff;   // the next class restarts at 0
        int at = 0;
#pragma unroll
        for (int half = 32; half > 0; half >>= 1)
            if (__shfl(seen_from, at + half) <= query) at += half;
        const int n_w = __shfl(seen.y, at), s0 = __shfl(seen.z, at);
        const int own_pos = s0 + (query - __shfl(seen.x, at));
        const int own_row = kSorted ? own_pos : a.n2n[own_pos];
        // the longest lane of the unit (entries are sorted by steps, but windows beyond the longest bin are not)
        int max_steps = (n_w + (1 << gshift) - 1) >> gshift;
#pragma unroll
        for (int other = 32; other > 0; other >>= 1) max_steps = max(max_steps, __shfl_xor(max_steps, other));
        max_steps = __builtin_amdgcn_readfirstlane(max_steps);
        // the lane's keys: sub, sub + 2^gshift, ... of the window's n_k
        const int n_k = n_w;
        const int k0 = s0;
        const int grp = sub;

        Slice<T, D> qv[HP];
        float ci[ND], acc[HP][D], m[HP], top[HP], l[HP];
#pragma unroll
        for (int hh = 0; hh < HP; ++hh) {
            qv[hh].load(gq + static_cast<int64_t>(own_row) * a.row_stride + (h + hh) * D);
#pragma unroll
            for (int c = 0; c < D; ++c) acc[hh][c] = 0.0f;
            m[hh] = top[hh] = -INFINITY;
            l[hh] = 0.0f;
        }
#pragma unroll
        for (int n = 0; n < ND; ++n) ci[n] = a.n_coords[static_cast<int64_t>(own_pos) * ND + n];

        // kKeys streamed keys per iteration: their loads and dependent chains interleave, which hides the
        // LDS and cache round trips a single chain would wait out one after the other
        int row_next[kKeys];
#pragma unroll
        for (int u = 0; u < kKeys; ++u) row_next[u] = kSorted ? 0 : a.n2n[k0 + min((u << gshift) + grp, n_k - 1)];
        for (int it = 0; it < max_steps; it += kKeys) {
            // the next unit's ticket is drawn during the last iteration: the atomic's round trip overlaps that
            // work, and a unit is not held back (out of reach of idle wavefronts) for longer than one step
            if (it + kKeys >= max_steps && lane == 0) drawn = atomicAdd(counters + queue * kCounterStride, 1);
            Slice<T, D> kv[kKeys][HP], v_in[kKeys][HP];
            float logit[kKeys][HP];
            uint32_t off[kKeys][ND];
            bool valid[kKeys];
#pragma unroll
            for (int u = 0; u < kKeys; ++u) {
                const int st = ((it + u) << gshift) + grp;
                valid[u] = st < n_k;
                const int st_pos = k0 + min(st, n_k - 1);
                const int st_row = kSorted ? st_pos : row_next[u];
                if (!kSorted) row_next[u] = a.n2n[k0 + min(st + (kKeys << gshift), n_k - 1)];
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
            if constexpr (!kLazy) {
                // online softmax: the running maximum moves with every key that raises it
                if (valid[0]) {   // the lowest key of the iteration; lanes whose block has ended sit the step out
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
            } else {
                // Online softmax against a reference exponent m that follows the running maximum lazily: it moves
                // (and the sums are rescaled) only when the lane's logit exceeds it by more than kSlack, which
                // after the first keys of a unit is rare, so most steps skip the rescaling of l and the D outputs;
                // weights stay below e^kSlack.  `top` is the true running maximum.
                float hi[HP];
                bool moved = false;
#pragma unroll
                for (int hh = 0; hh < HP; ++hh) {
                    hi[hh] = logit[0][hh];
#pragma unroll
                    for (int u = 1; u < kKeys; ++u) {
                        logit[u][hh] = valid[u] ? logit[u][hh] : -INFINITY;
                        hi[hh] = fmaxf(hi[hh], logit[u][hh]);
                    }
                    moved = moved || hi[hh] > m[hh] + kSlack;
                }
                // each lane decides for itself, so the bits of a query's result do not depend on which other queries
                // share its wavefront
                if (valid[0] && moved) {
#pragma unroll
                    for (int hh = 0; hh < HP; ++hh) {
                        const float m_new = fmaxf(m[hh], hi[hh]);
                        const float scale = __expf(m[hh] - m_new);   // exp(-inf) = 0 on the first key
                        l[hh] *= scale;
#pragma unroll
                        for (int c = 0; c < D; ++c) acc[hh][c] *= scale;
                        m[hh] = m_new;
                    }
                }
                if (valid[0]) {   // the lowest key of the iteration; lanes whose block has ended sit the step out
#pragma unroll
                    for (int hh = 0; hh < HP; ++hh) {
                        top[hh] = fmaxf(top[hh], hi[hh]);
#pragma unroll
                        for (int u = 0; u < kKeys; ++u) {
                            const float p = __expf(logit[u][hh] - m[hh]);
                            l[hh] += p;
                            v_in[u][hh].fma_to(acc[hh], p);
                            // The pair's value-table rows are added three at a time in packed fp16, two channels per
                            // instruction, before they enter the fp32 sums: 56 instructions per pair and head at
                            // head_dim 8 instead of 80 mixed-precision FMAs.  Groups of three keep the fp16 roundings
                            // at two per element, on sums of three rows (one chain over all nine rows saves eight
                            // more instructions, measured 13 % slower - eight dependent adds - and used up the 2e-3
                            // error budget on tables of magnitude 0.1); adding the value here as well measured -4 %
                            // for the same reason not to.  The reference's half path adds all rows and the value in
                            // half2 (self_attn_aio_fwd.cu:147).
                            constexpr int kGroup = 3;
#pragma unroll
                            for (int n0 = 0; n0 < ND; n0 += kGroup) {
                                Slice<T, D> tv_sum;
                                tv_sum.load_lds(off[u][n0] + hh * kHeadBytes + 2 * D * sizeof(T));
#pragma unroll
                                for (int g = 1; g < kGroup && n0 + g < ND; ++g) {
                                    Slice<T, D> tv_r;
                                    tv_r.load_lds(off[u][n0 + g] + hh * kHeadBytes + 2 * D * sizeof(T));
                                    tv_sum.add(tv_r);
                                }
                                tv_sum.fma_to(acc[hh], p);
                            }
                        }
                    }
                }
            }
        }
        // from the reference exponent to the true maximum (lanes that saw no key: both are -inf, nothing to scale)
        if constexpr (kLazy) {
#pragma unroll
            for (int hh = 0; hh < HP; ++hh) {
                const float scale = top[hh] == -INFINITY ? 1.0f : __expf(m[hh] - top[hh]);
                l[hh] *= scale;
#pragma unroll
                for (int c = 0; c < D; ++c) acc[hh][c] *= scale;
                m[hh] = top[hh];
            }
        }
#pragma unroll
        for (int hh = 0; hh < HP; ++hh) {
            // lanes that share a query saw alternate keys: merge their softmax states
            for (int other = 1; other < (1 << gshift); other <<= 1) {
                const float m_o = __shfl_xor(m[hh], other), l_o = __shfl_xor(l[hh], other);
                const float m_all = fmaxf(m[hh], m_o);
                const float w_me = (m[hh] == -INFINITY) ? 0.0f : __expf(m[hh] - m_all);
                const float w_ot = (m_o == -INFINITY) ? 0.0f : __expf(m_o - m_all);
                l[hh] = l[hh] * w_me + l_o * w_ot;
#pragma unroll
                for (int c = 0; c < D; ++c) acc[hh][c] = acc[hh][c] * w_me + __shfl_xor(acc[hh][c], other) * w_ot;
                m[hh] = m_all;
            }
            if (own_valid && sub == 0) {
                const float inv = 1.0f / l[hh];
#pragma unroll
                for (int c = 0; c < D; ++c) acc[hh][c] *= inv;
                store_row<D>(static_cast<T *>(a.out) + static_cast<int64_t>(own_row) * HD + (h + hh) * D, acc[hh]);
                if (a.out_max) a.out_max[static_cast<int64_t>(own_row) * H + h + hh] = m[hh];
                if (a.out_sum) a.out_sum[static_cast<int64_t>(own_row) * H + h + hh] = l[hh];
            }
        }
    }
    // The work list can serve further launches (a plan kept by the caller): the last wavefront of the launch to
    // leave its loop - by then no wavefront draws tickets any more - puts every queue counter back to zero.  The
    // exits are counted in three levels (workgroup in LDS, one of kQueues cache lines, all lines), so that no
    // cache line sees more than a few hundred of these atomics.
    if (lane == 0 && atomicAdd(&group_exited, 1) == kThreads / 64 - 1) {
        __threadfence();
        int *total = static_cast<int *>(a.workspace) + ws_total_offset(H) / sizeof(int);
        const int groups = static_cast<int>(gridDim.x), line = static_cast<int>(blockIdx.x) % kQueues;
        const int on_line = (groups - line + kQueues - 1) / kQueues;
        int *line_counter = total + (1 + line) * kCounterStride;
        if (atomicAdd(line_counter, 1) == on_line - 1) {
            *line_counter = 0;
            if (atomicAdd(total + 1, 1) == min(groups, kQueues) - 1) {
                total[1] = 0;
                int *all_counters = static_cast<int *>(a.workspace);
                for (int t = 0; t < H * kQueues; ++t) all_counters[t * kCounterStride] = 0;
                __threadfence();
            }
        }
    }
}

// ---- backward: the pair sweeps ------------------------------------------------------------------------------
// dq, dk, dv of the attention backward (Swin3D/src/attn/self_attn_aio_bwd.cu:197-509 adds every term with a global
// atomic) on the forward's work list: a lane owns one voxel of some window and streams the window's other side,
//   kKeyOwned = false: lane = query i, streams the keys j:    dq_i += dL (k_j + Tq(i,j))
//   kKeyOwned = true:  lane = key j, streams the queries i:   dk_j += dL (q_i + Tk(i,j)),  dv_j += P dout_i
// with P = exp(L - max_i) / sum_i from the forward's saved statistics, dP = dout_i . (v_j + Tv(i,j)) and
// dL = P (dP - dout_i . o_i).  Every gradient row has one owner and is stored once.  The sweeps also leave dL and
// P of every (pair, head) for the table-gradient kernels, each in the order its reader wants: the key-owned sweep
// writes (dL, P) at [head][pairs before the window + i n + j], the query-owned sweep dL at [.. + j n + i] - in both
// the lanes of a window write consecutive addresses.
template <typename T, int D, int HP> __host__ __device__ constexpr int bwd_pair_threads() { return 256; }

// TF is the type the feature rows are stored in (q, k, v, dout and the gradients dq, dk, dv); T the type of the
// tables and of the arithmetic.  TF = __half with T = float serves an fp16 forward whose backward runs in fp32: the
// rows are widened as they are loaded and the gradients rounded as they are stored, the arithmetic is that of T = TF
// = float on widened copies.
template <typename T, typename TF, int D, int ND, int HP, bool kKeyOwned, bool kShared>
// Wavefronts per SIMD, by register cap.  fp16 at head_dim 8: four (128 registers; -1 to -2 % against the three that
// the key-owned sweep's 133 registers allow).  fp16 at head_dim 16 and fp32 at head_dim 8: three (168 registers, 3 to
// 20 of them spilled: the backward of the window-7 layer with 6 heads of 16 2.05 -> 1.99 ms, of the headline layer
// in fp32 2.28 -> 2.05 ms).  fp32 at head_dim 16: two - uncapped it takes 286 registers and runs one wavefront per
// SIMD (6-head window-7 layer 3.16 ms; capped at 256 with 24 spilled 2.89).
__global__ __launch_bounds__((bwd_pair_threads<T, D, HP>()), (sizeof(T) == 2 ? (D == 8 ? 4 : 3) : (D == 8 ? 3 : 2))) void attn_bwd_pairs_kernel(BwdPairArgs b)
{
    const AttnArgs &a = b.f;
    constexpr int kThreads = bwd_pair_threads<T, D, HP>();
    extern __shared__ __align__(16) float smem[];
    __shared__ __align__(16) int group_exit_counter[4];
    int &group_exited = group_exit_counter[0];
    if (threadIdx.x == 0) group_exited = 0;
    const int H = a.H;
    const int HD = H * D;
    const int hg = a.spread_groups ? blockIdx.x % (H / HP) : (blockIdx.x / kQueues) % (H / HP);
    const int h = hg * HP;
    constexpr int kRowStride = table_row_stride_heads<T, D, HP>();
    T *tab = reinterpret_cast<T *>(smem);
    {
        const T *gq = static_cast<const T *>(a.table_q);
        const T *gk = static_cast<const T *>(a.table_k);
        const T *gv = static_cast<const T *>(a.table_v);
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
    const TF *gq = static_cast<const TF *>(a.q);
    const TF *gk = static_cast<const TF *>(a.k);
    const TF *gv = static_cast<const TF *>(a.v);
    const TF *ggo = static_cast<const TF *>(b.dout);
    const char *ws = static_cast<const char *>(a.workspace);
    const int4 *unit_info = reinterpret_cast<const int4 *>(ws + ws_units_offset(H));
    const int4 *entries = reinterpret_cast<const int4 *>(ws + ws_entries_offset(H, a.N));
    const int total_units = __builtin_amdgcn_readfirstlane(reinterpret_cast<const int *>(ws + ws_total_offset(H))[0]);
    int *counters = static_cast<int *>(a.workspace) + hg * kQueues * kCounterStride;
    constexpr int kRowBytes = kRowStride * static_cast<int>(sizeof(T));
    constexpr uint32_t kHeadBytes = 3 * D * sizeof(T);
    const uint32_t tab_addr = __builtin_amdgcn_readfirstlane(lds_address(tab));
    const uint32_t row_bytes = kRowBytes;
    float half_rows[ND], upper[ND];
    uint32_t base_off[ND];
#pragma unroll
    for (int n = 0; n < ND; ++n) {
        half_rows[n] = static_cast<float>(a.rows[n] / 2);
        upper[n] = crse_upper(a.rows[n]);
        base_off[n] = __builtin_amdgcn_readfirstlane(tab_addr + a.base[n] * kRowBytes);
    }
    // the one table-row sum that enters the owned gradient as a vector (Tq for dq_i, Tk for dk_j) sits behind the
    // q-side slice in the query-owned sweep and behind the k-side slice in the key-owned one
    // kShared: the key-owned sweep reads dL and P from records that the query-owned sweep, which ran before it,
    // wrote beside its own
    constexpr bool kRead = kKeyOwned && kShared;
    constexpr bool kWriteBoth = !kKeyOwned && kShared;

    int queue = xcd_id() % kQueues;
    int tried = 0;
    int drawn = 0;
    if (lane == 0) drawn = atomicAdd(counters + queue * kCounterStride, 1);
    for (;;) {
        int unit = __builtin_amdgcn_readfirstlane(drawn) * kQueues + queue;
        while (unit >= total_units && ++tried < kQueues) {
            queue = (queue + 1) % kQueues;
            if (lane == 0) drawn = atomicAdd(counters + queue * kCounterStride, 1);
            unit = __builtin_amdgcn_readfirstlane(drawn) * kQueues + queue;
        }
        if (unit >= total_units) break;
        // the unit, as in the forward sweep: 64 >> gshift owned voxels, each on 2^gshift adjacent lanes that take
        // alternate elements of the streamed side
        const int4 info = unit_info[unit];
        const int first = __builtin_amdgcn_readfirstlane(info.x);
        const int gshift = __builtin_amdgcn_readfirstlane(info.y);
        const int owners = __builtin_amdgcn_readfirstlane(info.w);
        const int sub = lane & ((1 << gshift) - 1);
        const bool own_valid = (lane >> gshift) < owners;
        const int slot = __builtin_amdgcn_readfirstlane(info.z) + min(lane >> gshift, owners - 1);
        const int4 seen = entries[first + lane];
        const int seen_from = seen.w == __builtin_amdgcn_readfirstlane(seen.w) ? seen.x : 0x7fffffff;
        int at = 0;
#pragma unroll
        for (int half = 32; half > 0; half >>= 1)
            if (__shfl(seen_from, at + half) <= slot) at += half;
        const int n_w = __shfl(seen.y, at), s0 = __shfl(seen.z, at);
        const int own_in = slot - __shfl(seen.x, at);     // position inside the window
        const int own_pos = s0 + own_in;
        const int own_row = a.n2n[own_pos];
        int max_steps = (n_w + (1 << gshift) - 1) >> gshift;
#pragma unroll
        for (int other = 32; other > 0; other >>= 1) max_steps = max(max_steps, __shfl_xor(max_steps, other));
        max_steps = __builtin_amdgcn_readfirstlane(max_steps);
        // pairs before the window; a window that does not fit the caller's pair store is skipped as a whole
        const int64_t pair_base = b.pos_base[s0];
        const bool fits = pair_base + static_cast<int64_t>(n_w) * n_w <= b.pairs;

        Slice<T, D> own_x[HP], own_y[HP];     // q_i, dout_i  or  k_j, v_j
        float own_m[HP], own_inv[HP], own_delta[HP];
        float ci[ND], res_x[HP][D], res_y[kKeyOwned ? HP : 1][D];
#pragma unroll
        for (int hh = 0; hh < HP; ++hh) {
            const int64_t at_row = static_cast<int64_t>(own_row) * HD + (h + hh) * D;
            if constexpr (kKeyOwned) {
                own_x[hh].load(gk + at_row);
                if constexpr (!kRead) own_y[hh].load(gv + at_row);
            } else {
                own_x[hh].load(gq + at_row);
                own_y[hh].load(ggo + at_row);
                own_m[hh] = b.stat_max[static_cast<int64_t>(own_row) * H + h + hh];
                own_inv[hh] = 1.0f / b.stat_sum[static_cast<int64_t>(own_row) * H + h + hh];
                own_delta[hh] = b.delta[static_cast<int64_t>(own_row) * H + h + hh];
            }
#pragma unroll
            for (int c = 0; c < D; ++c) res_x[hh][c] = 0.0f;
            if constexpr (kKeyOwned) {
#pragma unroll
                for (int c = 0; c < D; ++c) res_y[hh][c] = 0.0f;
            }
        }
#pragma unroll
        for (int n = 0; n < ND; ++n) ci[n] = a.n_coords[static_cast<int64_t>(own_pos) * ND + n];

        int row_next = a.n2n[s0 + min(sub, n_w - 1)];
        for (int it = 0; it < max_steps; ++it) {
            if (it + 1 >= max_steps && lane == 0) drawn = atomicAdd(counters + queue * kCounterStride, 1);
            const int st = (it << gshift) + sub;
            const bool valid = st < n_w && own_valid && fits;
            const int st_in = min(st, n_w - 1);
            const int st_pos = s0 + st_in;
            const int st_row = row_next;
            row_next = a.n2n[s0 + min(st + (1 << gshift), n_w - 1)];
            Slice<T, D> st_x[HP], st_y[HP];   // k_j, v_j  or  q_i, dout_i
            float st_m[HP], st_inv[HP], st_delta[HP];
#pragma unroll
            for (int hh = 0; hh < HP; ++hh) {
                const int64_t at_row = static_cast<int64_t>(st_row) * HD + (h + hh) * D;
                if constexpr (kRead) {
                    st_x[hh].load(gq + at_row);
                    st_y[hh].load(ggo + at_row);
                    st_m[hh] = st_inv[hh] = st_delta[hh] = 0.0f;
                } else if constexpr (kKeyOwned) {
                    st_x[hh].load(gq + at_row);
                    st_y[hh].load(ggo + at_row);
                    st_m[hh] = b.stat_max[static_cast<int64_t>(st_row) * H + h + hh];
                    st_inv[hh] = b.stat_sum[static_cast<int64_t>(st_row) * H + h + hh];
                    st_delta[hh] = b.delta[static_cast<int64_t>(st_row) * H + h + hh];
                } else {
                    st_x[hh].load(gk + at_row);
                    st_y[hh].load(gv + at_row);
                }
            }
            uint32_t off[ND];
            {
                float cj[ND];
#pragma unroll
                for (int n = 0; n < ND; ++n) cj[n] = a.n_coords[static_cast<int64_t>(st_pos) * ND + n];
#pragma unroll
                for (int n = 0; n < ND; ++n) {
                    // row_n(i, j): the query's coordinate first
                    const float c_i = kKeyOwned ? cj[n] : ci[n], c_j = kKeyOwned ? ci[n] : cj[n];
                    off[n] = mad_u24(static_cast<uint32_t>(crse_row(c_i, c_j, half_rows[n], upper[n])), row_bytes, base_off[n]);
                }
            }
#pragma unroll
            for (int hh = 0; hh < HP; ++hh) {
                const Slice<T, D> &qv = kKeyOwned ? st_x[hh] : own_x[hh];
                const Slice<T, D> &kv = kKeyOwned ? own_x[hh] : st_x[hh];
                const Slice<T, D> &vv = kKeyOwned ? own_y[hh] : st_y[hh];
                const Slice<T, D> &gov = kKeyOwned ? st_y[hh] : own_y[hh];
                const int64_t head_at = static_cast<int64_t>(h + hh) * b.pairs + pair_base;
                float2 rec = make_float2(0.0f, 0.0f);
                if constexpr (kRead) {
                    if (valid) rec = b.pd[head_at + static_cast<int64_t>(st_in) * n_w + own_in];
                }
                float logit = 0.0f, dp = 0.0f;
                if constexpr (!kRead) {
                    logit = qv.dot(kv, 0.0f);
                    dp = gov.dot(vv, 0.0f);
                }
                // sums of three rows of the table that enters the owned gradient as a vector (packed fp16 adds for
                // fp16 I/O, as the forward adds its value-table rows)
                // (fp32: one sum of all rows - plain adds, no packing to gain, and two sums fewer to hold)
                constexpr int kGroup = sizeof(T) == 4 ? ND : 3;
                Slice<T, D> vec_sum[(ND + kGroup - 1) / kGroup];
#pragma unroll
                for (int n = 0; n < ND; ++n) {
                    Slice<T, D> tq_r, tk_r, tv_r;
                    tk_r.load_lds(off[n] + hh * kHeadBytes + D * sizeof(T));
                    if constexpr (!kRead) {
                        tq_r.load_lds(off[n] + hh * kHeadBytes);
                        tv_r.load_lds(off[n] + hh * kHeadBytes + 2 * D * sizeof(T));
                        if (Slice<T, D>::kChainLogit) logit = kv.dot(tk_r, qv.dot(tq_r, logit));
                        else logit += kv.dot(tk_r, qv.dot(tq_r, 0.0f));
                        if (Slice<T, D>::kChainLogit) dp = gov.dot(tv_r, dp);
                        else dp += gov.dot(tv_r, 0.0f);
                    }
                    const Slice<T, D> &vec_r = kKeyOwned ? tk_r : tq_r;
                    if (n % kGroup == 0) vec_sum[n / kGroup] = vec_r;
                    else vec_sum[n / kGroup].add(vec_r);
                }
                const float m_i = kKeyOwned ? st_m[hh] : own_m[hh];
                const float inv_i = kKeyOwned ? 1.0f / st_inv[hh] : own_inv[hh];
                const float delta_i = kKeyOwned ? st_delta[hh] : own_delta[hh];
                const float p = kRead ? rec.y : valid ? __expf(logit - m_i) * inv_i : 0.0f;
                const float dl = kRead ? rec.x : p * (dp - delta_i);
                // dq_i += dL (k_j + Tq)   or   dk_j += dL (q_i + Tk)
                st_x[hh].fma_to(res_x[hh], dl);
#pragma unroll
                for (int g = 0; g < (ND + kGroup - 1) / kGroup; ++g) vec_sum[g].fma_to(res_x[hh], dl);
                if constexpr (kKeyOwned) st_y[hh].fma_to(res_y[hh], p);     // dv_j += P dout_i
                if (valid) {
                    if constexpr (kRead) {
                        // nothing to leave: the records are the query-owned sweep's
                    } else if constexpr (kKeyOwned) {
                        b.pd[head_at + static_cast<int64_t>(st_in) * n_w + own_in] = make_float2(dl, p);
                    } else {
                        b.dl_t[head_at + static_cast<int64_t>(st_in) * n_w + own_in] = dl;
                        // (dL, P) at [i][j] as well: a lane's records of successive steps are consecutive, the lanes'
                        // n records apart
                        if constexpr (kWriteBoth) b.pd[head_at + static_cast<int64_t>(own_in) * n_w + st_in] = make_float2(dl, p);
                    }
                }
            }
        }
#pragma unroll
        for (int hh = 0; hh < HP; ++hh) {
            // lanes that share an owned voxel saw alternate elements of the stream
            for (int other = 1; other < (1 << gshift); other <<= 1) {
#pragma unroll
                for (int c = 0; c < D; ++c) res_x[hh][c] += __shfl_xor(res_x[hh][c], other);
                if constexpr (kKeyOwned) {
#pragma unroll
                    for (int c = 0; c < D; ++c) res_y[hh][c] += __shfl_xor(res_y[hh][c], other);
                }
            }
            if (own_valid && sub == 0) {
                // a window beyond the caller's pair store was skipped: its rows say so
                if (!fits) {
#pragma unroll
                    for (int c = 0; c < D; ++c) res_x[hh][c] = __int_as_float(0x7fc00000);
                    if constexpr (kKeyOwned) {
#pragma unroll
                        for (int c = 0; c < D; ++c) res_y[hh][c] = __int_as_float(0x7fc00000);
                    }
                }
                const int64_t at_row = static_cast<int64_t>(own_row) * HD + (h + hh) * D;
                if constexpr (kKeyOwned) {
                    store_row<D>(static_cast<TF *>(b.dk) + at_row, res_x[hh]);
                    store_row<D>(static_cast<TF *>(b.dv) + at_row, res_y[hh]);
                } else {
                    store_row<D>(static_cast<TF *>(b.dq) + at_row, res_x[hh]);
                }
            }
        }
    }
    // the last wavefront of the launch to leave puts the queue counters back to zero (as in the forward sweep):
    // the next sweep runs on the same list
    if (lane == 0 && atomicAdd(&group_exited, 1) == kThreads / 64 - 1) {
        __threadfence();
        int *total = static_cast<int *>(a.workspace) + ws_total_offset(H) / sizeof(int);
        const int groups = static_cast<int>(gridDim.x), line = static_cast<int>(blockIdx.x) % kQueues;
        const int on_line = (groups - line + kQueues - 1) / kQueues;
        int *line_counter = total + (1 + line) * kCounterStride;
        if (atomicAdd(line_counter, 1) == on_line - 1) {
            *line_counter = 0;
            if (atomicAdd(total + 1, 1) == min(groups, kQueues) - 1) {
                total[1] = 0;
                int *all_counters = static_cast<int *>(a.workspace);
                for (int t = 0; t < H * kQueues; ++t) all_counters[t * kCounterStride] = 0;
                __threadfence();
            }
        }
    }
}

template <typename T, int D, int ND, int HP, bool kSorted>
int launch_sweep_heads(const AttnArgs &a, hipStream_t stream, int what)
{
    const size_t lds = align_up(sizeof(T) * static_cast<size_t>(a.total_rows) * table_row_stride_heads<T, D, HP>(), 16);
    if (lds > 160 * 1024)
        return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd: %d table rows x D=%d need %zu B of LDS (> 160 KiB)",
                    a.total_rows, D, lds);
    auto kernel = attn_fwd_sweep_kernel<T, D, ND, HP, kSorted>;
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), lds)) return rc;
    // A workgroup serves one head group for its whole life: as many workgroups per CU as registers and LDS allow.
    // They come in whole sets of (XCDs x head groups) - runs of eight consecutive workgroups, one per XCD, serve one
    // head group, so every XCD serves every head group and the rows of a unit reach one L2 - unless whole sets
    // would leave more than a tenth of the slots empty (many head groups): then the head groups take the workgroups
    // in turn and every slot is used, at the price of that locality (the kernel is not bound by memory traffic).
    int per_cu = groups_per_cu<T, D, HP>();
    while (per_cu > 1 && per_cu * lds > 160 * 1024) --per_cu;
    const int groups = a.H / HP;
    const int cus = device_cus();
    const int slots = per_cu * cus;
    const int set = kQueues * groups;
    const int whole = (slots / set) * set;
    AttnArgs b = a;
    b.spread_groups = 10 * whole < 9 * slots;
    const int grid = b.spread_groups ? (slots >= groups ? slots / groups * groups : groups) : whole;
    constexpr int kThreads = group_threads<T, D, HP>();
    b.target_items = grid / groups * (kThreads / 64);   // wavefronts that serve one head group
    b.block_shift = target_shift_for(a.N, a.W, b.target_items);
    const int64_t list_want = (a.W + kListThreads - 1) / kListThreads;
    const dim3 list_grid(static_cast<unsigned>(list_want < 1 ? 1 : (list_want > kListGroups ? kListGroups : list_want)));
    if (what & 1) {
        hipLaunchKernelGGL(sweep_count_kernel, list_grid, dim3(kListThreads), 0, stream, b);
        hipLaunchKernelGGL(sweep_place_kernel, list_grid, dim3(kListThreads), 0, stream, b);
        S3D_HIP_CHECK(hipGetLastError());
    }
    if (what & 2) {
        hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(kThreads), lds, stream, b);
        S3D_HIP_CHECK(hipGetLastError());
    }
    return S3D_OK;
}

template <typename T, int D, int ND>
int launch_sweep(const AttnArgs &a, hipStream_t stream, int what)
{
    // Two heads per wavefront where the registers allow it (fp16) and the heads pair up: the cRSE rows and LDS
    // addresses of a pair are spent once for both.  At head_dim 16 that means one workgroup of twelve wavefronts per
    // CU (75 KB of tables): it measured -10 % at 6 heads.
    if constexpr (sizeof(T) == 2 && D <= 16) {
        // three heads where they go in threes and fit (head_dim 8: 168 registers, three workgroups of 45 KB of
        // tables per CU): -2 % against pairs at 6 and 12 heads
        if constexpr (D == 8) {
            if (a.H % 3 == 0)
                return a.n2n ? launch_sweep_heads<T, D, ND, 3, false>(a, stream, what)
                             : launch_sweep_heads<T, D, ND, 3, true>(a, stream, what);
        }
        if (a.H % 2 == 0)
            return a.n2n ? launch_sweep_heads<T, D, ND, 2, false>(a, stream, what)
                         : launch_sweep_heads<T, D, ND, 2, true>(a, stream, what);
    }
    // fp32 at head_dim 8: pairs of heads as well
    if constexpr (sizeof(T) == 4 && D == 8) {
        if (a.H % 2 == 0)
            return a.n2n ? launch_sweep_heads<T, D, ND, 2, false>(a, stream, what)
                         : launch_sweep_heads<T, D, ND, 2, true>(a, stream, what);
    }
    return a.n2n ? launch_sweep_heads<T, D, ND, 1, false>(a, stream, what)
                 : launch_sweep_heads<T, D, ND, 1, true>(a, stream, what);
}

template <typename T>
int dispatch_shape(const AttnArgs &a, hipStream_t stream, int what)
{
#define S3D_CASE(DD, NN) \
    if (a.D == DD && a.nd == NN) return launch_sweep<T, DD, NN>(a, stream, what);
    S3D_CASE(8, 3) S3D_CASE(8, 6) S3D_CASE(8, 9)
    S3D_CASE(16, 3) S3D_CASE(16, 6) S3D_CASE(16, 9)
    S3D_CASE(32, 3) S3D_CASE(32, 6) S3D_CASE(32, 9)
#undef S3D_CASE
    return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd: unsupported head_dim %d / cRSE axes %d "
                "(head_dim in {8,16,32}, axes in {3,6,9})", a.D, a.nd);
}

}  // namespace

namespace {

template <typename T, typename TF, int D, int ND, int HP, bool kShared>
int launch_bwd_pairs_heads(const BwdPairArgs &b0, hipStream_t stream)
{
    const AttnArgs &a = b0.f;
    const size_t lds = align_up(sizeof(T) * static_cast<size_t>(a.total_rows) * table_row_stride_heads<T, D, HP>(), 16);
    if (lds > 160 * 1024)
        return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_bwd: %d table rows x D=%d need %zu B of LDS (> 160 KiB)",
                    a.total_rows, D, lds);
    auto q_sweep = attn_bwd_pairs_kernel<T, TF, D, ND, HP, false, kShared>;
    auto k_sweep = attn_bwd_pairs_kernel<T, TF, D, ND, HP, true, kShared>;
    constexpr int kThreads = bwd_pair_threads<T, D, HP>();
    int per_cu = 1;
    for (auto kernel : {q_sweep, k_sweep}) {
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), lds)) return rc;
    }
    {
        // workgroups per CU: what the registers of the heavier sweep and the tables in LDS allow
        int fit_q = 0, fit_k = 0;
        S3D_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&fit_q, reinterpret_cast<const void *>(q_sweep), kThreads, lds));
        S3D_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&fit_k, reinterpret_cast<const void *>(k_sweep), kThreads, lds));
        per_cu = fit_q < fit_k ? fit_q : fit_k;
        if (per_cu < 1) per_cu = 1;
    }
    const int groups = a.H / HP;
    const int cus = device_cus();
    const int slots = per_cu * cus;
    const int set = kQueues * groups;
    const int whole = (slots / set) * set;
    BwdPairArgs b = b0;
    b.f.spread_groups = 10 * whole < 9 * slots;
    const int grid = b.f.spread_groups ? (slots >= groups ? slots / groups * groups : groups) : whole;
    b.f.target_items = grid / groups * (kThreads / 64);
    b.f.block_shift = target_shift_for(a.N, a.W, b.f.target_items);
    const int64_t list_want = (a.W + kListThreads - 1) / kListThreads;
    const dim3 list_grid(static_cast<unsigned>(list_want < 1 ? 1 : (list_want > kListGroups ? kListGroups : list_want)));
    hipLaunchKernelGGL(sweep_count_kernel, list_grid, dim3(kListThreads), 0, stream, b.f);
    hipLaunchKernelGGL(sweep_place_kernel, list_grid, dim3(kListThreads), 0, stream, b.f);
    S3D_HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL(q_sweep, dim3(static_cast<unsigned>(grid)), dim3(kThreads), lds, stream, b);
    hipLaunchKernelGGL(k_sweep, dim3(static_cast<unsigned>(grid)), dim3(kThreads), lds, stream, b);
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}

template <typename T, typename TF, int D, int ND>
int launch_bwd_pairs(const BwdPairArgs &b, hipStream_t stream)
{
    // one head per wavefront: with two (fp16, head_dim 8) the key-owned sweep needs more than 256 registers and the
    // pair of sweeps measured 0.3 ms slower at the 6-head layer
    //
    // Who computes dL and P for the key-owned sweep.  Either it does, as the query-owned sweep does (the logits, dP,
    // the exponential: 125 of its 280 instructions per pair and head), or the query-owned sweep, which runs first,
    // leaves its values at [i][j] as well and the key-owned sweep reads them.  That second copy is written with the
    // lanes n records apart (a lane's own records of successive steps are consecutive); windows of more than 64
    // voxels, whose queries have several lanes each on adjacent records, write it in longer runs.  Measured, whole
    // backward, own values / shared: 1.76 / 1.87 ms on 26-voxel windows (6 heads of 8), 2.24 / 2.12 and 2.33 / 2.25
    // ms on the window-7 layers of 57 voxels a window (6 heads of 16, 12 of 8).  Shared where the mean window has
    // more than 32 voxels.
    if (b.f.N > 32 * b.f.W) return launch_bwd_pairs_heads<T, TF, D, ND, 1, true>(b, stream);
    return launch_bwd_pairs_heads<T, TF, D, ND, 1, false>(b, stream);
}

template <typename T, typename TF>
int dispatch_bwd_pairs(const BwdPairArgs &b, hipStream_t stream)
{
#define S3D_CASE(DD, NN) \
    if (b.f.D == DD && b.f.nd == NN) return launch_bwd_pairs<T, TF, DD, NN>(b, stream);
    S3D_CASE(8, 3) S3D_CASE(8, 6) S3D_CASE(8, 9)
    S3D_CASE(16, 3) S3D_CASE(16, 6) S3D_CASE(16, 9)
#undef S3D_CASE
    return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_bwd: unsupported head_dim %d / cRSE axes %d", b.f.D, b.f.nd);
}

}  // namespace

int launch_attn_bwd_pairs(const BwdPairArgs &b, int dtype, hipStream_t stream)
{
    switch (dtype) {
    case S3D_DTYPE_F32: return dispatch_bwd_pairs<float, float>(b, stream);
    case S3D_DTYPE_F16: return dispatch_bwd_pairs<__half, __half>(b, stream);
    case S3D_DTYPE_F32_F16_ROWS: return dispatch_bwd_pairs<float, __half>(b, stream);
    default: return fail(S3D_ERR_BAD_DTYPE, "s3d_attn_bwd: dtype %d (0 = fp32, 1 = fp16, 2 = fp32 on fp16 rows)", dtype);
    }
}

size_t attn_sweep_workspace_bytes(int H, int64_t W, int64_t N)
{
    // queue counters, the totals, one record per unit, the sorted window list and the list builder's notes
    return ws_end_offset(H, W, N);
}

int launch_attn_sweep(const AttnArgs &a, int dtype, hipStream_t stream, int what)
{
    switch (dtype) {
    case S3D_DTYPE_F32: return dispatch_shape<float>(a, stream, what);
    case S3D_DTYPE_F16: return dispatch_shape<__half>(a, stream, what);
    default: return fail(S3D_ERR_BAD_DTYPE, "s3d_attn_fwd: dtype %d (0 = fp32, 1 = fp16)", dtype);
    }
}

}  // namespace s3d
