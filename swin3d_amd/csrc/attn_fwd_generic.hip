// Sparse-voxel windowed self-attention forward with cRSE tables (gfx950): sweep kernel.
//
// Covers every dtype / shape the library accepts on the vector ALU (fp32 arithmetic; fp16 inputs enter through
// packed dot products and mixed-precision FMAs with fp32 accumulation).  A workgroup serves one head (or two)
// for its whole life and keeps the slices of the three relative-signal tables in LDS (loaded once, not once
// per window).  Lane = slot = one query against a block of at most 64 keys of its window: q_i, the running
// maximum, sum and output stay in the lane's registers while the lane streams its own window's keys, one per
// step, so there is no cross-lane reduction, no atomic on data and no O(pairs) index array; the result is
// deterministic.  The slots of all windows, sorted by step count, are packed into units of 64 (the lanes of a
// wavefront carry queries of several small windows); wavefronts draw units from the head's work queues.
// Windows of more than 64 voxels leave one partial result per key block, combined by generic_merge_kernel.
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
constexpr int kChunk = 64;   // slots per unit at most = lanes of a wavefront
constexpr int kListThreads = 256, kListGroups = 128;   // the list builder's workgroups: size, and how many at most
constexpr float kSlack = 10.0f;   // how far a logit may exceed the softmax reference exponent before it moves
constexpr int kMaxBlockSteps = 256;   // the longest key block a launch may choose
// key blocks a window of n voxels is split into when a slot streams at most 2^shift keys, and their even size
__host__ __device__ inline int key_blocks(int n, int shift) { return (n + (1 << shift) - 1) >> shift; }
__host__ __device__ inline int key_block_size(int n, int shift) { const int b = key_blocks(n, shift); return (n + b - 1) / b; }
// The key block length of a launch, 64 << shift.  A window longer than that is split and passes partial results
// through memory (72 bytes per voxel, head and block at head_dim 16, written and read back), so longer blocks
// are better as long as the longest slot stays short against what a wavefront does in the whole launch:
// N^2 / W pairs at least, H heads, over the lanes of about 3072 resident wavefronts.  64 unless two thirds of
// that cover a longer block.
__host__ inline int block_shift_for(int H, int64_t N, int64_t W, int max_window_voxels)
{
    if (N <= 0 || W <= 0) return 6;
    const double steps_per_wave = static_cast<double>(N) * static_cast<double>(N) / static_cast<double>(W) * H / (64.0 * 3072.0);
    int shift = 6;
    while ((1 << shift) < kMaxBlockSteps && (1 << shift) < max_window_voxels && 1.5 * (2 << shift) <= steps_per_wave) ++shift;
    return shift;
}

// byte offsets inside the workspace: the queue counters, the totals (units, split windows, slots), the first
// entry of every unit, the sorted window entries, the placement notes and per-workgroup bin totals of the list
// builder, the list of split windows, the partial results
__host__ __device__ inline size_t ws_round(size_t bytes) { return (bytes + 255) / 256 * 256; }
__host__ __device__ inline size_t ws_total_offset(int H) { return sizeof(int32_t) * static_cast<size_t>(H) * kQueues * kCounterStride; }
__host__ __device__ inline size_t ws_units_offset(int H) { return ws_total_offset(H) + 256; }
// a voxel of a window with b key blocks takes b slots; a unit is at least 16 slots
__host__ __device__ inline size_t ws_max_units(int64_t N, int max_blocks)
{
    return static_cast<size_t>(N > 0 ? N : 0) * max_blocks / (kChunk / 4) + 4;
}
__host__ __device__ inline size_t ws_entries_offset(int H, int64_t N, int max_blocks)
{
    return ws_units_offset(H) + ws_round(sizeof(int32_t) * ws_max_units(N, max_blocks));
}
__host__ __device__ inline size_t ws_place_offset(int H, int64_t W, int64_t N, int max_blocks)
{
    return ws_entries_offset(H, N, max_blocks) + ws_round(sizeof(int4) * (static_cast<size_t>(W > 0 ? W : 0) + kChunk));
}
__host__ __device__ inline size_t ws_bins_offset(int H, int64_t W, int64_t N, int max_blocks)
{
    return ws_place_offset(H, W, N, max_blocks) + ws_round(sizeof(int2) * static_cast<size_t>(W > 0 ? W : 1));
}
__host__ __device__ inline size_t ws_split_offset(int H, int64_t W, int64_t N, int max_blocks)
{
    return ws_bins_offset(H, W, N, max_blocks) + ws_round(sizeof(unsigned long long) * kListGroups * (kMaxBlockSteps + 1));
}
__host__ __device__ inline size_t ws_partials_offset(int H, int64_t W, int64_t N, int max_blocks)
{
    return ws_split_offset(H, W, N, max_blocks) + ws_round(sizeof(int32_t) * static_cast<size_t>(W > 0 ? W : 1));
}

// How the slots of a launch (sorted by steps, longest first) are cut into units.  A unit is one pass of a
// wavefront: 64 slots, or 32 slots whose lanes l and l + 32 share a query and take alternate keys (half the
// steps), or 16 slots in four such groups (a quarter).  The launch ends when the last wavefront ends, so the
// last slots go into the finer units: about two 16-slot units and one 32-slot unit per wavefront of a head
// group (`waves`), everything before them into 64-slot units.
struct UnitPlan {
    int units[3];   // units of 64, 32 and 16 slots, in this order along the slots
    __host__ __device__ int first_slot(int g) const { return g == 0 ? 0 : g == 1 ? units[0] * kChunk : units[0] * kChunk + units[1] * (kChunk / 2); }
    __host__ __device__ int first_unit(int g) const { return g == 0 ? 0 : g == 1 ? units[0] : units[0] + units[1]; }
};
__host__ __device__ inline UnitPlan plan_units(int total_slots, int waves)
{
    const int fine = 32 * (waves > 0 ? waves : 1);   // slots of each finer kind
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

// Work list of the launch, built by two small kernels.  A voxel of a window that is split into b key blocks
// (b = 1 up to the launch's block length of 64, 128 or 256 voxels) takes b slots, one per key block, and a slot
// streams the block's keys: at most that many steps.  The windows are sorted by that step count, longest first
// (a counting sort over the possible counts), their slots laid out back to back in that order -
// [window][key block][voxel] - and cut into units,
// so a wavefront's lanes carry queries of several windows when the windows are small, every lane of a unit
// runs (almost) the same number of steps, and the launch ends on its shortest units.
//
// generic_count_kernel: every workgroup takes a run of windows; a window takes a place in the workgroup's bin
// of its step count - its rank there and the slots before it (one 64-bit LDS atomic returns both, so the two
// orders agree; the order inside a bin does not affect results) - and the workgroup leaves its bin totals.
__global__ __launch_bounds__(kListThreads) void generic_count_kernel(AttnArgs a)
{
    __shared__ unsigned long long bin[kMaxBlockSteps + 1];   // per step count: windows << 32 | slots
    for (int t = threadIdx.x; t <= kMaxBlockSteps; t += kListThreads) bin[t] = 0;
    __syncthreads();
    char *ws = static_cast<char *>(a.workspace);
    int *total = reinterpret_cast<int *>(ws + ws_total_offset(a.H));
    int2 *place = reinterpret_cast<int2 *>(ws + ws_place_offset(a.H, a.W, a.N, a.max_key_tiles));
    unsigned long long *group_bins =
        reinterpret_cast<unsigned long long *>(ws + ws_bins_offset(a.H, a.W, a.N, a.max_key_tiles));
    const int W = static_cast<int>(a.W);
    const int per = (W + static_cast<int>(gridDim.x) - 1) / static_cast<int>(gridDim.x);
    const int begin = min(static_cast<int>(blockIdx.x) * per, W), end = min(begin + per, W);
    for (int w = begin + threadIdx.x; w < end; w += kListThreads) {
        const int n = a.w_sizes[w];
        const int blocks = key_blocks(n, a.block_shift);
        int2 got = make_int2(-1, 0);
        if (n > 0 && blocks <= a.max_key_tiles) {
            const unsigned long long before =
                atomicAdd(&bin[key_block_size(n, a.block_shift)], (1ull << 32) | static_cast<unsigned>(n * blocks));
            got = make_int2(static_cast<int>(before >> 32), static_cast<int>(before & 0xffffffffu));
        }
        place[w] = got;
    }
    __syncthreads();
    for (int t = threadIdx.x; t <= kMaxBlockSteps; t += kListThreads)
        group_bins[blockIdx.x * (kMaxBlockSteps + 1) + t] = bin[t];
    if (blockIdx.x == 0 && threadIdx.x == 0) total[1] = 0;   // split windows, counted by the second kernel
}

// generic_place_kernel (same grid): bins in descending step order, workgroups in order inside a bin.  Writes one
// entry (first slot, voxels, first sorted position, steps) per window in sorted order, the entry that holds
// the first slot of every unit, the list of split windows for the merge, the totals, and the queue counters
// at zero.  Windows beyond the caller's size bound get no slots.
__global__ __launch_bounds__(kListThreads) void generic_place_kernel(AttnArgs a)
{
    __shared__ int bin_entry[kMaxBlockSteps + 1], bin_slot[kMaxBlockSteps + 1];
    __shared__ int wave_c[kListThreads / 64], wave_s[kListThreads / 64];
    __shared__ int sums[2];
    char *ws = static_cast<char *>(a.workspace);
    int *counters = reinterpret_cast<int *>(ws);
    int *total = reinterpret_cast<int *>(ws + ws_total_offset(a.H));
    int *unit_first = reinterpret_cast<int *>(ws + ws_units_offset(a.H));
    int4 *entries = reinterpret_cast<int4 *>(ws + ws_entries_offset(a.H, a.N, a.max_key_tiles));
    const int2 *place = reinterpret_cast<const int2 *>(ws + ws_place_offset(a.H, a.W, a.N, a.max_key_tiles));
    const unsigned long long *group_bins =
        reinterpret_cast<const unsigned long long *>(ws + ws_bins_offset(a.H, a.W, a.N, a.max_key_tiles));
    int *split = reinterpret_cast<int *>(ws + ws_split_offset(a.H, a.W, a.N, a.max_key_tiles));
    static_assert(kListThreads == kMaxBlockSteps, "one thread per bin");
    // thread t holds the bin of (longest block) - t steps: the launch's total, and what the workgroups before
    // this one put there; an exclusive scan over the threads gives the bins their places
    {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const int steps = (1 << a.block_shift) - static_cast<int>(threadIdx.x);
        unsigned long long all = 0, before = 0;
        if (steps >= 1) {
#pragma unroll 8
            for (int g = 0; g < static_cast<int>(gridDim.x); ++g) {
                const unsigned long long v = group_bins[g * (kMaxBlockSteps + 1) + steps];
                all += v;
                before += g < static_cast<int>(blockIdx.x) ? v : 0;
            }
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
        if (steps >= 1) {
            bin_entry[steps] = base_c + incl_c - cnt + static_cast<int>(before >> 32);
            bin_slot[steps] = base_s + incl_s - slots + static_cast<int>(before & 0xffffffffu);
        }
        if (threadIdx.x == kListThreads - 1) { sums[0] = base_c + incl_c; sums[1] = base_s + incl_s; }
    }
    __syncthreads();
    const int total_entries = sums[0], total_slots = sums[1];
    const UnitPlan plan = plan_units(total_slots, a.target_items);
    const int W = static_cast<int>(a.W);
    const int per = (W + static_cast<int>(gridDim.x) - 1) / static_cast<int>(gridDim.x);
    const int begin = min(static_cast<int>(blockIdx.x) * per, W), end = min(begin + per, W);
    for (int w = begin + threadIdx.x; w < end; w += kListThreads) {
        const int2 got = place[w];
        if (got.x < 0) continue;
        const int n = a.w_sizes[w];
        const int blocks = key_blocks(n, a.block_shift), steps = key_block_size(n, a.block_shift);
        const int e = bin_entry[steps] + got.x;
        const int s = bin_slot[steps] + got.y;
        entries[e] = make_int4(s, n, a.w2n[w], steps);
        // the units whose first slot is one of this window's
        const int s_end = s + n * blocks;
#pragma unroll
        for (int g = 0; g < 3; ++g) {
            const int size = kChunk >> g, from = plan.first_slot(g), count = plan.units[g];
            int v = s <= from ? 0 : (s - from + size - 1) / size;
            for (; v < count && from + v * size < s_end; ++v) unit_first[plan.first_unit(g) + v] = e;
        }
        if (blocks > 1) split[atomicAdd(total + 1, 1)] = w;   // any order: the merge treats windows independently
    }
    if (blockIdx.x == 0) {
        // a wavefront reads 64 entries from a unit's first one: pad the list with entries no slot belongs to
        if (threadIdx.x < kChunk) entries[total_entries + threadIdx.x] = make_int4(total_slots, 1, 0, 1);
        if (threadIdx.x == 0) {
            total[0] = plan.units[0] + plan.units[1] + plan.units[2];
            total[2] = total_slots;
            total[3] = plan.units[0];
            total[4] = plan.units[1];
        }
        for (int t = threadIdx.x; t < a.H * kQueues; t += kListThreads) counters[t * kCounterStride] = 0;
    }
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
        const int blocks = key_blocks(n_w, a.block_shift);
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
template <typename T, int D, int HP> __host__ __device__ constexpr int groups_per_cu()
{
    return D > 8 || HP == 2 ? 3 : 4;
}

// elements of T between table rows in LDS when a workgroup holds the slices of HP heads side by side
template <typename T, int D, int HP> __host__ __device__ constexpr int table_row_stride_heads()
{
    return HP * 3 * D + ((HP * 3 * D * static_cast<int>(sizeof(T)) / 4) % 8 == 0 ? 16 / static_cast<int>(sizeof(T)) : 0);
}

// HP: heads a wavefront carries through a unit (adjacent heads HP * g .. HP * g + HP - 1).  The cRSE rows and
// LDS addresses of a pair do not depend on the head, so two heads share that part of the work.
template <typename T, int D, int ND, int HP>
__global__ __launch_bounds__(kThreads, (groups_per_cu<T, D, HP>())) void attn_fwd_sweep_kernel(AttnArgs a)
{
    // streamed keys per loop iteration: at head_dim 16 two interleaved chains hide the LDS round trips,
    // at head_dim 8 the extra registers cost more than they bring
    constexpr int kKeys = D <= 8 ? 1 : 2;
    // lazy softmax reference (see the loop): -4 % for fp16; fp32 measured no gain (head_dim 8) or a loss (16)
    constexpr bool kLazy = sizeof(T) == 2;
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
    const int *unit_first = reinterpret_cast<const int *>(ws + ws_units_offset(H));
    const int4 *entries = reinterpret_cast<const int4 *>(ws + ws_entries_offset(H, a.N, a.max_key_tiles));
    const int total_units = __builtin_amdgcn_readfirstlane(reinterpret_cast<const int *>(ws + ws_total_offset(H))[0]);
    const int total_slots = __builtin_amdgcn_readfirstlane(reinterpret_cast<const int *>(ws + ws_total_offset(H))[2]);
    UnitPlan plan;
    plan.units[0] = __builtin_amdgcn_readfirstlane(reinterpret_cast<const int *>(ws + ws_total_offset(H))[3]);
    plan.units[1] = __builtin_amdgcn_readfirstlane(reinterpret_cast<const int *>(ws + ws_total_offset(H))[4]);
    plan.units[2] = 0;
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
        // the lane's slot: a query of a window and one block of at most 64 of the window's keys.  The unit's 64
        // slots lie in at most 64 consecutive entries from the unit's first one; each lane reads one entry and
        // finds its own (the last entry that starts at or before its slot) by a search across the lanes.
        const int first = __builtin_amdgcn_readfirstlane(unit_first[unit]);
        const int4 seen = entries[first + lane];
        // the unit's kind: 2^gshift groups of lanes that share queries and take alternate keys
        const int gshift = unit < plan.first_unit(1) ? 0 : unit < plan.first_unit(2) ? 1 : 2;
        const int gs = kChunk >> gshift;
        const int grp = lane >> (6 - gshift);
        const int slot_raw = plan.first_slot(gshift) + (unit - plan.first_unit(gshift)) * gs + (lane & (gs - 1));
        const bool own_valid = slot_raw < total_slots;
        const int slot = min(slot_raw, total_slots - 1);   // lanes past the end repeat the last slot
        int at = 0;
#pragma unroll
        for (int half = 32; half > 0; half >>= 1)
            if (__shfl(seen.x, at + half) <= slot) at += half;
        const int n_w = __shfl(seen.y, at), s0 = __shfl(seen.z, at), block_size = __shfl(seen.w, at);
        const int in_window = slot - __shfl(seen.x, at);               // [key block][voxel]
        // entries are sorted by steps, longest first
        const int max_steps = (__builtin_amdgcn_readfirstlane(seen.w) + (1 << gshift) - 1) >> gshift;
        const int blocks = key_blocks(n_w, a.block_shift);
        const int kb = blocks == 1 ? 0 : in_window / n_w;
        const int own_pos = s0 + (in_window - kb * n_w);
        const int own_row = a.n2n[own_pos];
        // the slot's keys: block kb of the window's even split into blocks of at most 64
        const int k_begin = kb * block_size;
        const int n_k = min(block_size, n_w - k_begin);
        const int k0 = s0 + k_begin;

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
        for (int u = 0; u < kKeys; ++u) row_next[u] = a.n2n[k0 + min((u << gshift) + grp, n_k - 1)];
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
                const int st_row = row_next[u];
                row_next[u] = a.n2n[k0 + min(st + (kKeys << gshift), n_k - 1)];
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
                // (and the sums are rescaled) only when some lane's logit exceeds it by more than kSlack, which
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
                if (__builtin_amdgcn_ballot_w64(valid[0] && moved) != 0) {   // uniform: all lanes move their reference
                    if (valid[0]) {
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
#pragma unroll
                            for (int n = 0; n < ND; ++n) {
                                Slice<T, D> tv_r;
                                tv_r.load_lds(off[u][n] + hh * kHeadBytes + 2 * D * sizeof(T));
                                tv_r.fma_to(acc[hh], p);
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
            // groups saw alternate keys of the same queries: merge their softmax states
            for (int other = 32; other >= gs; other >>= 1) {
                const float m_o = __shfl_xor(m[hh], other), l_o = __shfl_xor(l[hh], other);
                const float m_all = fmaxf(m[hh], m_o);
                const float w_me = (m[hh] == -INFINITY) ? 0.0f : __expf(m[hh] - m_all);
                const float w_ot = (m_o == -INFINITY) ? 0.0f : __expf(m_o - m_all);
                l[hh] = l[hh] * w_me + l_o * w_ot;
#pragma unroll
                for (int c = 0; c < D; ++c) acc[hh][c] = acc[hh][c] * w_me + __shfl_xor(acc[hh][c], other) * w_ot;
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
    if (a.N * a.max_key_tiles > INT32_MAX - kChunk)
        return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd: %lld voxels x %d key blocks exceed the 32-bit slot count",
                    (long long)a.N, a.max_key_tiles);
    auto kernel = attn_fwd_sweep_kernel<T, D, ND, HP>;
    S3D_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    int device = 0, cus = 256;
    if (hipGetDevice(&device) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && v > 0) cus = v;
    }
    // a workgroup serves one head group for its whole life: as many workgroups per CU as registers and LDS allow,
    // in whole sets of (XCDs x head groups)
    int per_cu = groups_per_cu<T, D, HP>();
    while (per_cu > 1 && per_cu * lds > 160 * 1024) --per_cu;
    const int set = kQueues * (a.H / HP);
    const int sets = per_cu * cus / set > 0 ? per_cu * cus / set : 1;
    AttnArgs b = a;
    b.target_items = sets * kQueues * (kThreads / 64);   // wavefronts that serve one head group
    const int64_t list_want = (a.W + kListThreads - 1) / kListThreads;
    const dim3 list_grid(static_cast<unsigned>(list_want < 1 ? 1 : (list_want > kListGroups ? kListGroups : list_want)));
    hipLaunchKernelGGL(generic_count_kernel, list_grid, dim3(kListThreads), 0, stream, b);
    hipLaunchKernelGGL(generic_place_kernel, list_grid, dim3(kListThreads), 0, stream, b);
    S3D_HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(sets * set)), dim3(kThreads), lds, stream, b);
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

int attn_generic_block_shift(int H, int64_t N, int64_t W, int max_window_voxels)
{
    return block_shift_for(H, N, W, max_window_voxels);
}

int attn_generic_key_blocks(int H, int64_t N, int64_t W, int max_window_voxels)
{
    return key_blocks(max_window_voxels > 0 ? max_window_voxels : 1, block_shift_for(H, N, W, max_window_voxels));
}

size_t attn_generic_workspace_bytes(int H, int D, int64_t W, int64_t N, int max_window_voxels)
{
    // queue counters, the totals, the unit list and sorted window list, and one partial record per (key block, head,
    // voxel) when some window may be split along its keys
    const int blocks = attn_generic_key_blocks(H, N, W, max_window_voxels);
    const size_t partials = blocks <= 1 ? 0 : sizeof(float) * static_cast<size_t>(N) * blocks * H * (D + 2);
    return ws_partials_offset(H, W, N, blocks) + align_up(partials, 256);
}

float *attn_generic_partials(void *workspace, int H, int64_t W, int64_t N, int max_window_voxels)
{
    return reinterpret_cast<float *>(static_cast<char *>(workspace) +
                                     ws_partials_offset(H, W, N, attn_generic_key_blocks(H, N, W, max_window_voxels)));
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
