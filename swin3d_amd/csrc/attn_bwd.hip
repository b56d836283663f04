// Sparse-voxel windowed self-attention BACKWARD with cRSE tables (gfx950): fp32 arithmetic, fp16 or fp32 I/O.
//
// Math (Swin3D/src/attn/self_attn_aio_bwd.cu:14-113, Swin3D/sparse_dl/attn/attn_coff.py:191-232), per
// window, head h, query i, key j, with P = softmax weights and o the forward output:
//   dP(i,j) = dout_i . (v_j + Tv(i,j))            dL(i,j) = P(i,j) (dP(i,j) - dout_i . o_i)
//   dv_j  += P dout_i                              dTv[n][row_n(i,j)] += P dout_i
//   dq_i  += dL (k_j + Tq(i,j))                    dTq[n][row_n(i,j)] += dL q_i
//   dk_j  += dL (q_i + Tk(i,j))                    dTk[n][row_n(i,j)] += dL k_j
// The reference adds every term with a global atomic.  Here every output element has ONE owner, and the call has two
// forms.  With the window set's pair count it runs the pair sweeps of attn_sweep.hip (dq; dk and dv; on the
// forward's packed work list), which leave dL and P of every (pair, head) in the workspace, and the table-gradient
// kernels below (attn_bwd_tables_kernel), which read them.  Without it, the fused sweeps (attn_bwd_sweep_kernel),
// which recompute the logits and need no store:
//
//  * a key-owned sweep gives a lane one key j and streams the window's queries through the wavefront:
//    dk_j, dv_j accumulate in the lane's registers and are stored once;
//  * a query-owned sweep gives a lane one query i and streams the keys: dq_i likewise;
//  * table gradients: within one step of a sweep the streamed side is the same for all lanes (q_i and
//    dout_i in the key-owned sweep, k_j in the query-owned one), so
//        dTq[n][r] += (sum over lanes with row_n = r of dL) * q_i
//    is a histogram over table rows (integer LDS atomics, one per pair and axis, on a fixed-point image
//    scaled by the largest |dL| of the step) followed by a rank-1 update in which lane r owns row r.
//    The wavefront keeps its table gradients in registers for all the units it processes and adds them
//    to the global tables once, at the end (a workgroup works on one head for its whole life and keeps
//    that head's slices of the three tables in LDS).
//
// Windows of at most 32 voxels put two streamed elements in one wavefront step (two 32-lane groups).
#include "attn_kernels.h"
#include "sweep_common.h"

#include <type_traits>

namespace s3d {
namespace {

using namespace sweep;

constexpr int kCounterSets = 4;
constexpr int kBwdThreads = 256;
constexpr int kBwdWaves = kBwdThreads / 64;
constexpr int kChunk = 64;            // owned elements per unit = lanes of a wavefront
constexpr float kFixP = 16777216.0f;  // 2^24: softmax weights of one query sum to at most 1
constexpr float kFixL = 8388608.0f;   // 2^23: |dL| / max|dL| <= 1, at most 64 lanes meet in one bin

struct BwdArgs {
    const void *q, *k, *v, *table_q, *table_k, *table_v, *dout, *out;
    const float *out_max, *out_sum;
    const int32_t *w_sizes, *w2n, *n2n;
    const float *n_coords;
    void *dq, *dk, *dv;
    float *dtq, *dtk, *dtv;
    float *delta;     // [N,H] dout_i . o_i
    float *tgrad;     // per-wavefront table gradients of a sweep: [wavefront][kind][64 * BLK rows][D]
    int64_t *pos_base;   // [N]: at a window's first sorted position, the pairs (n^2) of the windows before it
    const float2 *pd;    // [H][pairs]: (dL, P) of the pair sweeps at base + i n + j
    const float *dl_t;   // [H][pairs]: dL at base + j n + i
    int64_t pairs;       // capacity of pd and dl_t per head
    int32_t *units;   // H * kQueues work counters (kCounterStride apart), the unit count, (window, chunk) per unit
    int32_t H, D, nd, total_rows;
    int64_t N, W, table_len;
    int32_t rows[kMaxAxes];
    int32_t base[kMaxAxes];
};

__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
}

// max of a non-negative value over the lanes of each group (32-lane halves when two_groups, else the wavefront),
// returned in every lane: DPP moves inside the 16-lane rows and across them, two scalar reads; no LDS permutes
__device__ __forceinline__ float group_max_nonneg(float v, bool two_groups, int grp)
{
    auto step = [](float x, auto ctrl, auto row_mask) {
        const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(x), decltype(ctrl)::value, decltype(row_mask)::value,
                                                      0xf, true);
        return fmaxf(x, __int_as_float(moved));
    };
    v = step(v, std::integral_constant<int, 0xB1>{}, std::integral_constant<int, 0xf>{});    // quad_perm [1,0,3,2]
    v = step(v, std::integral_constant<int, 0x4E>{}, std::integral_constant<int, 0xf>{});    // quad_perm [2,3,0,1]
    v = step(v, std::integral_constant<int, 0x141>{}, std::integral_constant<int, 0xf>{});   // row_half_mirror
    v = step(v, std::integral_constant<int, 0x140>{}, std::integral_constant<int, 0xf>{});   // row_mirror
    v = step(v, std::integral_constant<int, 0x142>{}, std::integral_constant<int, 0xa>{});   // row_bcast15 into rows 1, 3
    const float lo = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 31));
    const float hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
    return two_groups ? (grp ? hi : lo) : fmaxf(lo, hi);
}

// value of x in lane `src` (src uniform): a scalar read instead of an LDS permute
__device__ __forceinline__ float lane_value(float x, int src)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), src));
}

// delta[i][h] = dout_i . o_i; the table gradients and the work counters start at zero
template <typename T>
__global__ void bwd_prepare_kernel(BwdArgs a)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    const int64_t t0 = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const T *go = static_cast<const T *>(a.dout);
    const T *o = static_cast<const T *>(a.out);
    for (int64_t t = t0; t < a.N * a.H; t += stride) {
        // head_dim is a multiple of 8: rows in pieces of eight channels (16- or 32-byte loads)
        float s = 0.0f;
        for (int c0 = 0; c0 < a.D; c0 += 8) {
            float x[8], y[8];
            load_row<8>(go + t * a.D + c0, x);
            load_row<8>(o + t * a.D + c0, y);
#pragma unroll
            for (int c = 0; c < 8; ++c) s += x[c] * y[c];
        }
        a.delta[t] = s;
    }
    for (int64_t t = t0; t < a.table_len; t += stride) {
        a.dtq[t] = 0.0f;
        a.dtk[t] = 0.0f;
        a.dtv[t] = 0.0f;
    }
    for (int64_t t = t0; t < kCounterSets * a.H * kQueues; t += stride) a.units[t * kCounterStride] = 0;
}

// kCounterSets sets of H * kQueues work counters: every table-gradient kernel of a call draws from a set of its own
// (sets 0..3 by kind), so none has to wait for the counters to be put back; the fused sweeps share set 0 and reset it
__host__ __device__ inline size_t units_total_index(int H) { return static_cast<size_t>(kCounterSets) * H * kQueues * kCounterStride; }
__host__ __device__ inline size_t units_list_index(int H) { return units_total_index(H) + 64; }

// unit list: one (window, chunk of 64 owned elements, segment of 64 streamed elements) descriptor per unit, and the
// unit count; one workgroup.  The table-gradient kernels (a.pairs > 0) take a window of more than 64 voxels in
// segments of 64 streamed voxels - what a unit adds to the table gradients is a sum over the streamed side, and one
// unit for all 343 voxels of a full window was three times the average wavefront's share of a launch; the fused
// sweeps, whose owned gradients need the whole stream, get one unit per chunk (segment 0).
__global__ __launch_bounds__(1024) void bwd_units_kernel(BwdArgs a)
{
    // units are listed longest first, in classes of window size (a unit streams the whole window: n steps, or
    // n / 2 up to 32 voxels), windows in order inside a class: the launch then ends on its shortest units
    constexpr int kClasses = 6;
    auto class_of = [](int n) { return n > 256 ? 0 : n > 128 ? 1 : n > 64 ? 2 : n > 32 ? 3 : n > 16 ? 4 : 5; };
    __shared__ int wave_sum[16][kClasses];
    __shared__ int class_start[kClasses + 1];
    __shared__ long long wave_pairs[16];       // pairs (n^2) of the windows of each wavefront's threads
    const int W = static_cast<int>(a.W);
    const int per = (W + 1023) / 1024;
    const int begin = min(static_cast<int>(threadIdx.x) * per, W), end = min(begin + per, W);
    int mine[kClasses];
#pragma unroll
    for (int c = 0; c < kClasses; ++c) mine[c] = 0;
    long long pairs_mine = 0;
    for (int w = begin; w < end; ++w) {
        const int n = a.w_sizes[w];
        const int chunks = n > 0 ? (n + kChunk - 1) / kChunk : 0, cls = class_of(n);
        const int units_w = a.pairs > 0 ? chunks * chunks : chunks;
#pragma unroll
        for (int c = 0; c < kClasses; ++c) mine[c] += c == cls ? units_w : 0;
        pairs_mine += static_cast<long long>(n) * n;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    long long pairs_incl = pairs_mine;
    for (int off = 1; off < 64; off <<= 1) {
        const long long up = __shfl_up(pairs_incl, off);
        if (lane >= off) pairs_incl += up;
    }
    if (lane == 63) wave_pairs[wave] = pairs_incl;
    int incl[kClasses];
#pragma unroll
    for (int c = 0; c < kClasses; ++c) {
        incl[c] = mine[c];
        for (int off = 1; off < 64; off <<= 1) {
            const int up = __shfl_up(incl[c], off);
            if (lane >= off) incl[c] += up;
        }
        if (lane == 63) wave_sum[wave][c] = incl[c];
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int c = 0; c < kClasses; ++c) {
            class_start[c] = run;
            for (int v = 0; v < 16; ++v) {
                const int t = wave_sum[v][c];
                wave_sum[v][c] = run;   // units of this class in the wavefronts before v
                run += t;
            }
        }
        class_start[kClasses] = run;
        long long before = 0;
        for (int v = 0; v < 16; ++v) {
            const long long add = wave_pairs[v];
            wave_pairs[v] = before;
            before += add;
        }
        // a pair store shorter than the window set's pairs: the call's results are marked (NaN), see the reduction
        a.units[units_total_index(a.H) + 1] = a.pairs > 0 && before > a.pairs;
    }
    __syncthreads();
    // where the (pair, head) records of a window start in the pair store: written at the window's first position
    long long before = wave_pairs[wave] + pairs_incl - pairs_mine;
    int run[kClasses];
#pragma unroll
    for (int c = 0; c < kClasses; ++c) run[c] = wave_sum[wave][c] + incl[c] - mine[c];
    int2 *list = reinterpret_cast<int2 *>(a.units + units_list_index(a.H));
    // four windows at a time: their sizes and first positions are loaded before any of their stores (a load after
    // a store through another pointer waits for it)
    for (int w0 = begin; w0 < end; w0 += 4) {
        int n4[4], s4[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int w = min(w0 + e, end - 1);
            n4[e] = a.w_sizes[w];
            s4[e] = a.w2n[w];
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int w = w0 + e;
            if (w >= end) break;
            const int n = n4[e];
            if (n > 0) a.pos_base[s4[e]] = before;
            before += static_cast<long long>(n) * n;
            const int chunks = n > 0 ? (n + kChunk - 1) / kChunk : 0, cls = class_of(n);
            const int segs = a.pairs > 0 ? chunks : 1;
            int at = 0;
#pragma unroll
            for (int c = 0; c < kClasses; ++c) {
                if (c == cls) { at = run[c]; run[c] += chunks * segs; }
            }
            for (int c = 0; c < chunks; ++c)
                for (int sg = 0; sg < segs; ++sg) list[at + c * segs + sg] = make_int2(w, c | (sg << 16));
        }
    }
    if (threadIdx.x == 0) a.units[units_total_index(a.H)] = class_start[kClasses];
}

// the work counters are re-armed between sweeps
__global__ void bwd_reset_counters_kernel(BwdArgs a)
{
    for (int t = threadIdx.x; t < a.H * kQueues; t += blockDim.x) a.units[t * kCounterStride] = 0;
}

// MODE (key-owned sweep only): 0 = dk, dv, dTq, dTv in one sweep - what the library launches: two wavefronts per
// SIMD at head_dim 8, one at head_dim 16 (up to 512 registers, 192 to 256 of them MFMA accumulation registers
// for the two sets of table gradients); 1 = dk, dTq and 2 = dv, dTv are the halves of that sweep, used at
// head_dim 16 when the table has more than 384 rows per head; at 360 rows they measured 3.44 ms as two launches
// against 2.83 ms fused (the logits are computed once).
// The query-owned sweep produces dq and dTk.
// BLK: 64-row blocks of the head's flat table (all axes back to back) that the wavefront's
// table-gradient registers cover; lane l of block m owns flat row 64 m + l.
template <typename T, int D, int ND, bool KEY_OWNED, int MODE, int BLK>
__global__ __launch_bounds__(kBwdThreads, (D <= 8 ? 2 : 1)) void attn_bwd_sweep_kernel(BwdArgs a)
{
    constexpr bool kNeedDl = !KEY_OWNED || MODE != 2;          // dP / dL are needed
    constexpr bool kAccA = kNeedDl;                            // dTq (key-owned) or dTk (query-owned)
    constexpr bool kAccB = KEY_OWNED && MODE != 1;             // dTv
    constexpr int kHistKinds = (kAccA ? 1 : 0) + (kAccB ? 1 : 0);
    constexpr int kFlat = BLK * 64;                            // flat table rows covered (>= total_rows)
    constexpr int kHistWords = kHistKinds * 2 * kFlat;         // [kind][group][flat row]

    extern __shared__ float smem[];
    const int H = a.H;
    const int HD = H * D;
    // workgroups go to the XCDs in turn: consecutive runs of eight serve one head, so every XCD gets every head
    const int h = (blockIdx.x / kQueues) % H;
    // table slices of the head in the I/O type; a row holds the q-side, k-side and v-side slices back to back (one
    // LDS address per pair and axis)
    constexpr int kRowStride = table_row_stride<T, D>();
    constexpr int kRowBytes = kRowStride * static_cast<int>(sizeof(T));
    T *tab = reinterpret_cast<T *>(smem);
    int *hist_all = reinterpret_cast<int *>(reinterpret_cast<char *>(smem) +
                                            (static_cast<size_t>(a.total_rows) * kRowBytes + 15) / 16 * 16);

    {
        const T *gq = static_cast<const T *>(a.table_q);
        const T *gk = static_cast<const T *>(a.table_k);
        const T *gv = static_cast<const T *>(a.table_v);
        for (int t = threadIdx.x; t < a.total_rows * D; t += kBwdThreads) {
            const int r = t / D, c = t - r * D;
            const int64_t g = static_cast<int64_t>(r) * HD + h * D + c;
            tab[r * kRowStride + c] = gq[g];
            tab[r * kRowStride + D + c] = gk[g];
            tab[r * kRowStride + 2 * D + c] = gv[g];
        }
        for (int t = threadIdx.x; t < kBwdWaves * kHistWords; t += kBwdThreads) hist_all[t] = 0;
    }
    __syncthreads();   // the only workgroup barrier

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    int *hist_a = hist_all + wave * kHistWords;                 // dL histogram
    int *hist_b = hist_a + (kAccA ? 2 * kFlat : 0);             // P histogram
    unsigned long long *hist_ab = reinterpret_cast<unsigned long long *>(hist_a);   // both, [group][flat row]

    const T *gq = static_cast<const T *>(a.q);
    const T *gk = static_cast<const T *>(a.k);
    const T *gv = static_cast<const T *>(a.v);
    const T *ggo = static_cast<const T *>(a.dout);

    // table-gradient accumulators.  VALU updates (head_dim 8): acc[m][c] of lane l is (flat row 64 m + l, channel
    // c).  MFMA updates (head_dim 16, where one wavefront per SIMD leaves room for accumulation registers and the
    // update as matrix instructions measured 3-5 % faster; at head_dim 8 it measured 4 % slower): acc[m] holds
    // D / 4 four-element results in the layout of the 4x4x1 MFMA (16 blocks of 4 rows x 4 channels), element i of
    // quad c4 in lane l is (flat row 64 m + 4 (l / 4) + i, channel 4 c4 + l % 4)
    constexpr bool kMfmaUpdate = D > 8;
    float acc_a[BLK][D], acc_b[BLK][D];
#pragma unroll
    for (int m = 0; m < BLK; ++m)
#pragma unroll
        for (int c = 0; c < D; ++c) acc_a[m][c] = acc_b[m][c] = 0.0f;
    auto mfma_update = [](float (&acc)[D], float row_sum, const float (&b)[D / 4]) {
#pragma unroll
        for (int c = 0; c < D / 4; ++c) {
            f32x4_t r = {acc[4 * c], acc[4 * c + 1], acc[4 * c + 2], acc[4 * c + 3]};
            r = __builtin_amdgcn_mfma_f32_4x4x1f32(row_sum, b[c], r, 0, 0, 0);
            acc[4 * c] = r[0]; acc[4 * c + 1] = r[1]; acc[4 * c + 2] = r[2]; acc[4 * c + 3] = r[3];
        }
    };

    // 1.0 the optimiser cannot see through: x * one + sum keeps an fp16 row widened inside one mixed-precision FMA
    float one = 1.0f;
    asm volatile("" : "+v"(one));
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

    const int2 *unit_list = reinterpret_cast<const int2 *>(a.units + units_list_index(H));
    const int total_units = __builtin_amdgcn_readfirstlane(a.units[units_total_index(H)]);
    int *counters = a.units + h * kQueues * kCounterStride;

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
        const int2 desc = unit_list[unit];
        const int w = __builtin_amdgcn_readfirstlane(desc.x);
        const int chunk = __builtin_amdgcn_readfirstlane(desc.y) & 0xffff;
        const int n_w = __builtin_amdgcn_readfirstlane(a.w_sizes[w]);
        const int s0 = __builtin_amdgcn_readfirstlane(a.w2n[w]);
        // group size: a window of at most 32 voxels streams two elements per step
        const int gs = n_w <= 32 ? 32 : 64;
        const int ng = 64 / gs;
        const int grp = lane / gs;
        const int own = chunk * kChunk + (lane - grp * gs);
        const bool own_valid = own < n_w;
        const int own_pos = s0 + min(own, n_w - 1);
        const int own_row = a.n2n[own_pos];

        // owned side, in the I/O type (fp16: packed pairs)
        Slice<T, D> own_x, own_y;
        float own_c[ND], own_m = 0.0f, own_inv = 0.0f, own_delta = 0.0f;
        if constexpr (KEY_OWNED) {
            own_x.load(gk + static_cast<int64_t>(own_row) * HD + h * D);   // k_j
            if constexpr (kNeedDl) own_y.load(gv + static_cast<int64_t>(own_row) * HD + h * D);   // v_j
        } else {
            own_x.load(gq + static_cast<int64_t>(own_row) * HD + h * D);   // q_i
            own_y.load(ggo + static_cast<int64_t>(own_row) * HD + h * D);  // dout_i
            own_m = a.out_max[static_cast<int64_t>(own_row) * H + h];
            own_inv = 1.0f / a.out_sum[static_cast<int64_t>(own_row) * H + h];
            own_delta = a.delta[static_cast<int64_t>(own_row) * H + h];
        }
#pragma unroll
        for (int n = 0; n < ND; ++n) own_c[n] = a.n_coords[static_cast<int64_t>(own_pos) * ND + n];
        float res_x[D], res_y[D];   // dk_j, dv_j  or  dq_i
#pragma unroll
        for (int c = 0; c < D; ++c) res_x[c] = res_y[c] = 0.0f;

        const int steps = (n_w + ng - 1) / ng;
        int st_row_next = a.n2n[s0 + min(grp, n_w - 1)];
        for (int it = 0; it < steps; ++it) {
            // the next unit's ticket is drawn during the last step: the atomic's round trip overlaps that work, and
            // a unit is not held back, out of reach of idle wavefronts, for the length of a unit
            if (it + 1 == steps && lane == 0) drawn = atomicAdd(counters + queue * kCounterStride, 1);
            const int st = it * ng + grp;
            const bool st_valid = st < n_w;
            const int st_pos = s0 + min(st, n_w - 1);
            const int st_row = st_row_next;
            if (it + 1 < steps) st_row_next = a.n2n[s0 + min(st + ng, n_w - 1)];
            // streamed side (the same for all lanes of a group)
            Slice<T, D> st_x, st_y;
            float st_c[ND], st_m = 0.0f, st_inv = 0.0f, st_delta = 0.0f;
            if constexpr (KEY_OWNED) {
                st_x.load(gq + static_cast<int64_t>(st_row) * HD + h * D);    // q_i
                st_y.load(ggo + static_cast<int64_t>(st_row) * HD + h * D);   // dout_i
                st_m = a.out_max[static_cast<int64_t>(st_row) * H + h];
                st_inv = 1.0f / a.out_sum[static_cast<int64_t>(st_row) * H + h];
                st_delta = a.delta[static_cast<int64_t>(st_row) * H + h];
            } else {
                st_x.load(gk + static_cast<int64_t>(st_row) * HD + h * D);    // k_j
                st_y.load(gv + static_cast<int64_t>(st_row) * HD + h * D);    // v_j
            }
#pragma unroll
            for (int n = 0; n < ND; ++n) st_c[n] = a.n_coords[static_cast<int64_t>(st_pos) * ND + n];

            const Slice<T, D> &qv = KEY_OWNED ? st_x : own_x;
            const Slice<T, D> &kv = KEY_OWNED ? own_x : st_x;
            const Slice<T, D> &vv = KEY_OWNED ? own_y : st_y;
            const Slice<T, D> &gov = KEY_OWNED ? st_y : own_y;
            const float m_i = KEY_OWNED ? st_m : own_m;
            const float inv_i = KEY_OWNED ? st_inv : own_inv;
            const float delta_i = KEY_OWNED ? st_delta : own_delta;

            // L = q.k + q.Tq + k.Tk and dP = dout.(v + Tv) as dot products against the gathered rows; the one
            // row sum that enters an owned gradient as a vector is kept: Tk (dk_j) or Tq (dq_i)
            constexpr bool kChain = Slice<T, D>::kChainLogit;
            int r[ND];
            float tsum[D];
#pragma unroll
            for (int c = 0; c < D; ++c) tsum[c] = 0.0f;
            float logit = qv.dot(kv, 0.0f);
            float dp = 0.0f;
            if constexpr (kNeedDl) dp = gov.dot(vv, 0.0f);
#pragma unroll
            for (int n = 0; n < ND; ++n) {
                const float ci = KEY_OWNED ? st_c[n] : own_c[n];
                const float cj = KEY_OWNED ? own_c[n] : st_c[n];
                r[n] = crse_row(ci, cj, half_rows[n], upper[n]);
                const uint32_t off = mad_u24(static_cast<uint32_t>(r[n]), row_bytes, base_off[n]);
                Slice<T, D> tq_r, tk_r;
                tq_r.load_lds(off);
                tk_r.load_lds(off + D * sizeof(T));
                if constexpr (KEY_OWNED) {
                    if (kChain) logit = qv.dot(tq_r, logit); else logit += qv.dot(tq_r, 0.0f);
                    tk_r.fma_to(tsum, one);
                } else {
                    tq_r.fma_to(tsum, one);
                    if (kChain) logit = kv.dot(tk_r, logit); else logit += kv.dot(tk_r, 0.0f);
                }
                if constexpr (kNeedDl) {
                    Slice<T, D> tv_r;
                    tv_r.load_lds(off + 2 * D * sizeof(T));
                    if (kChain) dp = gov.dot(tv_r, dp); else dp += gov.dot(tv_r, 0.0f);
                }
            }
            if (kChain) logit = (KEY_OWNED ? kv : qv).dot_f32(tsum, logit);
            else logit += (KEY_OWNED ? kv : qv).dot_f32(tsum, 0.0f);
            const bool valid = own_valid && st_valid;
            const float p = valid ? __expf(logit - m_i) * inv_i : 0.0f;
            float dl = 0.0f;
            if constexpr (kNeedDl) dl = p * (dp - delta_i);
            if constexpr (KEY_OWNED) {
                if constexpr (MODE != 2) {
                    qv.fma_to(res_x, dl);                                           // dk_j += dl (q_i + Tk)
#pragma unroll
                    for (int c = 0; c < D; ++c) res_x[c] += dl * tsum[c];
                }
                if constexpr (MODE != 1) gov.fma_to(res_y, p);                      // dv_j += p dout_i
            } else {
                kv.fma_to(res_x, dl);                                               // dq_i += dl (k_j + Tq)
#pragma unroll
                for (int c = 0; c < D; ++c) res_x[c] += dl * tsum[c];
            }

            // table gradients: histogram of the step over table rows, then a rank-1 update (lane = row)
            float amax = 0.0f;
            int qd = 0, qp = 0;
            if constexpr (kAccA) {
                amax = group_max_nonneg(fabsf(dl), ng == 2, grp);
                qd = __float2int_rn(dl * (amax > 0.0f ? kFixL / amax : 0.0f));
            }
            if constexpr (kAccB) qp = __float2int_rn(p * kFixP);
            if constexpr (kAccA && kAccB) {
                // both histograms hit the same rows: one 64-bit cell per row, dL in the upper half and P (never
                // negative, at most 64 * 2^24 per cell: no carry) in the lower, one atomic per pair and axis
                const unsigned long long both =
                    (static_cast<unsigned long long>(static_cast<unsigned>(qd)) << 32) + static_cast<unsigned>(qp);
                if (valid && both != 0) {
#pragma unroll
                    for (int n = 0; n < ND; ++n) atomicAdd(hist_ab + grp * kFlat + a.base[n] + r[n], both);
                }
            } else if constexpr (kAccA) {
                if (valid && qd != 0) {
#pragma unroll
                    for (int n = 0; n < ND; ++n) atomicAdd(hist_a + grp * kFlat + a.base[n] + r[n], qd);
                }
            } else {
                if (valid && qp != 0) {
#pragma unroll
                    for (int n = 0; n < ND; ++n) atomicAdd(hist_b + grp * kFlat + a.base[n] + r[n], qp);
                }
            }
            wave_lds_fence();
            // rank-1 updates acc[row][c] += hist[row] * x[c]; as 4x4x1 MFMAs the A operand of lane l is the sum of
            // flat row 64 m + l (A of block l / 4, row l % 4), the B operand channel 4 c4 + l % 4 of the
            // streamed element (the same 1 x 4 row for all 16 blocks)
            for (int g = 0; g < ng; ++g) {
                const int src = __builtin_amdgcn_readfirstlane(g * gs);   // a lane of group g: its streamed registers are the group's
                if constexpr (kAccA && kAccB) {
                    const float sc = lane_value(amax, src) * (1.0f / kFixL);
                    const Slice<T, D> sx = st_x.lane(src);   // q_i
                    const Slice<T, D> sy = st_y.lane(src);   // dout_i
                    float bx[D / 4], by[D / 4];
                    if constexpr (kMfmaUpdate) {
                        sx.quad_channels(lane, bx);
                        sy.quad_channels(lane, by);
                    }
#pragma unroll
                    for (int m = 0; m < BLK; ++m) {
                        unsigned long long *cell = hist_ab + g * kFlat + m * 64 + lane;
                        const unsigned long long both = *cell;
                        *cell = 0;
                        const float gsum = static_cast<float>(static_cast<int>(both >> 32)) * sc;
                        const float psum = static_cast<float>(static_cast<unsigned>(both)) * (1.0f / kFixP);
                        if constexpr (kMfmaUpdate) {
                            mfma_update(acc_a[m], gsum, bx);
                            mfma_update(acc_b[m], psum, by);
                        } else {
                            sx.fma_to(acc_a[m], gsum);
                            sy.fma_to(acc_b[m], psum);
                        }
                    }
                } else if constexpr (kAccA) {
                    const float sc = lane_value(amax, src) * (1.0f / kFixL);
                    const Slice<T, D> sx = st_x.lane(src);   // q_i (key-owned) or k_j
                    float bx[D / 4];
                    if constexpr (kMfmaUpdate) sx.quad_channels(lane, bx);
#pragma unroll
                    for (int m = 0; m < BLK; ++m) {
                        int *cell = hist_a + g * kFlat + m * 64 + lane;
                        const float gsum = static_cast<float>(*cell) * sc;
                        *cell = 0;
                        if constexpr (kMfmaUpdate) mfma_update(acc_a[m], gsum, bx);
                        else sx.fma_to(acc_a[m], gsum);
                    }
                } else {
                    const Slice<T, D> sy = st_y.lane(src);   // dout_i
                    float by[D / 4];
                    if constexpr (kMfmaUpdate) sy.quad_channels(lane, by);
#pragma unroll
                    for (int m = 0; m < BLK; ++m) {
                        int *cell = hist_b + g * kFlat + m * 64 + lane;
                        const float psum = static_cast<float>(*cell) * (1.0f / kFixP);
                        *cell = 0;
                        if constexpr (kMfmaUpdate) mfma_update(acc_b[m], psum, by);
                        else sy.fma_to(acc_b[m], psum);
                    }
                }
            }
            wave_lds_fence();
        }

        if (ng == 2) {
            // the two groups own the same elements and saw alternate steps of the stream
#pragma unroll
            for (int c = 0; c < D; ++c) {
                res_x[c] += __shfl_xor(res_x[c], 32);
                res_y[c] += __shfl_xor(res_y[c], 32);
            }
        }
        if (own_valid && grp == 0) {
            if constexpr (KEY_OWNED) {
                if constexpr (MODE != 2)
                    store_row<D>(static_cast<T *>(a.dk) + static_cast<int64_t>(own_row) * HD + h * D, res_x);
                if constexpr (MODE != 1)
                    store_row<D>(static_cast<T *>(a.dv) + static_cast<int64_t>(own_row) * HD + h * D, res_y);
            } else {
                store_row<D>(static_cast<T *>(a.dq) + static_cast<int64_t>(own_row) * HD + h * D, res_x);
            }
        }
    }

    // lane l of block m = flat table row 64 m + l: the wavefront leaves its table gradients in a slot of its own
    // (no atomics: thousands of wavefronts adding to the same few thousand addresses cost 15 % of the backward);
    // bwd_reduce_tables_kernel sums the slots of a head
    float *slot = a.tgrad + (static_cast<size_t>(blockIdx.x) * kBwdWaves + wave) * (2 * kFlat * D);
#pragma unroll
    for (int m = 0; m < BLK; ++m) {
        if constexpr (kMfmaUpdate) {
#pragma unroll
            for (int c = 0; c < D / 4; ++c) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const size_t at = static_cast<size_t>(m * 64 + (lane & ~3) + i) * D + 4 * c + (lane & 3);
                    if constexpr (kAccA) slot[at] = acc_a[m][4 * c + i];
                    if constexpr (kAccB) slot[static_cast<size_t>(kFlat) * D + at] = acc_b[m][4 * c + i];
                }
            }
        } else {
            const int row = m * 64 + lane;
            if constexpr (kAccA) store_row<D>(slot + static_cast<size_t>(row) * D, acc_a[m]);
            if constexpr (kAccB) store_row<D>(slot + static_cast<size_t>(kFlat + row) * D, acc_b[m]);
        }
    }
}

// Table gradients from the dL and P that the pair sweeps left for every (pair, head): the histogram and rank-1
// machinery of the sweeps above without their logits, table rows and owned gradients.
//   KIND 0: lanes = queries i of a 64-voxel chunk, the window's keys stream:   dTk += hist(dL) x k_j
//   KIND 1: lanes = keys j, the queries stream:   dTq += hist(dL) x q_i  and  dTv += hist(P) x dout_i
//   KIND 2, 3: the two halves of KIND 1 as kernels of their own (dTq; dTv), for the shapes where both sets of
//           accumulators leave one wavefront per SIMD
// A step's inputs - the lane's record, the streamed rows and coordinates - are fetched one step ahead: the records
// come from HBM and a step is a short dependent chain (rows, histogram atomics, read-back), so their latency would
// be most of it.
// Wavefronts per SIMD: two for KIND 1 at head_dim 8 (80 accumulators; capped at 168 registers for three it spills
// and measured 1.7x the time), three for the one-table kinds; at head_dim 16 one for KIND 1 and two for the
// one-table kinds (KIND 0 capped at 256 registers spills 40 of them and is still 2-3 % of the call faster than at one).
template <typename T, int D, int ND, int KIND, int BLK>
__global__ __launch_bounds__(kBwdThreads, (D <= 8 ? (KIND == 1 ? 2 : 3) : (KIND != 1 ? 2 : 1))) void attn_bwd_tables_kernel(BwdArgs a)
{
    constexpr bool KEY_OWNED = KIND != 0;
    constexpr bool kAccB = KIND == 1;                          // two histograms and two sets of accumulators
    constexpr bool kFromP = KIND == 3;                         // the one histogram is of P, the vector dout_i
    constexpr int kHistKinds = 1 + (kAccB ? 1 : 0);
    constexpr int kFlat = BLK * 64;
    // A histogram cell exists in kCopies copies, chosen by the low bits of the lane number: lanes that hit the
    // same table row - neighbouring voxels share colours and normals - serialise on a cell, and the copies divide
    // that by up to kCopies; the copies of a row lie side by side, 16 bytes that the read-back fetches at once.
    constexpr int kCopies = kAccB ? 2 : 4;
    constexpr int kHistWords = kHistKinds * 2 * kFlat * kCopies;   // [group][flat row][copy] of 32- or 64-bit cells
    extern __shared__ float smem[];
    const int H = a.H;
    const int HD = H * D;
    const int h = (blockIdx.x / kQueues) % H;
    int *hist_all = reinterpret_cast<int *>(smem);
    for (int t = threadIdx.x; t < kBwdWaves * kHistWords; t += kBwdThreads) hist_all[t] = 0;
    __syncthreads();   // the only workgroup barrier

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    int *hist_a = hist_all + wave * kHistWords;
    unsigned long long *hist_ab = reinterpret_cast<unsigned long long *>(hist_a);
    // the streamed row of the first rank-1 update (k_j, q_i or, for the dTv half, dout_i) and of the second (KIND 1)
    const T *gx = static_cast<const T *>(KIND == 0 ? a.k : KIND == 3 ? a.dout : a.q);
    const T *gy = static_cast<const T *>(a.dout);

    // The rank-1 updates as 4x4x1 MFMAs wherever the VALU form would not fit the registers: the accumulators may
    // then live in accumulation registers.  Measured at head_dim 8 (us, VALU / MFMA form): fp16 with five 64-row
    // blocks 658 / 1017 key-owned and 387 / 510 query-owned; six blocks 1804 / 817 and 843 / 508 (the VALU form
    // spills); fp32 with five blocks 1256 / 644 and 384 / 380.
    constexpr bool kMfmaUpdate = D > 8 || BLK > 5 || (KIND == 1 && sizeof(T) == 4);
    float acc_a[BLK][D], acc_b[kAccB ? BLK : 1][D];
#pragma unroll
    for (int m = 0; m < BLK; ++m)
#pragma unroll
        for (int c = 0; c < D; ++c) {
            acc_a[m][c] = 0.0f;
            if (kAccB) acc_b[m][c] = 0.0f;
        }
    auto mfma_update = [](float (&acc)[D], float row_sum, const float (&b)[D / 4]) {
#pragma unroll
        for (int c = 0; c < D / 4; ++c) {
            f32x4_t r = {acc[4 * c], acc[4 * c + 1], acc[4 * c + 2], acc[4 * c + 3]};
            r = __builtin_amdgcn_mfma_f32_4x4x1f32(row_sum, b[c], r, 0, 0, 0);
            acc[4 * c] = r[0]; acc[4 * c + 1] = r[1]; acc[4 * c + 2] = r[2]; acc[4 * c + 3] = r[3];
        }
    };
    // per-axis constants, kept in scalar registers
    float half_rows[ND], upper[ND];
#pragma unroll
    for (int n = 0; n < ND; ++n) {
        half_rows[n] = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(static_cast<float>(a.rows[n] / 2))));
        upper[n] = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(crse_upper(a.rows[n]))));
    }
    const int copy = lane & (kCopies - 1);

    const int2 *unit_list = reinterpret_cast<const int2 *>(a.units + units_list_index(H));
    const int total_units = __builtin_amdgcn_readfirstlane(a.units[units_total_index(H)]);
    int *counters = a.units + (KIND * H + h) * kQueues * kCounterStride;

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
        const int2 desc = unit_list[unit];
        const int w = __builtin_amdgcn_readfirstlane(desc.x);
        const int chunk = __builtin_amdgcn_readfirstlane(desc.y) & 0xffff;
        const int seg = __builtin_amdgcn_readfirstlane(desc.y) >> 16;   // segment of 64 streamed voxels (windows > 64)
        const int n_w = __builtin_amdgcn_readfirstlane(a.w_sizes[w]);
        const int s0 = __builtin_amdgcn_readfirstlane(a.w2n[w]);
        const int gs = n_w <= 32 ? 32 : 64;
        const int ng = 64 / gs;
        const int grp = lane / gs;
        const int own = chunk * kChunk + (lane - grp * gs);
        const bool own_valid = own < n_w;
        const int own_in = min(own, n_w - 1);
        // records of this window and head in the pair store; a window beyond the store contributes nothing
        const int64_t before = a.pos_base[s0];
        const int64_t before_u = (static_cast<int64_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(before >> 32))) << 32) |
                                 static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(before)));
        const bool fits = before_u + static_cast<int64_t>(n_w) * n_w <= a.pairs;
        const int64_t stored_at = static_cast<int64_t>(h) * a.pairs + before_u + own_in;
        float own_c[ND];
#pragma unroll
        for (int n = 0; n < ND; ++n) own_c[n] = a.n_coords[static_cast<int64_t>(s0 + own_in) * ND + n];

        // the unit's steps: the whole window, or the segment's 64 streamed voxels (one per step: ng = 1 there)
        const int it_begin = seg * kChunk;
        const int steps = n_w > kChunk ? min(n_w, it_begin + kChunk) : (n_w + ng - 1) / ng;
        // The inputs of step `it` for this lane's group (streamed element st = it ng + grp): the streamed rows and
        // coordinates are fetched one step ahead, the lane's records kPrefetch steps ahead.  Every load of the loop is
        // unconditional (clamped positions; what lies past the end is masked where it is used), so the waits count
        // loads statically and a step waits for the oldest record only.
        constexpr int kPrefetch = 4;
        struct StepIn {
            Slice<T, D> x, y;
            float c[ND];
        };
        auto fetch = [&](int it, int st_row, StepIn &in) {
            const int st = min(it * ng + grp, n_w - 1);
            in.x.load(gx + static_cast<int64_t>(st_row) * HD + h * D);
            if constexpr (kAccB) in.y.load(gy + static_cast<int64_t>(st_row) * HD + h * D);
#pragma unroll
            for (int n = 0; n < ND; ++n) in.c[n] = a.n_coords[static_cast<int64_t>(s0 + st) * ND + n];
        };
        // a window beyond the store reads the first record of the head instead (never used: `fits` masks it)
        const int64_t rec_base = fits ? stored_at : static_cast<int64_t>(h) * a.pairs;
        const int rec_stride = fits ? n_w : 0;
        auto fetch_record = [&](int it) {
            const int st = min(it * ng + grp, n_w - 1);
            const int64_t rec_at = rec_base + static_cast<int64_t>(st) * rec_stride;
            float2 rec = make_float2(0.0f, 0.0f);
            if constexpr (KIND == 1) rec = a.pd[rec_at];
            else if constexpr (KIND == 2) rec.x = a.pd[rec_at].x;
            else if constexpr (KIND == 3) rec.x = a.pd[rec_at].y;
            else rec.x = a.dl_t[rec_at];
            return rec;
        };
        // the next unit's ticket, drawn here: its round trip overlaps the unit's first loads
        if (lane == 0) drawn = atomicAdd(counters + queue * kCounterStride, 1);
        StepIn next;
        float2 rec_ahead[kPrefetch];
#pragma unroll
        for (int e = 0; e < kPrefetch; ++e) rec_ahead[e] = fetch_record(it_begin + e);
        int row_after = a.n2n[s0 + min((it_begin + 1) * ng + grp, n_w - 1)];   // row of the second step's element
        fetch(it_begin, a.n2n[s0 + min(it_begin * ng + grp, n_w - 1)], next);
        for (int it = it_begin; it < steps; ++it) {
            const StepIn cur = next;
            const bool have = own_valid && fits && it * ng + grp < n_w;
            const float2 rec = rec_ahead[0];
#pragma unroll
            for (int e = 0; e + 1 < kPrefetch; ++e) rec_ahead[e] = rec_ahead[e + 1];
            rec_ahead[kPrefetch - 1] = fetch_record(it + kPrefetch);
            {
                const int row_next = row_after;
                row_after = a.n2n[s0 + min((it + 2) * ng + grp, n_w - 1)];
                fetch(it + 1, row_next, next);
            }
            // dl: the value of the first histogram (P for the dTv half, whose fixed-point scale is constant)
            const float dl = have ? rec.x : 0.0f, p = have ? rec.y : 0.0f;
            const float amax = kFromP ? 1.0f : group_max_nonneg(fabsf(dl), ng == 2, grp);
            const int qd = kFromP ? __float2int_rn(dl * kFixP)
                                  : __float2int_rn(dl * (amax > 0.0f ? kFixL * __builtin_amdgcn_rcpf(amax) : 0.0f));
            if constexpr (kAccB) {
                const int qp = __float2int_rn(p * kFixP);
                const unsigned long long both =
                    (static_cast<unsigned long long>(static_cast<unsigned>(qd)) << 32) + static_cast<unsigned>(qp);
                if (both != 0) {
#pragma unroll
                    for (int n = 0; n < ND; ++n) {
                        const float ci = KEY_OWNED ? cur.c[n] : own_c[n], cj = KEY_OWNED ? own_c[n] : cur.c[n];
                        atomicAdd(hist_ab + (grp * kFlat + a.base[n] + crse_row(ci, cj, half_rows[n], upper[n])) * kCopies + copy, both);
                    }
                }
            } else {
                if (qd != 0) {
#pragma unroll
                    for (int n = 0; n < ND; ++n) {
                        const float ci = KEY_OWNED ? cur.c[n] : own_c[n], cj = KEY_OWNED ? own_c[n] : cur.c[n];
                        atomicAdd(hist_a + (grp * kFlat + a.base[n] + crse_row(ci, cj, half_rows[n], upper[n])) * kCopies + copy, qd);
                    }
                }
            }
            wave_lds_fence();
            for (int g = 0; g < ng; ++g) {
                const int src = __builtin_amdgcn_readfirstlane(g * gs);
                const float sc = kFromP ? 1.0f / kFixP : lane_value(amax, src) * (1.0f / kFixL);
                const Slice<T, D> sx = cur.x.lane(src);
                float bx[D / 4], by[D / 4];
                if constexpr (kMfmaUpdate) sx.quad_channels(lane, bx);
                if constexpr (kAccB) {
                    const Slice<T, D> sy = cur.y.lane(src);
                    if constexpr (kMfmaUpdate) sy.quad_channels(lane, by);
#pragma unroll
                    for (int m = 0; m < BLK; ++m) {
                        // both copies of the row in one 16-byte read; the halves add without carry (see above)
                        uint4 *cell = reinterpret_cast<uint4 *>(hist_ab + (g * kFlat + m * 64 + lane) * kCopies);
                        const uint4 two = *cell;
                        *cell = make_uint4(0, 0, 0, 0);
                        const unsigned long long both = ((static_cast<unsigned long long>(two.y) << 32) | two.x) +
                                                        ((static_cast<unsigned long long>(two.w) << 32) | two.z);
                        const float gsum = static_cast<float>(static_cast<int>(both >> 32)) * sc;
                        const float psum = static_cast<float>(static_cast<unsigned>(both)) * (1.0f / kFixP);
                        if constexpr (kMfmaUpdate) {
                            mfma_update(acc_a[m], gsum, bx);
                            mfma_update(acc_b[m], psum, by);
                        } else {
                            sx.fma_to(acc_a[m], gsum);
                            sy.fma_to(acc_b[m], psum);
                        }
                    }
                } else {
#pragma unroll
                    for (int m = 0; m < BLK; ++m) {
                        int4 *cell = reinterpret_cast<int4 *>(hist_a + (g * kFlat + m * 64 + lane) * kCopies);
                        const int4 four = *cell;
                        *cell = make_int4(0, 0, 0, 0);
                        const int cells = four.x + four.y + four.z + four.w;
                        const float gsum = (kFromP ? static_cast<float>(static_cast<unsigned>(cells)) : static_cast<float>(cells)) * sc;
                        if constexpr (kMfmaUpdate) mfma_update(acc_a[m], gsum, bx);
                        else sx.fma_to(acc_a[m], gsum);
                    }
                }
            }
            wave_lds_fence();
        }
    }

    float *slot = a.tgrad + (static_cast<size_t>(blockIdx.x) * kBwdWaves + wave) * (2 * kFlat * D);
#pragma unroll
    for (int m = 0; m < BLK; ++m) {
        if constexpr (kMfmaUpdate) {
#pragma unroll
            for (int c = 0; c < D / 4; ++c) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const size_t at = static_cast<size_t>(m * 64 + (lane & ~3) + i) * D + 4 * c + (lane & 3);
                    slot[at] = acc_a[m][4 * c + i];
                    if constexpr (kAccB) slot[static_cast<size_t>(kFlat) * D + at] = acc_b[m][4 * c + i];
                }
            }
        } else {
            const int row = m * 64 + lane;
            store_row<D>(slot + static_cast<size_t>(row) * D, acc_a[m]);
            if constexpr (kAccB) store_row<D>(slot + static_cast<size_t>(kFlat + row) * D, acc_b[m]);
        }
    }
}

// Sums the per-wavefront table gradients of a sweep over the wavefronts of each head.  One wavefront per (kind, flat
// row, head): its lanes are the D channels of the row times 64 / D shares of the head's slots, which they read 4 D
// bytes at a time and add up by shuffles at the end.  dst_a / dst_b: the gradient tables of kind 0 / 1 (null = not
// produced).
__global__ __launch_bounds__(256) void bwd_reduce_tables_kernel(BwdArgs a, float *dst_a, float *dst_b, int flat_rows,
                                                                 int groups)
{
    const int H = a.H, D = a.D;
    const int lane = threadIdx.x & 63;
    const int item = blockIdx.x * (blockDim.x / 64) + (threadIdx.x >> 6);   // (kind, row, head)
    if (item >= 2 * a.total_rows * H) return;
    const int kind = item / (a.total_rows * H);
    float *dst = kind == 0 ? dst_a : dst_b;
    if (!dst) return;
    const int e = item - kind * a.total_rows * H;
    const int h = e % H, row = e / H;
    const int c = lane % D, share = lane / D, shares = 64 / D;
    const size_t slot_floats = 2 * static_cast<size_t>(flat_rows) * D;
    const size_t in_slot = (static_cast<size_t>(kind) * flat_rows + row) * D + c;
    // workgroup b of the sweep serves head (b / kQueues) % H: the head's slots are those of workgroups
    // (set * H + h) * kQueues + x, x < kQueues, four wavefronts each
    const int sets = groups / (H * kQueues);
    const int head_slots = sets * kQueues * kBwdWaves;
    float sum = 0.0f;
    for (int x = share; x < head_slots; x += shares) {
        const int set = x / (kQueues * kBwdWaves), in_set = x - set * (kQueues * kBwdWaves);
        const size_t slot = (static_cast<size_t>(set) * H + h) * (kQueues * kBwdWaves) + in_set;
        sum += a.tgrad[slot * slot_floats + in_slot];
    }
    for (int other = D; other < 64; other <<= 1) sum += __shfl_xor(sum, other);
    // the caller's pair count was too small for the window set: windows were skipped, so no sum is valid
    if (a.pairs > 0 && a.units[units_total_index(H) + 1]) sum = __int_as_float(0x7fc00000);
    if (share == 0) dst[(static_cast<size_t>(row) * H + h) * D + c] = sum;
}


// ---- the general form ---------------------------------------------------------------------------------------
// Shapes that the register-blocked kernels above do not cover - head_dim 32, or more than 64 table rows per axis
// on average (quant 8 with wide windows) - in the manner of the reference (Swin3D/src/attn/self_attn_aio_bwd.cu:
// 197-509, one thread per term and a global atomic for each): a thread owns one (window-sorted position, head),
// walks the keys of its window, keeps dq_i in registers and adds the other terms atomically - dk_j and dv_j into
// fp32 accumulators in global memory that a second kernel rounds to the output type (the lanes of a wavefront start
// at different keys, so that they do not meet on one row), the table gradients into a copy of the head's three
// tables in LDS (a workgroup serves one head and leaves its sums with global atomics at the end; kLdsTables = false,
// for tables beyond 160 KB per head: global atomics for every term).  No work list; the order of the atomic adds
// varies, so only dq is the same bits on every call.  Bound by the LDS atomics (27 D per pair and head): 205 ms for
// 200 000 voxels in windows of 5 at 6 heads of 32 channels, 11.5 ms for 50 000 voxels at window 7, quant 8, 6 heads
// of 8 with position tables only - some fifty times the forms above per pair; it exists so that every shape the
// forward takes has a backward.  T: type of the feature rows, TT: of the tables.
constexpr int kGeneralThreads = 256;

template <typename T, typename TT, int D, bool kLdsTables>
__global__ __launch_bounds__(kGeneralThreads) void attn_bwd_general_kernel(BwdArgs a, float *dk_acc, float *dv_acc)
{
    extern __shared__ float general_tables[];      // [flat row][q-side, k-side, v-side][D] sums of this workgroup
    const int H = a.H, nd = a.nd;
    const int64_t HD = static_cast<int64_t>(H) * D;
    const int h = blockIdx.x % H;
    const int slot = blockIdx.x / H, slots = gridDim.x / H;
    const T *gq = static_cast<const T *>(a.q), *gk = static_cast<const T *>(a.k), *gv = static_cast<const T *>(a.v);
    const T *ggo = static_cast<const T *>(a.dout);
    const TT *tq = static_cast<const TT *>(a.table_q), *tk = static_cast<const TT *>(a.table_k);
    const TT *tv = static_cast<const TT *>(a.table_v);
    if constexpr (kLdsTables) {
        for (int t = threadIdx.x; t < a.total_rows * 3 * D; t += kGeneralThreads) general_tables[t] = 0.0f;
        __syncthreads();
    }
    // chunks of kGeneralThreads consecutive window-sorted positions, dealt to the workgroups of the head in turn
    const int64_t chunks = (a.N + kGeneralThreads - 1) / kGeneralThreads;
    for (int64_t chunk = slot; chunk < chunks; chunk += slots) {
        const int64_t pos = chunk * kGeneralThreads + threadIdx.x;
        if (pos >= a.N) continue;
        // the window of the position: the last one that starts at or before it
        int64_t lo = 0, hi = a.W - 1;
        while (lo < hi) {
            const int64_t mid = (lo + hi + 1) >> 1;
            if (a.w2n[mid] <= pos) lo = mid;
            else hi = mid - 1;
        }
        const int n_w = a.w_sizes[lo], s0 = a.w2n[lo];
        const int i = static_cast<int>(pos - s0);
        if (i >= n_w) continue;      // positions that no window covers (none for a valid index)
        const int qi = a.n2n[pos];
        const int64_t q_at = static_cast<int64_t>(qi) * HD + h * D;
        float q[D], go[D], dq[D], ci[kMaxAxes];
#pragma unroll
        for (int c = 0; c < D; c += 8) {
            load_row<8>(gq + q_at + c, q + c);
            load_row<8>(ggo + q_at + c, go + c);
        }
#pragma unroll
        for (int c = 0; c < D; ++c) dq[c] = 0.0f;
        for (int n = 0; n < nd; ++n) ci[n] = a.n_coords[pos * nd + n];
        const float m_i = a.out_max[static_cast<int64_t>(qi) * H + h];
        const float inv_i = 1.0f / a.out_sum[static_cast<int64_t>(qi) * H + h];
        const float delta_i = a.delta[static_cast<int64_t>(qi) * H + h];
        for (int step = 0; step < n_w; ++step) {
            int j = i + step;                      // every query starts at its own key
            if (j >= n_w) j -= n_w;
            const int kj = a.n2n[s0 + j];
            const int64_t k_at = static_cast<int64_t>(kj) * HD + h * D;
            float kr[D], vs[D], tqs[D], tks[D];
#pragma unroll
            for (int c = 0; c < D; c += 8) {
                load_row<8>(gk + k_at + c, kr + c);
                load_row<8>(gv + k_at + c, vs + c);
            }
#pragma unroll
            for (int c = 0; c < D; ++c) tqs[c] = tks[c] = 0.0f;
            int row[kMaxAxes];
            for (int n = 0; n < nd; ++n) {
                const float cj = a.n_coords[static_cast<int64_t>(s0 + j) * nd + n];
                row[n] = a.base[n] + crse_row(ci[n], cj, static_cast<float>(a.rows[n] / 2), crse_upper(a.rows[n]));
                const int64_t row_at = static_cast<int64_t>(row[n]) * HD + h * D;
#pragma unroll
                for (int c = 0; c < D; c += 8) {
                    float x[8], y[8], z[8];
                    load_row<8>(tq + row_at + c, x);
                    load_row<8>(tk + row_at + c, y);
                    load_row<8>(tv + row_at + c, z);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        tqs[c + e] += x[e];
                        tks[c + e] += y[e];
                        vs[c + e] += z[e];
                    }
                }
            }
            float logit = 0.0f, dp = 0.0f;
#pragma unroll
            for (int c = 0; c < D; ++c) {
                logit += q[c] * (kr[c] + tqs[c]) + kr[c] * tks[c];
                dp += go[c] * vs[c];
            }
            const float p = __expf(logit - m_i) * inv_i;
            const float dl = p * (dp - delta_i);
#pragma unroll
            for (int c = 0; c < D; ++c) {
                dq[c] += dl * (kr[c] + tqs[c]);
                atomicAdd(dk_acc + k_at + c, dl * (q[c] + tks[c]));
                atomicAdd(dv_acc + k_at + c, p * go[c]);
            }
            for (int n = 0; n < nd; ++n) {
                if constexpr (kLdsTables) {
                    float *cell = general_tables + row[n] * 3 * D;
#pragma unroll
                    for (int c = 0; c < D; ++c) {
                        atomicAdd(cell + c, dl * q[c]);
                        atomicAdd(cell + D + c, dl * kr[c]);
                        atomicAdd(cell + 2 * D + c, p * go[c]);
                    }
                } else {
                    const int64_t row_at = static_cast<int64_t>(row[n]) * HD + h * D;
#pragma unroll
                    for (int c = 0; c < D; ++c) {
                        atomicAdd(a.dtq + row_at + c, dl * q[c]);
                        atomicAdd(a.dtk + row_at + c, dl * kr[c]);
                        atomicAdd(a.dtv + row_at + c, p * go[c]);
                    }
                }
            }
        }
#pragma unroll
        for (int c = 0; c < D; c += 8) store_row<8>(static_cast<T *>(a.dq) + q_at + c, dq + c);
    }
    if constexpr (kLdsTables) {
        __syncthreads();
        for (int t = threadIdx.x; t < a.total_rows * 3 * D; t += kGeneralThreads) {
            const int r = t / (3 * D), rest = t - r * (3 * D), which = rest / D, c = rest - which * D;
            float *dst = which == 0 ? a.dtq : which == 1 ? a.dtk : a.dtv;
            const float sum = general_tables[t];
            if (sum != 0.0f) atomicAdd(dst + static_cast<int64_t>(r) * HD + h * D + c, sum);
        }
    }
}

__global__ void bwd_general_zero_kernel(float *x, int64_t count)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; t < count; t += stride) x[t] = 0.0f;
}

// dk, dv from their fp32 accumulators, eight channels per thread
template <typename T>
__global__ void bwd_general_store_kernel(BwdArgs a, const float *dk_acc, const float *dv_acc)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    const int64_t pieces = a.N * a.H * a.D / 8;
    for (int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; t < pieces; t += stride) {
        float x[8], y[8];
        load_row<8>(dk_acc + 8 * t, x);
        load_row<8>(dv_acc + 8 * t, y);
        store_row<8>(static_cast<T *>(a.dk) + 8 * t, x);
        store_row<8>(static_cast<T *>(a.dv) + 8 * t, y);
    }
}

// head_dim 32, or more table rows than the register blocks of the table-gradient kernels cover
inline bool bwd_general_form(int H, int D, int nd, int64_t table_len)
{
    return D == 32 || table_len / (static_cast<int64_t>(H) * D) > 64 * nd;
}
size_t bwd_general_acc_bytes(int64_t N, int H, int D) { return align_up(sizeof(float) * static_cast<size_t>(N) * H * D, 256); }

template <typename T, typename TT, int D>
int launch_bwd_general_dim(const BwdArgs &a, float *dk_acc, float *dv_acc, hipStream_t stream)
{
    const int64_t work = a.N * a.H + a.table_len;
    const int prep_grid = static_cast<int>(ceil_div(work, 256) < 4096 ? ceil_div(work, 256) : 4096);
    hipLaunchKernelGGL(bwd_prepare_kernel<T>, dim3(static_cast<unsigned>(prep_grid)), dim3(256), 0, stream, a);
    const int64_t count = 2 * static_cast<int64_t>(bwd_general_acc_bytes(a.N, a.H, a.D) / sizeof(float));
    hipLaunchKernelGGL(bwd_general_zero_kernel, dim3(2048), dim3(256), 0, stream, dk_acc, count);
    S3D_HIP_CHECK(hipGetLastError());
    // workgroups: about four per CU, a whole number per head, no more than the chunks of positions give work to
    const size_t lds = sizeof(float) * static_cast<size_t>(a.total_rows) * 3 * D;
    const int64_t chunks = (a.N + kGeneralThreads - 1) / kGeneralThreads;
    int device = 0, cus = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus < 1)
        cus = 256;
    int64_t per_head = (4 * cus + a.H - 1) / a.H;
    if (per_head > chunks) per_head = chunks;
    if (per_head < 1) per_head = 1;
    const unsigned grid = static_cast<unsigned>(per_head * a.H);
    if (lds <= 160 * 1024) {
        auto kernel = attn_bwd_general_kernel<T, TT, D, true>;
        S3D_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(kGeneralThreads), lds, stream, a, dk_acc, dv_acc);
    } else {
        hipLaunchKernelGGL((attn_bwd_general_kernel<T, TT, D, false>), dim3(grid), dim3(kGeneralThreads), 0, stream, a,
                           dk_acc, dv_acc);
    }
    hipLaunchKernelGGL(bwd_general_store_kernel<T>, dim3(2048), dim3(256), 0, stream, a, dk_acc, dv_acc);
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}

template <typename T, typename TT>
int launch_bwd_general(const BwdArgs &a, float *dk_acc, float *dv_acc, hipStream_t stream)
{
    switch (a.D) {
    case 8: return launch_bwd_general_dim<T, TT, 8>(a, dk_acc, dv_acc, stream);
    case 16: return launch_bwd_general_dim<T, TT, 16>(a, dk_acc, dv_acc, stream);
    case 32: return launch_bwd_general_dim<T, TT, 32>(a, dk_acc, dv_acc, stream);
    default: return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_bwd: head_dim %d (8, 16 or 32)", a.D);
    }
}

template <typename T, int D>
size_t bwd_lds_bytes(const BwdArgs &a, int kinds, int blk)
{
    return align_up(sizeof(T) * static_cast<size_t>(a.total_rows) * table_row_stride<T, D>(), 16) +
           sizeof(int) * kBwdWaves * kinds * 2 * static_cast<size_t>(blk) * 64;
}

template <typename T, int D, int ND, bool KEY_OWNED, int MODE, int BLK>
int launch_sweep_blk(const BwdArgs &a, int grid, hipStream_t stream)
{
    constexpr bool need_dl = !KEY_OWNED || MODE != 2;
    constexpr int kinds = (need_dl ? 1 : 0) + ((KEY_OWNED && MODE != 1) ? 1 : 0);
    auto kernel = attn_bwd_sweep_kernel<T, D, ND, KEY_OWNED, MODE, BLK>;
    const size_t lds = bwd_lds_bytes<T, D>(a, kinds, BLK);
    if (lds > 160 * 1024)
        return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_bwd: the tables of one head (%d rows x %d) do not fit LDS",
                    a.total_rows, a.D);
    S3D_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    hipLaunchKernelGGL(bwd_reset_counters_kernel, dim3(1), dim3(64), 0, stream, a);
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(kBwdThreads), lds, stream, a);
    S3D_HIP_CHECK(hipGetLastError());
    float *dst_a = need_dl ? (KEY_OWNED ? a.dtq : a.dtk) : nullptr;
    float *dst_b = (KEY_OWNED && MODE != 1) ? a.dtv : nullptr;
    const int items = 2 * a.total_rows * a.H;
    hipLaunchKernelGGL(bwd_reduce_tables_kernel, dim3(static_cast<unsigned>((items + 3) / 4)), dim3(256), 0, stream,
                       a, dst_a, dst_b, BLK * 64, grid);
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}

// workgroups of a sweep: whole sets of (XCDs x heads), about two per CU (a workgroup serves one head for its
// whole life).  At head_dim 16 only one fits a CU at a time; the others start as the first heads run out of
// units and go to the heads that still have some, which measured 5 % faster than a grid of one per CU (whole
// sets leave 16 of 256 CUs without a workgroup at six heads).
constexpr int kTablesPerCu = 4;   // workgroups per CU of the table-gradient kernels, at most
int bwd_grid(int H, int per_cu = 2)
{
    int device = 0, cus = 256;
    if (hipGetDevice(&device) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && v > 0) cus = v;
    }
    const int set = kQueues * H;
    return (per_cu * cus / set > 0 ? per_cu * cus / set : 1) * set;
}

template <typename T, int D, int ND, int KIND, int BLK>
int launch_tables_blk(const BwdArgs &a, int grid, hipStream_t stream)
{
    constexpr int kinds = KIND == 1 ? 2 : 1;
    auto kernel = attn_bwd_tables_kernel<T, D, ND, KIND, BLK>;
    constexpr int copies = KIND == 1 ? 2 : 4;
    const size_t lds = sizeof(int) * kBwdWaves * kinds * 2 * static_cast<size_t>(BLK) * 64 * copies;
    S3D_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    // as many workgroups per CU as registers and histograms allow (at most kTablesPerCu: the slots of the
    // workspace), in whole sets of (XCDs x heads)
    int fit = 0;
    S3D_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&fit, reinterpret_cast<const void *>(kernel), kBwdThreads, lds));
    grid = bwd_grid(a.H, fit < 1 ? 1 : fit > kTablesPerCu ? kTablesPerCu : fit);
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(kBwdThreads), lds, stream, a);
    S3D_HIP_CHECK(hipGetLastError());
    const int items = 2 * a.total_rows * a.H;
    float *first = KIND == 0 ? a.dtk : KIND == 3 ? a.dtv : a.dtq;
    hipLaunchKernelGGL(bwd_reduce_tables_kernel, dim3(static_cast<unsigned>((items + 3) / 4)), dim3(256), 0, stream,
                       a, first, KIND == 1 ? a.dtv : nullptr, BLK * 64, grid);
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}

template <typename T, int D, int ND, int KIND>
int launch_tables(const BwdArgs &a, int grid, hipStream_t stream)
{
    const int blocks = (a.total_rows + 63) / 64;
    constexpr int kSmall = 2 * ND / 3;
    if constexpr (ND == 9) {
        if (blocks <= 5) return launch_tables_blk<T, D, ND, KIND, 5>(a, grid, stream);
    }
    if (blocks <= kSmall) return launch_tables_blk<T, D, ND, KIND, kSmall>(a, grid, stream);
    return launch_tables_blk<T, D, ND, KIND, ND>(a, grid, stream);
}

// table-gradient registers for as many 64-row blocks as the head's flat table has: 5 for window 5 at four steps
// per cell with all nine axes (312 rows), 6 for window 7 (360 rows); every block costs 2 * D registers and a
// share of the per-step histogram flush
template <typename T, int D, int ND, bool KEY_OWNED, int MODE>
int launch_sweep(const BwdArgs &a, int grid, hipStream_t stream)
{
    const int blocks = (a.total_rows + 63) / 64;
    constexpr int kSmall = 2 * ND / 3;
    if constexpr (ND == 9) {
        if (blocks <= 5) return launch_sweep_blk<T, D, ND, KEY_OWNED, MODE, 5>(a, grid, stream);
    }
    if (blocks <= kSmall) return launch_sweep_blk<T, D, ND, KEY_OWNED, MODE, kSmall>(a, grid, stream);
    return launch_sweep_blk<T, D, ND, KEY_OWNED, MODE, ND>(a, grid, stream);
}

// T is the type of the feature rows (q, k, v, out, dout, dq, dk, dv); the tables have it too unless dtype says
// that they are fp32 beside fp16 rows: the pair sweeps, the only kernels of the pair form that read tables, are
// chosen by dtype, the other kernels of that form read rows and records only.
template <typename T, int D, int ND>
int launch_bwd(const BwdArgs &a, const BwdPairArgs &pairs, int dtype, hipStream_t stream)
{
    const int64_t work = a.N * a.H + a.table_len;
    const int prep_grid = static_cast<int>(ceil_div(work > 0 ? work : 1, 256) < 4096 ? ceil_div(work > 0 ? work : 1, 256) : 4096);
    hipLaunchKernelGGL(bwd_prepare_kernel<T>, dim3(static_cast<unsigned>(prep_grid)), dim3(256), 0, stream, a);
    S3D_HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL(bwd_units_kernel, dim3(1), dim3(1024), 0, stream, a);
    S3D_HIP_CHECK(hipGetLastError());
    const int grid = bwd_grid(a.H);
    if (a.pairs > 0) {
        // dq, dk, dv by the pair sweeps, which leave dL and P of every (pair, head); the table gradients from those
        if (int rc = launch_attn_bwd_pairs(pairs, dtype, stream)) return rc;
        // head_dim 16: dTq and dTv as kernels of their own, two wavefronts per SIMD each instead of one for both
        // (2.37 -> 2.27 ms at the 6-head window-7 layer; at head_dim 8 the split measured +8 %)
        if constexpr (D > 8) {
            if (int rc = launch_tables<T, D, ND, 2>(a, grid, stream)) return rc;
            if (int rc = launch_tables<T, D, ND, 3>(a, grid, stream)) return rc;
        } else {
            if (int rc = launch_tables<T, D, ND, 1>(a, grid, stream)) return rc;
        }
        return launch_tables<T, D, ND, 0>(a, grid, stream);
    }
    // one key-owned sweep for dk, dv and both of its table gradients; at head_dim 16 with more than six 64-row
    // blocks of table rows (quant 8) the two sets of accumulation registers no longer fit one wavefront
    // (250-320 registers spilled) and the sweep runs as its two halves
    if (D <= 8 || (a.total_rows + 63) / 64 <= 6) {
        if (int rc = launch_sweep<T, D, ND, true, 0>(a, grid, stream)) return rc;
    } else {
        if (int rc = launch_sweep<T, D, ND, true, 1>(a, grid, stream)) return rc;
        if (int rc = launch_sweep<T, D, ND, true, 2>(a, grid, stream)) return rc;
    }
    return launch_sweep<T, D, ND, false, 0>(a, grid, stream);
}

int fill_bwd_axes(BwdArgs &a, const int32_t *table_sizes, int nd, int64_t table_len)
{
    const int64_t hd = static_cast<int64_t>(a.H) * a.D;
    int64_t total = 0;
    int base = 0;
    for (int n = 0; n < nd; ++n) {
        const int64_t size = table_sizes[n];
        if (size <= 0 || size % hd != 0)
            return fail(S3D_ERR_BAD_SHAPE, "s3d_attn_bwd: table_sizes[%d] = %lld is not a positive multiple of "
                        "H*D = %lld", n, (long long)size, (long long)hd);
        total += size;
        a.rows[n] = static_cast<int32_t>(size / hd);
        a.base[n] = base;
        base += a.rows[n];
    }
    for (int n = nd; n < kMaxAxes; ++n) a.rows[n] = a.base[n] = 0;
    if (total != table_len)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_attn_bwd: sum(table_sizes) = %lld differs from table_len = %lld",
                    (long long)total, (long long)table_len);
    a.total_rows = base;
    return S3D_OK;
}

// units: one per (window, chunk), and with a pair count one per (window, chunk, segment): the sum over the windows of
// ceil(n / 64)^2 <= n^2 / 4096 + n / 32 + 1
size_t bwd_units_bytes(int64_t W, int64_t N, int H, int64_t pairs)
{
    const size_t max_units = static_cast<size_t>(W > 0 ? W : 1) + static_cast<size_t>(N > 0 ? N : 0) / 32 +
                             static_cast<size_t>(pairs > 0 ? pairs : 0) / 4096;
    return align_up(sizeof(int32_t) * (units_list_index(H) + 2 * max_units), 256);
}

size_t bwd_delta_bytes(int64_t N, int H) { return align_up(sizeof(float) * static_cast<size_t>(N) * H, 256); }

// one slot per wavefront of a sweep: two kinds x (64 rows per axis at most) x D floats
size_t bwd_tgrad_bytes(int H, int D, int nd)
{
    return align_up(sizeof(float) * static_cast<size_t>(bwd_grid(H, kTablesPerCu)) * kBwdWaves * 2 * (64 * nd) * D, 256);
}

// the pair path's part of the workspace: window pair offsets, (dL, P) and transposed dL of every (pair, head), and
// the pair sweeps' work list
size_t bwd_pos_base_bytes(int64_t N) { return align_up(sizeof(int64_t) * static_cast<size_t>(N > 0 ? N : 1), 256); }
size_t bwd_pd_bytes(int H, int64_t pairs) { return align_up(sizeof(float2) * static_cast<size_t>(H) * pairs, 256); }
size_t bwd_dlt_bytes(int H, int64_t pairs) { return align_up(sizeof(float) * static_cast<size_t>(H) * pairs, 256); }
// the last part of every form's workspace: the identity row map that stands in for a null n2n
size_t bwd_row_map_bytes(int64_t N) { return align_up(sizeof(int32_t) * static_cast<size_t>(N > 0 ? N : 1), 256); }

__global__ void bwd_identity_rows_kernel(int32_t *map, int64_t n)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) map[i] = static_cast<int32_t>(i);
}

}  // namespace
}  // namespace s3d

extern "C" __attribute__((visibility("default"))) size_t s3d_attn_bwd_workspace_bytes(int32_t H, int32_t D,
                                                                                      int32_t nd, int64_t table_len,
                                                                                      int64_t N, int64_t W,
                                                                                      int64_t pairs)
{
    using namespace s3d;
    if (H < 1 || D < 1 || nd < 1 || nd > kMaxAxes || table_len < 1 || N < 0 || W < 0 || pairs < 0) return 0;
    if (bwd_general_form(H, D, nd, table_len))
        return bwd_units_bytes(W, N, H, 0) + bwd_delta_bytes(N, H) + 2 * bwd_general_acc_bytes(N, H, D) +
               bwd_row_map_bytes(N);
    size_t need = bwd_units_bytes(W, N, H, pairs) + bwd_delta_bytes(N, H) + bwd_tgrad_bytes(H, D, nd) +
                  bwd_pos_base_bytes(N) + bwd_row_map_bytes(N);
    if (pairs > 0)
        need += bwd_pd_bytes(H, pairs) + bwd_dlt_bytes(H, pairs) + align_up(attn_sweep_workspace_bytes(H, W, N), 256);
    return need;
}

extern "C" __attribute__((visibility("default"))) int s3d_attn_bwd(
    const void *q, const void *k, const void *v, const void *table_q, const void *table_k,
    const void *table_v, const int32_t *table_sizes, int32_t nd, int64_t table_len,
    const int32_t *w_sizes, const int32_t *w2n, const int32_t *n2n, const float *n_coords, const void *out,
    const float *out_max, const float *out_sum, const void *dout, void *dq, void *dk, void *dv,
    float *dtable_q, float *dtable_k, float *dtable_v, int64_t N, int32_t H, int32_t D, int64_t W,
    int64_t pairs, int32_t dtype, void *workspace, size_t workspace_bytes, void *stream)
{
    using namespace s3d;
    if (N < 0 || W < 0 || H < 1 || D < 1 || nd < 1 || table_len < 1 || pairs < 0)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_attn_bwd: bad sizes N=%lld W=%lld H=%d D=%d nd=%d table_len=%lld pairs=%lld",
                    (long long)N, (long long)W, H, D, nd, (long long)table_len, (long long)pairs);
    if (nd != 3 && nd != 6 && nd != 9)
        return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_bwd: %d cRSE axes (3, 6 or 9)", nd);
    if (D != 8 && D != 16 && D != 32) return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_bwd: head_dim %d (8, 16 or 32)", D);
    if (W > 0x7fffffffLL || N > 0x7fffffffLL || H > 65535)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_attn_bwd: N, W must fit 31 bits and H 16 bits");
    if (dtype != S3D_DTYPE_F32 && dtype != S3D_DTYPE_F16 && dtype != S3D_DTYPE_F32_F16_ROWS)
        return fail(S3D_ERR_BAD_DTYPE, "s3d_attn_bwd: dtype %d (0 = fp32, 1 = fp16, 2 = fp32 on fp16 rows)", dtype);
    const bool general = bwd_general_form(H, D, nd, table_len);
    if (dtype == S3D_DTYPE_F32_F16_ROWS && pairs == 0 && !general)
        return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_bwd: fp32 arithmetic on fp16 rows (dtype 2) needs the pair count; "
                    "without it pass fp32 copies of the rows with dtype 0");
    if (!table_sizes) return fail(S3D_ERR_NULL_POINTER, "s3d_attn_bwd: table_sizes (host) is null");
    BwdArgs a{};
    a.H = H;
    a.D = D;
    a.nd = nd;
    a.N = N;
    a.W = W;
    a.table_len = table_len;
    if (int rc = fill_bwd_axes(a, table_sizes, nd, table_len)) return rc;
    if (!dtable_q || !dtable_k || !dtable_v)
        return fail(S3D_ERR_NULL_POINTER, "s3d_attn_bwd: null table-gradient pointer");
    const size_t need = s3d_attn_bwd_workspace_bytes(H, D, nd, table_len, N, W, pairs);
    if (!workspace || workspace_bytes < need)
        return fail(S3D_ERR_WORKSPACE, "s3d_attn_bwd: workspace %zu B < required %zu B",
                    workspace ? workspace_bytes : size_t(0), need);
    if (N > 0 && W > 0 &&
        (!q || !k || !v || !table_q || !table_k || !table_v || !w_sizes || !w2n || !n_coords || !out ||
         !out_max || !out_sum || !dout || !dq || !dk || !dv))
        return fail(S3D_ERR_NULL_POINTER, "s3d_attn_bwd: null device pointer");
    if (!n2n && N > 0 && W > 0) {
        // rows in window order: the kernels read the identity map from the end of the workspace
        int32_t *map = reinterpret_cast<int32_t *>(static_cast<char *>(workspace) + need - bwd_row_map_bytes(N));
        hipLaunchKernelGGL(bwd_identity_rows_kernel, dim3(static_cast<unsigned>((N + 255) / 256)), dim3(256), 0,
                           static_cast<hipStream_t>(stream), map, N);
        S3D_HIP_CHECK(hipGetLastError());
        n2n = map;
    }
    a.q = q; a.k = k; a.v = v;
    a.table_q = table_q; a.table_k = table_k; a.table_v = table_v;
    a.dout = dout; a.out = out; a.out_max = out_max; a.out_sum = out_sum;
    a.w_sizes = w_sizes; a.w2n = w2n; a.n2n = n2n; a.n_coords = n_coords;
    a.dq = dq; a.dk = dk; a.dv = dv;
    a.dtq = dtable_q; a.dtk = dtable_k; a.dtv = dtable_v;
    a.units = static_cast<int32_t *>(workspace);
    if (general) {
        // the form for shapes outside the register-blocked kernels: units | delta | dk accumulator | dv accumulator
        hipStream_t gs = static_cast<hipStream_t>(stream);
        a.pairs = 0;
        if (N == 0 || W == 0) {
            a.N = 0;
            hipLaunchKernelGGL((bwd_prepare_kernel<float>), dim3(64), dim3(256), 0, gs, a);
            S3D_HIP_CHECK(hipGetLastError());
            return S3D_OK;
        }
        char *g_at = static_cast<char *>(workspace) + bwd_units_bytes(W, N, H, 0);
        a.delta = reinterpret_cast<float *>(g_at);
        g_at += bwd_delta_bytes(N, H);
        float *dk_acc = reinterpret_cast<float *>(g_at);
        float *dv_acc = reinterpret_cast<float *>(g_at + bwd_general_acc_bytes(N, H, D));
        switch (dtype) {
        case S3D_DTYPE_F32: return launch_bwd_general<float, float>(a, dk_acc, dv_acc, gs);
        case S3D_DTYPE_F16: return launch_bwd_general<__half, __half>(a, dk_acc, dv_acc, gs);
        default: return launch_bwd_general<__half, float>(a, dk_acc, dv_acc, gs);
        }
    }
    a.delta = reinterpret_cast<float *>(static_cast<char *>(workspace) + bwd_units_bytes(W, N, H, pairs));
    char *at = static_cast<char *>(workspace) + bwd_units_bytes(W, N, H, pairs) + bwd_delta_bytes(N, H);
    a.tgrad = reinterpret_cast<float *>(at);
    at += bwd_tgrad_bytes(H, D, nd);
    a.pos_base = reinterpret_cast<int64_t *>(at);
    at += bwd_pos_base_bytes(N);
    a.pairs = pairs;
    BwdPairArgs pr{};
    if (pairs > 0) {
        float2 *pd = reinterpret_cast<float2 *>(at);
        at += bwd_pd_bytes(H, pairs);
        float *dl_t = reinterpret_cast<float *>(at);
        at += bwd_dlt_bytes(H, pairs);
        a.pd = pd;
        a.dl_t = dl_t;
        pr.f.q = q; pr.f.k = k; pr.f.v = v;
        pr.f.row_stride = static_cast<int64_t>(H) * D;
        pr.f.table_q = table_q; pr.f.table_k = table_k; pr.f.table_v = table_v;
        pr.f.w_sizes = w_sizes; pr.f.w2n = w2n; pr.f.n2n = n2n;
        pr.f.n_coords = n_coords;
        pr.f.workspace = at;
        pr.f.H = H; pr.f.D = D; pr.f.nd = nd; pr.f.total_rows = a.total_rows;
        pr.f.N = N; pr.f.W = W;
        for (int n = 0; n < kMaxAxes; ++n) { pr.f.rows[n] = a.rows[n]; pr.f.base[n] = a.base[n]; }
        pr.dout = dout;
        pr.stat_max = out_max; pr.stat_sum = out_sum; pr.delta = a.delta;
        pr.dq = dq; pr.dk = dk; pr.dv = dv;
        pr.pos_base = a.pos_base;
        pr.pd = pd; pr.dl_t = dl_t; pr.pairs = pairs;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (N == 0 || W == 0) {
        // nothing to differentiate: the table gradients are zero
        a.N = 0;
        hipLaunchKernelGGL((bwd_prepare_kernel<float>), dim3(64), dim3(256), 0, s, a);
        S3D_HIP_CHECK(hipGetLastError());
        return S3D_OK;
    }
#define S3D_BWD_CASE(DD, NN)                                                              \
    if (D == DD && nd == NN)                                                              \
        return dtype == S3D_DTYPE_F32 ? launch_bwd<float, DD, NN>(a, pr, dtype, s) : launch_bwd<__half, DD, NN>(a, pr, dtype, s);
    S3D_BWD_CASE(8, 3) S3D_BWD_CASE(8, 6) S3D_BWD_CASE(8, 9)
    S3D_BWD_CASE(16, 3) S3D_BWD_CASE(16, 6) S3D_BWD_CASE(16, 9)
#undef S3D_BWD_CASE
    return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_bwd: D=%d nd=%d", D, nd);
}
