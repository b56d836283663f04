// Sparse-voxel windowed self-attention forward with cRSE tables: MFMA kernel (gfx950, fp16).
//
// A wavefront draws work items from a device-side queue.  An item is one 32-query x 32-key tile
// pair of a window and a group of heads; for the tile pair and each head of the group
//   S^T   = K Q^T                       one MFMA, lands directly in the logit registers
//   QT_n  = Tq_n Q^T,  KT_n = Tk_n K^T  per signal axis n, MFMA -> LDS ("every table row
//                                       against every query / key of the tile")
// so that the table terms of a pair's logit become two 4-byte LDS gathers per axis
//   L(i,j) = S(i,j) + sum_n QT_n[row_n(i,j)][i] + KT_n[j][row_n(i,j)]
// instead of 2*D-element table row gathers.  The value side uses the transposed trick:
//   sum_j P(i,j) Tv_n[row_n(i,j)] = sum_r H_n[r][i] Tv_n[r],  H_n[r][i] = sum_{j: row_n(i,j)=r} P(i,j)
// a per-query histogram of the softmax weights over table rows, followed by MFMAs against a
// transposed copy of the value table.  P V is an MFMA as well.
//
// The histogram is accumulated with INTEGER LDS atomics on 2^-24 fixed point (softmax weights
// are in [0,1], at most 32 of them meet in one bin): a wavefront's ds_add_u32 measured about
// 5 clocks of the LDS pipe (a 4-byte gather: 2.7), ds_add_f32 many times more.
//
// Lane layout = the 32x32 MFMA accumulator layout: lane l holds query i = l % 32 and, in
// register v, key j = 8*(v/4) + 4*(l/32) + v%4, so logits, softmax weights and the B operand
// of the value MFMAs never move between lanes.  QT / H are stored [row][query] (bank = query,
// conflict-free for any row pattern), KT is stored [key][row] (one key per half-wave: the
// gathers hit consecutive words of one row).
//
// The row indices depend on the pair only; they are computed once per item (fp32, in the
// reference's operation order, Swin3D/src/attn/attn_utils.cuh:444-450) and kept as bytes in
// registers across the heads of the item.  A window of at most 32 voxels is finished by its item;
// a larger one leaves one partial result (max, sum, unnormalised output) per key tile and head,
// which attn_merge_partials_kernel combines.
//
// Latency: an item is a long chain of small dependent steps, so every global load is issued
// one step ahead of its use (next head's q/k/v fragments, next axis' table fragments) and the
// transposed value table of all heads sits in LDS, shared by the wavefronts of the workgroup.
#include "attn_kernels.h"
#include "sweep_common.h"

namespace s3d {
namespace {

typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));

constexpr int kWaves = 8;             // wavefronts per workgroup (they share the value table in LDS)
constexpr int kTile = 32;             // queries / keys per tile
constexpr float kFix = 16777216.0f;   // 2^24 fixed point of the histogram
constexpr int kItemsPerWave = 2;      // heads are grouped so that a wavefront draws about this many items

// index (in ints) of the first work counter inside the item list: after the [W + 3] header, on a 256-byte boundary
__host__ __device__ inline size_t queue_counters_index(int64_t W)
{
    return (static_cast<size_t>(W > 0 ? W : 1) + 3 + 63) / 64 * 64;
}

// LDS operations of one wavefront execute in order; this only stops the compiler from moving
// LDS accesses across the point where lanes exchange data (global loads stay free to move).
__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
}

template <int D> struct Frag;
template <> struct Frag<8> {
    typedef h4 type;
    static __device__ __forceinline__ f16v mfma(h4 a, h4 b, f16v c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x8f16(a, b, c, 0, 0, 0);
    }
};
template <> struct Frag<16> {
    typedef h8 type;
    static __device__ __forceinline__ f16v mfma(h8 a, h8 b, f16v c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

// channels [ (D/2)*half, (D/2)*half + D/2 ) of one (row, head): what a lane feeds to the MFMA
template <int D>
__device__ __forceinline__ typename Frag<D>::type load_frag(const _Float16 *row_head, int half)
{
    return *reinterpret_cast<const typename Frag<D>::type *>(row_head + (D / 2) * half);
}

__device__ __forceinline__ int crse_row(float ci, float cj, int rows)
{
    float rel = ci - cj;
    rel = rel + static_cast<float>(rows / 2);
    rel = fminf(fmaxf(rel, 0.0f), static_cast<float>(rows));
    return min(static_cast<int>(rel), rows - 1);
}

// key index held by accumulator register v of a lane in half-wave `half`
__device__ __forceinline__ constexpr int key_of(int v, int half) { return 8 * (v / 4) + 4 * half + (v % 4); }

// RMAX: rows of the largest axis table rounded up to 16 (32, 48 or 64)
template <int RMAX> struct WaveLds {
    static constexpr int kTiles = (RMAX + kTile - 1) / kTile;  // 32-row MFMA tiles per axis table
    static constexpr int kQtRows = RMAX;                       // QT / H rows kept in LDS
    static constexpr int kKtStride = RMAX + 4;                 // words per key row of KT
    static constexpr int kCrd = kTile * kMaxAxes;
    static constexpr int kQt = kQtRows * kTile;                // QT[row][query], reused as H[row][query]
    static constexpr int kKt = kTile * kKtStride;
    static constexpr int kVt = kTile * 16 / 2;                 // V tile [key][D] in halves
    static constexpr int kWords = kCrd + kQt + kKt + kVt;
};

// TVT_LDS: the transposed value table of all heads is staged in LDS (it must fit next to the
// per-wavefront staging); otherwise its fragments are read from the L2-resident workspace copy.
template <int D, int ND, int RMAX, bool TVT_LDS>
__global__ __launch_bounds__(kWaves * 64) void attn_fwd_mfma_kernel(AttnArgs a)
{
    extern __shared__ float smem[];
    typedef typename Frag<D>::type frag_t;
    typedef WaveLds<RMAX> L;
    constexpr int kIdxWords = (16 * ND + 3) / 4;

    const int H = a.H;
    const int HD = H * D;
    const int prow = a.padded_rows;

    // transposed value table of all heads: tvt[(h*D + c)*prow + padded row]
    int tvt_words = 0;
    if constexpr (TVT_LDS) {
        const h8 *src = static_cast<const h8 *>(a.workspace);
        h8 *dst = reinterpret_cast<h8 *>(smem);
        const int chunks = HD * prow / 8;   // prow is a multiple of 16
        for (int t = threadIdx.x; t < chunks; t += kWaves * 64) dst[t] = src[t];
        __syncthreads();   // the only workgroup barrier; every wavefront reaches it
        tvt_words = HD * prow / 2;
    }

    // the wavefront index is uniform: tell the compiler, so that everything derived from the
    // work item (sizes, tile counts, loop bounds) lives in scalar registers and branches are scalar
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int il = lane & 31;
    const int half = lane >> 5;

    float *crd_k = smem + (tvt_words + 3) / 4 * 4 + wave * L::kWords;   // [32][ND]
    float *qt = crd_k + L::kCrd;                                          // [kQtRows][32]
    unsigned int *hist = reinterpret_cast<unsigned int *>(qt);
    float *kt = qt + L::kQt;                                              // [32][kKtStride]
    _Float16 *vt = reinterpret_cast<_Float16 *>(kt + L::kKt);             // [32][D]

    const _Float16 *gq = static_cast<const _Float16 *>(a.q);
    const _Float16 *gk = static_cast<const _Float16 *>(a.k);
    const _Float16 *gv = static_cast<const _Float16 *>(a.v);
    const _Float16 *gtq = static_cast<const _Float16 *>(a.table_q);
    const _Float16 *gtk = static_cast<const _Float16 *>(a.table_k);
    _Float16 *gout = static_cast<_Float16 *>(a.out);

    // work list written by attn_prepare_kernel: inclusive prefix of (query tile, key tile) pairs per
    // window, then the work counter, the number of head groups and the heads per group
    const int *item_end = static_cast<const int *>(a.items);
    const int groups = __builtin_amdgcn_readfirstlane(item_end[a.W + 1]);
    const int group_heads = __builtin_amdgcn_readfirstlane(item_end[a.W + 2]);
    const int total_items = __builtin_amdgcn_readfirstlane(item_end[a.W - 1]) * groups;
    // work items are handed out through a device counter (zeroed by attn_prepare_kernel), so a
    // wavefront that drew long items simply draws fewer of them
    // eight queues, each counter on a cache line of its own (atomics on one line retire one at a time); item i
    // belongs to queue i % 8 and a wavefront starts on the queue of the XCD it runs on
    int *counters = static_cast<int *>(a.items) + queue_counters_index(a.W);
    int queue = sweep::xcd_id() % sweep::kQueues;
    int tried = 0;

    const int cc = min(il, D - 1);               // channel this lane feeds to the value MFMAs
    const bool c_valid = il < D;
    // per-lane bases such that key slot v sits at a compile-time offset: key_of(v, half) =
    // key_of(v, 0) + 4*half
    const float *kt_lane = kt + 4 * half * L::kKtStride;
    const _Float16 *vt_lane = vt + 4 * half * D + cc;

    f16v zero16;
#pragma unroll
    for (int v = 0; v < 16; ++v) zero16[v] = 0.0f;

    for (;;) {
        int item = 0;
        if (lane == 0) item = atomicAdd(counters + queue * sweep::kCounterStride, 1);
        item = __builtin_amdgcn_readfirstlane(item) * sweep::kQueues + queue;
        if (item >= total_items) {
            if (++tried == sweep::kQueues) break;
            queue = (queue + 1) % sweep::kQueues;
            continue;
        }
        // item = (tile pair, head group); consecutive items share the tile pair
        const int pair = item / groups;
        const int h_begin = (item - pair * groups) * group_heads;
        const int h_end = min(H, h_begin + group_heads);
        // window of this tile pair: first w with item_end[w] > pair
        int lo = 0, hi = static_cast<int>(a.W) - 1;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (__builtin_amdgcn_readfirstlane(item_end[mid]) > pair) hi = mid; else lo = mid + 1;
        }
        const int w = lo;
        const int n_w = __builtin_amdgcn_readfirstlane(a.w_sizes[w]);
        const int s0 = __builtin_amdgcn_readfirstlane(a.w2n[w]);
        const int nkt = (n_w + kTile - 1) / kTile;   // key tiles (= query tiles)
        const bool single_key_tile = nkt == 1;
        // A window beyond the caller's size bound has no room for its partial results.  Its rows are not left
        // as the buffer held them: the item of a query tile's first key tile fills them (and the statistics)
        // with NaN, so an understated bound shows in the result.
        if (nkt > a.max_key_tiles) {
            const int local = pair - (w > 0 ? __builtin_amdgcn_readfirstlane(item_end[w - 1]) : 0);
            const int q_in = (local / nkt) * kTile + il;
            if (local % nkt == 0 && half == 0 && q_in < n_w) {
                const int row = a.n2n[s0 + q_in];
                const _Float16 nan16 = static_cast<_Float16>(__builtin_nanf(""));
                for (int h = h_begin; h < h_end; ++h) {
                    for (int c = 0; c < D; ++c) gout[static_cast<int64_t>(row) * HD + h * D + c] = nan16;
                    if (a.out_max) a.out_max[static_cast<int64_t>(row) * H + h] = __builtin_nanf("");
                    if (a.out_sum) a.out_sum[static_cast<int64_t>(row) * H + h] = __builtin_nanf("");
                }
            }
            continue;
        }
        // one item = one (query tile, key tile) pair of a window and a group of heads: the pair row
        // indices are computed once and reused by every head of the group.  A window of at most 32
        // voxels writes the final output; larger windows write per-key-tile partial results
        // (running max, sum, unnormalised output) that attn_merge_partials_kernel combines.
        const int local = pair - (w > 0 ? __builtin_amdgcn_readfirstlane(item_end[w - 1]) : 0);
        const int q0 = (local / nkt) * kTile;
        const int kt_i = local % nkt;
        const int k0 = kt_i * kTile;
        const int nk = min(kTile, n_w - k0);

        const bool q_valid = q0 + il < n_w;
        const int q_pos = s0 + min(q0 + il, n_w - 1);   // lanes past the window repeat the last voxel
        const int q_row = a.n2n[q_pos];
        float ci[ND];
#pragma unroll
        for (int n = 0; n < ND; ++n) ci[n] = a.n_coords[static_cast<int64_t>(q_pos) * ND + n];

        uint32_t idx[kIdxWords];

        // stage the key coordinates of a key tile and derive the row indices of all pairs
        auto build_pair_rows = [&](int k0, int nk) {
            wave_lds_fence();
            for (int t = lane; t < kTile * ND; t += 64) {
                const int j = t / ND, n = t - j * ND;
                crd_k[t] = a.n_coords[static_cast<int64_t>(s0 + k0 + min(j, nk - 1)) * ND + n];
            }
            wave_lds_fence();
#pragma unroll
            for (int t = 0; t < kIdxWords; ++t) idx[t] = 0;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int j = key_of(v, half);
#pragma unroll
                for (int n = 0; n < ND; ++n) {
                    const int r = crse_row(ci[n], crd_k[j * ND + n], a.rows[n]);
                    idx[(v * ND + n) >> 2] |= static_cast<uint32_t>(r) << (8 * ((v * ND + n) & 3));
                }
            }
        };
        build_pair_rows(k0, nk);

        // fragments of the head ahead: issued one head early
        const int k_row = a.n2n[s0 + k0 + min(il, nk - 1)];
        frag_t qf_next, kf_next;
        h8 vv_next;
        auto prefetch_head = [&](int hh) {
            qf_next = load_frag<D>(gq + static_cast<int64_t>(q_row) * a.row_stride + hh * D, half);
            kf_next = load_frag<D>(gk + static_cast<int64_t>(k_row) * a.row_stride + hh * D, half);
            vv_next = *reinterpret_cast<const h8 *>(gv + static_cast<int64_t>(k_row) * a.row_stride + hh * D +
                                                    (D == 16 ? 8 * half : 0));
        };
        prefetch_head(h_begin);

        for (int h = h_begin; h < h_end; ++h) {
            // the packed row indices are loop invariant; hide that from the optimiser, which would
            // otherwise hoist the ~300 LDS addresses derived from them out of the head loop and
            // spill them all
#pragma unroll
            for (int t = 0; t < kIdxWords; ++t) asm volatile("" : "+v"(idx[t]));
            const frag_t qf = qf_next, kf = kf_next;
            const h8 vv = vv_next;
            // first axis' table fragments for this head, then the next step's q/k/v
            frag_t tq_cur[L::kTiles], tk_cur[L::kTiles];
            auto load_axis = [&](int n, frag_t *tq_dst, frag_t *tk_dst) {
                const int rows = a.rows[n];
#pragma unroll
                for (int t = 0; t < L::kTiles; ++t) {
                    const int trow = a.base[n] + min(kTile * t + il, rows - 1);
                    tq_dst[t] = load_frag<D>(gtq + static_cast<int64_t>(trow) * HD + h * D, half);
                    tk_dst[t] = load_frag<D>(gtk + static_cast<int64_t>(trow) * HD + h * D, half);
                }
            };
            load_axis(0, tq_cur, tk_cur);
            if (h + 1 < h_end) prefetch_head(h + 1);

            // V tile -> LDS, [key][D] halves
            wave_lds_fence();
            if (half * 8 < D) *reinterpret_cast<h8 *>(vt + il * D + 8 * half) = vv;

            // logits: S^T[j][i] = sum_c K[j][c] Q[i][c]; copied out of the MFMA accumulator so that
            // the per-axis updates below are plain VALU adds on VGPRs
            float lg[16];
            {
                const f16v s_acc = Frag<D>::mfma(kf, qf, zero16);
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    lg[v] = s_acc[v];
                    asm volatile("" : "+v"(lg[v]));   // one VGPR each, not a 16-register tuple
                }
            }

#pragma unroll
            for (int n = 0; n < ND; ++n) {
                frag_t tq_nxt[L::kTiles], tk_nxt[L::kTiles];
                if (n + 1 < ND) load_axis(n + 1, tq_nxt, tk_nxt);
                const int tiles = (a.rows[n] + kTile - 1) / kTile;
#pragma unroll
                for (int t = 0; t < L::kTiles; ++t) {
                    if (t < tiles) {
                        const f16v dq = Frag<D>::mfma(tq_cur[t], qf, zero16);   // QT[r][i]
                        const f16v dk = Frag<D>::mfma(tk_cur[t], kf, zero16);   // KT[r][j]
                        // registers 4g..4g+3 hold rows 32t + 8g + 4*half + (0..3); rows >= RMAX are not kept
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            if (kTile * t + 8 * (v / 4) + 8 <= RMAX)
                                qt[(kTile * t + key_of(v, half)) * kTile + il] = dq[v];
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            if (kTile * t + 8 * g + 8 <= RMAX) {
                                f4 x = {dk[4 * g], dk[4 * g + 1], dk[4 * g + 2], dk[4 * g + 3]};
                                *reinterpret_cast<f4 *>(kt + il * L::kKtStride + kTile * t + 8 * g + 4 * half) = x;
                            }
                        }
                    }
                }
                wave_lds_fence();
                // straight-line over all 16 key slots: slots past the end of the tile read
                // staged duplicates of the last key and get weight 0 below
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r = (idx[(v * ND + n) >> 2] >> (8 * ((v * ND + n) & 3))) & 0xff;
                    lg[v] += qt[r * kTile + il] + kt_lane[key_of(v, 0) * L::kKtStride + r];
                }
                // pin the sums here: without it the scheduler keeps the gathered values of all
                // axes alive and adds them after the last axis (hundreds of spilled registers)
#pragma unroll
                for (int v = 0; v < 16; ++v) asm volatile("" : "+v"(lg[v]));
                wave_lds_fence();
                if (n + 1 < ND) {
#pragma unroll
                    for (int t = 0; t < L::kTiles; ++t) {
                        tq_cur[t] = tq_nxt[t];
                        tk_cur[t] = tk_nxt[t];
                    }
                }
            }

            // online softmax over this key tile
            float mx = -INFINITY;
#pragma unroll
            for (int v = 0; v < 16; ++v)
                if (key_of(v, half) < nk) mx = fmaxf(mx, lg[v]);
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = mx;
            float p[16];
            float psum = 0.0f;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                p[v] = (key_of(v, half) < nk) ? __expf(lg[v] - m_new) : 0.0f;
                psum += p[v];
            }
            psum += __shfl_xor(psum, 32);
            // 2^-24 fixed-point image of the weights for the integer histogram (0 for dead slots)
            unsigned int pfix[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) pfix[v] = static_cast<unsigned int>(p[v] * kFix + 0.5f);

            // value side: acc[c][i], c = 8*(v/4) + 4*half + v%4
            f16v acc = zero16;

            wave_lds_fence();   // V tile written above is visible to every lane
#pragma unroll
            for (int b = 0; b < 2; ++b) {   // 16 keys per MFMA: element e <-> key key_of(8b + e, half)
                h8 vf, pf;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const _Float16 x = vt_lane[key_of(8 * b + e, 0) * D];
                    vf[e] = c_valid ? x : static_cast<_Float16>(0.0f);
                    pf[e] = static_cast<_Float16>(p[8 * b + e]);
                }
                acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf, acc, 0, 0, 0);
            }

            const _Float16 *tvt_row;
            if constexpr (TVT_LDS)
                tvt_row = reinterpret_cast<const _Float16 *>(smem) + (h * D + cc) * prow;
            else
                tvt_row = static_cast<const _Float16 *>(a.workspace) + static_cast<int64_t>(h * D + cc) * prow;
#pragma unroll
            for (int n = 0; n < ND; ++n) {
                const int rows16 = (a.rows[n] + 15) / 16;
                // global copy of the value table: fetch this axis' fragments now, their latency hides
                // behind the histogram; the LDS copy is read right before each MFMA instead
                h8 tf[RMAX / 16];
                if constexpr (!TVT_LDS) {
#pragma unroll
                    for (int b = 0; b < RMAX / 16; ++b) {
                        tf[b] = h8{0, 0, 0, 0, 0, 0, 0, 0};
                        if (b < rows16 && c_valid)
                            tf[b] = *reinterpret_cast<const h8 *>(tvt_row + a.pbase[n] + 16 * b + 8 * half);
                    }
                }
                // clear H_n
                for (int t = lane; t < rows16 * 16 * kTile / 4; t += 64) {
                    f4 z = {0.0f, 0.0f, 0.0f, 0.0f};
                    *reinterpret_cast<f4 *>(qt + 4 * t) = z;
                }
                wave_lds_fence();
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r = (idx[(v * ND + n) >> 2] >> (8 * ((v * ND + n) & 3))) & 0xff;
                    atomicAdd(hist + r * kTile + il, pfix[v]);
                }
                wave_lds_fence();
                auto hist_frag = [&](int b) {
                    h8 hf;
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        hf[e] = static_cast<_Float16>(
                            static_cast<float>(hist[(16 * b + 8 * half + e) * kTile + il]) * (1.0f / kFix));
                    return hf;
                };
                if constexpr (TVT_LDS) {
                    for (int b = 0; b < rows16; ++b) {
                        h8 t = *reinterpret_cast<const h8 *>(tvt_row + a.pbase[n] + 16 * b + 8 * half);
                        if (!c_valid) t = h8{0, 0, 0, 0, 0, 0, 0, 0};
                        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(t, hist_frag(b), acc, 0, 0, 0);
                    }
                } else {
#pragma unroll
                    for (int b = 0; b < RMAX / 16; ++b)
                        if (b < rows16)
                            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(tf[b], hist_frag(b), acc, 0, 0, 0);
                }
                wave_lds_fence();
            }
            if (q_valid) {
                if (single_key_tile) {
                    const float inv = 1.0f / psum;
                    _Float16 *orow = gout + static_cast<int64_t>(q_row) * HD + h * D;
#pragma unroll
                    for (int g = 0; g < D / 8; ++g) {   // registers 4g..4g+3 hold channels 8g + 4*half + e
                        h4 ov;
#pragma unroll
                        for (int e = 0; e < 4; ++e) ov[e] = static_cast<_Float16>(acc[4 * g + e] * inv);
                        *reinterpret_cast<h4 *>(orow + 8 * g + 4 * half) = ov;
                    }
                    if (half == 0) {
                        if (a.out_max) a.out_max[static_cast<int64_t>(q_row) * H + h] = m_new;
                        if (a.out_sum) a.out_sum[static_cast<int64_t>(q_row) * H + h] = psum;
                    }
                } else {
                    // partial of this key tile: [key tile][head][sorted position][D channels, max, sum];
                    // the 32 queries of the tile fill one contiguous run
                    float *part = a.partials +
                                  ((static_cast<int64_t>(kt_i) * H + h) * a.N + q_pos) * (D + 2);
#pragma unroll
                    for (int g = 0; g < D / 8; ++g) {
                        f4 ov = {acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
                        *reinterpret_cast<f4 *>(part + 8 * g + 4 * half) = ov;
                    }
                    if (half == 0) {
                        part[D] = m_new;
                        part[D + 1] = psum;
                    }
                }
            }
        }
    }
}

// Windows of more than 32 voxels: combine the per-key-tile partial results of every (voxel, head).
// One thread per (sorted position, head); the window of a position is found by bisection of w2n.
template <int D>
__global__ __launch_bounds__(256) void attn_merge_partials_kernel(AttnArgs a)
{
    const int H = a.H;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= a.N * H) return;
    // position fastest: neighbouring threads read neighbouring partial records
    const int h = static_cast<int>(t / a.N), pos = static_cast<int>(t - static_cast<int64_t>(h) * a.N);
    int lo = 0, hi = static_cast<int>(a.W) - 1;   // last window that starts at or before pos
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (a.w2n[mid] <= pos) lo = mid; else hi = mid - 1;
    }
    const int nkt = (a.w_sizes[lo] + kTile - 1) / kTile;
    if (nkt <= 1 || nkt > a.max_key_tiles) return;
    const float *part = a.partials + (static_cast<int64_t>(h) * a.N + pos) * (D + 2);
    const int64_t tile_stride = static_cast<int64_t>(H) * a.N * (D + 2);
    float m = -INFINITY;
    for (int kt = 0; kt < nkt; ++kt) m = fmaxf(m, part[kt * tile_stride + D]);
    float l = 0.0f, o[D];
#pragma unroll
    for (int c = 0; c < D; ++c) o[c] = 0.0f;
    for (int kt = 0; kt < nkt; ++kt) {
        const float *pk = part + kt * tile_stride;
        const float wgt = __expf(pk[D] - m);
        l += pk[D + 1] * wgt;
#pragma unroll
        for (int c = 0; c < D; ++c) o[c] += pk[c] * wgt;
    }
    const int row = a.n2n[pos];
    const float inv = 1.0f / l;
    _Float16 *orow = static_cast<_Float16 *>(a.out) + (static_cast<int64_t>(row) * H + h) * D;
    _Float16 ov[D];
#pragma unroll
    for (int c = 0; c < D; ++c) ov[c] = static_cast<_Float16>(o[c] * inv);
#pragma unroll
    for (int g = 0; g < D / 8; ++g) *reinterpret_cast<h8 *>(orow + 8 * g) = *reinterpret_cast<const h8 *>(ov + 8 * g);
    if (a.out_max) a.out_max[static_cast<int64_t>(row) * H + h] = m;
    if (a.out_sum) a.out_sum[static_cast<int64_t>(row) * H + h] = l;
}

// Set-up of one attention launch, one kernel:
//  * workgroup 0 writes the work list: inclusive prefix sum of the (query tile, key tile) pairs of every
//    window (W is at most a few hundred thousand), the work counter and the split of the heads into groups;
//  * the other workgroups transpose the value table [axis][row][h][c] -> [h][c][padded row], every axis
//    padded to a multiple of 16 rows.
__global__ __launch_bounds__(1024) void attn_prepare_kernel(AttnArgs a)
{
    if (blockIdx.x > 0) {
        const int HD = a.H * a.D;
        _Float16 *dst = static_cast<_Float16 *>(a.workspace);
        const _Float16 *src = static_cast<const _Float16 *>(a.table_v);
        const int64_t total = static_cast<int64_t>(HD) * a.padded_rows;
        for (int64_t t = static_cast<int64_t>(blockIdx.x - 1) * blockDim.x + threadIdx.x; t < total;
             t += static_cast<int64_t>(gridDim.x - 1) * blockDim.x) {
            const int hc = static_cast<int>(t / a.padded_rows);
            const int pr = static_cast<int>(t - static_cast<int64_t>(hc) * a.padded_rows);
            _Float16 val = static_cast<_Float16>(0.0f);
            for (int n = 0; n < a.nd; ++n) {
                const int r = pr - a.pbase[n];
                if (r >= 0 && r < a.rows[n]) val = src[static_cast<int64_t>(a.base[n] + r) * HD + hc];
            }
            dst[t] = val;
        }
        return;
    }
    __shared__ int wave_total[16];
    int *item_end = static_cast<int *>(a.items);
    const int W = static_cast<int>(a.W);
    const int per = (W + 1023) / 1024;
    const int begin = threadIdx.x * per, end = min(begin + per, W);
    int sum = 0;
    for (int w = begin; w < end; ++w) {
        const int tiles = (a.w_sizes[w] + kTile - 1) / kTile;
        sum += tiles * tiles;
    }
    // inclusive scan over the 1024 threads: shuffles inside a wavefront, then the 16 wavefront totals
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
            if (static_cast<int>(threadIdx.x) >= off) v += up;
        }
        wave_total[threadIdx.x] = v;
    }
    __syncthreads();
    incl += wave > 0 ? wave_total[wave - 1] : 0;
    int run = incl - sum;
    for (int w = begin; w < end; ++w) {
        const int tiles = (a.w_sizes[w] + kTile - 1) / kTile;
        run += tiles * tiles;
        item_end[w] = run;
    }
    // the work counters of the attention kernel
    if (threadIdx.x < sweep::kQueues) item_end[queue_counters_index(a.W) + threadIdx.x * sweep::kCounterStride] = 0;
    if (threadIdx.x == 1023) {
        // heads are split into groups when the tile pairs alone are too few to keep every wavefront
        // of the persistent grid busy with several items (deep stages: few, large windows, many heads)
        const int pairs = incl;
        int groups = pairs > 0 ? (a.target_items + pairs - 1) / pairs : 1;
        groups = max(1, min(groups, a.H));
        const int group_heads = (a.H + groups - 1) / groups;
        item_end[W] = 0;
        item_end[W + 1] = (a.H + group_heads - 1) / group_heads;
        item_end[W + 2] = group_heads;
    }
}

size_t lds_bytes(const AttnArgs &a, int wave_words, bool tvt_lds)
{
    const size_t tvt_words = tvt_lds ? static_cast<size_t>(a.H) * a.D * a.padded_rows / 2 : 0;
    return sizeof(float) * ((tvt_words + 3) / 4 * 4 + static_cast<size_t>(kWaves) * wave_words);
}

constexpr size_t kLdsPerCu = 160 * 1024;

template <int D, int ND, int RMAX, bool TVT_LDS>
int launch(const AttnArgs &args, hipStream_t stream)
{
    AttnArgs a = args;
    auto kernel = attn_fwd_mfma_kernel<D, ND, RMAX, TVT_LDS>;
    const size_t lds = lds_bytes(a, WaveLds<RMAX>::kWords, TVT_LDS);
    S3D_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    // persistent grid: as many workgroups as fit the chip at once (LDS-bound), never more than the
    // windows can feed; wavefronts pull items in a strided loop
    int device = 0, cus = 256;
    if (hipGetDevice(&device) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && v > 0) cus = v;
    }
    const int per_cu = kLdsPerCu / lds > 0 ? static_cast<int>(kLdsPerCu / lds) : 1;
    int64_t grid = static_cast<int64_t>(cus) * per_cu;
    a.target_items = static_cast<int>(grid) * kWaves * kItemsPerWave;
    const int64_t cells = static_cast<int64_t>(a.H) * a.D * a.padded_rows;
    hipLaunchKernelGGL(attn_prepare_kernel, dim3(1 + static_cast<unsigned>(ceil_div(cells, 1024))), dim3(1024), 0,
                       stream, a);
    S3D_HIP_CHECK(hipGetLastError());
    // never more wavefronts than work items (upper bound: every window as large as the largest,
    // every head an item of its own)
    const int64_t need = ceil_div(a.W * a.max_key_tiles * a.max_key_tiles * a.H, kWaves);
    if (grid > need) grid = need;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(kWaves * 64), lds, stream, a);
    S3D_HIP_CHECK(hipGetLastError());
    if (a.max_key_tiles > 1)
        hipLaunchKernelGGL(attn_merge_partials_kernel<D>, dim3(static_cast<unsigned>(ceil_div(a.N * a.H, 256))),
                           dim3(256), 0, stream, a);
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}

int max_axis_rows(const AttnArgs &a)
{
    int m = 0;
    for (int n = 0; n < a.nd; ++n) m = a.rows[n] > m ? a.rows[n] : m;
    return m;
}

}  // namespace

int attn_mfma_padded_rows(const int32_t *rows, int nd)
{
    int padded = 16;   // slack so that 16-row reads of the last block stay inside the table
    for (int n = 0; n < nd; ++n) padded += (rows[n] + 15) / 16 * 16;
    return padded;
}

bool attn_mfma_supported(const AttnArgs &a, int dtype)
{
    if (dtype != S3D_DTYPE_F16) return false;
    if (a.D != 8 && a.D != 16) return false;
    if (a.nd != 3 && a.nd != 6 && a.nd != 9) return false;
    const int rmax = max_axis_rows(a);
    if (rmax > 64) return false;
    return true;
}

size_t attn_mfma_table_bytes(int H, int D, int padded_rows)
{
    return align_up(sizeof(_Float16) * static_cast<size_t>(H) * D * padded_rows, 256);
}

size_t attn_mfma_items_bytes(int64_t W)
{
    return sizeof(int32_t) * (queue_counters_index(W) + static_cast<size_t>(sweep::kQueues) * sweep::kCounterStride);
}

int attn_mfma_key_tiles(int max_window_voxels)
{
    return max_window_voxels <= kTile ? 1 : (max_window_voxels + kTile - 1) / kTile;
}

size_t attn_mfma_workspace_bytes(int H, int D, int padded_rows, int64_t W, int64_t N, int max_window_voxels)
{
    const int tiles = attn_mfma_key_tiles(max_window_voxels);
    const size_t partials = tiles <= 1 ? 0 : sizeof(float) * static_cast<size_t>(N) * tiles * H * (D + 2);
    return attn_mfma_table_bytes(H, D, padded_rows) + attn_mfma_items_bytes(W) + align_up(partials, 256);
}

int launch_attn_mfma(const AttnArgs &a, hipStream_t stream)
{
    const int rmax = max_axis_rows(a);
    const int words = rmax <= 32 ? WaveLds<32>::kWords : rmax <= 48 ? WaveLds<48>::kWords : WaveLds<64>::kWords;
    const bool tvt_lds = lds_bytes(a, words, true) <= kLdsPerCu;
#define S3D_RMAX(DD, NN, LDS)                                                    \
    return rmax <= 32   ? launch<DD, NN, 32, LDS>(a, stream)                     \
           : rmax <= 48 ? launch<DD, NN, 48, LDS>(a, stream)                     \
                        : launch<DD, NN, 64, LDS>(a, stream);
#define S3D_CASE(DD, NN)                                                         \
    if (a.D == DD && a.nd == NN) {                                               \
        if (tvt_lds) { S3D_RMAX(DD, NN, true) } else { S3D_RMAX(DD, NN, false) } \
    }
    S3D_CASE(8, 3) S3D_CASE(8, 6) S3D_CASE(8, 9)
    S3D_CASE(16, 3) S3D_CASE(16, 6) S3D_CASE(16, 9)
#undef S3D_CASE
#undef S3D_RMAX
    return fail(S3D_ERR_UNSUPPORTED, "s3d_attn_fwd: MFMA kernel does not cover D=%d nd=%d", a.D, a.nd);
}

}  // namespace s3d
