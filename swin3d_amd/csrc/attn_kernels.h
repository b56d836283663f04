// Internal interface between the attention entry point and its kernel families.
#pragma once

#include "s3d_common.h"

namespace s3d {

constexpr int kMaxAxes = 9;

// Everything a window-attention kernel needs, by value (lives in kernel-argument SGPRs).
struct AttnArgs {
    const void *q, *k, *v;                 // [N,H,D], voxel rows `row_stride` elements apart
    int64_t row_stride;
    const void *table_q, *table_k, *table_v;  // flat [sum rows][H][D]
    const int32_t *w_sizes, *w2n, *n2n;
    const int32_t *sizes_dev;              // sweep kernel: per-axis table sizes on the device (rows[] / base[] unset), or null
    const float *n_coords;                 // [N,nd], window-sorted
    void *out;                             // [N,H,D]
    float *out_max, *out_sum;              // [N,H] or null
    void *workspace;                       // the caller's workspace
    void *items;                           // int32 [W+1] work-item prefix + counter (MFMA path)
    float *partials;                       // MFMA path: per-key-tile partial results of multi-tile windows
    int32_t max_key_tiles;                 // MFMA path: key tiles of the largest window (stride of `partials`)
    int32_t block_shift;                   // sweep kernel: the step target, a lane streams about 2^block_shift keys
    int32_t target_items;                  // work items the launch wants at least (heads are split to reach it)
    int32_t spread_groups;                 // sweep kernel: head groups take the workgroups in turn (else in runs of eight)
    int32_t H, D, nd, total_rows;
    int64_t N, W;
    int32_t rows[kMaxAxes];                // rows of each axis table
    int32_t base[kMaxAxes];                // first row of each axis table in the flat table
    int32_t pbase[kMaxAxes];               // first row of each axis in the padded transposed table
    int32_t padded_rows;                   // row stride of the transposed value table
};

// Persistent workgroups, one head (or pair of heads) each with its table slices in LDS; lane = one query of some
// window, which streams that window's keys; VALU math, any dtype, windows of any size.  Needs a.workspace (work
// queues, sorted window list, unit list); a.n2n may be null (rows already in window-sorted order).
size_t attn_generic_workspace_bytes(int H, int64_t W, int64_t N);
// what: kAttnBuildList (the two list kernels: needs w_sizes, w2n and the shape only), kAttnSweep (the sweep on a
// work list that is already in a.workspace; the launch leaves it ready for the next one), or both.
constexpr int kAttnBuildList = 1, kAttnSweep = 2;
int launch_attn_generic(const AttnArgs &a, int dtype, hipStream_t stream, int what = kAttnBuildList | kAttnSweep);

// The pair sweeps of the backward on the sweep kernel's work list (built here, in b.f.workspace, which needs
// attn_generic_workspace_bytes): dq, dk, dv, and dL, P of every (pair, head) for the table-gradient kernels.
struct BwdPairArgs {
    AttnArgs f;                  // shape, q, k, v, tables, index arrays (n2n required), rows[] / base[], workspace
    const void *dout;            // [N,H,D]
    const float *stat_max, *stat_sum, *delta;   // [N,H]: the forward's statistics, dout_i . o_i
    void *dq, *dk, *dv;          // [N,H,D]
    const int64_t *pos_base;     // [N]: at a window's first sorted position, the pairs of the windows before it
    float2 *pd;                  // [H][pairs]: (dL, P) at base + i n + j  (i, j: query, key position inside the window)
    float *dl_t;                 // [H][pairs]: dL at base + j n + i
    int64_t pairs;               // capacity of pd and dl_t per head; windows beyond it are skipped
};
int launch_attn_bwd_pairs(const BwdPairArgs &b, int dtype, hipStream_t stream);

// One wavefront per window, MFMA products + LDS gathers; fp16 only.
bool attn_mfma_supported(const AttnArgs &a, int dtype);
// the shapes where it is the faster of the two kernels: head_dim 16 with full windows, 300 voxels or more on
// average.  Measured at window 7 on a 56 x 56 x 28 lattice filled to 100 / 80 / 60 / 30 % (343 / 274 / 206 / 103
// voxels per window), sweep against MFMA kernel in ms: 6 heads 2.01 / 1.96, 1.36 / 1.34, 0.83 / 0.83, 0.26 / 0.31;
// 20 heads 6.39 / 6.14, 4.24 / 4.22, 2.38 / 2.58, 0.76 / 0.85; 40 heads 12.86 / 12.15, 8.43 / 8.36, 4.68 / 5.08,
// 1.36 / 1.65.  Room scans (50 to 70 voxels per window at every stage of the encoder) are the sweep kernel's.  At
// head_dim 8 the sweep kernel's packed fp16 arithmetic wins everywhere.
inline bool attn_mfma_preferred(const AttnArgs &a)
{
    return a.D > 8 && a.N >= 300 * a.W;
}
size_t attn_mfma_table_bytes(int H, int D, int padded_rows);
size_t attn_mfma_items_bytes(int64_t W);
int attn_mfma_key_tiles(int max_window_voxels);
size_t attn_mfma_workspace_bytes(int H, int D, int padded_rows, int64_t W, int64_t N, int max_window_voxels);
int launch_attn_mfma(const AttnArgs &a, hipStream_t stream);

}  // namespace s3d
