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
    const int32_t *w_sizes, *w2n, *n2n;    // n2n may be null: rows already in window-sorted order
    const int32_t *sizes_dev;              // per-axis table sizes on the device (rows[] / base[] unset), or null
    const float *n_coords;                 // [N,nd], window-sorted
    void *out;                             // [N,H,D]
    float *out_max, *out_sum;              // [N,H] or null
    void *workspace;                       // the work list: queue counters, unit and window records
    int32_t block_shift;                   // the step target, a lane streams about 2^block_shift keys
    int32_t target_items;                  // wavefronts that serve one head group (sizes the finer units at the list's end)
    int32_t spread_groups;                 // head groups take the workgroups in turn (else in runs of eight)
    int32_t H, D, nd, total_rows;
    int64_t N, W;
    int32_t rows[kMaxAxes];                // rows of each axis table
    int32_t base[kMaxAxes];                // first row of each axis table in the flat table
};

// Persistent workgroups, one to three heads each with their table slices in LDS; lane = one query of some window,
// which streams that window's keys; VALU math (packed fp16 dot products for fp16 I/O), any dtype, windows of any
// size.  Needs a.workspace (work queues, sorted window list, unit list).
size_t attn_sweep_workspace_bytes(int H, int64_t W, int64_t N);
// what: kAttnBuildList (the two list kernels: needs w_sizes, w2n and the shape only), kAttnSweep (the sweep on a
// work list that is already in a.workspace; the launch leaves it ready for the next one), or both.
constexpr int kAttnBuildList = 1, kAttnSweep = 2;
int launch_attn_sweep(const AttnArgs &a, int dtype, hipStream_t stream, int what = kAttnBuildList | kAttnSweep);

// The pair sweeps of the backward on the sweep kernel's work list (built here, in b.f.workspace, which needs
// attn_sweep_workspace_bytes): dq, dk, dv, and dL, P of every (pair, head) for the table-gradient kernels.
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

}  // namespace s3d
