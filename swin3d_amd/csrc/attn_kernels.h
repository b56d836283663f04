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
    const float *n_coords;                 // [N,nd], window-sorted
    void *out;                             // [N,H,D]
    float *out_max, *out_sum;              // [N,H] or null
    void *workspace;                       // the caller's workspace
    void *items;                           // int32 [W+1] work-item prefix + counter (MFMA path)
    float *partials;                       // MFMA path: per-key-tile partial results of multi-tile windows
    int32_t max_key_tiles;                 // MFMA path: key tiles of the largest window (stride of `partials`)
    int32_t block_shift;                   // sweep kernel: the step target, a lane streams about 2^block_shift keys
    int32_t target_items;                  // work items the launch wants at least (heads are split to reach it)
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

// One wavefront per window, MFMA products + LDS gathers; fp16 only.
bool attn_mfma_supported(const AttnArgs &a, int dtype);
// the shapes where it is the faster of the two kernels: head_dim 16 with nearly full windows (256 voxels on
// average; measured at window 7 with 6 heads: 343-voxel windows 0.88 ms against 0.99 ms, 205 voxels 0.435 against
// 0.424, 104 voxels 0.165 against 0.145, a room scan with 57 voxels on average 0.43 against 0.35), or with many
// heads, over which it spreads the row indices of a tile pair, and 60 voxels on average (Swin3D-L, window 7: 20
// heads and 61 voxels 0.885 against 0.919 ms, 55 voxels 0.853 against 0.718; 40 heads and 69 voxels 0.571 against
// 0.700, 45 voxels 0.463 against 0.429; 10 heads and 58 voxels 1.57 against 1.37).  At head_dim 8 the sweep
// kernel's packed fp16 dot products win everywhere.
inline bool attn_mfma_preferred(const AttnArgs &a)
{
    return a.D > 8 && (a.N >= 256 * a.W || (a.H >= 16 && a.N >= 60 * a.W));
}
size_t attn_mfma_table_bytes(int H, int D, int padded_rows);
size_t attn_mfma_items_bytes(int64_t W);
int attn_mfma_key_tiles(int max_window_voxels);
size_t attn_mfma_workspace_bytes(int H, int D, int padded_rows, int64_t W, int64_t N, int max_window_voxels);
int launch_attn_mfma(const AttnArgs &a, hipStream_t stream);

}  // namespace s3d
