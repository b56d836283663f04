/*
 * swin3d_amd -- C ABI of the MI355X (gfx950) sparse window-attention forward,
 * window index builder and KNN helper.
 *
 * Plain pointers and sizes only: every pointer named "device" is a HIP device
 * address, `stream` is a hipStream_t passed as void* (NULL = the null stream).
 * All entry points enqueue work on `stream` and return without synchronising
 * unless stated otherwise.  Every output and every workspace is allocated by the
 * caller; the only device memory the library itself holds is the fixed scratch
 * array of s3d_attn_fwd_noalloc (8 MiB per GPU, part of the code object).
 *
 * Return value: 0 on success, a negative S3D_ERR_* code for a rejected argument,
 * a positive value = the hipError_t of a failed runtime call.  A human readable
 * description of the last failure on the calling thread is returned by
 * s3d_last_error_string().
 *
 * Each declaration cites the reference interface it replaces (paths relative to
 * the microsoft/Swin3D tree).
 */
#ifndef SWIN3D_AMD_H
#define SWIN3D_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define S3D_OK 0
#define S3D_ERR_NULL_POINTER (-1)
#define S3D_ERR_BAD_SHAPE (-2)
#define S3D_ERR_BAD_DTYPE (-3)
#define S3D_ERR_UNSUPPORTED (-4)
#define S3D_ERR_WORKSPACE (-5)

/* element type of q/k/v, the tables and the attention output */
#define S3D_DTYPE_F32 0
#define S3D_DTYPE_F16 1
/* s3d_attn_bwd only: fp32 tables beside fp16 rows (q, k, v, out, dout, dq, dk, dv): the backward of an fp16 forward
 * computed in fp32, as PrecisionMode.HALF_FORWARD asks (Swin3D/sparse_dl/attn/attn_coff.py:206-215 casts the rows
 * up and the gradients down; here they are widened as they are loaded and rounded as they are stored) */
#define S3D_DTYPE_F32_F16_ROWS 2

/* largest K of s3d_knn (K_MAX of Swin3D/src/knn/knn_cuda_kernel.cu:4) */
#define S3D_KNN_KMAX 64
/* squared distance stored in unfilled KNN slots: float(0x7fffffff)
 * (MAX_DIST of Swin3D/src/knn/knn_cuda_kernel.cu:5); their index is -1 */
#define S3D_KNN_PAD_DIST2 2147483648.0f

/* Library version, major*10000 + minor*100 + patch. */
int s3d_version(void);

/* Description of the last error raised on the calling thread ("" if none). */
const char *s3d_last_error_string(void);

/*
 * Windowed self-attention forward with contextual relative signal encoding.
 *
 * Replaces the pair of pybind entry points
 *   cal_max_coffs           Swin3D/src/attn/self_attn_aio_fwd.cu:255-455
 *   self_attn_cuda_forward  Swin3D/src/attn/self_attn_aio_fwd.cu:457-688
 * (declared in Swin3D/src/attn/self_attn_aio_fwd.h:11-26, exported at
 * Swin3D/src/attn/attn_api.cpp:20,23) and the division
 * Swin3D/sparse_dl/attn/attn_coff.py:184, for pos_mode SEPARATE (3) and
 * indice_mode INDIRECT (2), in ONE pass and without the O(M) pair arrays
 * m2w_indices / w2m_offsets.
 *
 *   q, k, v        device [N,H,D] of `dtype`, original voxel order (q pre-scaled); see qkv_row_stride
 *   table_q/k/v    device [table_len] of `dtype`, layout [axis][row][h][c]
 *   table_sizes    HOST int32 [nd], table_sizes[n] = rows_n * H * D (the values of the
 *                  reference's `table_offsets` tensor, fwd.cu:258,285; read on the host so
 *                  that the row counts travel as kernel arguments)
 *                  With the flag S3D_ATTN_SIZES_ON_DEVICE the pointer is a DEVICE int32 [nd] array instead - the
 *                  tensor the reference's caller builds on every call (Swin3D/modules/swin3d_layers.py:511) - and
 *                  the host never reads it: the sweep kernel takes the row counts from it (clipped so that no
 *                  access leaves the head's table; sizes that do not add up to table_len give a wrong result, not
 *                  a fault).  s3d_attn_plan accepts NULL for table_sizes for such callers.
 *   table_len      elements per table = sum_n table_sizes[n]
 *   w_sizes, w2n   device int32 [W]: voxels per window, exclusive prefix sum
 *   n2n            device int32 [N]: window-sorted position -> original row, or NULL when the rows of q, k,
 *                  v and out are in window-sorted order already (position = row): the kernels then read and
 *                  write the rows in place, without the gather of Swin3D/src/attn/attn_utils.cuh:391-409
 *   n_coords       device fp32 [N,nd], window-sorted order, scaled by the quant sizes
 *   out            device [N,H,D] of `dtype`: softmax-normalised attention output
 *   out_max        device fp32 [N,H] or NULL: max logit per (voxel, head)
 *                  (the tensor cal_max_coffs returns)
 *   out_sum        device fp32 [N,H] or NULL: sum_j exp(logit - max)
 *                  (second tensor of self_attn_cuda_forward; raw = out * sum)
 *   qkv_row_stride elements between consecutive voxel rows of q, k and v (0 = H*D, dense).  A multiple
 *                  of 8 that is >= H*D: with 3*H*D and q, k, v pointing H*D apart the kernels read the
 *                  [N, 3*H*D] output of the qkv projection (Swin3D/modules/swin3d_layers.py:502-509) in
 *                  place, without the reference's reshape / permute / contiguous copy.
 *   flags          0, or S3D_ATTN_PLANNED (`workspace` holds a work list built by s3d_attn_plan, see below)
 *                  and / or S3D_ATTN_SIZES_ON_DEVICE (see table_sizes)
 *   workspace      device scratch of at least s3d_attn_fwd_workspace_bytes(H, N, W) bytes: the work list of the
 *                  launch (work-queue counters, one record per unit of 8 to 64 queries and one per window, the
 *                  list builder's notes), about 2 N + 24 W bytes + 0.3 MB whatever the window sizes
 *   w2n must be ascending (the exclusive prefix sum of w_sizes, as the reference builds it:
 *   Swin3D/modules/swin3d_layers.py:100-103).
 *   D in {8,16,32}, nd in {3,6,9}, H >= 1 (the reference takes head_dim up to 32: self_attn_aio_fwd.cu:486).
 *
 * Row index of axis n for the pair (query i, key j), all in fp32:
 *   rel = (n_coords[i][n] - n_coords[j][n]) + float(rows_n / 2)
 *   row = min(int(min(max(rel, 0), rows_n)), rows_n - 1)
 * (Swin3D/src/attn/attn_utils.cuh:444-450; the reference indexes one row past
 * the axis table when the clamped value equals rows_n, this library folds that
 * case onto the last row).
 *
 * fp16: inputs, tables and output are fp16; products accumulate in fp32, exp in fp32.  The value-table rows of a
 * pair are added three at a time in fp16 before they enter the fp32 sums (the reference's half path adds all of
 * them and the value in half2, Swin3D/src/attn/self_attn_aio_fwd.cu:147).  Every call gives the same bits for the
 * same inputs (no atomics on data, work list in window order).
 *
 * One kernel family serves every shape: persistent workgroups that keep their heads' table slices in LDS, a lane
 * per query streaming its window's keys (VALU; packed fp16 dot products for fp16 I/O).
 */
#define S3D_ATTN_PLANNED 4   /* `workspace` holds a plan written by s3d_attn_plan: see there */
#define S3D_ATTN_SIZES_ON_DEVICE 8   /* `table_sizes` is a DEVICE int32 [nd] array (see s3d_attn_fwd) */
size_t s3d_attn_fwd_workspace_bytes(int32_t H, int64_t N, int64_t W);
int s3d_attn_fwd(const void *q, const void *k, const void *v, const void *table_q,
                 const void *table_k, const void *table_v, const int32_t *table_sizes, int32_t nd,
                 int64_t table_len, const int32_t *w_sizes, const int32_t *w2n, const int32_t *n2n,
                 const float *n_coords, void *out, float *out_max, float *out_sum, int64_t N,
                 int32_t H, int32_t D, int64_t W, int64_t qkv_row_stride, int32_t dtype, int32_t flags,
                 void *workspace, size_t workspace_bytes, void *stream);

/*
 * Work list of the sweep kernel, built once per window set ("plan").
 *
 * The reference builds its O(pairs) index arrays once per window set and hands them to every attention call
 * of the blocks that share the set (Swin3D/modules/swin3d_layers.py:857-871: one `get_index01` per window
 * set, `indices` reused by the blocks).  The counterpart here is O(N + W): the windows sorted by size and cut into
 * units of 64 lanes.  s3d_attn_fwd builds it on every call (two small kernels); a caller that keeps a window set
 * for several calls builds it once with s3d_attn_plan and passes the plan buffer as `workspace` together with
 * the flag S3D_ATTN_PLANNED, for calls with the same w_sizes, w2n, N, W, H, D, dtype and table_sizes.  Such a call
 * runs the sweep kernel and nothing else.  The plan holds the launch's work counters, which a launch leaves at
 * zero again: a plan serves one call at a time (calls in stream order; not two streams at once).
 *   plan           device buffer of at least s3d_attn_plan_bytes(H, N, W) bytes (= s3d_attn_fwd_workspace_bytes)
 */
size_t s3d_attn_plan_bytes(int32_t H, int64_t N, int64_t W);
int s3d_attn_plan(const int32_t *table_sizes, int32_t nd, int64_t table_len, const int32_t *w_sizes,
                  const int32_t *w2n, int64_t N, int32_t H, int32_t D, int64_t W, int32_t dtype, void *plan,
                  size_t plan_bytes, void *stream);

/*
 * The same forward without a workspace argument and without any allocation.
 *
 * It has no counterpart in the reference.  It is for callers that cannot allocate device memory around the
 * call: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The work list lives
 * in a device array of 8 MiB that is part of the library's code object, one copy per GPU, held until the process
 * ends.  The call fails with S3D_ERR_WORKSPACE when s3d_attn_fwd_workspace_bytes(H, N, W) exceeds 8 MiB (about
 * 2 N + 24 W bytes + 0.3 MB: e.g. one million voxels in up to 200 000 windows fit).  No call allocates or frees.
 * The first call on a device looks up the array's address there (hipGetSymbolAddress) and the first call of a
 * shape (dtype, head_dim, axes, heads per wavefront) raises that kernel's dynamic-LDS limit (hipFuncSetAttribute):
 * neither belongs into a stream capture, so make ONE eager call per device and shape before capturing; the calls
 * after it enqueue kernels only.
 * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two host
 * threads) race on it and must be serialised by the caller; calls in stream order on one stream are safe,
 * and nothing is carried over from one call to the next.
 * Arguments, results and status codes as for s3d_attn_fwd.
 */
int s3d_attn_fwd_noalloc(const void *q, const void *k, const void *v, const void *table_q,
                         const void *table_k, const void *table_v, const int32_t *table_sizes, int32_t nd,
                         int64_t table_len, const int32_t *w_sizes, const int32_t *w2n, const int32_t *n2n,
                         const float *n_coords, void *out, float *out_max, float *out_sum, int64_t N,
                         int32_t H, int32_t D, int64_t W, int64_t qkv_row_stride, int32_t dtype, void *stream);

/*
 * Windowed self-attention backward.
 *
 * Replaces cal_exp_sum_grads and self_attn_indir_backward
 * (Swin3D/src/attn/self_attn_aio_bwd.cu:14-47 and :49-113, 197-509, exported at
 * Swin3D/src/attn/attn_api.cpp:21,24; called from
 * Swin3D/sparse_dl/attn/attn_coff.py:219-224) for pos_mode SEPARATE and indice_mode INDIRECT,
 * without the O(M) pair arrays.  Arithmetic is fp32 for both dtypes.
 *
 *   q .. n_coords  as for s3d_attn_fwd (the forward's inputs; with n2n NULL - rows in window order - the call
 *                  writes the identity map into its workspace and reads that)
 *   out, out_max, out_sum   the forward's outputs for the same inputs (out of `dtype`, statistics fp32):
 *                  the tensors the reference saves for backward (attn_coff.py:186-187)
 *   dout           device [N,H,D] of `dtype`: gradient of the loss w.r.t. `out`
 *   dq, dk, dv     device [N,H,D] of `dtype`, overwritten (every row belongs to exactly one window)
 *   dtable_q/k/v   device FP32 [table_len], overwritten; layout of the tables
 *   pairs          M = sum of w_sizes^2, the pairs of the window set (counts[1] of s3d_window_index; the length
 *                  of the reference's index arrays), or 0.  With M the call runs two pair sweeps on the forward's
 *                  kind of work list (dq; dk and dv), which leave dL and P of every (pair, head) in the workspace
 *                  - 12 * H * pairs bytes -, and two table-gradient sweeps that read them.  With 0 it runs two fused
 *                  sweeps that recompute the logits for the table gradients and need no such store (about a third
 *                  more time).  A value below M cannot hold the records of every window: the rows of dq, dk, dv
 *                  that belong to the windows beyond it and all three table gradients then come out as NaN.
 *   workspace      device scratch of at least s3d_attn_bwd_workspace_bytes(H, D, nd, table_len, N, W, pairs) bytes
 *   dtype          S3D_DTYPE_F32, S3D_DTYPE_F16, or S3D_DTYPE_F32_F16_ROWS: the tables fp32, every [N,H,D] tensor
 *                  fp16, the results those of dtype S3D_DTYPE_F32 on fp32 copies of the rows with dq, dk, dv
 *                  rounded to fp16 (the same arithmetic; the two launches may pack the windows differently, which
 *                  reorders the fp32 sums); needs pairs > 0
 *   D in {8,16,32}, nd in {3,6,9}.  head_dim 32 and tables of more than 64 * nd rows per head in total (quant 8
 *                  with wide windows) run in a general form in the manner of the reference - one thread per
 *                  (query, head), atomic adds for dk, dv (fp32 accumulators in the workspace) and for the table
 *                  gradients (per workgroup in LDS, then global), so only dq is then the same bits on every
 *                  call; `pairs` is ignored.  It is some fifty times slower per pair than the forms described
 *                  here (0.2 s for 200 000 voxels at head_dim 32) and exists so that every shape of the forward
 *                  has a backward; its workspace is 8 * N * H * D bytes plus the statistics.
 *
 * No global atomics (the general form apart).  dq, dk, dv have one owning lane per row and are sums in a fixed order: the same bits on
 * every call.  The table gradients are accumulated per wavefront over the units it draws from the work queues,
 * left in a slot of the workspace and summed per head, slots in order, by a reduction kernel: which units a
 * wavefront draws varies from call to call, so these sums are regrouped and agree between calls to fp32 rounding
 * (about 1e-6 of the largest element), not bit for bit.
 */
size_t s3d_attn_bwd_workspace_bytes(int32_t H, int32_t D, int32_t nd, int64_t table_len, int64_t N, int64_t W,
                                    int64_t pairs);
int s3d_attn_bwd(const void *q, const void *k, const void *v, const void *table_q, const void *table_k,
                 const void *table_v, const int32_t *table_sizes, int32_t nd, int64_t table_len,
                 const int32_t *w_sizes, const int32_t *w2n, const int32_t *n2n, const float *n_coords,
                 const void *out, const float *out_max, const float *out_sum, const void *dout, void *dq,
                 void *dk, void *dv, float *dtable_q, float *dtable_k, float *dtable_v, int64_t N,
                 int32_t H, int32_t D, int64_t W, int64_t pairs, int32_t dtype, void *workspace,
                 size_t workspace_bytes, void *stream);

/*
 * Window sort + segment offsets.
 *
 * Replaces BasicLayer.get_map_pair / get_window_mapping
 * (Swin3D/modules/swin3d_layers.py:713-787, MinkowskiEngine pooling + kernel_map +
 * torch.sort) and the w2n / w_sizes part of sparse_self_attention (:96-103).
 *
 *   coords     device int32 [N,4] rows (batch, x, y, z); x,y,z multiples of `stride`
 *   stride     tensor stride of the voxel grid (>= 1)
 *   window     window size in voxels per side (1..10)
 *   shift      window shift in voxels (0 or window/2; get_shifted_sp, :824-838)
 *   n2n        device int32 [N]  out: window-sorted position -> original row
 *   w_w_id     device int32 [N]  out: local id lx*window^2 + ly*window + lz per sorted position
 *   w_sizes    device int32 [N]  out: first W entries = voxels per window
 *   w2n        device int32 [N]  out: first W entries = exclusive prefix sum of w_sizes
 *   counts     device int64 [4]  out: {W, M = sum w_sizes^2, max w_size, error flag}
 *                                 error flag != 0: a coordinate was outside the supported
 *                                 range (batch 0..4095, window coordinates -8192..8191)
 *   workspace  device scratch of at least s3d_window_index_workspace_bytes(N) bytes
 *
 * Window order: ascending (batch, wx, wy, wz) with floor division of the shifted
 * coordinate by window*stride; inside a window ascending local id; equal keys by
 * ascending original row.
 */
size_t s3d_window_index_workspace_bytes(int64_t N);
int s3d_window_index(const int32_t *coords, int64_t N, int32_t stride, int32_t window,
                     int32_t shift, int32_t *n2n, int32_t *w_w_id, int32_t *w_sizes, int32_t *w2n,
                     int64_t *counts, void *workspace, size_t workspace_bytes, void *stream);

/*
 * The same index by a counting sort over the lattice of windows, for scenes whose windows fit a dense lattice of
 * at most max(4096, 2 N) cells (capped at 2^24): the bounding box of (batch, wx, wy, wz) over the voxels.  Room-sized
 * scenes do; the call is then five launches of a few microseconds instead of a sort of all voxels.  Same arguments
 * and outputs as s3d_window_index (the results are identical, rows of equal coordinates in row order); own
 * workspace size.  When the lattice is too large, counts[3] has bit 1 (value 2) set and NO output is written: call
 * s3d_window_index instead.  counts[3] bit 0 (value 1): coordinates out of range, as for s3d_window_index.
 */
size_t s3d_window_index_grid_workspace_bytes(int64_t N);
int s3d_window_index_grid(const int32_t *coords, int64_t N, int32_t stride, int32_t window,
                          int32_t shift, int32_t *n2n, int32_t *w_w_id, int32_t *w_sizes, int32_t *w2n,
                          int64_t *counts, void *workspace, size_t workspace_bytes, void *stream);

/*
 * Representative voxel of every cell of a window sort: the member whose signal row is nearest (Euclidean, fp32) to
 * the mean of the cell's signal rows; ties go to the lower row.  With a sort at window = 2 a cell is a coarse voxel
 * of the stride-2 downsample (GridCoordsDown, Swin3D/modules/swin3d_layers.py:179-231, a chain of scatter
 * reductions there).  Members are summed in sorted order, so the result is deterministic.
 *
 *   n2n, w2n, w_sizes  device int32: outputs of s3d_window_index (W = counts[0] cells)
 *   signals            device fp32 rows of `signals_stride` floats, original row order; the first `num_signals`
 *                      columns (1..16) enter the distance
 *   out                device int64 [W]: the chosen row of every cell
 */
int s3d_cell_representatives(const int32_t *n2n, const int32_t *w2n, const int32_t *w_sizes, int64_t W,
                             const float *signals, int64_t signals_stride, int32_t num_signals, int64_t *out,
                             void *stream);

/*
 * Rows of the lattice neighbours of every voxel, from the voxels' sorted packed keys.
 *
 * A packed coordinate key is linear in (batch, x, y, z), so a neighbour's key is the voxel's key plus a constant
 * per offset.  Used for the 27 offsets of the stem's 3x3x3 sparse convolution (the reference takes the kernel map
 * from MinkowskiEngine, Swin3D/models/Swin3D.py:75-86); no counterpart kernel in the reference.
 *
 *   sorted_keys  device int64 [N] ascending, distinct      order  device int64 [N]: order[i] = row of sorted_keys[i]
 *   deltas       device int64 [M] key offsets (1 <= M <= 1024)
 *   out          device int64 [N,M]: out[order[i]][d] = order[p] with sorted_keys[p] = sorted_keys[i] + deltas[d],
 *                or N when no voxel has that key
 */
int s3d_key_neighbours(const int64_t *sorted_keys, const int64_t *order, int64_t N, const int64_t *deltas, int32_t M,
                       int64_t *out, void *stream);

/*
 * Signal matrix of the attention op in window-sorted order (the `n_coords` argument of s3d_attn_fwd), one pass.
 *
 * Replaces the tensor statements of BasicLayer.get_index01 (Swin3D/modules/swin3d_layers.py:800-804: window-local
 * voxel position + fractional position, other signals appended, both gathered into sorted order) and, with the
 * two scales, of WindowAttention.forward (:513-536: xyz columns times quant_size, the others times 2 * quant_size).
 *
 *   w_w_id, n2n   device int32 [N]   outputs of s3d_window_index
 *   frac          device fp32 [N,3]  position of the point inside its voxel, in voxels, original row order
 *   signals       device fp32 rows of `signals_stride` floats, original row order; the first `num_signals`
 *                 columns are used (0, 3 or 6: colour, normal); may be null when num_signals = 0
 *   out           device fp32 [N, 3 + num_signals]:
 *                 out[p] = ((lx, ly, lz) + frac[n2n[p]]) * xyz_scale, signals[n2n[p]] * other_scale
 *                 (sum and product rounded separately, as the tensor statements do)
 *   scales 1, 1 give the reference's unscaled n_coords.
 */
int s3d_window_signals(const int32_t *w_w_id, const int32_t *n2n, const float *frac, const float *signals,
                       int64_t signals_stride, int32_t num_signals, int32_t window, float xyz_scale,
                       float other_scale, float *out, int64_t N, void *stream);

/*
 * K nearest sources of every query inside the same batch segment.
 *
 * Replaces knn_cuda (Swin3D/src/knn/knn_cuda_kernel.cu:207-244, declared in
 * Swin3D/src/knn/knn_cuda_kernel.h:5-12, exported at Swin3D/src/knn/knn_api.cpp:5).
 *
 *   src_xyz      device fp32 [Ns,3]      query_xyz  device fp32 [Nq,3]
 *   src_offset   device int32 [B] cumulative END offsets of the batch segments of src
 *   query_offset device int32 [B] same for the queries
 *   ret_idx      device int32 [Nq,K] out: global source rows
 *   ret_dist2    device fp32 [Nq,K] out: SQUARED distances ((dx*dx + dy*dy) + dz*dz with
 *                every operation rounded to fp32, d = src - query)
 *   cell_size    edge of the bucketing grid in the units of xyz; <= 0 picks it from the data
 *   workspace    device scratch of at least s3d_knn_workspace_bytes(Ns, Nq, B) bytes
 *
 * Result per query: the K smallest sources under the order (distance, source row),
 * emitted in that order (ties go to the lower row).  Segments with fewer than K
 * sources are padded with row -1 and S3D_KNN_PAD_DIST2.  1 <= K <= S3D_KNN_KMAX.
 */
size_t s3d_knn_workspace_bytes(int64_t Ns, int64_t Nq, int32_t B);
int s3d_knn(int32_t K, const float *src_xyz, int64_t Ns, const float *query_xyz, int64_t Nq,
            const int32_t *src_offset, const int32_t *query_offset, int32_t B, int32_t *ret_idx,
            float *ret_dist2, float cell_size, void *workspace, size_t workspace_bytes,
            void *stream);

/*
 * Inverse-distance interpolation of source features at the queries, from the result of s3d_knn.
 *
 * Replaces the torch statement knn_linear_interpolation
 * (Swin3D/modules/swin3d_layers.py:53-73: K indexing passes over src_feat and the weight
 * arithmetic, about 3*K + 4 kernels) with one gather kernel:
 *   weight_i = 1 / (sqrt(dist2_i) + 1e-8), normalised over the K neighbours of the query
 *   out[q]   = sum_i weight_i * src_feat[idx[q][i]]
 *
 *   idx, dist2   device [Nq,K] as written by s3d_knn (squared distances)
 *   src_feat     device [Ns,C] of `dtype`        out   device [Nq,C] of `dtype`
 * Neighbour slots padded with row -1 carry no weight (the reference's torch indexing would read the
 * LAST source row there, with a weight of about 2e-5); a query with no neighbour at all gets zeros.
 * Accumulation is fp32, one rounding to `dtype`.
 */
/*
 * Channel-wise maximum of the source features over the K nearest sources of every query, from the result of s3d_knn.
 *
 * Replaces the gather + max of the KNN downsample (Swin3D/modules/swin3d_layers.py:292-312: query_knn_feature
 * builds [Nq,K,C], then max over K) with one kernel that never writes the gathered copies:
 *   out[q][c] = max_i src_feat[max(idx[q][i], 0)][c]
 * A slot padded with row -1 reads row 0, exactly as the clamped index of the tensor statement does.
 *   idx        device int32 [Nq,K] as written by s3d_knn
 *   src_feat   device [Ns,C] of `dtype` (Ns >= 1)        out   device [Nq,C] of `dtype`
 */
int s3d_knn_max_pool(const int32_t *idx, int32_t K, int64_t Nq, const void *src_feat, int64_t Ns, int32_t C,
                     int32_t dtype, void *out, void *stream);

int s3d_knn_interpolate(const int32_t *idx, const float *dist2, int32_t K, int64_t Nq, const void *src_feat,
                        int64_t Ns, int32_t C, int32_t dtype, void *out, void *stream);

/*
 * Residual add fused with LayerNorm, for the Swin block on either side of the attention operator.
 *
 * The reference block (Swin3D/modules/swin3d_layers.py:617-623) computes
 *   feats = short_cut + attn(norm1(feats));  feats = feats + mlp(norm2(feats))
 * with torch kernels (add, LayerNorm in fp32, and under autocast a cast in front of the next GEMM).  This call
 * does, per row of C channels,
 *   s = x + residual            (residual null: s = x)
 *   x_out = s                   (skipped when residual or x_out is null; x_out may be x)
 *   y = (s - mean(s)) / sqrt(var(s) + eps) * gamma + beta      (biased variance, as torch.nn.LayerNorm)
 *
 *   x              device [N,C] fp32 (the residual stream)
 *   residual       device [N,C] of residual_dtype (S3D_DTYPE_F32 / S3D_DTYPE_F16), or null
 *   gamma, beta    device [C] fp32
 *   y              device [N,C] of y_dtype
 * C a multiple of 4 and at most 1024; arithmetic in fp32.
 */
int s3d_add_layernorm(const float *x, const void *residual, int32_t residual_dtype, const float *gamma,
                      const float *beta, float eps, float *x_out, void *y, int32_t y_dtype, int64_t N, int32_t C,
                      void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SWIN3D_AMD_H */
