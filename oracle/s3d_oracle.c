/*
 * CPU oracle for the Swin3D sparse window-attention forward, its window index
 * builder and the KNN helper.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is a plain-C restatement of the
 * reference algorithm, written from the reference's source text, and is used
 * only as the checker in tests, in the smoke test and as the timed CPU
 * baseline of the benchmark.  No product code path may call into it.
 *
 * Reference files each function follows (paths relative to the Swin3D tree):
 *   s3d_oracle_window_index  Swin3D/modules/swin3d_layers.py:713-787 (get_map_pair,
 *                            get_window_mapping), :824-838 (get_shifted_sp)
 *   s3d_oracle_pair_index    Swin3D/modules/swin3d_layers.py:76-150 (sparse_self_attention)
 *                            and Swin3D/src/attn/attn_utils.cuh:372-381 (pair decode)
 *   s3d_oracle_crse_rows     Swin3D/src/attn/attn_utils.cuh:437-453 (set_qk_offset)
 *   s3d_oracle_attn_fwd_*    Swin3D/src/attn/self_attn_aio_fwd.cu:16-52 (max pass),
 *                            :111-188 (exp / accumulate pass),
 *                            Swin3D/src/attn/attn_utils.cuh:455-464 (table sum),
 *                            Swin3D/sparse_dl/attn/attn_coff.py:180-184 (raw / sum)
 *   s3d_oracle_attn_bwd_f64  Swin3D/src/attn/self_attn_aio_bwd.cu:14-113,
 *                            Swin3D/sparse_dl/attn/attn_coff.py:191-232
 *   s3d_oracle_knn           Swin3D/src/knn/knn_cuda_kernel.cu:139-204 with the
 *                            canonical (distance, index) order instead of heap order
 *   s3d_oracle_knn_heap      Swin3D/src/knn/knn_cuda_kernel.cu:29-62, 139-204, faithful
 *                            heap order (documentation of where the two differ)
 *
 * Parity status of each function (what pins it is in tests/test_oracle_*.py):
 *   window_index : pinned by dict-grouping brute force, permutation/scan invariants,
 *                  the shift property.  The reference's cross-window order comes from
 *                  MinkowskiEngine's hash map and is PARITY UNPINNED; the canonical
 *                  order here is lexicographic (batch, wx, wy, wz).
 *   pair_index   : pinned against both reference statements of the pair decode.
 *   crse_rows    : pinned by edge-value tests of the quantiser formula.
 *   attn_fwd     : pinned by a numpy fp64 brute force, softmax(QK^T)V special case,
 *                  closed forms and invariances.
 *   knn          : pinned by numpy lexsort brute force, scipy cKDTree, tie lattices.
 *   knn_heap     : restated from the source text only; PARITY UNPINNED (nothing
 *                  executable pins the reference's heap order here).
 *
 * Build: see oracle/Makefile (gcc -O2 -fopenmp -ffp-contract=off).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define S3D_MAX_ND 16

/* floor division for possibly negative numerators (MinkowskiEngine pools with
 * floor semantics on signed coordinates). */
static inline int32_t floordiv_i32(int32_t a, int32_t b)
{
    int32_t q = a / b;
    if ((a % b != 0) && ((a < 0) != (b < 0))) --q;
    return q;
}

/* ------------------------------------------------------------------------- */
/* Window index                                                              */
/* ------------------------------------------------------------------------- */

typedef struct {
    int32_t b, wx, wy, wz, local, orig;
} s3d_wkey;

static int wkey_cmp(const void *pa, const void *pb)
{
    const s3d_wkey *a = (const s3d_wkey *)pa, *b = (const s3d_wkey *)pb;
    if (a->b != b->b) return a->b < b->b ? -1 : 1;
    if (a->wx != b->wx) return a->wx < b->wx ? -1 : 1;
    if (a->wy != b->wy) return a->wy < b->wy ? -1 : 1;
    if (a->wz != b->wz) return a->wz < b->wz ? -1 : 1;
    if (a->local != b->local) return a->local < b->local ? -1 : 1;
    if (a->orig != b->orig) return a->orig < b->orig ? -1 : 1;
    return 0;
}

/*
 * coords   [N,4] int32 (batch, x, y, z); x, y, z are multiples of `stride`.
 * shift    window shift in voxels (0, or window_size / 2 for the shifted set).
 * Outputs (caller allocated, capacity N each):
 *   n2n[N]      sorted position -> original row
 *   w_w_id[N]   local id lx*ws*ws + ly*ws + lz of the voxel at each sorted position
 *   w_sizes[W]  voxels per window, w2n[W] exclusive prefix sum of w_sizes
 *   counts[0] = W, counts[1] = M = sum w_sizes^2
 */
int s3d_oracle_window_index(const int32_t *coords, int64_t N, int32_t stride, int32_t ws,
                            int32_t shift, int32_t *n2n, int32_t *w_w_id, int32_t *w_sizes,
                            int32_t *w2n, int64_t *counts)
{
    if (N < 0 || stride <= 0 || ws <= 0) return -1;
    s3d_wkey *keys = (s3d_wkey *)malloc(sizeof(s3d_wkey) * (size_t)(N > 0 ? N : 1));
    if (!keys) return -2;
    const int32_t span = ws * stride;
    for (int64_t i = 0; i < N; ++i) {
        int32_t c[3], w[3], l[3];
        for (int a = 0; a < 3; ++a) {
            c[a] = coords[i * 4 + 1 + a] + shift * stride;
            w[a] = floordiv_i32(c[a], span);
            l[a] = floordiv_i32(c[a] - w[a] * span, stride);
        }
        keys[i].b = coords[i * 4];
        keys[i].wx = w[0];
        keys[i].wy = w[1];
        keys[i].wz = w[2];
        keys[i].local = (l[0] * ws + l[1]) * ws + l[2];
        keys[i].orig = (int32_t)i;
    }
    qsort(keys, (size_t)N, sizeof(s3d_wkey), wkey_cmp);
    int64_t W = 0, M = 0;
    for (int64_t i = 0; i < N; ++i) {
        n2n[i] = keys[i].orig;
        w_w_id[i] = keys[i].local;
        int new_window = (i == 0) || keys[i].b != keys[i - 1].b || keys[i].wx != keys[i - 1].wx ||
                         keys[i].wy != keys[i - 1].wy || keys[i].wz != keys[i - 1].wz;
        if (new_window) {
            w2n[W] = (int32_t)i;
            w_sizes[W] = 0;
            ++W;
        }
        ++w_sizes[W - 1];
    }
    for (int64_t w = 0; w < W; ++w) M += (int64_t)w_sizes[w] * w_sizes[w];
    counts[0] = W;
    counts[1] = M;
    free(keys);
    return 0;
}

/*
 * The O(M) pair index the reference materialises ("v2" protocol): for every
 * pair m: its window, and the sorted positions of its query (x) and key (y).
 * w2m[W] is the exclusive prefix sum of w_sizes^2.
 */
int s3d_oracle_pair_index(const int32_t *w_sizes, int64_t W, int64_t *w2m, int64_t *m2w,
                          int64_t *x_offset, int64_t *y_offset)
{
    int64_t m = 0, base = 0;
    for (int64_t w = 0; w < W; ++w) {
        int64_t n = w_sizes[w];
        w2m[w] = m;
        for (int64_t off = 0; off < n * n; ++off) {
            if (m2w) m2w[m] = w;
            if (x_offset) x_offset[m] = base + off / n;
            if (y_offset) y_offset[m] = base + off % n;
            ++m;
        }
        base += n;
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* cRSE quantiser                                                            */
/* ------------------------------------------------------------------------- */

/*
 * Row of the axis-n table hit by the (query i, key j) pair.  The arithmetic is
 * fp32 in exactly the reference's operation order:
 *     rel = c_i - c_j;  rel += (Wn / 2);  rel = min(max(0, rel), float(Wn - 1e-10))
 * where float(Wn - 1e-10) == float(Wn).  A clamped value equal to Wn indexes
 * one row past the axis table in the reference; here it is folded onto the
 * last row (Wn - 1) and reported through *edge.
 */
static inline int32_t crse_row(float ci, float cj, int32_t Wn, int *edge)
{
    float rel = ci - cj;
    rel = rel + (float)(Wn / 2);
    float hi = (float)((double)Wn - 1e-10);
    float r = fminf(fmaxf(0.0f, rel), hi);
    int32_t row = (int32_t)r;
    if (row > Wn - 1) {
        row = Wn - 1;
        if (edge) *edge = 1;
    }
    return row;
}

/* rows[n] for one pair of sorted positions (i, j); returns number of edge hits. */
int s3d_oracle_crse_rows(const float *n_coords, int32_t nd, const int32_t *table_sizes,
                         int32_t HD, int64_t i, int64_t j, int32_t *rows)
{
    int edges = 0;
    for (int n = 0; n < nd; ++n) {
        int e = 0;
        rows[n] = crse_row(n_coords[i * nd + n], n_coords[j * nd + n], table_sizes[n] / HD, &e);
        edges += e;
    }
    return edges;
}

/* ------------------------------------------------------------------------- */
/* Attention forward                                                         */
/* ------------------------------------------------------------------------- */

/*
 * q, k, v      [N,H,D] float, original voxel order (fp16 callers pass the fp16 values widened)
 * tq, tk, tv   flat tables, layout [axis][row][h][c]; table_sizes[n] = rows_n*H*D
 * n_coords     [N,nd] float, window-sorted order, already scaled by the quant sizes
 * n2n          sorted position -> original row;  w_sizes / w2n per window
 * out          [N,H,D] normalised output (original order)
 * out_max      [N,H] max logit per (query, head)          (may be NULL)
 * out_sum      [N,H] sum_j exp(logit - max)                (may be NULL)
 * edge_pairs   number of (pair, axis) hits at the folded upper edge (may be NULL)
 *
 * The body lives in s3d_oracle_attn.inc and is instantiated twice: with double
 * accumulation for the parity oracle, with float for the timed CPU baseline.
 */
#define S3D_ATTN_NAME s3d_oracle_attn_fwd_f64
#define S3D_ATTN_ACC double
#define S3D_ATTN_EXP exp
#include "s3d_oracle_attn.inc"
#undef S3D_ATTN_NAME
#undef S3D_ATTN_ACC
#undef S3D_ATTN_EXP

#define S3D_ATTN_NAME s3d_oracle_attn_fwd_f32
#define S3D_ATTN_ACC float
#define S3D_ATTN_EXP expf
#include "s3d_oracle_attn.inc"
#undef S3D_ATTN_NAME
#undef S3D_ATTN_ACC
#undef S3D_ATTN_EXP

/*
 * Attention backward (double accumulation).
 *
 * Follows Swin3D/sparse_dl/attn/attn_coff.py:191-232 and
 * Swin3D/src/attn/self_attn_aio_bwd.cu:14-113 in the reference's own terms:
 *   raw_i        = out_i * sum_i                                    (attn_coff.py:219)
 *   sum_grad_i   = - sum_c raw_i[c] / sum_i^2 * dout_i[c]           (cal_exp_sum_grad_kernel, bwd.cu:38)
 *   exp_ij       = exp(logit_ij - max_i),  norm_ij = exp_ij / sum_i (bwd.cu:91-92)
 *   value_ij     = v_j + Tv(i,j)
 *   dv_j, dTv rows  += dout_i * norm_ij                             (bwd.cu:99-101)
 *   coff_grad_ij = (sum_c dout_i[c] value_ij[c] / sum_i + sum_grad_i) * exp_ij   (bwd.cu:103-106)
 *   dk_j += coff_grad (q_i + Tk(i,j));  dq_i += coff_grad (k_j + Tq(i,j))        (bwd.cu:107-108)
 *   dTq rows += coff_grad q_i;  dTk rows += coff_grad k_j                        (bwd.cu:109-110)
 * max_i and sum_i are recomputed here (the reference passes the forward's tensors in).
 * dq, dk, dv [N,H,D] and dtq, dtk, dtv [table_len] are overwritten.
 * Pinned by automatic differentiation of an independent dense statement of the forward
 * (tests/test_oracle_attn_bwd.py) and by central differences of the forward oracle.
 */
int s3d_oracle_attn_bwd_f64(const float *q, const float *k, const float *v, const float *tq, const float *tk,
                            const float *tv, const int32_t *table_sizes, int32_t nd, const int32_t *w_sizes,
                            const int32_t *w2n, const int32_t *n2n, const float *n_coords, const float *dout,
                            double *dq, double *dk, double *dv, double *dtq, double *dtk, double *dtv,
                            int64_t N, int32_t H, int32_t D, int64_t W)
{
    if (nd < 1 || nd > S3D_MAX_ND || H < 1 || D < 1) return -1;
    const int32_t HD = H * D;
    int32_t base[S3D_MAX_ND], rowsz[S3D_MAX_ND];
    int64_t table_len = 0;
    for (int n = 0; n < nd; ++n) {
        if (table_sizes[n] <= 0 || table_sizes[n] % HD != 0) return -3;
        base[n] = (int32_t)table_len;
        rowsz[n] = table_sizes[n] / HD;
        table_len += table_sizes[n];
    }
    memset(dq, 0, sizeof(double) * (size_t)N * HD);
    memset(dk, 0, sizeof(double) * (size_t)N * HD);
    memset(dv, 0, sizeof(double) * (size_t)N * HD);
    memset(dtq, 0, sizeof(double) * (size_t)table_len);
    memset(dtk, 0, sizeof(double) * (size_t)table_len);
    memset(dtv, 0, sizeof(double) * (size_t)table_len);
    for (int64_t w = 0; w < W; ++w) {
        const int64_t s0 = w2n[w];
        const int64_t n_w = w_sizes[w];
        double *logit = (double *)malloc(sizeof(double) * (size_t)(n_w > 0 ? n_w : 1));
        int32_t *rows = (int32_t *)malloc(sizeof(int32_t) * (size_t)(n_w > 0 ? n_w : 1) * (size_t)nd);
        double *bq = (double *)malloc(sizeof(double) * 3 * (size_t)D);
        double *bk = bq + D, *bv = bk + D;
        for (int64_t a = 0; a < n_w; ++a) {
            const int64_t i = s0 + a;
            const int64_t qi = n2n[i];
            for (int64_t b = 0; b < n_w; ++b) {
                int e = 0;
                for (int n = 0; n < nd; ++n)
                    rows[b * nd + n] = crse_row(n_coords[i * nd + n], n_coords[(s0 + b) * nd + n], rowsz[n], &e);
            }
            for (int32_t h = 0; h < H; ++h) {
                const float *qv = q + qi * HD + h * D;
                const float *go = dout + qi * HD + h * D;
                /* forward quantities of the row: logits, max, sum, unnormalised output */
                double mx = -INFINITY;
                for (int64_t b = 0; b < n_w; ++b) {
                    const float *kv = k + (int64_t)n2n[s0 + b] * HD + h * D;
                    double l = 0;
                    for (int32_t c = 0; c < D; ++c) {
                        double tq_c = 0, tk_c = 0;
                        for (int n = 0; n < nd; ++n) {
                            const int64_t f = (int64_t)base[n] + (int64_t)rows[b * nd + n] * HD + h * D + c;
                            tq_c += (double)tq[f];
                            tk_c += (double)tk[f];
                        }
                        l += (double)qv[c] * (double)kv[c] + (double)qv[c] * tq_c + (double)kv[c] * tk_c;
                    }
                    logit[b] = l;
                    if (l > mx) mx = l;
                }
                double sum = 0, raw_dot = 0;
                for (int64_t b = 0; b < n_w; ++b) sum += exp(logit[b] - mx);
                for (int64_t b = 0; b < n_w; ++b) {
                    const float *vv = v + (int64_t)n2n[s0 + b] * HD + h * D;
                    const double e = exp(logit[b] - mx);
                    for (int32_t c = 0; c < D; ++c) {
                        double tv_c = 0;
                        for (int n = 0; n < nd; ++n)
                            tv_c += (double)tv[(int64_t)base[n] + (int64_t)rows[b * nd + n] * HD + h * D + c];
                        raw_dot += e * ((double)vv[c] + tv_c) * (double)go[c];
                    }
                }
                const double sum_grad = -raw_dot / (sum * sum);
                for (int64_t b = 0; b < n_w; ++b) {
                    const int64_t kj = n2n[s0 + b];
                    const float *kv = k + kj * HD + h * D;
                    const float *vv = v + kj * HD + h * D;
                    for (int32_t c = 0; c < D; ++c) {
                        bq[c] = bk[c] = bv[c] = 0;
                        for (int n = 0; n < nd; ++n) {
                            const int64_t f = (int64_t)base[n] + (int64_t)rows[b * nd + n] * HD + h * D + c;
                            bq[c] += (double)tq[f];
                            bk[c] += (double)tk[f];
                            bv[c] += (double)tv[f];
                        }
                    }
                    const double e = exp(logit[b] - mx);
                    const double norm = e / sum;
                    double pv = 0;
                    for (int32_t c = 0; c < D; ++c) {
                        const double vg = (double)go[c] * norm;
                        dv[kj * HD + h * D + c] += vg;
                        for (int n = 0; n < nd; ++n)
                            dtv[(int64_t)base[n] + (int64_t)rows[b * nd + n] * HD + h * D + c] += vg;
                        pv += (double)go[c] * ((double)vv[c] + bv[c]) / sum;
                    }
                    const double cg = (pv + sum_grad) * e;
                    for (int32_t c = 0; c < D; ++c) {
                        dk[kj * HD + h * D + c] += cg * ((double)qv[c] + bk[c]);
                        dq[qi * HD + h * D + c] += cg * ((double)kv[c] + bq[c]);
                        for (int n = 0; n < nd; ++n) {
                            const int64_t f = (int64_t)base[n] + (int64_t)rows[b * nd + n] * HD + h * D + c;
                            dtq[f] += cg * (double)qv[c];
                            dtk[f] += cg * (double)kv[c];
                        }
                    }
                }
            }
        }
        free(logit);
        free(rows);
        free(bq);
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* KNN                                                                       */
/* ------------------------------------------------------------------------- */

#define S3D_KNN_KMAX 64
#define S3D_KNN_PAD_DIST 2147483648.0f /* float(0x7fffffff) */

/* squared distance, every operation rounded to fp32, d = src - query,
 * ((dx*dx) + (dy*dy)) + (dz*dz); the file is compiled with -ffp-contract=off. */
static inline float knn_dist2(const float *s, float qx, float qy, float qz)
{
    const float dx = s[0] - qx, dy = s[1] - qy, dz = s[2] - qz;
    const float xx = dx * dx, yy = dy * dy, zz = dz * dz;
    const float xy = xx + yy;
    return xy + zz;
}

static inline void knn_segment(int64_t g, const int32_t *src_offset, const int32_t *query_offset,
                               int32_t B, int64_t *begin, int64_t *end)
{
    int32_t b = 0;
    for (; b < B; ++b)
        if (g < query_offset[b]) break;
    if (b >= B) { /* query beyond the last offset: empty candidate set */
        *begin = 0;
        *end = 0;
        return;
    }
    *begin = b > 0 ? src_offset[b - 1] : 0;
    *end = src_offset[b];
}

/*
 * Canonical KNN: the K smallest sources of the query's batch segment under the
 * lexicographic order (squared distance, source index), emitted in that order.
 * Segments with fewer than K sources are padded with index -1, distance 2^31.
 * ret_dist2 holds SQUARED distances (the Python wrapper takes the root).
 */
int s3d_oracle_knn(int32_t K, const float *src_xyz, int64_t Ns, const float *query_xyz, int64_t Nq,
                   const int32_t *src_offset, const int32_t *query_offset, int32_t B,
                   int32_t *ret_idx, float *ret_dist2, int32_t num_threads)
{
    if (K < 1 || K > S3D_KNN_KMAX) return -1;
    (void)Ns;
#pragma omp parallel for schedule(dynamic, 64) num_threads(num_threads)
    for (int64_t g = 0; g < Nq; ++g) {
        float bd[S3D_KNN_KMAX];
        int32_t bi[S3D_KNN_KMAX];
        int32_t cnt = 0;
        int64_t s0, s1;
        knn_segment(g, src_offset, query_offset, B, &s0, &s1);
        const float qx = query_xyz[g * 3], qy = query_xyz[g * 3 + 1], qz = query_xyz[g * 3 + 2];
        for (int64_t i = s0; i < s1; ++i) {
            const float d = knn_dist2(src_xyz + i * 3, qx, qy, qz);
            /* sources arrive in ascending index, so a candidate equal to the
             * current worst never displaces it (lower index wins). */
            if (cnt == K && !(d < bd[K - 1])) continue;
            int32_t p = cnt < K ? cnt : K - 1;
            while (p > 0 && bd[p - 1] > d) {
                bd[p] = bd[p - 1];
                bi[p] = bi[p - 1];
                --p;
            }
            bd[p] = d;
            bi[p] = (int32_t)i;
            if (cnt < K) ++cnt;
        }
        for (int32_t t = 0; t < K; ++t) {
            ret_idx[g * K + t] = t < cnt ? bi[t] : -1;
            ret_dist2[g * K + t] = t < cnt ? bd[t] : S3D_KNN_PAD_DIST;
        }
    }
    return 0;
}

/* ---- faithful heap-order restatement (documentation only) ---------------- */

static void heap_sift(float *heap, int32_t *idx, int32_t start, int32_t end)
{
    int32_t curr = start, child = 2 * start + 1;
    while (child < end) {
        if (child + 1 < end && heap[child] < heap[child + 1]) ++child;
        if (heap[curr] > heap[child]) return;
        float tf = heap[curr];
        heap[curr] = heap[child];
        heap[child] = tf;
        int32_t ti = idx[curr];
        idx[curr] = idx[child];
        idx[child] = ti;
        curr = child;
        child = 2 * curr + 1;
    }
}

/*
 * Heap-order KNN as the reference kernel computes it: strict `dist < heap[0]`
 * replacement, sift that also swaps on equality, heap initialised to 2^31,
 * final heap sort.  Slots never filled keep distance 2^31 and index -1 here
 * (the reference leaves those indices uninitialised).
 */
int s3d_oracle_knn_heap(int32_t K, const float *src_xyz, int64_t Ns, const float *query_xyz,
                        int64_t Nq, const int32_t *src_offset, const int32_t *query_offset,
                        int32_t B, int32_t *ret_idx, float *ret_dist2)
{
    if (K < 1 || K > S3D_KNN_KMAX) return -1;
    (void)Ns;
    for (int64_t g = 0; g < Nq; ++g) {
        float heap[S3D_KNN_KMAX];
        int32_t idx[S3D_KNN_KMAX];
        for (int32_t t = 0; t < K; ++t) {
            heap[t] = S3D_KNN_PAD_DIST;
            idx[t] = -1;
        }
        int64_t s0, s1;
        knn_segment(g, src_offset, query_offset, B, &s0, &s1);
        const float qx = query_xyz[g * 3], qy = query_xyz[g * 3 + 1], qz = query_xyz[g * 3 + 2];
        for (int64_t i = s0; i < s1; ++i) {
            const float d = knn_dist2(src_xyz + i * 3, qx, qy, qz);
            if (d < heap[0]) {
                heap[0] = d;
                idx[0] = (int32_t)i;
                heap_sift(heap, idx, 0, K);
            }
        }
        for (int32_t t = K - 1; t > 0; --t) {
            float tf = heap[0];
            heap[0] = heap[t];
            heap[t] = tf;
            int32_t ti = idx[0];
            idx[0] = idx[t];
            idx[t] = ti;
            heap_sift(heap, idx, 0, t);
        }
        for (int32_t t = 0; t < K; ++t) {
            ret_idx[g * K + t] = idx[t];
            ret_dist2[g * K + t] = heap[t];
        }
    }
    return 0;
}

/*
 * Inverse-distance interpolation over KNN results, Swin3D/modules/swin3d_layers.py:53-73:
 *   dist = sqrt(dist2) in fp32 (Swin3D/sparse_dl/knn/knn.py:24), weight = 1 / (dist + 1e-8),
 *   weight /= sum of the weights of the query, out = sum_i src_feat[idx_i] * weight_i.
 * Double accumulation.  Slots padded with row -1 carry no weight (decision of this build: the
 * reference's torch indexing reads the last source row there).
 * Pinned by closed forms (tests/test_oracle_knn.py): constant field, coincident query,
 * hand-computed two-neighbour weights.
 */
int s3d_oracle_knn_interpolate(const int32_t *idx, const float *dist2, int32_t K, int64_t Nq,
                               const float *src_feat, int32_t C, double *out)
{
    if (K < 1 || C < 1 || Nq < 0) return -1;
    for (int64_t q = 0; q < Nq; ++q) {
        double norm = 0;
        for (int i = 0; i < K; ++i)
            if (idx[q * K + i] >= 0) norm += 1.0 / ((double)sqrtf(dist2[q * K + i]) + 1e-8);
        for (int32_t c = 0; c < C; ++c) out[q * C + c] = 0;
        for (int i = 0; i < K; ++i) {
            const int32_t row = idx[q * K + i];
            if (row < 0) continue;
            const double w = (1.0 / ((double)sqrtf(dist2[q * K + i]) + 1e-8)) / norm;
            for (int32_t c = 0; c < C; ++c) out[q * C + c] += w * (double)src_feat[(int64_t)row * C + c];
        }
    }
    return 0;
}

int s3d_oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
