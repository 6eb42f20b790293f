/*
 * fgnn.h -- C ABI of libfgnn_hip.so: fused GNN sparse operators for AMD gfx950 (MI355X).
 *
 * Every entry point takes plain device pointers and sizes, launches on the HIP stream handed
 * in (`stream` is a hipStream_t passed as void*; NULL = the null stream) and returns
 *      0            success
 *      < 0          argument error (FGNN_ERR_*), nothing was launched
 *      > 0          a hipError_t from a launch or runtime call
 * fgnn_last_error() gives a thread-local message for the last non-zero return.  Nothing in the
 * library aborts, exits or prints.  The caller owns every buffer (inputs, outputs, workspace);
 * the library owns only the schedule objects it hands out.  All index arrays are int32, all
 * value arrays are contiguous float32.  Graphs are CSR indexed by DESTINATION node (row = dst,
 * col_ind = src); per-edge arrays are in CSR position order; the CSC arrays (col_ptr, row_ind)
 * are the transpose with `permute[q]` = CSR position of CSC entry q.
 *
 * Each declaration cites the interface of the reference (mlsysAE2022/ae_mlsys_gnn) that it
 * stands in for.
 */
#ifndef FGNN_H
#define FGNN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
/* the library is built with hidden visibility; only the declarations below are exported */
#pragma GCC visibility push(default)

#define FGNN_ERR_NULL      (-1)  /* a required pointer is NULL */
#define FGNN_ERR_SHAPE     (-2)  /* a size is negative or inconsistent */
#define FGNN_ERR_ALIGN     (-3)  /* a float buffer is not 16-byte aligned */
#define FGNN_ERR_LIMIT     (-4)  /* a size exceeds what the kernels support */
#define FGNN_ERR_WORKSPACE (-5)  /* workspace missing or too small */
#define FGNN_ERR_SCHEDULE  (-6)  /* schedule does not match the arrays it is used with */

int         fgnn_version(void);
const char *fgnn_last_error(void);

/* ---------------------------------------------------------------- row schedules
 * A schedule is the degree-binned work list of one pointer array (row_ptr for forward passes,
 * col_ptr for backward passes): rows longer than `seg_len` edges are cut into segments that are
 * reduced separately and merged, and the work items are ordered longest first.  The reference
 * has no counterpart (it launches one block per row: src/fused_gat/fused_gat_SM.cu:518-532);
 * passing sched == NULL to an operator selects the same one-wave-per-row mapping.
 * The list is built on the device (segment counts per row, two scans, a stable radix sort by length); only a dozen
 * counters come back to the host for the allocation sizes, which synchronises `stream` once or twice.  The
 * reference prepares its graphs on the host with scipy (script/train/train_gatconv_our.py:87-121).
 * FGNN_SCHEDULE_BUILDER=host in the environment selects the first implementation instead (the pointer array read
 * back and the list built by the host): item for item the same list, kept as the cross-check. */
typedef struct fgnn_schedule fgnn_schedule_t;
int     fgnn_schedule_create(const int32_t *ptr_dev, int n_rows, int seg_len, void *stream,
                             fgnn_schedule_t **out);
/* XCD-aware variant for the gather kernels (fused GAT, mhspmm, GMMConv): rows longer than min_deg
 * (<= 0: 64) entries are cut by source bucket (8 buckets, one per XCD) and workgroup w only gets
 * segments of bucket w % 8, so each XCD's L2 sees one eighth of the gathered feature rows.  The
 * schedule keeps its own bucket-ordered copy of `idx` (4*E bytes of device memory) and, with
 * with_positions != 0, the original position of every entry (another 4*E bytes): operators with
 * per-edge tensors (stashed GAT attention, mhspmm weights, GMMConv pseudo-coordinates) need it and
 * return FGNN_ERR_SCHEDULE without; the recomputing fused GAT does not.  `idx` must be the array later
 * passed to the operator.
 * The layout assumes that workgroup w of a dispatch runs on XCD w % 8, which is how a gfx950 device that shows all 256
 * compute units behaves; the call checks the device (architecture name and compute-unit count, once per device) and on
 * anything else (a partition of the part, another part) builds the plain list of fgnn_schedule_create instead:
 * fgnn_schedule_num_buckets() of the result tells (8 or 0).  FGNN_XCD_MAPPING=0 / 1 in the environment overrides the
 * check.  fgnn_xcd_mapping_for() is the rule itself (XCD count for an architecture name and a compute-unit count, 0 =
 * mapping unknown), exported so that it can be tested without a device. */
int     fgnn_xcd_mapping_for(const char *gcn_arch, int compute_units);
int     fgnn_schedule_num_buckets(const fgnn_schedule_t *s);
int     fgnn_schedule_create_bucketed(const int32_t *ptr_dev, const int32_t *idx_dev, int n_rows,
                                      int seg_len, int min_deg, int with_positions, void *stream,
                                      fgnn_schedule_t **out);
/* Copies the map from the schedule's entry order to the caller's edge positions into pos_out[E]
 * (identity for a plain schedule), frees the schedule's copy and switches the schedule to "own order":
 * operators then index per-edge tensors (pseudo-coordinates, stashed attention, mhspmm weights, the
 * per-edge gradients they return) and `permute` by the schedule's entry order q, i.e. the caller passes
 * t_own[q] = t[pos_out[q]].  Worth it for per-edge data that is constant or produced elementwise: under an
 * XCD-aware schedule every XCD then touches contiguous runs instead of scattered elements (fused GMMConv at
 * 114.8 M edges: backward 3.6 -> 2.5 ms).  Once per schedule; FGNN_ERR_SCHEDULE for an XCD-aware schedule
 * built without positions.  No counterpart in the reference.  Synchronises `stream`. */
int     fgnn_schedule_take_positions(fgnn_schedule_t *s, int32_t *pos_out_dev, void *stream);
void    fgnn_schedule_destroy(fgnn_schedule_t *s);
int     fgnn_schedule_num_items(const fgnn_schedule_t *s);
int     fgnn_schedule_num_partials(const fgnn_schedule_t *s);   /* segments of split rows */
int64_t fgnn_schedule_num_edges(const fgnn_schedule_t *s);
/* Device memory the schedule itself holds (work items, split table, the bucket-ordered index copy and the
 * position map of an XCD-aware schedule): allocated by the library outside the caller's allocator, so a
 * caller that reports peak memory adds it.  No counterpart in the reference. */
size_t  fgnn_schedule_device_bytes(const fgnn_schedule_t *s);
/* For inspection and tests: the work items (4 ints each: row, begin, end, partial slot or -1; row -1 = padding of an
 * XCD-aware list) and the table of split rows (4 ints each: row, first slot, segments, 0) copied to device memory of
 * the caller; items_out holds 4 * fgnn_schedule_num_items ints, splits_out 4 * fgnn_schedule_num_splits; either
 * may be NULL. */
int     fgnn_schedule_num_splits(const fgnn_schedule_t *s);
/* The lists are sorted longest first: every work item at a slot >= this number has at most 64 entries (a multiple of 64
 * slots per source bucket, or fgnn_schedule_num_items).  On graphs of short rows the kernels for rows narrower than a wave
 * (fused GAT up to 128 floats, multi-head SpMM and GMMConv up to 64) put a whole wave on each item before it and one lane
 * group of a wave on each item after it, in one launch.  No counterpart in the reference. */
int     fgnn_schedule_num_wave_slots(const fgnn_schedule_t *s);
int     fgnn_schedule_export(const fgnn_schedule_t *s, int32_t *items_out, int32_t *splits_out, void *stream);

/* Checks a CSR (or CSC) pair before any gather kernel sees it: ptr[0] == 0, ptr non-decreasing,
 * ptr[n_rows] == E and every idx in [0, n_cols).  One reduction kernel and a 4-byte read-back (synchronises
 * `stream`); returns FGNN_ERR_SHAPE with the findings in fgnn_last_error().  The operators themselves do not
 * range-check indices (the reference's do not either: src/fused_gat/fused_gat_SM.cpp:22-36 only asserts
 * device, dtype and contiguity), so a loader of untrusted files calls this first. */
int     fgnn_validate_graph(const int32_t *ptr_dev, const int32_t *idx_dev, int n_rows, int n_cols, int64_t E,
                            void *stream);

/* Two numbers about the row lengths of a pointer array, for the caller's choice between the plain and the
 * XCD-aware schedule: stats_host[0] = entries held by rows longer than long_len, stats_host[1] = the longest
 * row.  One reduction kernel and a 16-byte read-back (synchronises `stream`).  No counterpart in the
 * reference, whose kernels take one row per thread block whatever its length
 * (src/fused_gat/fused_gat_SM.cu:139-145 launches N blocks). */
int     fgnn_row_length_stats(const int32_t *ptr_dev, int n_rows, int long_len, int64_t *stats_host, void *stream);

/* ---------------------------------------------------------------- fused GAT
 * Replaces fused_gat_SM.gat_forward (src/fused_gat/fused_gat_SM.cpp:14-38, host launcher
 * fused_gat_SM.cu:536-558) and, with e_lrelu/e_softmax non-NULL, fused_gat_stash.gat_forward
 * and fused_gat.gat_forward (src/fused_gat/fused_gat_stash.cu:420-442, fused_gat.cu:365-386).
 *   out[i,h,:] = sum_p softmax_p(lrelu(attn_row[i,h] + attn_col[col_ind[p],h])) * in_feat[col_ind[p],h,:]
 * Outputs: out [N,H,F], edge_max, edge_sum [N,H].  Optional (NULL to skip):
 *   aux_out2 [N,H,F], aux_c [N,H]  -- sum_p alpha*lrelu'(e) * in_feat and sum_p alpha*lrelu'(e);
 *                                     they let the backward run in a single gather pass
 *   e_lrelu, e_softmax [E,H]       -- the stashed per-edge tensors of the stash variants; e_lrelu may be
 *                                     NULL alone (fgnn_gat_backward does not read it)
 * Workspace: fgnn_gat_forward_workspace_bytes(sched, H, F) bytes (0 when sched is NULL). */
size_t fgnn_gat_forward_workspace_bytes(const fgnn_schedule_t *sched, int H, int F);
int    fgnn_gat_forward(int N, int64_t E, int H, int F,
                        const float *attn_row, const float *attn_col,
                        const int32_t *row_ptr, const int32_t *col_ind, float negative_slope,
                        const float *in_feat, float *out, float *edge_max, float *edge_sum,
                        float *aux_out2, float *aux_c, float *e_lrelu, float *e_softmax,
                        const fgnn_schedule_t *sched, void *workspace, size_t workspace_bytes,
                        void *stream);

/* Replaces fused_gat_SM.gat_backward (src/fused_gat/fused_gat_SM.cpp:40-124, host launcher
 * fused_gat_SM.cu:865-893); with permute/e_softmax non-NULL it reads the stashed attention
 * instead of recomputing it (fused_gat_stash.gat_backward, fused_gat_stash.cu:776-804;
 * fused_gat.gat_backward, fused_gat.cu:641-670): e_softmax is then the CSR-ordered [E,H] array of fgnn_gat_forward and
 * permute is required (FGNN_ERR_NULL without it; a stash written by fgnn_gat_stash_own_order has another layout and goes
 * to fgnn_gat_backward_own_order).  e_lrelu is accepted for the reference's argument list and not read: the sign of the
 * pre-activation is that of attn_row + attn_col.
 * Rows of more than 1024 floats (any number of heads <= 64 of up to 1024 floats each, the range of
 * fused_gat_SM.cu:518-522, :843-847) are served in passes over groups of heads through contiguous slices kept in the
 * workspace; they need a schedule (FGNN_ERR_SCHEDULE otherwise), and the workspace functions include the slices.
 * need_recompute of the workspace function: bit 0 = out_feat/aux_out2/aux_c will be NULL, bit 1 = a stash will be passed
 * (only rows of more than 1024 floats need room for it).
 * Inputs as the reference's plus out_feat/aux_out2/aux_c from the forward; when those three are
 * NULL they are recomputed into the workspace from (row_ptr, col_ind) first.
 * Outputs: grad_feat [N,H,F], grad_attn_row, grad_attn_col [N,H]; all fully overwritten and
 * bit-reproducible from run to run (no atomics).
 * sched_csr is only used for the recompute case. */
size_t fgnn_gat_backward_workspace_bytes(int N, int H, int F, const fgnn_schedule_t *sched_csc,
                                         const fgnn_schedule_t *sched_csr, int need_recompute);
int    fgnn_gat_backward(int N, int64_t E, int H, int F, float negative_slope,
                         const int32_t *row_ptr, const int32_t *col_ind,
                         const int32_t *col_ptr, const int32_t *row_ind,
                         const int32_t *permute, const float *e_lrelu, const float *e_softmax,
                         const float *edge_max, const float *edge_sum,
                         const float *in_feat, const float *attn_row, const float *attn_col,
                         const float *out_feat, const float *aux_out2, const float *aux_c,
                         const float *grad_out,
                         float *grad_feat, float *grad_attn_row, float *grad_attn_col,
                         const fgnn_schedule_t *sched_csc, const fgnn_schedule_t *sched_csr,
                         void *workspace, size_t workspace_bytes, void *stream);

/* fgnn_gat_backward reading the stash of fgnn_gat_stash_own_order (below): e_softmax_own[q,h] in the entry order of this
 * pass under the same sched_csc, sign bit set where the pre-activation is not positive.  The layout is a property of the
 * entry point, not of a NULL argument: a CSR-ordered stash handed in here (or the reverse) would be read as the wrong
 * edges' weights without any error.  No counterpart in the reference, whose stash is CSR-ordered
 * (src/fused_gat/fused_gat_stash.cu:444-464). */
int    fgnn_gat_backward_own_order(int N, int64_t E, int H, int F, float negative_slope,
                                   const int32_t *row_ptr, const int32_t *col_ind,
                                   const int32_t *col_ptr, const int32_t *row_ind,
                                   const float *e_softmax_own, const float *edge_max, const float *edge_sum,
                                   const float *in_feat, const float *attn_row, const float *attn_col,
                                   const float *out_feat, const float *aux_out2, const float *aux_c,
                                   const float *grad_out,
                                   float *grad_feat, float *grad_attn_row, float *grad_attn_col,
                                   const fgnn_schedule_t *sched_csc, const fgnn_schedule_t *sched_csr,
                                   void *workspace, size_t workspace_bytes, void *stream);

/* The reference's fuse-scatter GAT variant as it defines it (operators/fused_gat.py:36-50; src/fused_gat/fused_gat.cu):
 * forward = fused_scatter_kernel (:235-300: scores, LeakyReLU and row softmax in one pass that writes [E,H]) + mhspmm;
 * backward = permuted mhspmm + mhsddmm + fused_gather_row (:502-556) + gather_col (:558-586).
 * fgnn_gat_scatter is the first kernel: e_softmax[p,h] = softmax over row(p) of lrelu(attn_row[row(p),h] +
 * attn_col[col_ind[p],h]); e_lrelu (optional, NULL to skip) gets the LeakyReLU values the reference stashes next to it.
 * fgnn_gat_gather_row is fused_gather_row: grad_edge_out[p,h] = lrelu'(e) * e_softmax * (grad_edge - sum_row e_softmax *
 * grad_edge) and grad_attn_row = its row sums, in one pass; the sign of the pre-activation is read from e_lrelu when that
 * is given and formed again from col_ind / attn_row / attn_col otherwise (4 bytes per entry read instead of 4*H, and no
 * second [E,H] array kept between the passes).  grad_edge_out may be grad_edge (in place).  The SpMM steps are fgnn_mhspmm
 * and fgnn_mhsddmm, gather_col is fgnn_edge_colsum.  H <= 64. */
int    fgnn_gat_scatter(int N, int64_t E, int H, const int32_t *row_ptr, const int32_t *col_ind, const float *attn_row,
                        const float *attn_col, float negative_slope, float *e_lrelu, float *e_softmax, void *stream);
int    fgnn_gat_gather_row(int N, int64_t E, int H, const int32_t *row_ptr, const int32_t *col_ind, const float *attn_row,
                           const float *attn_col, const float *e_lrelu, float negative_slope, const float *e_softmax,
                           const float *grad_edge, float *grad_edge_out, float *grad_attn_row, void *stream);

/* The stashed attention of the stash variants in the ORDER OF THE BACKWARD PASS: e_softmax_own[q,h] = alpha of
 * entry q of the walk of (col_ptr, row_ind) under sched_csc (its bucket-ordered entry order when it is XCD-aware,
 * plain CSC order otherwise or with sched_csc == NULL), computed from the forward's row statistics; the sign bit of
 * the stored value is set when the edge's pre-activation is not positive (alpha itself is >= 0), so the backward
 * needs no other per-edge or per-destination data than <grad_out, out>.
 * fgnn_gat_backward_own_order called with this array and the same sched_csc then streams the
 * stash instead of gathering it through permute (114.8 M edges, 8 heads: backward 10.5 -> about 7 ms).  The
 * reference keeps its stash in CSR order and transposes while reading (src/fused_gat/fused_gat_stash.cu:444-464);
 * a caller that owns the stashed tensor (the autograd function does) is free to keep it in this order instead. */
int    fgnn_gat_stash_own_order(int N, int64_t E, int H, float negative_slope, const int32_t *col_ptr,
                                const int32_t *row_ind, const float *attn_row, const float *attn_col,
                                const float *edge_max, const float *edge_sum, float *e_softmax_own,
                                const fgnn_schedule_t *sched_csc, void *stream);

/* ---------------------------------------------------------------- fused EdgeConv
 * Replaces fused_edgeconv.edgeconv_forward / edgeconv_backward
 * (src/fused_edgeconv/fused_edgeconv.cpp:12-51; fused_edgeconv.cu:148-200).
 *   out[i,f] = max_{p in [i*k,(i+1)*k)} (h_dst[i,f] + h_src[src_ind[p],f]);  argmax[i,f] = the
 *   source node id at the FIRST maximal position (int32; the reference stores a float).
 * backward: grad_src[n_src,F] = scatter-add of grad_out at argmax (zero-filled first). */
int fgnn_edgeconv_forward(int N, int n_src, int F, int k, const int32_t *src_ind,
                          const float *h_src, const float *h_dst, float *out, int32_t *argmax,
                          void *stream);
int fgnn_edgeconv_backward(int N, int n_src, int F, const int32_t *argmax, const float *grad_out,
                           float *grad_src, void *stream);

/* EdgeConv with the LeakyReLU that follows every EdgeConv of the reference's DGCNN stack
 * (script/train/train_edgeconv_our.py:56, `h = F.leaky_relu(h, 0.2)`) fused in: the forward stores
 * lrelu(max, out_slope); the backward replays the mask from that output (out > 0 <=> pre-activation > 0 for
 * out_slope > 0, which is required) while it scatters, and writes the masked gradient -- the gradient of h_dst --
 * to grad_dst.  block > 0 selects the blocked form (workspace of fgnn_edgeconv_backward_blocked_workspace_bytes),
 * block <= 0 the plain scatter (workspace unused). */
int fgnn_edgeconv_forward_lrelu(int N, int n_src, int F, int k, const int32_t *src_ind, const float *h_src,
                                const float *h_dst, float out_slope, float *out, int32_t *argmax, void *stream);
int fgnn_edgeconv_backward_lrelu(int N, int n_src, int F, int block, const int32_t *argmax, const float *out,
                                 float out_slope, const float *grad_out, float *grad_src, float *grad_dst,
                                 void *workspace, size_t workspace_bytes, void *stream);

/* The same backward for batched point clouds.  `block` is a hint that the neighbours of destination
 * rows [b*block, (b+1)*block) lie in source rows of the same range, as in a kNN graph of clouds of
 * `block` points (fgnn_knn_graph): those contributions are accumulated in LDS and written with plain
 * stores; any others go through an overflow list in the workspace and global atomics, so a wrong hint
 * only costs time.  Falls back to fgnn_edgeconv_backward when n_src != N or block > 4096.  No
 * counterpart in the reference (its backward is the plain scatter, fused_edgeconv.cu:175-187). */
size_t fgnn_edgeconv_backward_blocked_workspace_bytes(int N, int F);
int    fgnn_edgeconv_backward_blocked(int N, int n_src, int F, int block, const int32_t *argmax,
                                      const float *grad_out, float *grad_src, void *workspace,
                                      size_t workspace_bytes, void *stream);

/* fgnn_edgeconv_backward_blocked for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): same arguments without the workspace.  The overflow list
 * lives in a fixed device array inside the library (16 MiB + 256 B, held by every GPU the library runs on until
 * the process ends); the call allocates nothing and rejects N*F above
 * fgnn_edgeconv_backward_blocked_static_max_elems() (4 Mi elements) with FGNN_ERR_LIMIT.  All calls on one GPU
 * share that array: calls that overlap on one GPU (different streams, different threads) race; calls on one
 * stream are safe, each call rebuilds the list from a counter it clears first.  The first call on a device looks the
 * array's device address up (hipGetSymbolAddress, under a mutex): make one ordinary call on each device before a call
 * under stream capture.  Shapes that take the plain fill-and-scatter form (n_src != N, block > 4096) use no scratch and
 * are not bound by the size limit.  No counterpart in the reference. */
size_t fgnn_edgeconv_backward_blocked_static_max_elems(void);
int    fgnn_edgeconv_backward_blocked_static(int N, int n_src, int F, int block, const int32_t *argmax,
                                             const float *grad_out, float *grad_src, void *stream);

/* k-nearest-neighbour graph of batched point clouds, the input of fgnn_edgeconv_forward: points
 * [n_clouds*P, D]; src_ind [n_clouds*P*k] gets, for every point, the global ids of the k nearest
 * points of its own cloud (itself included), nearest first, ties to the smaller id; 1 <= k <= min(P,
 * 128).  Stands in for
 * the DGL KNNGraph call of the reference's DGCNN loop (script/train/train_edgeconv_our.py:51-55). */
int fgnn_knn_graph(int n_clouds, int P, int D, int k, const float *points, int32_t *src_ind,
                   void *stream);

/* ---------------------------------------------------------------- fused GMMConv (MoNet)
 * Replaces gmmconv.gmmconv / gmmconveb / gmmconvstash (src/fused_gmmconv/gmmconv.cc:43-78;
 * gmmconv.cu:201-263):  w[p,k] = exp(-0.5 sum_d ((pseudo[p,d]-mu[k,d])*inv_sigma[k,d])^2),
 *   out[i,k,:] = sum_p w[p,k] * node_feat[col_ind[p],k,:].
 * pseudo [E,dim] is in the position order of (ptr, idx); when pos_map is non-NULL the row
 * pseudo[pos_map[p]] is used instead (lets a CSC pass read CSR-ordered pseudo without the
 * mhtranspose copy of operators/fused_gmmconv.py:55).  gauss_out [E,K] optional.
 * sum_kernels == 1 fuses the layer's `.sum(1)` (layers/gmmconv_layer.py:69) into the store:
 * out is then [N,F] = sum_k out[i,k,:].
 * sum_kernels == 2: node_feat is ONE [N,F] matrix shared by the K kernels (node_feat[j,k,:] == node_feat[j,:]
 * for every k), out stays [N,K,F].  A layer whose input is narrower than K x its output aggregates the
 * input this way and multiplies by the fc weights afterwards, which is the same sum with the two linear
 * steps exchanged; an edge then gathers F floats instead of K x out.  Needs F % 4 == 0, F <= 256, K <= 4,
 * gauss_out == NULL (FGNN_ERR_LIMIT / FGNN_ERR_SHAPE otherwise). */
size_t fgnn_gmm_forward_workspace_bytes(const fgnn_schedule_t *sched, int K, int F);
int    fgnn_gmm_forward(int N, int64_t E, int K, int dim, int F,
                        const int32_t *ptr, const int32_t *idx, const int32_t *pos_map,
                        const float *node_feat, const float *pseudo, const float *mu,
                        const float *inv_sigma, float *out, float *gauss_out, int sum_kernels,
                        const fgnn_schedule_t *sched, void *workspace, size_t workspace_bytes,
                        void *stream);

/* fgnn_gmm_forward with sum_kernels == 1 and the layer's epilogue (layers/gmmconv_layer.py:69-75: `rst = rst +
 * res_fc(feat)`, `rst = rst + bias`) in the same store: out[i,:] = sum_k out[i,k,:] + residual[i,:] + bias[:], bias [F]
 * and residual [N,F] optional (NULL).  Their gradients are the gradient of out (summed over the nodes for the
 * bias), so fgnn_gmm_backward serves unchanged. */
int    fgnn_gmm_forward_epilogue(int N, int64_t E, int K, int dim, int F,
                                 const int32_t *ptr, const int32_t *idx, const int32_t *pos_map,
                                 const float *node_feat, const float *pseudo, const float *mu,
                                 const float *inv_sigma, const float *bias, const float *residual,
                                 float *out, float *gauss_out, const fgnn_schedule_t *sched,
                                 void *workspace, size_t workspace_bytes, void *stream);

/* Replaces the backward sequence of operators/fused_gmmconv.py:51-58 (mhsddmm + mhtranspose +
 * gmmconv over CSC + GaussianBp, gmmconv.cu:265-285) with one pass over the CSC arrays:
 * grad_feat [N,K,F], grad_pseudo [E,dim] (CSR order), grad_mu, grad_sigma [K,dim].
 * The pass writes gw*w per edge into the workspace; a second edge-parallel kernel finishes the
 * Gaussian derivatives, grad_mu / grad_sigma reduced in a fixed order (bit-reproducible).
 * A schedule of col_ptr is required.
 * permute == NULL: pseudo is given in the order of (col_ptr, row_ind) itself and grad_pseudo comes back
 * in that order.  A caller that keeps its per-edge inputs in both orders (they are often an
 * elementwise function of constant edge data) thereby avoids the per-edge gather and scatter through
 * permute, which is most of this pass on large graphs. */
size_t fgnn_gmm_backward_workspace_bytes(const fgnn_schedule_t *sched_csc, int K, int dim, int F);
/* sum_kernels == 1: grad_out is [N,F], the gradient of the fused sum over kernels (every kernel of a
 * node sees the same row, so the pass gathers F instead of K*F floats per edge).
 * sum_kernels == 2: node_feat is [N,F], shared by the K kernels (see fgnn_gmm_forward); grad_out is [N,K,F]
 * and grad_feat [N,K,F] receives kernel k's share in slice k: the gradient of node_feat is their sum over k. */
int    fgnn_gmm_backward(int N, int64_t E, int K, int dim, int F,
                         const int32_t *col_ptr, const int32_t *row_ind, const int32_t *permute,
                         const float *node_feat, const float *pseudo, const float *mu,
                         const float *inv_sigma, const float *grad_out, int sum_kernels,
                         float *grad_feat, float *grad_pseudo, float *grad_mu, float *grad_sigma,
                         const fgnn_schedule_t *sched_csc, void *workspace, size_t workspace_bytes,
                         void *stream);

/* gmmconv.Gaussian / gmmconv.GaussianBp (gmmconv.cc:36-41,80-86; gmmconv.cu:187-199,265-285).
 * The backward implements the closed-form derivatives of the Gaussian weight; grad_mu and
 * grad_sigma are reduced in a fixed order (bit-reproducible). */
int    fgnn_gaussian(int64_t E, int K, int dim, const float *pseudo, const float *mu,
                     const float *inv_sigma, float *out, void *stream);
size_t fgnn_gaussian_backward_workspace_bytes(int64_t E, int K, int dim);
int    fgnn_gaussian_backward(int64_t E, int K, int dim, const float *pseudo, const float *mu,
                              const float *inv_sigma, const float *grad_w,
                              float *grad_pseudo, float *grad_mu, float *grad_sigma,
                              void *workspace, size_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------- small operators
 * mhspmm.mhspmm (src/spmm/mhspmm.cc; mhspmm.cu:44-66): out[i,h,:] = sum_p att[p,h]*feat[idx[p],h,:];
 * att row used is att[pos_map[p]] when pos_map is non-NULL.  With H == 1 and att == NULL it is
 * the unweighted single-head SpMM of operators/spmm.py:38-41.
 * Workspace: the partial results of split rows and, for an XCD-aware schedule with a head count that is neither a
 * multiple of four nor below three, E*H floats more into which the weights are first copied in the list's entry order
 * (the gather pass then streams them; with H % 4 == 0 it reads them in place as 128-bit words).  With att == NULL, or
 * with a workspace that only holds the partials (fgnn_gmm_forward_workspace_bytes of the same shape), the weights are
 * always read in place. */
size_t fgnn_mhspmm_workspace_bytes(const fgnn_schedule_t *sched, int H, int F);
int    fgnn_mhspmm(int N, int64_t E, int H, int F, const int32_t *ptr, const int32_t *idx,
                   const int32_t *pos_map, const float *att, const float *feat, float *out,
                   const fgnn_schedule_t *sched, void *workspace, size_t workspace_bytes,
                   void *stream);
/* mhsddmm.mhsddmm (src/sddmm/mhsddmm.cc; mhsddmm.cu:83-99) and, with H == 1, sddmm.csr_sddmm
 * (src/sddmm/sddmm.cpp): out[p,h] = <a[row(p),h,:], b[col_ind[p],h,:]>. */
int    fgnn_mhsddmm(int N, int64_t E, int H, int F, const int32_t *row_ptr, const int32_t *col_ind,
                    const float *a, const float *b, float *out, void *stream);
/* The same operator walked under a work list of (row_ptr, col_ind) that carries its edge positions (NULL = the
 * call above): with an XCD-aware list every XCD gathers from one eighth of the b-rows; results are stored at the
 * caller's CSR positions either way, unless the list's position map was handed out (fgnn_schedule_take_positions):
 * then out is in the list's entry order, written as contiguous runs. */
int    fgnn_mhsddmm_scheduled(int N, int64_t E, int H, int F, const int32_t *row_ptr, const int32_t *col_ind,
                              const float *a, const float *b, float *out, const fgnn_schedule_t *sched,
                              void *stream);
/* sddmm.coo_sddmm (src/sddmm/sddmm.cpp:12-27), with heads: out[e,h] = <a[row_ind[e],h,:],
 * b[col_ind[e],h,:]> for an edge list; a is [n_rows,H,F], b is [n_cols,H,F].  Indices are not
 * range-checked on the device. */
int    fgnn_sddmm_coo(int64_t E, int n_rows, int n_cols, int H, int F, const int32_t *row_ind,
                      const int32_t *col_ind, const float *a, const float *b, float *out,
                      void *stream);
/* mhtranspose.mhtranspose (src/csr2csc/mhtranspose.cc; mhtranspose.cu:28-47): out[q,:] = in[permute[q],:]. */
int    fgnn_gather_rows(int64_t E, int W, const int32_t *permute, const float *in, float *out,
                        void *stream);
/* edge_softmax.edge_softmax / edge_softmax_backward (src/edge_softmax/edge_softmax.cc;
 * edge_softmax.cu:100-128). */
int    fgnn_edge_softmax(int N, int64_t E, int H, const int32_t *row_ptr, const float *in, float *out,
                         void *stream);
int    fgnn_edge_softmax_backward(int N, int64_t E, int H, const int32_t *row_ptr, const float *sm,
                                  const float *grad_out, float *grad_in, void *stream);
/* u_add_v.u_add_v_forward / u_add_v_backward (src/u_add_v/u_add_v.cpp; u_add_v.cu:28-90):
 * out[p,w] = row_val[row(p),w] + col_val[col_ind[p],w]; backward grad_row[i,:] = sum of grad_out over row i,
 * grad_col[j,:] = sum of grad_out over the entries with col_ind == j.  fgnn_u_add_v_backward takes the reference's
 * arguments and, like the reference, forms the column sums with float atomics (into a buffer it zero-fills first):
 * the summation order, and with it the last bits of grad_col, vary from run to run.  fgnn_u_add_v_backward_planned
 * below is the atomic-free form. */
int    fgnn_u_add_v(int N, int64_t E, int W, const int32_t *row_ptr, const int32_t *col_ind,
                    const float *row_val, const float *col_val, float *out, void *stream);
int    fgnn_u_add_v_backward(int N, int64_t E, int W, const int32_t *row_ptr, const int32_t *col_ind,
                             const float *grad_out, float *grad_row, float *grad_col, void *stream);

/* Column sums of a per-edge array without global atomics, bit-reproducible: out[j,:] = sum of g[p,:] over the CSR
 * positions p with col_ind[p] == j (the grad_col of u_add_v's backward, u_add_v.cu:43-90, and the gather_col step of
 * the fuse-scatter GAT backward, src/fused_gat/fused_gat.cu:558-586, which reads g through `permute`: 32 bytes out
 * of every 128-byte line it pulls).  A plan belongs to one (row_ptr, col_ind) pair, which must outlive it and keep
 * its contents, and needs the columns of every row in ascending order to pay off (any order is summed correctly).
 * It cuts the columns into ranges whose accumulators (columns x W floats, W rounded up to a multiple of 4) fit
 * lds_bytes of LDS (<= 0: 8 KiB, which lets twenty waves share a compute unit; at most 64 KiB) and keeps 6 bytes of device memory per entry: every range's
 * entries in CSR order, so that a range's pass reads g in contiguous runs.  task_len (<= 0: chosen from E) is the
 * number of entries one wave sums; ranges longer than that are summed in pieces and merged in a fixed order through
 * the workspace.  A plan built for W serves every narrower array too.  Building it sorts the entries once (a radix
 * sort pass or two) and synchronises `stream`.  W <= 64, or <= 256 in multiples of 4 on 16-byte aligned arrays. */
typedef struct fgnn_colsum_plan fgnn_colsum_plan_t;
int    fgnn_colsum_plan_create(const int32_t *row_ptr, const int32_t *col_ind, int n_rows, int n_cols, int64_t E, int W,
                               int lds_bytes, int task_len, void *stream, fgnn_colsum_plan_t **out);
void   fgnn_colsum_plan_destroy(fgnn_colsum_plan_t *p);
size_t fgnn_colsum_plan_device_bytes(const fgnn_colsum_plan_t *p);
int    fgnn_colsum_plan_columns_per_range(const fgnn_colsum_plan_t *p);
int    fgnn_colsum_plan_num_tasks(const fgnn_colsum_plan_t *p);
int    fgnn_colsum_plan_matches(const fgnn_colsum_plan_t *p, const int32_t *row_ptr, const int32_t *col_ind, int n_rows,
                                int n_cols, int64_t E);
size_t fgnn_colsum_workspace_bytes(const fgnn_colsum_plan_t *p, int W);
int    fgnn_edge_colsum(const fgnn_colsum_plan_t *p, int W, const float *g, float *out, void *workspace,
                        size_t workspace_bytes, void *stream);
/* Row sums of a per-edge array in a fixed order: out[i,:] = sum of g[p,:] over the CSR positions of row i (the grad_row
 * of u_add_v's backward, u_add_v.cu:43-66).  Any width. */
int    fgnn_edge_rowsum(int N, int64_t E, int W, const int32_t *row_ptr, const float *g, float *out, void *stream);
/* fgnn_u_add_v_backward with both sums in a fixed order: fgnn_edge_rowsum + fgnn_edge_colsum under a plan of
 * (row_ptr, col_ind) with n_cols == N; workspace of fgnn_colsum_workspace_bytes(plan, W). */
int    fgnn_u_add_v_backward_planned(int N, int64_t E, int W, const int32_t *row_ptr, const int32_t *col_ind,
                                     const float *grad_out, float *grad_row, float *grad_col,
                                     const fgnn_colsum_plan_t *plan, void *workspace, size_t workspace_bytes, void *stream);

/* The per-edge pseudo-coordinate projection of the MoNet drivers, nn.Sequential(nn.Linear(2, D),
 * nn.Tanh()) on the [E, 2] edge coordinates (script/train/train_gmmconv_our.py:46-57), in one pass
 * over the edges each way: y[e,o] = tanh(x[e,0]*W[o,0] + x[e,1]*W[o,1] + b[o]), 1 <= D <= 4,
 * W [D,2] and b [D] as in nn.Linear.  The backward returns the parameter gradients (the coordinates are
 * data): grad_W[o,c] = sum_e gt[e,o]*x[e,c], grad_b[o] = sum_e gt[e,o], gt = grad_y*(1 - y^2), summed in
 * a fixed order.  x must be 8-byte aligned. */
int    fgnn_edge_linear_tanh(int64_t E, int D, const float *x, const float *W, const float *b, float *y,
                             void *stream);
size_t fgnn_edge_linear_tanh_backward_workspace_bytes(int64_t E, int D);
int    fgnn_edge_linear_tanh_backward(int64_t E, int D, const float *x, const float *y,
                                      const float *grad_y, float *grad_W, float *grad_b,
                                      void *workspace, size_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------- loss of the training drivers
 * torch.nn.CrossEntropyLoss over the labelled rows (script/train/train_gatconv_our.py:166-175) as two passes over the
 * logits instead of a dozen elementwise and reduction kernels: the forward writes, per row, lse = log sum_c exp(x[c]) and
 * row_loss = lse - x[label] (the loss is their mean); the backward writes grad[row, c] = (exp(x[c] - lse) - [c == label])
 * * upstream[row].  logits rows are ld floats apart (ld >= C: a [N, C] view of a padded array is read in place), gradient
 * rows ld_grad floats apart, their columns C .. ld_grad - 1 get zeros (the gradient of a padded array needs no second
 * copy).  labels are int64 (torch's default); a label outside [0, C) indexes nothing and gives a NaN row loss.  Nothing
 * synchronises: the calls can be captured into a HIP graph.  C <= 256 (1024 when ld and ld_grad are multiples of four and
 * the arrays 16-byte aligned). */
int    fgnn_cross_entropy_forward(int64_t N, int C, int64_t ld, const float *logits, const int64_t *labels, float *lse,
                                  float *row_loss, void *stream);
int    fgnn_cross_entropy_backward(int64_t N, int C, int64_t ld, int64_t ld_grad, const float *logits,
                                   const int64_t *labels, const float *lse, const float *upstream,
                                   float *grad_logits, void *stream);

/* ---------------------------------------------------------------- csr2csc
 * Replaces csrtocsc.csr2csc (src/csr2csc/csr2csc.cc; csr2csc.cu:7-43, a cuSPARSE
 * cusparseCsr2cscEx2 call).  Stable: entries of a column keep ascending CSR position.
 * Outputs col_ptr [n_cols+1], row_ind [E], permute [E] (int32 positions; the reference carries
 * them as float values). */
size_t fgnn_csr2csc_workspace_bytes(int n_rows, int n_cols, int64_t E);
int    fgnn_csr2csc(int n_rows, int n_cols, int64_t E, const int32_t *row_ptr, const int32_t *col_ind,
                    int32_t *col_ptr, int32_t *row_ind, int32_t *permute,
                    void *workspace, size_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------- coo2csr
 * Edge list (dst[e], src[e]) -> CSR by destination with ascending sources inside a row; with
 * dedupe != 0 duplicate (dst, src) pairs are merged.  Replaces the host-side scipy csr_matrix call of
 * the reference's drivers (script/train/train_gatconv_our.py:87-91).  Outputs: row_ptr [n_rows+1],
 * col_ind (first *n_out entries valid; capacity E), n_out (device int64: number of CSR entries),
 * edge_pos [E] optional: CSR position of every input edge (to carry per-edge data along). */
size_t fgnn_coo2csr_workspace_bytes(int n_rows, int n_cols, int64_t E);
int    fgnn_coo2csr(int n_rows, int n_cols, int64_t E, const int32_t *dst, const int32_t *src, int dedupe,
                    int32_t *row_ptr, int32_t *col_ind, int64_t *n_out, int32_t *edge_pos,
                    void *workspace, size_t workspace_bytes, void *stream);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* FGNN_H */
