/*
 * hiscache_hip.h -- C ABI of libhiscache_hip.so, the MI355X (gfx950) kernel
 * library for HisCache's history-aware aggregation and cache admission.
 *
 * It replaces the reference's pybind11 operator module `hiscache_backend`
 * (/root/reference: src/cpp/python_bindings/binding.cpp:9-24).  The reference
 * passes torch::Tensor handles; this ABI passes raw DEVICE pointers, sizes,
 * dtype enums and a hipStream_t (as void*).  Conventions:
 *
 *   - every function returns an hc_status (0 = ok); nothing aborts the process
 *     (the reference exits on ASSERT, src/cpp/include/common.h:13-34);
 *   - the library never allocates or frees device memory: outputs and
 *     workspaces are caller-owned; hc_*_workspace_bytes() sizes them;
 *   - all launches are asynchronous on the given stream; nothing synchronises;
 *   - indices are int64 (reference: common.h:12) unless a name says otherwise;
 *   - feature/history data may be fp32, fp16 or bf16 (hc_dtype); accumulation
 *     and all outputs of the aggregation are fp32;
 *   - row-major, densely packed 2-D arrays; a NULL optional pointer means
 *     "absent" as documented per argument.
 */
#ifndef HISCACHE_HIP_H
#define HISCACHE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  HC_OK = 0,
  HC_EINVAL = 1,       /* null pointer, negative size, inconsistent shapes */
  HC_EDTYPE = 2,       /* unknown dtype enum */
  HC_ELAUNCH = 3,      /* the HIP runtime reported a launch error */
  HC_EWORKSPACE = 4,   /* workspace missing or too small */
  HC_EUNSUPPORTED = 5, /* valid request outside what the kernels cover */
  HC_ENODEVICE = 6     /* no usable GPU */
} hc_status;

typedef enum { HC_F32 = 0, HC_F16 = 1, HC_BF16 = 2 } hc_dtype;

/* Which rows a history map substitutes. */
typedef enum {
  HC_SUBST_ROW = 0, /* reference rule: hmap[R] flags DESTINATION rows, hbuf[R,hsize] is row-aligned */
  HC_SUBST_SRC = 1  /* extension: hmap[n_src] maps SOURCE ids to rows of a history table hbuf[Hn,hsize] */
} hc_subst_mode;

typedef enum { HC_NORM_L2 = 0, HC_NORM_L1 = 1 } hc_norm_kind;
typedef enum {
  HC_CMP_LT = 0,    /* admit when score <  thres            (hiscache/history_cache.py:215) */
  HC_CMP_NOT_GT = 1 /* admit unless thres != 0 && score > thres (src/cpp/src/grad_check.cu:18) */
} hc_cmp_kind;

const char *hc_version(void);
const char *hc_strerror(int status);
/* Number of visible GPUs; 0 when there is none (never fails). */
int hc_device_count(void);

/* ---------------------------------------------------------------- aggregation forward
 * Replaces aggr_forward_history (src/cpp/include/history_aggr.h:34-37, kernels
 * src/cpp/src/history_aggr.cu:7-40) and aggr_forward_history_edge_value
 * (history_aggr.h:39-42, kernels history_aggr.cu:42-125).
 *
 *   edge_value == NULL : mean aggregation.  Row r with hmap[r] != -1 copies
 *       hbuf[r, :F]; otherwise vout[r,:] = (sum_j vin[idx[j],:]) / deg(r); a
 *       zero-degree row is written as 0.
 *   edge_value != NULL : vout[r,h,:] = sum_j edge_value[j,h] * vin[idx[j],h,:]
 *       (fused multiply-add, no division); history rows copy hbuf[r,:F]
 *       (hsize == F) or hbuf[r, h*F:(h+1)*F] (hsize == F*n_head).
 *   mode == HC_SUBST_SRC (mean only): every neighbour row is read from
 *       hbuf[hmap[idx[j]], :F] when hmap[idx[j]] != -1, else from vin; hmap has
 *       n_src entries; the table has vin's element type, or vin is fp32 and
 *       the table fp16 / bf16 (other pairs return HC_EUNSUPPORTED).
 *
 * ptr[R+1], idx[>= ptr[R]], vin[n_src, n_head, F] (in_dtype), hmap NULL = no
 * history, hbuf (hist_dtype), vout[R, n_head, F] fp32.  n_head >= 1; n_head > 1
 * requires edge_value.
 * Summation order (fp32, fixed, so results are bit-reproducible): a row is
 * summed in CSR order; when hc_aggr_fwd_long_row_edges() reports a threshold
 * T > 0 for the shape (mean and single-head weighted aggregation on widths
 * that are a multiple of 64), a row with more than T edges is summed as four
 * contiguous quarters of ceil(deg/4) edges, each in CSR order, combined left to
 * right ((q0+q1)+q2)+q3, then divided (mean only).
 * workspace (optional, NULL allowed; 256-byte aligned, of
 * hc_aggr_fwd_workspace_bytes(mode, R, E, n_src) bytes, E = an upper bound of
 * ptr[R]): on large blocks the long rows are listed first and scheduled at the
 * start of the launch, which shortens its tail; with HC_SUBST_SRC over a
 * million sources or more, one bit per source ("has an entry") is derived from
 * hmap first, so that sources without an entry never touch the map.  Results
 * do not depend on the workspace. */
size_t hc_aggr_fwd_workspace_bytes(int mode, int64_t R, int64_t E, int64_t n_src);
int hc_aggr_fwd(int mode, const int64_t *ptr, const int64_t *idx, const void *vin, int in_dtype,
                const int64_t *hmap, const void *hbuf, int hist_dtype, int64_t hsize,
                const float *edge_value, int64_t n_head, float *vout, int64_t R, int64_t F,
                int64_t n_src, void *workspace, size_t workspace_bytes, void *stream);

/* The long-row threshold T that hc_aggr_fwd applies to a mean aggregation with
 * rows of F elements of in_dtype; 0 when every row is summed strictly in CSR
 * order.  No reference counterpart (the reference sums every row with one
 * warp per 32 columns, history_aggr.cu:27-37). */
int64_t hc_aggr_fwd_long_row_edges(int64_t F, int in_dtype);

/* ---------------------------------------------------------------- transpose (CSC view)
 * No reference counterpart: the reference backward scatters with float
 * atomicAdd (history_aggr.cu:164); this library gathers over a transposed view
 * instead, which makes the sums deterministic.
 *
 * Stable sort of the first E edge slots by source id.  Edge slots >= ptr[R],
 * when hmap_row != NULL the edges of rows with hmap_row[r] != -1, and when
 * hmap_src != NULL (n_src entries) the edges whose source s has
 * hmap_src[s] != -1 are dropped: a row that took its history row, and a source
 * that was substituted by a history-table row, pass no gradient to vin.
 * Outputs: ptrT[n_src+1] (int64), rowT[E] (destination row per
 * transposed edge, ascending inside a source), edgeT[E] (original edge slot);
 * only the first ptrT[n_src] entries of rowT/edgeT are meaningful.
 * Requires R, E, n_src < 2^31 - 1.
 * Blocks of more than 2^20 edge slots (up to 2^28, with up to about 44 M
 * sources) are sorted by this library's own two-level bucket sort; smaller
 * ones by a counting sort or a library sort.  All of these record kernels only
 * under stream capture.  Beyond those sizes the sort library underneath clears
 * its counters with hipMemsetAsync, which a captured graph would replay as
 * memset nodes: on a capturing stream such a call returns HC_EUNSUPPORTED and
 * records nothing. */
size_t hc_transpose_workspace_bytes(int64_t R, int64_t E, int64_t n_src);
int hc_build_transpose(const int64_t *ptr, const int64_t *idx, const int64_t *hmap_row,
                       const int64_t *hmap_src, int64_t R, int64_t E, int64_t n_src, int64_t *ptrT,
                       int32_t *rowT, int32_t *edgeT, void *workspace, size_t workspace_bytes,
                       void *stream);

/* hc_build_transpose_dev: the same view (no history maps: nothing is left out)
 * for a block whose sizes the host does not know yet -- a mini-batch that
 * hc_sample_layers has just drawn, whose layer sizes are still in its `counts`
 * array on the device.  *R_dev, *E_dev, *n_src_dev are read by the kernels;
 * max_E / max_src (the capacities of idx and of the node list, at most 2^24
 * each) size the launches, the workspace and the outputs: ptrT[max_src+1],
 * rowT[max_E], edgeT[max_E] (nullable).  Only ptrT[0..n_src] and the first
 * ptrT[n_src] entries of rowT/edgeT are written.  Sizes beyond the capacities
 * (*E_dev > max_E, *n_src_dev > max_src, or a negative size) are clamped, so
 * that no access leaves idx or the outputs, and the view is then that of the
 * truncated block (ptr must hold *R_dev + 1 offsets: the rows have no capacity
 * argument): *overflow (one
 * int32 in device memory, nullable) is set to 1 in that case and to 0
 * otherwise, for the caller to check when it reads the sizes back.  Four launches, kernels only
 * (safe under stream capture), nothing is read back: this is how the sampler
 * emits the batch's transposed view together with the batch, so that backward
 * (hc_aggr_bwd_batch_view) builds none.  The loader of the reference hands over
 * one shared CSR per batch (hiscache/history_model.py:124-128); the CSC is this
 * library's addition to that wire format. */
size_t hc_transpose_dev_workspace_bytes(int64_t max_E, int64_t max_src);
int hc_build_transpose_dev(const int64_t *ptr, const int64_t *idx, const int64_t *R_dev,
                           const int64_t *E_dev, const int64_t *n_src_dev, int64_t max_E,
                           int64_t max_src, int64_t *ptrT, int32_t *rowT, int32_t *edgeT,
                           int32_t *overflow, void *workspace, size_t workspace_bytes, void *stream);
/* hc_build_transpose_dev_deg: the same call with one more output, *max_in_degree
 * (one int64 in device memory, nullable): the largest number of edges that one
 * source has in the view, found by the block that scans the counters.  A caller
 * that reads it back with the sizes knows whether the batch holds a source above
 * hc_aggr_bwd_chunk_edges and may then call hc_aggr_bwd_batch_view without
 * workspace, which runs it without its hub blocks and its second launch. */
int hc_build_transpose_dev_deg(const int64_t *ptr, const int64_t *idx, const int64_t *R_dev,
                               const int64_t *E_dev, const int64_t *n_src_dev, int64_t max_E,
                               int64_t max_src, int64_t *ptrT, int32_t *rowT, int32_t *edgeT,
                               int32_t *overflow, int64_t *max_in_degree, void *workspace,
                               size_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------- aggregation backward
 * Replaces AggrHistoryFunction::backward / AggrHistoryEdgeValueFunction::backward
 * (history_aggr.cu:493-596; kernels :127-397).
 *
 *   grad_vin[n_src, n_head, F] : for every source s, the sum over its incoming
 *       edges (ascending destination row) of g[r,h,:]/deg(r) (mean) or
 *       g[r,h,:]*edge_value[j,h] (weighted); rows without edges are written 0.
 *   grad_hbuf[R, hsize] (nullable; HC_SUBST_ROW with hmap only): g[r,:] for
 *       history rows, 0 elsewhere.  With n_head > 1 and hsize == F the heads
 *       are summed in head order; with hsize == F*n_head they are concatenated.
 *   edge_grad[E_total, n_head] (nullable; needs edge_value and vin):
 *       edge_grad[j,h] = <g[r,h,:], vin[idx[j],h,:]> for edges of non-history
 *       rows, 0 for the others.  E_total = number of edge slots to fill.
 *
 * ptrT/rowT/edgeT come from hc_build_transpose called with the same hmap_row
 * (so edges of history rows are already gone); ptrT[n_src] <= E_total.  After
 * a forward pass in HC_SUBST_SRC mode pass hmap = NULL here and build the view
 * with hmap_src: substituted sources then have no incoming edges and their
 * rows of grad_vin are written 0 (vin[s] was never read for them).  A view
 * built without hmap_src gives every source the gradient of the row that was
 * read for it, whichever table it came from; the caller routes the rows of
 * substituted sources to the history table's gradient if it wants one.
 * Summation order (fp32, fixed): ascending destination row.  When a workspace
 * of hc_aggr_bwd_workspace_bytes() is given and hc_aggr_bwd_chunk_edges(F)
 * reports C > 0, a source with more than C incoming edges is summed in chunks
 * of C consecutive edges (each chunk in order, by its own wave) and the chunk
 * sums are combined left to right; without a workspace (NULL), and always for
 * weighted sums, every source is summed strictly in order by one wave.  The workspace must be 256-byte
 * aligned. */
size_t hc_aggr_bwd_workspace_bytes(int64_t E_total, int64_t F);
int64_t hc_aggr_bwd_chunk_edges(int64_t F);
int hc_aggr_bwd(const int64_t *ptr, const int64_t *idx, const int64_t *ptrT, const int32_t *rowT,
                const int32_t *edgeT, const float *g, const int64_t *hmap, const float *edge_value,
                const void *vin, int in_dtype, int64_t n_head, float *grad_vin, float *grad_hbuf,
                int64_t hsize, float *edge_grad, int64_t E_total, int64_t R, int64_t F,
                int64_t n_src, void *workspace, size_t workspace_bytes, void *stream);

/* hc_aggr_bwd_batch_view: the mean aggregation's backward over ONE transposed
 * view of the whole mini-batch CSR, shared by every layer of the batch and
 * built before the cache has been consulted (hc_build_transpose over all rows
 * of the batch with hmap_row = hmap_src = NULL, or hc_build_transpose_dev
 * behind the sampler), so that no view is built inside backward.  The
 * reference's layers share one CSR per batch the same way
 * (hiscache/history_model.py:124-128) and scatter with atomics
 * (history_aggr.cu:127-168).
 *
 * A layer owns the first R rows of the batch CSR and the first n_src sources;
 * ptrT[0..n_src] is a prefix of the batch view's offsets.  Transposed edges
 * whose destination row is >= R, or has hmap[row] != -1 (hmap nullable), are
 * stepped over here instead of being left out of the view.  grad_vin[n_src, F]
 * and grad_hbuf (nullable) as in hc_aggr_bwd.  E_view bounds ptrT[n_src] (the
 * entries of rowT that may be read; it sizes the workspace:
 * hc_aggr_bwd_workspace_bytes(E_view, F)).
 * Summation order: ascending destination row over the live edges.  With a
 * workspace and C = hc_aggr_bwd_chunk_edges(F) > 0, a source with more than C
 * edges IN THE BATCH VIEW is summed in chunks of C consecutive view positions
 * (live edges only, each chunk from zero), combined left to right.  For a
 * source with at most C edges in the batch view the result has the same bits
 * as hc_aggr_bwd over a view built for the layer.
 * Plain mean, one head, fp32 gradient; any F. */
int hc_aggr_bwd_batch_view(const int64_t *ptr, const int64_t *ptrT, const int32_t *rowT,
                           const float *g, const int64_t *hmap, float *grad_vin, float *grad_hbuf,
                           int64_t hsize, int64_t E_view, int64_t R, int64_t F, int64_t n_src,
                           void *workspace, size_t workspace_bytes, void *stream);

/* hc_aggr_bwd_batch_view_typed: the input gradient of the relational layer
 * (hiscache/history_model.py:220-278; forward: hc_typed_csr, then hc_aggr_fwd
 * with its 1/deg edge weights over the (row, relation) groups) over the batch's
 * shared view, which must carry edgeT.  g is [R*num_rel, F]: the gradient of
 * the groups' sums.  For every source s
 *   grad_vin[s,:] = sum over its kept edges e (row r, relation k = edge_types[e])
 *                   of g[r*num_rel + k, :] * (1 / deg(r))
 * in ascending (row, edge slot) order, product rounded, then added.  Kept as in
 * hc_typed_csr: r < R, e < E, k in [0, num_rel), used_mask (n_src bytes,
 * nullable) != 0 for s; deg(r) = ptr[r+1] - ptr[r].  Sources without kept edges
 * get 0.  F must be one of the fast widths (64, 128, 192, 256, 384, 512, 768,
 * 1024), else HC_EUNSUPPORTED.  (The order differs from hc_aggr_bwd over a view
 * of the regrouped block only where parallel edges of one (source, row) pair
 * carry different relations.) */
int hc_aggr_bwd_batch_view_typed(const int64_t *ptr, const int64_t *ptrT, const int32_t *rowT,
                                 const int32_t *edgeT, const int64_t *edge_types, int64_t E,
                                 int num_rel, const uint8_t *used_mask, const float *g,
                                 float *grad_vin, int64_t R, int64_t F, int64_t n_src, void *stream);

/* ---------------------------------------------------------------- used masks
 * Replaces count_history_reconstruct (src/cpp/include/grad_check.h:18-20,
 * src/cpp/src/grad_check.cu:70-130).  masks is (num_layer+1) x n_all bytes
 * (0/1), written in full: masks[num_layer] is the seed level, masks[0] the
 * raw-feature level.  hmap (nullable) covers rows [0, hmap_len); rows beyond
 * it count as "no history". */
int hc_count_history(const int64_t *ptr, const int64_t *idx, const int64_t *hmap, int64_t hmap_len,
                     uint8_t *masks, int64_t ptr_rows, int64_t n_all, int64_t n_seed, int num_layer,
                     void *stream);

/* ---------------------------------------------------------------- admission
 * hc_row_scores: score[r] = ||grad[r,:]||_2 (hiscache/history_cache.py:205) or
 * sum|grad[r,:]| (hiscache/history_table.py:161).  Summation order: element e
 * of a row belongs to lane (e/4)%64; a lane folds its elements in increasing e
 * (L2: acc = fma(x,x,acc)); the 64 partials are combined by a butterfly with
 * partner distance 32,16,8,4,2,1; L2 takes sqrtf (correctly rounded). */
int hc_row_scores(const float *grad, float *score, int64_t M, int64_t F, int norm_kind, void *stream);

/* hc_quantile_threshold: the admission threshold `torch.quantile(score, rate)`
 * (hiscache/history_cache.py:211, hiscache/history_table.py:173) without a
 * sort: out[0] = a + w*(b - a) for w < 0.5, else b - (b - a)*one_minus_w, where
 * a and b are the order statistics of rank lo and hi (0-based, hi = lo or
 * lo + 1) of score[0, n) and every step is rounded to fp32 on its own -- the
 * caller works out lo, hi and w from rate and n the way torch.quantile does
 * (pos = fp32(rate) * fp32(n - 1), lo = floor(pos), w = pos - lo).  One launch
 * (a radix select by one block); n <= hc_quantile_max_scores(), else
 * HC_EUNSUPPORTED (hc_quantile_threshold_ws takes any size).  NaN scores rank behind +inf, as in a sort;
 * -0 ranks in front of +0. */
int64_t hc_quantile_max_scores(void);
int hc_quantile_threshold(const float *score, int64_t n, int64_t lo, int64_t hi, float w,
                          float one_minus_w, float *out, void *stream);
/* The same threshold for any n < 2^31.  Up to 32 768 scores it is
 * hc_quantile_threshold and needs no workspace; above, the select runs over the
 * whole chip in seven small launches (a clear, one launch per 8-bit digit of the
 * key, one for the upper order statistic, one for the interpolation) and needs
 * hc_quantile_workspace_bytes(n) bytes, 4-byte aligned.  Same bits either way. */
size_t hc_quantile_workspace_bytes(int64_t n);
int hc_quantile_threshold_ws(const float *score, int64_t n, int64_t lo, int64_t hi, float w,
                             float one_minus_w, float *out, void *workspace, size_t workspace_bytes,
                             void *stream);

/* hc_grad_check: the fused admission pass.  Replaces record_history
 * (grad_check.h:12-16, grad_check.cu:6-68) and the torch sequence of
 * HistoryCache.update_history (hiscache/history_cache.py:205-221,243-254).
 *
 *   score[r] = row score of grad (grad != NULL) or score_in[r] (grad == NULL)
 *   pass[r]  = cmp(score[r], *thres)                 (thres: 1 fp32 on device)
 *   admit[r] = (used == NULL || used[r]) && pass[r] &&
 *              (slot[r] == -1 || (age != NULL && age[r] >= age_limit))
 *   mask_out[r] = admit[r]; score_out[r] = score[r] (nullable)
 *
 * Admitted rows take ring slots in ROW ORDER: the k-th admitted row gets
 * (header + k) mod capacity; header advances by the admitted count (the
 * reference hands slots out in atomic arrival order, grad_check.cu:25).  Per
 * admitted row: the slot's previous owner is un-mapped if it still points at
 * the slot (grad_check.cu:26-30), emb[r,:F] is stored into table[slot,:F]
 * (converted to table_dtype, round to nearest even), full2slot[sub_to_full[r]]
 * = slot, slot2full[slot] = sub_to_full[r], checkin[slot] = glb_iter
 * (:40-45; checkin nullable).  slot_out[r] (nullable) = slot or -1.
 * If more rows are admitted than the ring holds, the result equals inserting
 * them one by one in row order.  sub_to_full[0:M) must not repeat an id.
 * header is 1 int64 on the device, updated in place. */
size_t hc_grad_check_workspace_bytes(int64_t M);
int hc_grad_check(const float *grad, const float *score_in, const float *emb, const int64_t *slot,
                  const int32_t *age, const uint8_t *used, const int64_t *sub_to_full,
                  const float *thres, int32_t age_limit, int norm_kind, int cmp_kind,
                  uint8_t *mask_out, float *score_out, int64_t *slot_out, void *table,
                  int table_dtype, int64_t capacity, int64_t *full2slot, int64_t *slot2full,
                  int64_t *checkin, int64_t *header, int64_t glb_iter, int64_t M, int64_t F,
                  void *workspace, size_t workspace_bytes, void *stream);

/* hc_grad_check_static: hc_grad_check without a workspace argument, for callers
 * that cannot allocate device memory (code under stream capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same arguments, results and kernels as hc_grad_check; the scratch
 * the passes share lives in a fixed device array inside the library (about
 * 0.33 MB per GPU, held until the process ends), whose address is looked up on
 * the first call on each device.  The call allocates and frees nothing.
 * M > HC_GRAD_CHECK_STATIC_MAX_ROWS returns HC_EUNSUPPORTED.  All calls on one
 * GPU share that array: calls that overlap on one GPU (two streams, two
 * threads) race; calls on one stream are ordered and safe. */
#define HC_GRAD_CHECK_STATIC_MAX_ROWS 16777216
int hc_grad_check_static(const float *grad, const float *score_in, const float *emb,
                         const int64_t *slot, const int32_t *age, const uint8_t *used,
                         const int64_t *sub_to_full, const float *thres, int32_t age_limit,
                         int norm_kind, int cmp_kind, uint8_t *mask_out, float *score_out,
                         int64_t *slot_out, void *table, int table_dtype, int64_t capacity,
                         int64_t *full2slot, int64_t *slot2full, int64_t *checkin, int64_t *header,
                         int64_t glb_iter, int64_t M, int64_t F, void *stream);

/* hc_record_history: the reference's argument set, in its order
 * (grad_check.h:12-16): precomputed score, device threshold, used mask,
 * "not greater" comparison, fp32 table buffer_all[history_num, history_size].
 * Same row-order slot rule as hc_grad_check. */
int hc_record_history(const float *buffer_new, float *buffer_all, const uint8_t *used_mask,
                      const int64_t *sub_to_full, const int64_t *sub_to_history,
                      int64_t *history_to_full, int64_t *full_to_history, int64_t *header,
                      const float *score, const float *thres, int64_t *checkin_iter,
                      int64_t glb_iter, int64_t M, int64_t history_num, int64_t history_size,
                      void *workspace, size_t workspace_bytes, void *stream);

/* hc_cache_append: the append-only admission of HistoryCache.update_history
 * (hiscache/history_cache.py:215-254) as one sequence of launches.
 *   mask[r] = (score[r] < *thres) && (sub2embed[r] == -1)                    (:215)
 *   the k-th admitted row is written to embedding slot header + k            (:216-221)
 *   feature slots overlapped by [header, header+A) are invalidated:
 *     full2embed[feat2full[b:e]] = -1, b = header*H/F_in,
 *     e = ceil((header+A)*H/F_in), clipped to n_feat                         (:223-226)
 *   previous owners of the overwritten slots are un-mapped when they point
 *     into [header, header+A)                                                (:230-240)
 *   full2embed[sub_to_full[r]] = slot, embed2full[slot] = sub_to_full[r]     (:243-253)
 *   header += A                                                              (:254)
 * buffer is the flat fp32 cache viewed as [capacity, H]; rows that would land
 * at or beyond `capacity` are dropped and *overflow (1 int64, nullable) is set
 * to their count (the reference raises a shape error there).  header is 1
 * int64 on the device. */
int hc_cache_append(const float *score, const float *thres, const float *emb,
                    const int64_t *sub2embed, const int64_t *sub_to_full, uint8_t *mask_out,
                    float *buffer, int64_t capacity, int64_t H, int64_t F_in, int64_t *full2embed,
                    int64_t *embed2full, const int64_t *feat2full, int64_t n_feat, int64_t *header,
                    int64_t *overflow, int64_t M, void *workspace, size_t workspace_bytes,
                    void *stream);

/* hc_evict replaces the torch sequences of HistoryTable.evict_by_staleness and
 * evict_by_both (hiscache/history_table.py:189-251) for one table.  Gradient
 * rule (M > 0): batch row r with sub2slot[r] != -1 and score[r] >= *thres
 * gives up its slot (:234-244).  Staleness rule: every slot with
 * -1 < checkin <= stale_iter is given up (:193-200, :246-251); pass
 * stale_iter < 0 to skip it.  Giving up slot s: full2slot[slot2full[s]] = -1,
 * slot2full[s] = -1, checkin[s] = -1.  The final state is the one the
 * reference reaches by applying the gradient rule first and the staleness rule
 * second. */
int hc_evict(const int64_t *sub2slot, const float *score, const float *thres, int64_t M,
             int64_t stale_iter, int64_t *checkin, int64_t *slot2full, int64_t *full2slot,
             int64_t capacity, int64_t n_full, void *stream);

/* ---------------------------------------------------------------- sampler
 * Layered neighbour sampling on the device.  The reference takes its batches
 * from the external cxgnndl loader (hiscache/history_trainer.py:19,26); these
 * entry points produce the same wire format the model and the cache read
 * (hiscache/history_model.py:120-153, hiscache/history_cache.py:307-324):
 * sub-graph nodes numbered seeds first, then each hop's new nodes in
 * first-seen order; counts[k] = nodes within k hops; one shared CSR
 * (ptr, idx) with the sampled neighbours of the first counts[L-1] nodes.
 *
 * Rule for row u (full id f, degree d) at hop k: if d <= fanout[k] all
 * neighbours in list order, else neighbour j (j < fanout[k]) is list position
 * perm(j), a bijection of [0, d) keyed by (rng_seed, k, f): four Feistel
 * rounds over the next even power of two, round function splitmix64, with
 * cycle walking.  The picks of a row are therefore distinct list positions.
 *
 * node_map is int32[num_nodes], persistent between calls, all "unseen" on
 * entry and on return (hc_sample_map_init fills it once).  seeds must be
 * distinct valid ids.  fanout is a HOST array of num_hops entries
 * (<= HC_SAMPLE_MAX_HOPS).  Outputs are sized by hc_sample_capacity: ptr
 * [max_rows + 1], idx [max_edges], sub_to_full [max_nodes]; counts is
 * int64[2*num_hops + 1] on the device: counts[0..L] node counts, then the
 * cumulative edge count after every hop.  Nothing is read back: the caller
 * copies counts to the host when it needs the sizes.  Calls that share a
 * node_map must not overlap. */
#define HC_SAMPLE_MAX_HOPS 8
int hc_sample_capacity(int64_t n_seed, const int64_t *fanout, int num_hops, int64_t num_nodes,
                       int64_t *max_rows, int64_t *max_edges, int64_t *max_nodes);
size_t hc_sample_workspace_bytes(int64_t n_seed, const int64_t *fanout, int num_hops,
                                 int64_t num_nodes);
int hc_sample_map_init(int32_t *node_map, int64_t num_nodes, void *stream);
int hc_sample_layers(const int64_t *indptr, const int64_t *indices, int64_t num_nodes,
                     const int64_t *seeds, int64_t n_seed, const int64_t *fanout, int num_hops,
                     uint64_t rng_seed, int32_t *node_map, int64_t *ptr, int64_t *idx,
                     int64_t *sub_to_full, int64_t *counts, void *workspace, size_t workspace_bytes,
                     void *stream);
/* hc_sample_layers_seed_at: the same call with the seed read from *rng_seed_at
 * (memory the device can read: device memory or pinned host memory) when its
 * first kernel runs, not when the call is made -- so that a call recorded in a
 * HIP graph (every launch of it has the same shape for the same n_seed and
 * fanout, the sizes stay on the device) can be replayed for the next batch
 * after the host has stored a new seed there and new ids in `seeds`. */
int hc_sample_layers_seed_at(const int64_t *indptr, const int64_t *indices, int64_t num_nodes,
                             const int64_t *seeds, int64_t n_seed, const int64_t *fanout, int num_hops,
                             const uint64_t *rng_seed_at, int32_t *node_map, int64_t *ptr, int64_t *idx,
                             int64_t *sub_to_full, int64_t *counts, void *workspace,
                             size_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------- helpers
 * hc_count_num replaces count_num (grad_check.h:26, grad_check.cu:165-182):
 * histogram of arr into out[mmax+1] (int32, zeroed here) that skips value 0.
 * Values outside [0, mmax] are ignored. */
int hc_count_num(const int64_t *arr, int64_t n, int64_t mmax, int32_t *out, void *stream);

/* hc_typed_csr regroups the edges of the first R rows by (row, relation) for
 * the relational convolution (hiscache/history_model.py:248-270, where the
 * reference marks unused edges with an extra relation and lets cxgnncomp's
 * RGCNOP_sorted sort the edges by relation on every call).  Group
 * v = r*num_rel + k of (ptr2, idx2) holds, in their original order, the source
 * ids of row r's edges e with edge_types[e] == k whose source is in
 * [0, n_src) and, when used_mask (n_src bytes, nullable) is given, has
 * used_mask[src] != 0.  Only edge slots below E are read (E = entries
 * available in idx and in edge_types).  Outputs: ptr2[R*num_rel + 1],
 * idx2[E] (only the first ptr2[R*num_rel] entries are written),
 * cnt[R*num_rel] = group sizes, deg[R] = full row degrees ptr[r+1]-ptr[r],
 * edge_weight[E] (fp32, nullable; written where idx2 is) = 1/deg of the edge's
 * row: with these weights the weighted aggregation over the groups gives each
 * group's share of the row's mean over all its edges directly
 * (sum over the group / deg), without a pass that rescales group means.
 * num_rel <= 64 (HC_EUNSUPPORTED above).  Results are exact and independent of
 * scheduling.  ticket (nullable): one 32-bit word of device memory that is zero
 * on entry and zero again when the call's kernels have run; with it, blocks of
 * up to 2^20 (row, relation) groups take two launches, need no workspace and
 * make no library call (calls that share a ticket must not overlap). */
size_t hc_typed_csr_workspace_bytes(int64_t R, int num_rel);
int hc_typed_csr(const int64_t *ptr, const int64_t *idx, const int64_t *edge_types,
                 const uint8_t *used_mask, int64_t R, int64_t E, int64_t n_src, int num_rel,
                 int64_t *ptr2, int64_t *idx2, int64_t *cnt, int64_t *deg, float *edge_weight,
                 void *workspace, size_t workspace_bytes, unsigned *ticket, void *stream);

/* hc_edge_types_by_ranges: relation of every edge of the first R rows from the
 * node types of its ends, out[e] = pair_to_rel[type(row) * T + type(idx[e])]
 * with T = n_bounds + 1 and type(v) = number of bounds[b] <= sub_to_full[v]
 * (node types stored as consecutive full-id ranges, as mag240M stores papers,
 * authors and institutions).  Stands in for cxgnncomp_backend.gen_edge_type_mag240m
 * (called at hiscache/history_model.py:356), which is not part of the
 * reference repository.  Edge slots in [ptr[R], E) are set to -1 (out needs no
 * initialisation); a source outside [0, n_all) gets -1.  n_bounds <= 64. */
int hc_edge_types_by_ranges(const int64_t *ptr, const int64_t *idx, const int64_t *sub_to_full,
                            int64_t n_all, const int64_t *bounds, int n_bounds,
                            const int64_t *pair_to_rel, int64_t *out, int64_t R, int64_t E,
                            void *stream);

/* hc_check_csr: input check a caller can run before handing a block to the
 * aggregation entry points, which (like the reference kernels) trust their
 * indices.  report is int64[4] on the device: [0] rows whose end offset lies
 * before their start, [1] offsets outside [0, E], [2] neighbour ids outside
 * [0, n_src) among the slots [ptr[0], ptr[R]), [3] zero.  No reference
 * counterpart. */
int hc_check_csr(const int64_t *ptr, const int64_t *idx, int64_t R, int64_t E, int64_t n_src,
                 int64_t *report, void *stream);

/* hc_structure_score replaces get_graph_structure_score (grad_check.h:22-24,
 * grad_check.cu:132-163) with a level-synchronous, deterministic reading of
 * the same rule: per pass, seeds hold 1; a row with a non-zero value offers
 * value*deg to each neighbour that was 0 before the pass; the smallest offer
 * wins.  out[n_all] int64; scratch[n_all] int64 is caller-provided. */
int hc_structure_score(const int64_t *ptr, const int64_t *idx, int64_t ptr_rows, int64_t n_all,
                       int64_t n_seed, int num_layer, int64_t *out, int64_t *scratch, void *stream);

/* hc_gather_rows: dst[i,:] = (mask == NULL || mask[i]) ? src[ids[i],:] : 0,
 * optionally accumulated (dst += ...) when accumulate != 0.  A negative id
 * addresses from the end (-1 = last row), as the torch indexing it replaces
 * does (hiscache/history_cache.py:312-313,345-350).  src may be device memory
 * or pinned, mapped host memory (zero-copy read over the host link); dst is
 * [n, F] of dst_dtype; src is [n_rows, F] of src_dtype. */
int hc_gather_rows(const void *src, int src_dtype, int64_t n_rows, const int64_t *ids,
                   const uint8_t *mask, void *dst, int dst_dtype, int accumulate, int64_t n,
                   int64_t F, void *stream);

/* hc_stream_create_cu_limited: a HIP stream (non-default, default priority)
 * whose kernels run on n_cus compute units only, spread over the chip; for the
 * zero-copy feature read that runs beside the previous batch's forward and
 * backward (the side stream of cxgnndl.UVM's role, hiscache/history_cache.py:
 * 283,301,345): a kernel that waits on the host link slows the kernels beside
 * it unless it is kept to a few compute units (16 - 32 still saturate the
 * link), and the overlap only pays when the compute itself runs on a
 * non-default stream.  The handle is a hipStream_t; release it with
 * hc_stream_destroy once its work has finished. */
int hc_stream_create_cu_limited(int n_cus, void **stream);
int hc_stream_destroy(void *stream);

/* hc_fixup_rows: rows that were gathered ahead of time under a guess of which
 * are needed -- the zero-copy read of a batch's features started one batch
 * early, under the cache state of that moment (uvm.masked_get of
 * hiscache/history_cache.py:345 moved off the critical path) -- brought to the
 * exact answer: dst[i,:] = src[ids[i],:] where need[i] && !have[i]; dst[i,:] = 0
 * where !need[i] && have[i]; other rows are left untouched.  need / have: one
 * byte per row.  Afterwards dst equals hc_gather_rows with mask = need. */
int hc_fixup_rows(const void *src, int src_dtype, int64_t n_rows, const int64_t *ids,
                  const uint8_t *need, const uint8_t *have, void *dst, int dst_dtype, int64_t n,
                  int64_t F, void *stream);

/* hc_gather_rows_hot / hc_gather_rows_flagged: a feature matrix in two tiers.
 * The reference keeps the features of the most requested nodes in GPU memory
 * beside the embeddings (hotness order from sorted_indices.dat,
 * hiscache/history_cache.py:121-142) and merges them with the rows read
 * through UVM (:345-350).  Here copies of the hot rows form a matrix
 * hot[n_hot, F] in device memory, slot_map[n_map] (int32) holds a node's row in
 * it or -1, and the whole matrix stays in pinned host memory.  A batch's rows
 * come in two launches that write disjoint rows of dst[n, F]:
 *   hc_gather_rows_hot: for every i, with take = (mask == NULL || mask[i]) and
 *     ids[i] inside [0, n_map) (a negative id addresses from the end):
 *     dst[i,:] = hot[slot_map[ids[i]],:] when taken and the slot lies in
 *     [0, n_hot); dst[i,:] = 0 when not taken; otherwise the row is left alone
 *     and cold[i] = 1 (cold[i] = 0 for the rows written here).  cold: n bytes.
 *   hc_gather_rows_flagged: dst[i,:] = src[ids[i],:] for the rows with
 *     flag[i] != 0 (cleared if ids[i] lies outside [0, n_rows)), other rows are
 *     not touched.  src may be pinned, mapped host memory; ids may differ from
 *     the first call's (a caller that stores the host matrix under other row
 *     numbers).
 * After both, dst equals hc_gather_rows(src, ..., ids, mask) when hot holds
 * copies of src's rows. */
int hc_gather_rows_hot(const void *hot, int hot_dtype, int64_t n_hot, const int32_t *slot_map,
                       int64_t n_map, const int64_t *ids, const uint8_t *mask, void *dst, int dst_dtype,
                       uint8_t *cold, int64_t n, int64_t F, void *stream);
int hc_gather_rows_flagged(const void *src, int src_dtype, int64_t n_rows, const int64_t *ids,
                           const uint8_t *flag, void *dst, int dst_dtype, int64_t n, int64_t F,
                           void *stream);

/* hc_lookup: out[i] = map[ids[i] + offset]  (int64 gather; the id translation
 * of lookup_and_load, hiscache/history_cache.py:310,315). */
int hc_lookup(const int64_t *map, int64_t map_len, const int64_t *ids, int64_t offset, int64_t *out,
              int64_t n, void *stream);
/* hc_lookup_dev: hc_lookup for a batch padded to a fixed size (recorded
 * iterations): entries at or behind *n_valid_dev (one int64 in device memory)
 * are padding and come out as -1. */
int hc_lookup_dev(const int64_t *map, int64_t map_len, const int64_t *ids, int64_t offset,
                  const int64_t *n_valid_dev, int64_t *out, int64_t n, void *stream);

/* hc_load_mask: the rows of a batch that have to be read from the feature store,
 * and the cache's hit counters, in one launch.  The reference spells the mask as
 * load = used & ~(sub2feat != -1) with tensor operators
 * (hiscache/history_cache.py:327-330) and can print the counts from a debug
 * branch (:331-341); here they accumulate in device memory and are read only
 * when the caller asks for them.
 *   used[n_all]      bytes: row is still needed (used_masks[0] of hc_count_history)
 *   sub2feat[n_all]  nullable: feature-cache slot per node, -1 = not cached
 *   sub2embed[n1]    nullable: embedding slot per 1-hop node, -1 = not cached
 *   prev_mask[n_prev] nullable: the admission mask of the previous update
 *   hit_feat[n_all]  out, nullable: sub2feat[i] != -1
 *   load_mask[n_all] out, nullable: used[i] && !hit_feat[i]
 *   counters[8]      in/out, nullable, int64, += per call: [0] 1, [1] n_all, [2] n1,
 *                    [3] embedding hits, [4] nodes pruned (!used), [5] feature-cache
 *                    hits, [6] rows to load, [7] rows admitted by prev_mask. */
int hc_load_mask(const uint8_t *used, const int64_t *sub2feat, const int64_t *sub2embed,
                 const uint8_t *prev_mask, int64_t n_all, int64_t n1, int64_t n_prev,
                 uint8_t *hit_feat, uint8_t *load_mask, int64_t *counters, void *stream);

/* hc_ring_lookup: lookup of a ring table (full2slot / checkin / table as
 * hc_grad_check maintains them) for one batch, in one launch:
 *   slot_out[i] = full2slot[ids[i]], or -1 when the id has no entry or its entry
 *                 is stale: now - checkin[slot] >= age_limit (checkin nullable:
 *                 then no entry is stale);
 *   rows_out[i,:F] (fp32, nullable) = table[slot_out[i], :F], zeros for -1.
 * A stale entry is reported as absent so that the caller recomputes the row and
 * may admit the fresh value; the reference bounds the age of an entry the same
 * way by un-mapping old slots (hiscache/history_table.py:189-200) and looks
 * slots up with torch indexing (hiscache/history_cache.py:307-313). */
int hc_ring_lookup(const int64_t *full2slot, int64_t n_full, const int64_t *ids,
                   const int64_t *checkin, int64_t now, int64_t age_limit, const void *table,
                   int table_dtype, int64_t capacity, int64_t F, int64_t *slot_out, float *rows_out,
                   int64_t n, void *stream);

/* ---------------------------------------------------------------- layer epilogue
 * hc_bn_relu_fwd / hc_bn_relu_bwd: the training-mode epilogue of a hidden
 * layer, `x = self.bns[i](x); x = F.relu(x)` (hiscache/history_model.py:139-140,
 * 386-387) behind a convolution whose linear layer adds a bias
 * (history_model.py:66,94), as two launches forward and two backward.
 *   forward:  mean[c], var[c] (biased) over the n rows of x[n, C] (fp32);
 *             save_mean = mean, save_invstd = 1/sqrt(var + eps);
 *             y = max(0, (x - mean) * invstd * gamma + beta);
 *             running_mean = (1 - momentum) * running_mean + momentum * (mean + bias),
 *             running_var  = (1 - momentum) * running_var + momentum * var * n/(n-1)
 *             (torch.nn.BatchNorm1d's rule; both nullable);
 *             *num_batches_tracked += 1 (one int64 on the device, nullable:
 *             the module's batch counter, which costs a launch of its own otherwise).
 *   backward: dy' = dy where y > 0, else 0; dbeta = sum dy', dgamma = sum dy' * xhat,
 *             dx = gamma * invstd * (dy' - dbeta/n - xhat * dgamma/n), dbias = 0.
 * bias (nullable) is a per-column constant that the caller has NOT added to x:
 * in front of a normalisation it cancels in y and has zero gradient; it only
 * shifts the mean that the running statistics record.  gamma / beta nullable
 * (1 / 0).  x is the forward's input in both calls.  C % 4 == 0, C <= 1024
 * (HC_EUNSUPPORTED otherwise).  Column statistics are summed per slab of rows and
 * the slabs merged in slab order: results do not depend on scheduling.
 * ticket: one 32-bit word of device memory that is zero on entry and zero again
 * when the call's kernels have run; calls that share a ticket must not overlap.
 * workspace: hc_bn_relu_workspace_bytes(n, C), 16-byte aligned; not preserved. */
size_t hc_bn_relu_workspace_bytes(int64_t n, int64_t C);
int hc_bn_relu_fwd(const float *x, const float *bias, const float *gamma, const float *beta,
                   float *running_mean, float *running_var, int64_t *num_batches_tracked,
                   float momentum, float eps, float *y, float *save_mean, float *save_invstd,
                   int64_t n, int64_t C, void *workspace, size_t workspace_bytes, unsigned *ticket,
                   void *stream);
int hc_bn_relu_bwd(const float *dy, const float *x, const float *gamma, const float *beta,
                   const float *save_mean, const float *save_invstd, float *dx, float *dgamma,
                   float *dbeta, float *dbias, int64_t n, int64_t C, void *workspace,
                   size_t workspace_bytes, unsigned *ticket, void *stream);

/* hc_weight_grad: the gradient of a layer's linear maps, dw[H, F] = g^T x for
 * g [n, H] and x [n, F] (fp32, row-major, contiguous) -- what autograd computes
 * for `self.lin_l(out)` and `self.lin_r(x[:num_node])`
 * (hiscache/history_model.py:94-98), whose weights are [H, F].  x1 / dw1
 * (both or neither NULL) is a second operand that shares g: the aggregated rows
 * and the root rows of a SAGE layer go through the same two launches.  The rows
 * are split into slabs, every slab's product is computed on the matrix cores in
 * fp32 and the slabs are added in slab order: no atomics, the result does not
 * depend on scheduling (the slab partition is a function of n, H, F and the
 * operand count).  H % 64 == 0, F % 64 == 0, both at most 4096
 * (HC_EUNSUPPORTED otherwise); dw 16-byte aligned.
 * workspace: hc_weight_grad_workspace_bytes(n, H, F, operands), 16-byte aligned. */
size_t hc_weight_grad_workspace_bytes(int64_t n, int64_t H, int64_t F, int n_operands);
int hc_weight_grad(const float *g, const float *x0, const float *x1, int64_t n, int64_t H, int64_t F,
                   float *dw0, float *dw1, void *workspace, size_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------- recorded iterations
 * Entry points for callers that record the launches of one training iteration
 * once (a HIP graph over arrays of a fixed, padded size) and replay them for
 * every batch.  None of them has a counterpart in the reference, whose loop
 * (hiscache/history_trainer.py:176-193) launches operator by operator.  What a
 * replay cannot change -- a launch's arguments -- is read from device memory
 * here: the number of rows in use and the iteration number.  Each is the entry
 * point of the same name without the suffix in every other respect, the same
 * kernels included.
 *
 * hc_stage_arrays: dst[a][i] = i < n_copy[a] ? src[a][i] : fill[a] for
 * i in [0, n_total[a]) and up to 16 arrays of elements of 8, 4, 2 or 1 bytes
 * (elem_bytes[a]; integers, or the bit patterns of floating-point rows with
 * fill 0), and scalars_dst[k] = scalars[k] for up to 16 int64 values, in one
 * launch: a batch's arrays padded into fixed-size ones (row offsets continued
 * at the edge count, ids at -1) together with its sizes.  The argument arrays
 * are host arrays, read before the call returns.  Every layer of a padded
 * batch gets row offsets of its own, flat behind the layer's real rows: the
 * rows between a layer's count and its padded count are real rows of the next
 * hop, whose sources lie beyond the layer's input, and must stay empty.
 *
 * hc_ring_lookup_dev: hc_ring_lookup with now = *now_dev and ids[i] for
 * i >= *n_valid_dev taken as padding (slot -1, zero row).
 *
 * hc_grad_check_dev: hc_grad_check with glb_iter = *glb_iter_dev.  Padding rows
 * are kept out with the `used` mask.
 *
 * hc_quantile_threshold_dev: hc_quantile_threshold over score[0, n) with
 * n = *n_dev kept inside [1, n_max] and the rank worked out on the device as the
 * host works it out for hc_quantile_threshold (pos = fp32(rate) * fp32(n - 1),
 * lo = floor(pos), w = pos - lo): the same bits.  n_max <= hc_quantile_max_scores().
 *
 * hc_bn_relu_fwd_dev / hc_bn_relu_bwd_dev: hc_bn_relu_fwd / _bwd over a matrix
 * of n rows of which the first *n_dev (kept inside [1, n]; n_dev NULL = all) are
 * in use: only those enter the statistics and the column sums, y and dx of the
 * others are zero.  The slab partition is that of n. */
int hc_stage_arrays(const void *const *src, void *const *dst, const int64_t *n_copy, const int64_t *n_total,
                    const int64_t *fill, const int *elem_bytes, int n_arrays, int64_t *scalars_dst,
                    const int64_t *scalars, int n_scalars, void *stream);
int hc_ring_lookup_dev(const int64_t *full2slot, int64_t n_full, const int64_t *ids, const int64_t *checkin,
                       const int64_t *now_dev, const int64_t *n_valid_dev, int64_t age_limit,
                       const void *table, int table_dtype, int64_t capacity, int64_t F, int64_t *slot_out,
                       float *rows_out, int64_t n, void *stream);
int hc_grad_check_dev(const float *grad, const float *score_in, const float *emb, const int64_t *slot,
                      const int32_t *age, const uint8_t *used, const int64_t *sub_to_full,
                      const float *thres, int32_t age_limit, int norm_kind, int cmp_kind,
                      uint8_t *mask_out, float *score_out, int64_t *slot_out, void *table,
                      int table_dtype, int64_t capacity, int64_t *full2slot, int64_t *slot2full,
                      int64_t *checkin, int64_t *header, const int64_t *glb_iter_dev, int64_t M, int64_t F,
                      void *workspace, size_t workspace_bytes, void *stream);
int hc_quantile_threshold_dev(const float *score, const int64_t *n_dev, int64_t n_max, float rate, float *out,
                              void *stream);
int hc_bn_relu_fwd_dev(const float *x, const float *bias, const float *gamma, const float *beta,
                       float *running_mean, float *running_var, int64_t *num_batches_tracked,
                       float momentum, float eps, float *y, float *save_mean, float *save_invstd,
                       int64_t n, int64_t C, const int64_t *n_dev, void *workspace, size_t workspace_bytes,
                       unsigned *ticket, void *stream);
int hc_bn_relu_bwd_dev(const float *dy, const float *x, const float *gamma, const float *beta,
                       const float *save_mean, const float *save_invstd, float *dx, float *dgamma,
                       float *dbeta, float *dbias, int64_t n, int64_t C, const int64_t *n_dev,
                       void *workspace, size_t workspace_bytes, unsigned *ticket, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HISCACHE_HIP_H */
