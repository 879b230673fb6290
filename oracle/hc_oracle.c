/*
 * hc_oracle.c -- TEST INFRASTRUCTURE ONLY.  Never linked into, imported by or
 * shipped with the product library; only tests, the smoke check and the CPU
 * baseline leg of the benchmark may load it.
 *
 * Plain-C, single-threaded restatement of the HisCache hot path, written from
 * the reference's source text.  Every function cites the reference lines it
 * follows.  Loops walk rows and edges in CSR order and accumulate in fp32, so
 * per output element the order of additions is the order a sequential reader
 * of the reference kernel would produce.
 *
 * Index type is int64 everywhere (reference: src/cpp/include/common.h:12).
 *
 * Every function here is pinned by the tests against closed forms, brute
 * force or library routines, except (PARITY UNPINNED against the reference):
 *   orc_structure_score   the reference result depends on thread scheduling;
 *                         only the level-synchronous reading is pinned;
 *   orc_sample_layers     the reference has no sampler (external loader); the
 *                         rule is pinned through its consequences only;
 *   edge_types_by_ranges  (hc_oracle.py) stands in for an external library
 *                         routine whose numbering is not available.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef int64_t Index;

#define ORC_OK 0
#define ORC_EINVAL 1

/* ------------------------------------------------------------------------- */
/* fp32 -> fp16 / bf16, round-to-nearest-even (used for reduced-precision     */
/* history tables, a build extension: the reference tables are fp32 only).    */
/* ------------------------------------------------------------------------- */
static uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

uint16_t orc_f32_to_f16(float f) {
  uint32_t x = f2u(f);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) { /* inf / nan */
    if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((ax >> 13) & 0x3ffu));
    return (uint16_t)(sign | 0x7c00u);
  }
  if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (ax < 0x33000001u) { /* |f| <= 2^-25 -> 0 (ties to even gives 0 at exactly 2^-25) */
    return (uint16_t)sign;
  }
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  uint32_t shift;
  uint32_t base;
  if (e < -14) { /* subnormal half */
    shift = (uint32_t)(13 + (-14 - e));
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(e + 15) << 10;
    m &= 0x7fffffu;
  }
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q += 1; /* carries propagate into the exponent */
  return (uint16_t)(sign | (base + q));
}

uint16_t orc_f32_to_bf16(float f) {
  uint32_t x = f2u(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u); /* quiet nan */
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7fffu + lsb;
  return (uint16_t)(x >> 16);
}

float orc_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu;
  uint32_t m = h & 0x3ffu;
  if (e == 0) {
    if (m == 0) return u2f(sign);
    float v = (float)m * (1.0f / 16777216.0f); /* m * 2^-24 */
    return (sign ? -v : v);
  }
  if (e == 31) return u2f(sign | 0x7f800000u | (m << 13));
  return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

float orc_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* ------------------------------------------------------------------------- */
/* Aggregation forward                                                        */
/* ------------------------------------------------------------------------- */

/* Mean aggregation with per-destination-row history substitution.
 * Follows gen_fwd_history_v2, src/cpp/src/history_aggr.cu:7-40:
 *   hmap[row] != -1 -> vout[row,:] = hbuf[row, :F]      (:21-25; hbuf is row-indexed)
 *   else            -> vout[row,:] = (sum_j vin[idx[j],:]) / deg   (:27-39)
 *   deg == 0        -> row is left as the caller's zero fill (:38, :425)
 * hmap may be NULL (no history at all). */
static void sum_rows_seq(const Index *idx, const float *vin, Index F, Index b, Index e, float *o) {
  for (Index j = b; j < e; ++j) {
    const float *x = vin + idx[j] * F;
    for (Index c = 0; c < F; ++c) o[c] += x[c];
  }
}

/* split_above == 0: every row is summed strictly in CSR order (the order a sequential reader of
 * the reference kernel produces).  split_above > 0 restates the device library's documented order
 * for long rows: a row with more than split_above edges is summed as four contiguous quarters of
 * ceil(deg/4) edges, each in CSR order, combined left to right ((q0+q1)+q2)+q3. */
int orc_fwd_mean_row(const Index *ptr, const Index *idx, const float *vin,
                     const Index *hmap, const float *hbuf, float *vout,
                     Index R, Index F, Index hsize, Index split_above) {
  float *part = (float *)malloc((size_t)F * sizeof(float));
  if (!part) return ORC_EINVAL;
  for (Index row = 0; row < R; ++row) {
    float *o = vout + row * F;
    memset(o, 0, (size_t)F * sizeof(float));
    if (hmap && hmap[row] != -1) {
      for (Index c = 0; c < F; ++c) o[c] = hbuf[row * hsize + c];
      continue;
    }
    Index b = ptr[row], e = ptr[row + 1];
    int n = (int)(e - b);
    if (n == 0) continue;
    if (split_above > 0 && n > split_above) {
      Index q = (n + 3) / 4;
      for (int w = 0; w < 4; ++w) {
        Index sb = b + w * q, se = sb + q;
        if (sb > e) sb = e;
        if (se > e) se = e;
        if (w == 0) {
          sum_rows_seq(idx, vin, F, sb, se, o);
        } else {
          memset(part, 0, (size_t)F * sizeof(float));
          sum_rows_seq(idx, vin, F, sb, se, part);
          for (Index c = 0; c < F; ++c) o[c] += part[c];
        }
      }
    } else {
      sum_rows_seq(idx, vin, F, b, e, o);
    }
    for (Index c = 0; c < F; ++c) o[c] = o[c] / (float)n;
  }
  free(part);
  return ORC_OK;
}

/* Weighted-sum aggregation, follows gen_fwd_history_v2_edge_value,
 * history_aggr.cu:42-78: no division, every non-history row is written
 * (0 for empty rows, :77).  `rs += vin * val` is one fused multiply-add. */
static void wsum_rows_seq(const Index *idx, const float *ev, const float *vin, Index F, Index b,
                          Index e, float *o) {
  for (Index j = b; j < e; ++j) {
    const float *x = vin + idx[j] * F;
    float w = ev[j];
    for (Index c = 0; c < F; ++c) o[c] = fmaf(x[c], w, o[c]);
  }
}

/* split_above as in orc_fwd_mean_row: the device library's quarter rule for rows with more than
 * split_above edges (four contiguous quarters, each from zero in CSR order, combined left to right). */
int orc_fwd_edge_value(const Index *ptr, const Index *idx, const float *ev,
                       const float *vin, const Index *hmap, const float *hbuf,
                       float *vout, Index R, Index F, Index hsize, Index split_above) {
  float *part = (float *)malloc((size_t)F * sizeof(float));
  if (!part) return ORC_EINVAL;
  for (Index row = 0; row < R; ++row) {
    float *o = vout + row * F;
    if (hmap && hmap[row] != -1) {
      for (Index c = 0; c < F; ++c) o[c] = hbuf[row * hsize + c];
      continue;
    }
    for (Index c = 0; c < F; ++c) o[c] = 0.0f;
    Index b = ptr[row], e = ptr[row + 1];
    Index n = e - b;
    if (split_above > 0 && n > split_above) {
      Index q = (n + 3) / 4;
      for (int w = 0; w < 4; ++w) {
        Index sb = b + w * q, se = sb + q;
        if (sb > e) sb = e;
        if (se > e) se = e;
        if (w == 0) {
          wsum_rows_seq(idx, ev, vin, F, sb, se, o);
        } else {
          memset(part, 0, (size_t)F * sizeof(float));
          wsum_rows_seq(idx, ev, vin, F, sb, se, part);
          for (Index c = 0; c < F; ++c) o[c] += part[c];
        }
      }
    } else {
      wsum_rows_seq(idx, ev, vin, F, b, e, o);
    }
  }
  free(part);
  return ORC_OK;
}

/* Multi-head weighted sum, follows gen_fwd_history_v2_edge_value_multi_head,
 * history_aggr.cu:80-125.  vin[N,H,F], ev[E,H], vout[R,H,F].
 * History rows: hsize == F -> every head copies hbuf[row,:F] (:97-99);
 * hsize == F*H -> head h copies hbuf[row, h*F:(h+1)*F] (:100-103);
 * anything else is an error (:104-106). */
int orc_fwd_edge_value_multi_head(const Index *ptr, const Index *idx,
                                  const float *ev, const float *vin,
                                  const Index *hmap, const float *hbuf,
                                  float *vout, Index R, Index F, Index hsize,
                                  Index H) {
  if (hmap && hsize != F && hsize != F * H) return ORC_EINVAL;
  for (Index row = 0; row < R; ++row) {
    for (Index h = 0; h < H; ++h) {
      float *o = vout + (row * H + h) * F;
      if (hmap && hmap[row] != -1) {
        const float *src = (hsize == F) ? hbuf + row * hsize : hbuf + row * hsize + h * F;
        for (Index c = 0; c < F; ++c) o[c] = src[c];
        continue;
      }
      for (Index c = 0; c < F; ++c) o[c] = 0.0f;
      for (Index j = ptr[row]; j < ptr[row + 1]; ++j) {
        const float *x = vin + (idx[j] * H + h) * F;
        float w = ev[j * H + h];
        for (Index c = 0; c < F; ++c) o[c] = fmaf(x[c], w, o[c]);
      }
    }
  }
  return ORC_OK;
}

/* Mean aggregation with per-SOURCE substitution (build extension, not in the
 * reference): x_j = hmap[idx[j]] != -1 ? hist[hmap[idx[j]], :F] : feat[idx[j], :F].
 * With an all -1 map it is orc_fwd_mean_row without history. */
static void sum_rows_src(const Index *idx, const float *feat, const Index *hmap_src, const float *hist,
                         Index F, Index hsize, Index b, Index e, float *o) {
  for (Index j = b; j < e; ++j) {
    Index s = idx[j];
    const float *x = (hmap_src && hmap_src[s] != -1) ? hist + hmap_src[s] * hsize : feat + s * F;
    for (Index c = 0; c < F; ++c) o[c] += x[c];
  }
}

int orc_fwd_mean_src(const Index *ptr, const Index *idx, const float *feat,
                     const Index *hmap_src, const float *hist, float *vout,
                     Index R, Index F, Index hsize, Index split_above) {
  float *part = (float *)malloc((size_t)F * sizeof(float));
  if (!part) return ORC_EINVAL;
  for (Index row = 0; row < R; ++row) {
    float *o = vout + row * F;
    memset(o, 0, (size_t)F * sizeof(float));
    Index b = ptr[row], e = ptr[row + 1];
    int n = (int)(e - b);
    if (n == 0) continue;
    if (split_above > 0 && n > split_above) {   /* same quarter rule as orc_fwd_mean_row */
      Index q = (n + 3) / 4;
      for (int w = 0; w < 4; ++w) {
        Index sb = b + w * q, se = sb + q;
        if (sb > e) sb = e;
        if (se > e) se = e;
        if (w == 0) {
          sum_rows_src(idx, feat, hmap_src, hist, F, hsize, sb, se, o);
        } else {
          memset(part, 0, (size_t)F * sizeof(float));
          sum_rows_src(idx, feat, hmap_src, hist, F, hsize, sb, se, part);
          for (Index c = 0; c < F; ++c) o[c] += part[c];
        }
      }
    } else {
      sum_rows_src(idx, feat, hmap_src, hist, F, hsize, b, e, o);
    }
    for (Index c = 0; c < F; ++c) o[c] = o[c] / (float)n;
  }
  free(part);
  return ORC_OK;
}

/* ------------------------------------------------------------------------- */
/* Aggregation backward                                                       */
/* ------------------------------------------------------------------------- */

/* Follows gen_bwd_history_grad_v2, history_aggr.cu:127-168, with the float
 * atomics replaced by a sequential walk (rows ascending, edges in CSR order):
 *   history row -> grads_history[row,:F] += g[row,:]        (:144-149, no division)
 *   else        -> grads_out[idx[j],:] += g[row,:] / deg    (:140-142, :161-166)
 * grads_out[n_src,F] and grads_history[R,hsize] are zero-filled first (:503-504). */
static int bwd_mean_row_impl(const Index *ptr, const Index *idx, const float *g,
                             const Index *hmap, float *grads_out, float *grads_history,
                             Index R, Index F, Index hsize, Index n_src, Index chunk, Index view_rows) {
  /* chunk == 0: every source row is summed strictly in (row, edge) order.  chunk > 0 restates the
   * device library's documented order for hubs: a source with more than `chunk` incoming edges is
   * summed in chunks of `chunk` consecutive incoming edges, each chunk from zero in order, and the
   * chunk sums are combined left to right.
   * view_rows < 0: "incoming edges" are the live ones (rows below R that did not take their history
   * row): the order over a transposed view built for this layer.  view_rows >= R: the order over one
   * view of the first view_rows rows of the whole mini-batch CSR (hc_aggr_bwd_batch_view): positions
   * are counted over every edge of those rows, a hub is a source with more than `chunk` of them, and
   * only the live edges of a chunk are added. */
  memset(grads_out, 0, (size_t)(n_src * F) * sizeof(float));
  if (grads_history) memset(grads_history, 0, (size_t)(R * hsize) * sizeof(float));
  Index *indeg = NULL, *seen = NULL, *hub_of = NULL;
  float *part = NULL;
  Index n_hubs = 0;
  const Index walk_rows = view_rows < 0 ? R : view_rows;
  if (chunk > 0) {
    indeg = (Index *)calloc((size_t)(n_src > 0 ? n_src : 1), sizeof(Index));
    seen = (Index *)calloc((size_t)(n_src > 0 ? n_src : 1), sizeof(Index));
    hub_of = (Index *)malloc((size_t)(n_src > 0 ? n_src : 1) * sizeof(Index));
    if (!indeg || !seen || !hub_of) return ORC_EINVAL;
    for (Index row = 0; row < walk_rows; ++row) {
      if (view_rows < 0 && hmap && hmap[row] != -1) continue;
      for (Index j = ptr[row]; j < ptr[row + 1]; ++j)
        if (idx[j] >= 0 && idx[j] < n_src) indeg[idx[j]]++;
    }
    for (Index s = 0; s < n_src; ++s) hub_of[s] = indeg[s] > chunk ? n_hubs++ : -1;
    part = (float *)calloc((size_t)((n_hubs > 0 ? n_hubs : 1) * F), sizeof(float));
    if (!part) return ORC_EINVAL;
  }
  for (Index row = 0; row < walk_rows; ++row) {
    const int live = row < R && !(hmap && hmap[row] != -1);
    const float *gr = row < R ? g + row * F : g;
    if (row < R && !live && grads_history) {
      for (Index c = 0; c < F; ++c) grads_history[row * hsize + c] += gr[c];
    }
    if (!live && (view_rows < 0 || chunk == 0)) continue;
    Index b = ptr[row], e = ptr[row + 1];
    int n = (int)(e - b);
    if (n == 0) continue;
    for (Index j = b; j < e; ++j) {
      Index s = idx[j];
      if (s < 0 || s >= n_src) continue;   /* a source of deeper layers: only rows >= R reach it */
      float *o = grads_out + s * F;
      if (chunk > 0 && hub_of[s] >= 0) {
        float *p = part + hub_of[s] * F;
        if (live)
          for (Index c = 0; c < F; ++c) p[c] += gr[c] / (float)n;
        seen[s]++;
        if (seen[s] % chunk == 0 || seen[s] == indeg[s]) { /* chunk complete: fold it in */
          for (Index c = 0; c < F; ++c) { o[c] += p[c]; p[c] = 0.0f; }
        }
      } else if (live) {
        for (Index c = 0; c < F; ++c) o[c] += gr[c] / (float)n;
      }
    }
  }
  free(indeg); free(seen); free(hub_of); free(part);
  return ORC_OK;
}

int orc_bwd_mean_row(const Index *ptr, const Index *idx, const float *g,
                     const Index *hmap, float *grads_out, float *grads_history,
                     Index R, Index F, Index hsize, Index n_src, Index chunk) {
  return bwd_mean_row_impl(ptr, idx, g, hmap, grads_out, grads_history, R, F, hsize, n_src, chunk, -1);
}

/* The same gradient in the summation order of hc_aggr_bwd_batch_view: `ptr` / `idx` hold at least
 * view_rows >= R rows (the whole mini-batch CSR), g and hmap the layer's first R rows. */
int orc_bwd_mean_row_batch_view(const Index *ptr, const Index *idx, const float *g,
                                const Index *hmap, float *grads_out, float *grads_history,
                                Index R, Index F, Index hsize, Index n_src, Index chunk, Index view_rows) {
  if (view_rows < R) return ORC_EINVAL;
  return bwd_mean_row_impl(ptr, idx, g, hmap, grads_out, grads_history, R, F, hsize, n_src, chunk, view_rows);
}

/* Source-substitution backward (build extension): the gradient of the mean
 * with respect to the substituted source row, whichever table it came from. */
int orc_bwd_mean_src(const Index *ptr, const Index *idx, const float *g,
                     float *grad_src, Index R, Index F, Index n_src) {
  return orc_bwd_mean_row(ptr, idx, g, NULL, grad_src, NULL, R, F, 0, n_src, 0);
}

/* Follows gen_bwd_history_grad_v2_edge_value (:170-213) and its _edge_grad
 * variant (:215-270).  grads_out[idx[j],:] += g[row,:] * ev[j]  (product
 * rounded, then added: the reference adds the product with atomicAdd).
 * edge_grad[j] = sum_c g[row,c] * vin[idx[j],c]  (:258-267) -- the reference's
 * summation order is arrival order, so it is computed here in double and
 * rounded once; compare with a tolerance.  edge_grad / vin may be NULL. */
int orc_bwd_edge_value(const Index *ptr, const Index *idx, const float *ev,
                       const float *g, const Index *hmap, const float *vin,
                       float *grads_out, float *grads_history, float *edge_grad,
                       Index R, Index F, Index hsize, Index n_src, Index E) {
  memset(grads_out, 0, (size_t)(n_src * F) * sizeof(float));
  if (grads_history) memset(grads_history, 0, (size_t)(R * hsize) * sizeof(float));
  if (edge_grad) memset(edge_grad, 0, (size_t)E * sizeof(float));
  for (Index row = 0; row < R; ++row) {
    const float *gr = g + row * F;
    if (hmap && hmap[row] != -1) {
      for (Index c = 0; c < F; ++c) grads_history[row * hsize + c] += gr[c];
      continue;
    }
    for (Index j = ptr[row]; j < ptr[row + 1]; ++j) {
      float *o = grads_out + idx[j] * F;
      float w = ev[j];
      for (Index c = 0; c < F; ++c) {
        float p = gr[c] * w;
        o[c] += p;
      }
      if (edge_grad) {
        const float *x = vin + idx[j] * F;
        double s = 0.0;
        for (Index c = 0; c < F; ++c) s += (double)gr[c] * (double)x[c];
        edge_grad[j] = (float)s;
      }
    }
  }
  return ORC_OK;
}

/* Follows gen_bwd_history_grad_v2_edge_value_multi_head (:272-327) and its
 * _edge_grad variant (:329-397).  g[R,H,F], ev[E,H], vin[N,H,F],
 * grads_out[N,H,F], grads_history[R,hsize], edge_grad[E,H].
 * History rows: hsize == F -> all heads accumulate into grads_history[row,:F]
 * in head order (:293-294); hsize == F*H -> per-head slices (:295-298). */
int orc_bwd_edge_value_multi_head(const Index *ptr, const Index *idx,
                                  const float *ev, const float *g,
                                  const Index *hmap, const float *vin,
                                  float *grads_out, float *grads_history,
                                  float *edge_grad, Index R, Index F,
                                  Index hsize, Index H, Index n_src, Index E) {
  if (hmap && hsize != F && hsize != F * H) return ORC_EINVAL;
  memset(grads_out, 0, (size_t)(n_src * H * F) * sizeof(float));
  if (grads_history) memset(grads_history, 0, (size_t)(R * hsize) * sizeof(float));
  if (edge_grad) memset(edge_grad, 0, (size_t)(E * H) * sizeof(float));
  for (Index row = 0; row < R; ++row) {
    for (Index h = 0; h < H; ++h) {
      const float *gr = g + (row * H + h) * F;
      if (hmap && hmap[row] != -1) {
        float *d = (hsize == F) ? grads_history + row * hsize : grads_history + row * hsize + h * F;
        for (Index c = 0; c < F; ++c) d[c] += gr[c];
        continue;
      }
      for (Index j = ptr[row]; j < ptr[row + 1]; ++j) {
        float *o = grads_out + (idx[j] * H + h) * F;
        float w = ev[j * H + h];
        for (Index c = 0; c < F; ++c) {
          float p = gr[c] * w;
          o[c] += p;
        }
        if (edge_grad) {
          const float *x = vin + (idx[j] * H + h) * F;
          double s = 0.0;
          for (Index c = 0; c < F; ++c) s += (double)gr[c] * (double)x[c];
          edge_grad[j * H + h] = (float)s;
        }
      }
    }
  }
  return ORC_OK;
}

/* ------------------------------------------------------------------------- */
/* Transposed (CSC) view used by the atomic-free backward.  Stable counting    */
/* sort of edges by source id; edges of history rows are dropped when          */
/* hmap_row is given.  ptrT[n_src+1], rowT[E], edgeT[E] (only the first        */
/* ptrT[n_src] entries are meaningful).  Build-defined, no reference twin.     */
/* ------------------------------------------------------------------------- */
int orc_build_transpose(const Index *ptr, const Index *idx, const Index *hmap_row,
                        Index R, Index n_src, Index *ptrT, int32_t *rowT,
                        int32_t *edgeT) {
  memset(ptrT, 0, (size_t)(n_src + 1) * sizeof(Index));
  for (Index row = 0; row < R; ++row) {
    if (hmap_row && hmap_row[row] != -1) continue;
    for (Index j = ptr[row]; j < ptr[row + 1]; ++j) {
      if (idx[j] < 0 || idx[j] >= n_src) return ORC_EINVAL;
      ptrT[idx[j] + 1]++;
    }
  }
  for (Index s = 0; s < n_src; ++s) ptrT[s + 1] += ptrT[s];
  Index *cur = (Index *)malloc((size_t)(n_src + 1) * sizeof(Index));
  if (!cur) return ORC_EINVAL;
  memcpy(cur, ptrT, (size_t)(n_src + 1) * sizeof(Index));
  for (Index row = 0; row < R; ++row) {
    if (hmap_row && hmap_row[row] != -1) continue;
    for (Index j = ptr[row]; j < ptr[row + 1]; ++j) {
      Index p = cur[idx[j]]++;
      rowT[p] = (int32_t)row;
      edgeT[p] = (int32_t)j;
    }
  }
  free(cur);
  return ORC_OK;
}

/* ------------------------------------------------------------------------- */
/* count_history_reconstruct                                                  */
/* ------------------------------------------------------------------------- */

/* Follows count_history_kernel + count_history_reconstruct,
 * src/cpp/src/grad_check.cu:70-130.  masks is (L+1) x n_all bytes, zero-filled
 * here (:107-110); masks[L] is the seed level, masks[0] the raw-feature level.
 * Pass i = 0..L-1 reads use_in = masks[L-i], writes use_out = masks[L-1-i]
 * (:125-127).  A row is active if it is a seed on the first pass (:79-82) or
 * use_in[row] is set (:83-84).  On pass i == 1 only (:122-124) an active row
 * with history stops without marking anything (:87-90); otherwise it marks
 * itself (:92-94) and all its neighbours (:97-100).
 * hmap covers rows [0, hmap_len); an active row beyond it on pass 1 is an
 * input error here (the reference would read out of bounds). */
int orc_count_history(const Index *ptr, const Index *idx, const Index *hmap,
                      Index hmap_len, uint8_t *masks, Index ptr_rows,
                      Index n_all, Index n_seed, int L) {
  memset(masks, 0, (size_t)((Index)(L + 1) * n_all));
  for (int i = 0; i < L; ++i) {
    uint8_t *use_in = masks + (Index)(L - i) * n_all;
    uint8_t *use_out = masks + (Index)(L - 1 - i) * n_all;
    int layer_id = L - 1 - i;
    const Index *hm = (i == 1) ? hmap : NULL;
    for (Index row = 0; row < ptr_rows; ++row) {
      if (row < n_seed && layer_id == L - 1) {
        use_in[row] = 1;
      } else if (use_in[row] != 1) {
        continue;
      }
      if (hm) {
        if (row >= hmap_len) return ORC_EINVAL;
        if (hm[row] != -1) continue;
      }
      use_out[row] = 1;
      for (Index j = ptr[row]; j < ptr[row + 1]; ++j) {
        if (idx[j] < 0 || idx[j] >= n_all) return ORC_EINVAL;
        use_out[idx[j]] = 1;
      }
    }
  }
  return ORC_OK;
}

/* ------------------------------------------------------------------------- */
/* Admission                                                                  */
/* ------------------------------------------------------------------------- */

/* One ring insert: the body of record_history_kernel_used_mask after the
 * predicate, grad_check.cu:22-45.  slot = old header; header advances modulo
 * the capacity (atomicInc semantics, :25); the slot's previous owner is
 * un-mapped only if it still points at the slot (:26-30). */
static void ring_insert(Index full, Index *header, Index cap, Index *slot2full,
                        Index *full2slot, Index *checkin, Index glb_iter,
                        Index *slot_out) {
  Index s = *header;
  *header = (s >= cap - 1) ? 0 : s + 1;
  Index old = slot2full[s];
  if (old != -1 && full2slot[old] == s) full2slot[old] = -1;
  full2slot[full] = s;
  slot2full[s] = full;
  if (checkin) checkin[s] = glb_iter;
  *slot_out = s;
}

/* Follows record_history_kernel_used_mask + record_history,
 * grad_check.cu:6-68, processed sequentially in row order (the reference
 * hands out slots in atomic arrival order; the admitted SET is the same).
 * Skip a row if sub_to_history != -1, or thres != 0 && score > thres, or
 * used_mask == 0 (:17-21).  mask_out (nullable) receives the admitted flag
 * per row -- the reference has no such output. */
int orc_record_history(const float *buffer_new, float *buffer_all,
                       const uint8_t *used_mask, const Index *sub_to_full,
                       const Index *sub_to_history, Index *history_to_full,
                       Index *full_to_history, Index *header,
                       const float *score, const float *thres_p,
                       Index *checkin_iter, Index glb_iter, Index M,
                       Index history_num, Index history_size,
                       uint8_t *mask_out) {
  float thres = thres_p[0];
  for (Index sub = 0; sub < M; ++sub) {
    int skip = (sub_to_history[sub] != -1) ||
               (thres != 0 && score[sub] > thres) ||
               (used_mask && used_mask[sub] == 0);
    if (mask_out) mask_out[sub] = (uint8_t)!skip;
    if (skip) continue;
    Index s;
    ring_insert(sub_to_full[sub], header, history_num, history_to_full,
                full_to_history, checkin_iter, glb_iter, &s);
    memcpy(buffer_all + s * history_size, buffer_new + sub * history_size,
           (size_t)history_size * sizeof(float));
  }
  return ORC_OK;
}

/* Row score with the summation order the device kernel documents: a row is
 * covered by 64 lanes; element e belongs to lane (e / 4) % 64; a lane folds
 * its elements in increasing e (L2: acc = fma(x, x, acc); L1: acc += |x|);
 * the 64 partials are combined by a butterfly, partner distance 32,16,8,4,2,1
 * (acc[l] = acc[l] + acc[l ^ d]); L2 takes sqrtf of the total.
 * Mathematically: L2 is Tensor.norm(dim=1) (hiscache/history_cache.py:205),
 * L1 is sum(abs(grad), 1) (hiscache/history_table.py:161). */
#define ORC_NORM_L2 0
#define ORC_NORM_L1 1
float orc_row_score(const float *row, Index F, int norm_kind) {
  float acc[64];
  for (int l = 0; l < 64; ++l) acc[l] = 0.0f;
  for (Index e = 0; e < F; ++e) {
    int l = (int)((e / 4) % 64);
    float x = row[e];
    if (norm_kind == ORC_NORM_L2) acc[l] = fmaf(x, x, acc[l]);
    else acc[l] = acc[l] + fabsf(x);
  }
  for (int d = 32; d >= 1; d >>= 1) {
    float nxt[64];
    for (int l = 0; l < 64; ++l) nxt[l] = acc[l] + acc[l ^ d];
    memcpy(acc, nxt, sizeof(acc));
  }
  return norm_kind == ORC_NORM_L2 ? sqrtf(acc[0]) : acc[0];
}

int orc_row_scores(const float *grad, float *score, Index M, Index F, int norm_kind) {
  for (Index r = 0; r < M; ++r) score[r] = orc_row_score(grad + r * F, F, norm_kind);
  return ORC_OK;
}

/* Fused admission (the "grad_check" pass; build-defined generalisation that
 * reduces to the two reference rules):
 *   score[r] = row norm of grad (or the given score when grad == NULL)
 *   pass[r]  = cmp == LT     ? score <  thres                   (history_cache.py:215)
 *              cmp == NOT_GT ? !(thres != 0 && score > thres)   (grad_check.cu:18)
 *   admit[r] = used[r] && pass[r] && (slot[r] == -1 || (age && age[r] >= age_limit))
 * Admitted rows are ring-inserted in row order exactly as in record_history;
 * the embedding row is stored as fp32, fp16 or bf16 (round to nearest even).
 * table_dtype: 0 = f32, 1 = f16, 2 = bf16. */
#define ORC_CMP_LT 0
#define ORC_CMP_NOT_GT 1
int orc_grad_check(const float *grad, const float *score_in, const float *emb,
                   const Index *slot, const int32_t *age, const uint8_t *used,
                   const Index *sub_to_full, float thres, int32_t age_limit,
                   int norm_kind, int cmp_kind, uint8_t *mask_out,
                   float *score_out, void *table, int table_dtype,
                   Index capacity, Index *full2slot, Index *slot2full,
                   Index *checkin, Index *header, Index glb_iter, Index M,
                   Index F, Index *slot_out) {
  for (Index r = 0; r < M; ++r) {
    float sc = grad ? orc_row_score(grad + r * F, F, norm_kind) : score_in[r];
    if (score_out) score_out[r] = sc;
    int pass = (cmp_kind == ORC_CMP_LT) ? (sc < thres) : !(thres != 0 && sc > thres);
    int fresh = (slot[r] == -1) || (age && age[r] >= age_limit);
    int admit = pass && fresh && (!used || used[r] != 0);
    mask_out[r] = (uint8_t)admit;
    if (slot_out) slot_out[r] = -1;
    if (!admit) continue;
    Index s;
    ring_insert(sub_to_full[r], header, capacity, slot2full, full2slot, checkin,
                glb_iter, &s);
    if (slot_out) slot_out[r] = s;
    const float *src = emb + r * F;
    if (table_dtype == 0) {
      memcpy((float *)table + s * F, src, (size_t)F * sizeof(float));
    } else if (table_dtype == 1) {
      uint16_t *d = (uint16_t *)table + s * F;
      for (Index c = 0; c < F; ++c) d[c] = orc_f32_to_f16(src[c]);
    } else if (table_dtype == 2) {
      uint16_t *d = (uint16_t *)table + s * F;
      for (Index c = 0; c < F; ++c) d[c] = orc_f32_to_bf16(src[c]);
    } else {
      return ORC_EINVAL;
    }
  }
  return ORC_OK;
}

/* ------------------------------------------------------------------------- */
/* Small helpers                                                              */
/* ------------------------------------------------------------------------- */

/* Follows count_kernel / count_num, grad_check.cu:165-182: histogram into
 * int32[mmax+1] that skips value 0 (:169). */
int orc_count_num(const Index *arr, Index n, Index mmax, int32_t *out) {
  memset(out, 0, (size_t)(mmax + 1) * sizeof(int32_t));
  for (Index i = 0; i < n; ++i) {
    Index a = arr[i];
    if (a == 0) continue;
    if (a < 0 || a > mmax) return ORC_EINVAL;
    out[a] += 1;
  }
  return ORC_OK;
}

/* Typed CSR for the relational convolution (hiscache/history_model.py:248-270:
 * edges whose source is unused get an extra relation and are ignored; the rest
 * are grouped by relation).  Group r*K+k of (ptr2, idx2) lists, in edge order,
 * the sources of row r's edges of relation k that are kept.  cnt = group
 * sizes, deg = full row degrees.  Pinned by the tests against a stable sort by
 * (row, relation) written with numpy. */
int orc_typed_csr(const Index *ptr, const Index *idx, const Index *et, const uint8_t *used,
                  Index R, Index E, Index n_src, int K, Index *ptr2, Index *idx2, Index *cnt,
                  Index *deg) {
  if (K < 1 || R < 0) return ORC_EINVAL;
  Index pos = 0;
  ptr2[0] = 0;
  for (Index r = 0; r < R; ++r) {
    Index begin = ptr[r], end = ptr[r + 1] < E ? ptr[r + 1] : E;
    deg[r] = ptr[r + 1] - ptr[r];
    for (int k = 0; k < K; ++k) {
      Index c = 0;
      for (Index e = begin; e < end; ++e) {
        Index s = idx[e];
        if (et[e] != k || s < 0 || s >= n_src) continue;
        if (used && !used[s]) continue;
        idx2[pos++] = s;
        ++c;
      }
      cnt[r * K + k] = c;
      ptr2[r * K + k + 1] = pos;
    }
  }
  return ORC_OK;
}

/* Input gradient of the relational layer in the order of hc_aggr_bwd_batch_view_typed: the forward
 * (history_model.py:248-270 with the grouping of orc_typed_csr) gives edge e of row r the weight
 * 1/deg(r) inside group r*K + et[e]; walking rows and edge slots in ascending order adds
 * g[r*K + et[e], :] * (1/deg(r)) to the edge's source, product rounded first. */
int orc_bwd_typed_batch_view(const Index *ptr, const Index *idx, const Index *et, const uint8_t *used,
                             const float *g, float *grads_out, Index R, Index E, Index F, int K,
                             Index n_src) {
  if (K < 1 || R < 0) return ORC_EINVAL;
  memset(grads_out, 0, (size_t)(n_src * F) * sizeof(float));
  for (Index r = 0; r < R; ++r) {
    Index begin = ptr[r], end = ptr[r + 1] < E ? ptr[r + 1] : E;
    Index d = ptr[r + 1] - ptr[r];
    float w = 1.0f / (float)(d > 0 ? d : 1);
    for (Index e = begin; e < end; ++e) {
      Index s = idx[e], k = et[e];
      if (k < 0 || k >= K || s < 0 || s >= n_src) continue;
      if (used && !used[s]) continue;
      const float *gr = g + (r * K + k) * F;
      float *o = grads_out + s * F;
      for (Index c = 0; c < F; ++c) {
        float prod = gr[c] * w;
        o[c] += prod;
      }
    }
  }
  return ORC_OK;
}

/* get_graph_structure_score, grad_check.cu:132-163.  The reference reads and
 * writes `output` across warps inside one pass, so its result depends on
 * scheduling.  This is the level-synchronous reading of the same rule: pass
 * p works on a snapshot; seeds hold 1 (:139); a row with a non-zero snapshot
 * value offers value*deg to every neighbour whose snapshot value is 0 (:145);
 * when several rows offer to one neighbour in the same pass the smallest
 * offer is kept.  PARITY UNPINNED against the reference (order-dependent). */
int orc_structure_score(const Index *ptr, const Index *idx, Index ptr_rows,
                        Index n_all, Index n_seed, int L, Index *out) {
  Index *prev = (Index *)calloc((size_t)n_all, sizeof(Index));
  if (!prev) return ORC_EINVAL;
  memset(out, 0, (size_t)n_all * sizeof(Index));
  for (int p = 0; p < L; ++p) {
    for (Index r = 0; r < n_seed && r < n_all; ++r) out[r] = 1;
    memcpy(prev, out, (size_t)n_all * sizeof(Index));
    for (Index row = 0; row < ptr_rows; ++row) {
      if (prev[row] == 0) continue;
      Index deg = ptr[row + 1] - ptr[row];
      Index offer = prev[row] * deg;
      for (Index j = ptr[row]; j < ptr[row + 1]; ++j) {
        Index n = idx[j];
        if (prev[n] != 0) continue;
        if (out[n] == 0 || offer < out[n]) out[n] = offer;
      }
    }
  }
  free(prev);
  return ORC_OK;
}

/* Row gather used by lookup_and_load (hiscache/history_cache.py:312-313,
 * 345-350): dst[i,:] = table[ids[i],:] when (mask == NULL || mask[i]) else 0.
 * A negative id addresses from the end, as Python indexing does (-1 -> last
 * row), which is what the reference's gather of un-cached slots reads. */
int orc_gather_rows(const float *table, Index n_rows, const Index *ids,
                    const uint8_t *mask, float *dst, Index n, Index F) {
  for (Index i = 0; i < n; ++i) {
    float *o = dst + i * F;
    if (mask && !mask[i]) { memset(o, 0, (size_t)F * sizeof(float)); continue; }
    Index id = ids[i];
    if (id < 0) id += n_rows;
    if (id < 0 || id >= n_rows) return ORC_EINVAL;
    memcpy(o, table + id * F, (size_t)F * sizeof(float));
  }
  return ORC_OK;
}

/* ------------------------------------------------------------------ sampler
 * Layered neighbour sampling, stated sequentially.  The reference has no
 * sampler of its own (batches come from the external cxgnndl loader,
 * hiscache/history_trainer.py:19,26), so this restates the library's published
 * rule, not reference code: PARITY UNPINNED against cxgnndl; the batch layout
 * is the one hiscache/history_model.py:120-153 reads.  Pinned by the tests
 * through what the rule implies: perm is a bijection of [0, d) (brute force),
 * rows hold min(d, fanout) distinct list positions, local ids are first-seen
 * order, and the pick frequencies are uniform (chi-square). */
uint64_t orc_mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

/* Keyed bijection of [0, d), d >= 2: 4 Feistel rounds on 2h bits (h = half of
 * the bit length of d-1, rounded up), cycle walking back into [0, d). */
uint64_t orc_sample_perm(uint64_t j, uint64_t d, uint64_t key) {
  int bits = 0;
  for (uint64_t t = d - 1; t; t >>= 1) ++bits;
  int h = (bits + 1) / 2;
  uint64_t mask = (1ull << h) - 1ull;
  uint64_t x = j;
  do {
    uint64_t l = x >> h, r = x & mask;
    for (int round = 0; round < 4; ++round) {
      uint64_t f = orc_mix64(r ^ key ^ ((uint64_t)round << 56)) & mask;
      uint64_t t = l ^ f;
      l = r;
      r = t;
    }
    x = (l << h) | r;
  } while (x >= d);
  return x;
}

int orc_sample_layers(const Index *indptr, const Index *indices, Index num_nodes,
                      const Index *seeds, Index n_seed, const Index *fanout, int L,
                      uint64_t rng_seed, Index *ptr, Index *idx, Index *sub_to_full,
                      Index *counts) {
  Index *loc = (Index *)malloc((size_t)num_nodes * sizeof(Index));
  if (!loc) return ORC_EINVAL;
  for (Index i = 0; i < num_nodes; ++i) loc[i] = -1;
  for (Index i = 0; i < n_seed; ++i) {
    sub_to_full[i] = seeds[i];
    loc[seeds[i]] = i;
  }
  Index lo = 0, hi = n_seed, E = 0;
  ptr[0] = 0;
  counts[0] = n_seed;
  for (int k = 0; k < L; ++k) {
    Index next = hi;
    uint64_t hop_key = orc_mix64(rng_seed + (uint64_t)k);
    for (Index u = lo; u < hi; ++u) {
      Index f = sub_to_full[u];
      Index first = indptr[f];
      Index d = indptr[f + 1] - first;
      Index c = d < fanout[k] ? d : fanout[k];
      uint64_t key = orc_mix64(hop_key ^ (uint64_t)f);
      for (Index j = 0; j < c; ++j) {
        Index pos = d > fanout[k] ? (Index)orc_sample_perm((uint64_t)j, (uint64_t)d, key) : j;
        Index v = indices[first + pos];
        if (loc[v] < 0) {
          loc[v] = next;
          sub_to_full[next++] = v;
        }
        idx[E++] = loc[v];
      }
      ptr[u + 1] = E;
    }
    lo = hi;
    hi = next;
    counts[k + 1] = hi;
    counts[L + 1 + k] = E;
  }
  free(loc);
  return ORC_OK;
}

