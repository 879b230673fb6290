/*
 * hc_cpu_mt.c -- TEST INFRASTRUCTURE ONLY: the CPU baseline leg of the benchmark.
 *
 * The reference has no CPU implementation of its kernels
 * (src/cpp/src/history_aggr.cu is CUDA only); this is what a CPU port of the
 * aggregation step looks like when it is written for all host cores: OpenMP over
 * destination rows in the forward (history_aggr.cu:7-40 with the per-source
 * substitution of the build), over source ranges in the transposed view, and over
 * sources in the backward (history_aggr.cu:127-168 as a gather, no atomics).
 * Rows and sources are independent and every sum keeps the order of hc_oracle.c,
 * so the results are bit-identical to the single-threaded statement whatever the
 * thread count; the tests check exactly that.
 */
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef int64_t Index;

#define ORC_OK 0
#define ORC_EINVAL 1

int mt_num_threads(void) { return omp_get_max_threads(); }

static void add_rows(const Index *idx, const float *feat, const Index *hmap_src, const float *hist, Index F,
                     Index hsize, Index b, Index e, float *o) {
  for (Index j = b; j < e; ++j) {
    const Index s = idx[j];
    const float *x = (hmap_src && hmap_src[s] != -1) ? hist + hmap_src[s] * hsize : feat + s * F;
    for (Index c = 0; c < F; ++c) o[c] += x[c];
  }
}

/* Mean forward with per-source substitution; rows above split_above edges as four quarters combined
 * left to right (the same rule as orc_fwd_mean_src). */
int mt_fwd_mean_src(const Index *ptr, const Index *idx, const float *feat, const Index *hmap_src,
                    const float *hist, float *vout, Index R, Index F, Index hsize, Index split_above) {
  int bad = 0;
#pragma omp parallel
  {
    float *part = (float *)malloc((size_t)F * sizeof(float));
    if (!part) {
#pragma omp atomic write
      bad = 1;
    }
#pragma omp for schedule(dynamic, 256)
    for (Index row = 0; row < R; ++row) {
      if (!part) continue;
      float *o = vout + row * F;
      memset(o, 0, (size_t)F * sizeof(float));
      const Index b = ptr[row], e = ptr[row + 1];
      const Index n = e - b;
      if (n == 0) continue;
      if (split_above > 0 && n > split_above) {
        const Index q = (n + 3) / 4;
        for (int w = 0; w < 4; ++w) {
          Index sb = b + w * q, se = sb + q;
          if (sb > e) sb = e;
          if (se > e) se = e;
          if (w == 0) {
            add_rows(idx, feat, hmap_src, hist, F, hsize, sb, se, o);
          } else {
            memset(part, 0, (size_t)F * sizeof(float));
            add_rows(idx, feat, hmap_src, hist, F, hsize, sb, se, part);
            for (Index c = 0; c < F; ++c) o[c] += part[c];
          }
        }
      } else {
        add_rows(idx, feat, hmap_src, hist, F, hsize, b, e, o);
      }
      const float d = (float)(int)n;
      for (Index c = 0; c < F; ++c) o[c] = o[c] / d;
    }
    free(part);
  }
  return bad ? ORC_EINVAL : ORC_OK;
}

/* Transposed view (stable by destination row): ptrT[n_src+1], rowT[E].  Every thread owns a range of
 * sources and walks all edges twice (count, place); no atomics, the order inside a source is the walk
 * order, i.e. ascending (row, edge). */
int mt_build_transpose(const Index *ptr, const Index *idx, Index R, Index n_src, Index *ptrT, int32_t *rowT) {
  const Index E = ptr[R];
  for (Index j = 0; j < E; ++j)
    if (idx[j] < 0 || idx[j] >= n_src) return ORC_EINVAL;
  memset(ptrT, 0, (size_t)(n_src + 1) * sizeof(Index));
  Index *cur = (Index *)malloc((size_t)(n_src + 1) * sizeof(Index));
  if (!cur) return ORC_EINVAL;
#pragma omp parallel
  {
    const int T = omp_get_num_threads(), t = omp_get_thread_num();
    const Index lo = n_src * t / T, hi = n_src * (t + 1) / T;
    for (Index j = 0; j < E; ++j) {
      const Index s = idx[j];
      if (s >= lo && s < hi) ptrT[s + 1]++;
    }
#pragma omp barrier
#pragma omp single
    {
      for (Index s = 0; s < n_src; ++s) ptrT[s + 1] += ptrT[s];
      memcpy(cur, ptrT, (size_t)(n_src + 1) * sizeof(Index));
    }
    for (Index row = 0; row < R; ++row) {
      for (Index j = ptr[row]; j < ptr[row + 1]; ++j) {
        const Index s = idx[j];
        if (s >= lo && s < hi) rowT[cur[s]++] = (int32_t)row;
      }
    }
  }
  free(cur);
  return ORC_OK;
}

/* Mean backward as a gather over the transposed view: grads_out[s] = sum over incoming edges, ascending
 * destination row, of g[row] / deg(row); a source with more than `chunk` incoming edges (chunk > 0) is
 * summed in chunks of `chunk` edges, each from zero, combined left to right (orc_bwd_mean_row's rule). */
int mt_bwd_mean(const Index *ptr, const Index *ptrT, const int32_t *rowT, const float *g, float *grads_out,
                Index n_src, Index F, Index chunk) {
  int bad = 0;
#pragma omp parallel
  {
    float *part = (float *)malloc((size_t)F * sizeof(float));
    if (!part) {
#pragma omp atomic write
      bad = 1;
    }
#pragma omp for schedule(dynamic, 1024)
    for (Index s = 0; s < n_src; ++s) {
      if (!part) continue;
      float *o = grads_out + s * F;
      memset(o, 0, (size_t)F * sizeof(float));
      const Index b = ptrT[s], e = ptrT[s + 1];
      if (chunk > 0 && e - b > chunk) {
        for (Index cb = b; cb < e; cb += chunk) {
          const Index ce = cb + chunk < e ? cb + chunk : e;
          memset(part, 0, (size_t)F * sizeof(float));
          for (Index k = cb; k < ce; ++k) {
            const Index row = rowT[k];
            const float d = (float)(int)(ptr[row + 1] - ptr[row]);
            const float *gr = g + row * F;
            for (Index c = 0; c < F; ++c) part[c] += gr[c] / d;
          }
          for (Index c = 0; c < F; ++c) o[c] += part[c];
        }
      } else {
        for (Index k = b; k < e; ++k) {
          const Index row = rowT[k];
          const float d = (float)(int)(ptr[row + 1] - ptr[row]);
          const float *gr = g + row * F;
          for (Index c = 0; c < F; ++c) o[c] += gr[c] / d;
        }
      }
    }
    free(part);
  }
  return bad ? ORC_EINVAL : ORC_OK;
}
