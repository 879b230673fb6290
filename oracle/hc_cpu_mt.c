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
/* hmap_src (nullable, n_src entries): edges whose source has hmap_src[s] != -1 are left out (a source that
 * was substituted by a history-table row in the forward pass passes no gradient to its feature row). */
int mt_build_transpose(const Index *ptr, const Index *idx, Index R, Index n_src, Index *ptrT, int32_t *rowT,
                       const Index *hmap_src) {
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
      if (s >= lo && s < hi && (!hmap_src || hmap_src[s] == -1)) ptrT[s + 1]++;
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
        if (s >= lo && s < hi && (!hmap_src || hmap_src[s] == -1)) rowT[cur[s]++] = (int32_t)row;
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

/* ---------------------------------------------------------------------------------------------- */
/* Fused admission (orc_grad_check's rule) for all host cores: scores and predicate per row in
 * parallel, ring slots in row order from a two-level prefix sum of the mask, then previous owners
 * un-mapped, then the new owners written and the rows copied (fp32 -> fp16, round to nearest even).
 * Un-mapping before mapping gives the sequential result as long as no slot is handed out twice in
 * one call; a call that admits more rows than the table holds is refused (ORC_EINVAL) and left to
 * the sequential statement.  Scores use the 64-lane order of orc_row_score.                         */
/* ---------------------------------------------------------------------------------------------- */
#include <math.h>

static uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static uint16_t f32_to_f16(float f) {
  const uint32_t x = f2u(f), sign = (x >> 16) & 0x8000u, mag = x & 0x7fffffffu;
  if (mag >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (mag > 0x7f800000u ? 0x200u | ((mag >> 13) & 0x3ffu) : 0));
  if (mag >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);          /* rounds to infinity */
  if (mag < 0x33000001u) return (uint16_t)sign;                        /* rounds to zero */
  int32_t e = (int32_t)(mag >> 23) - 127;
  uint32_t m = (mag & 0x7fffffu) | 0x800000u;
  int shift = e < -14 ? 13 + (-14 - e) : 13;
  uint32_t half = m >> shift, rem = m & ((1u << shift) - 1), mid = 1u << (shift - 1);
  if (rem > mid || (rem == mid && (half & 1))) half++;
  if (e < -14) return (uint16_t)(sign | half);                         /* subnormal (may carry into normal) */
  return (uint16_t)(sign | ((uint32_t)((e + 15) << 10) + (half - 0x400u)));
}

uint16_t mt_f32_to_f16(float f) { return f32_to_f16(f); }

/* acc[l] folds the elements of lane l in increasing index (fma), the 64 partials meet in a butterfly with
 * partner distance 32 ... 1: orc_row_score's order, laid out so that a 256-element block is one pass. */
static inline __attribute__((always_inline)) float row_score_l2(const float *row, Index F) {
  float acc[64];
  for (int l = 0; l < 64; ++l) acc[l] = 0.0f;
  Index e = 0;
  for (; e + 256 <= F; e += 256) {
    for (int l = 0; l < 64; ++l) {
      const float *x = row + e + 4 * l;
      float a = acc[l];
      a = fmaf(x[0], x[0], a);
      a = fmaf(x[1], x[1], a);
      a = fmaf(x[2], x[2], a);
      a = fmaf(x[3], x[3], a);
      acc[l] = a;
    }
  }
  for (; e < F; ++e) {
    const int l = (int)((e / 4) % 64);
    acc[l] = fmaf(row[e], row[e], acc[l]);
  }
  for (int d = 32; d >= 1; d >>= 1) {
    float nxt[64];
    for (int l = 0; l < 64; ++l) nxt[l] = acc[l] + acc[l ^ d];
    memcpy(acc, nxt, sizeof(acc));
  }
  return sqrtf(acc[0]);
}

/* Two builds of the two hot loops: plain C for any x86-64, and one for cores with FMA and F16C (a fused
 * multiply-add instruction instead of the library call, eight conversions per instruction; both round
 * exactly like the portable code).  Chosen once per call from the CPU's feature bits. */
#include <immintrin.h>

static void score_rows_any(const float *grad, Index lo, Index hi, Index F, float *score) {
  for (Index r = lo; r < hi; ++r) score[r] = row_score_l2(grad + r * F, F);
}
__attribute__((target("avx2,fma"))) static void score_rows_fma(const float *grad, Index lo, Index hi, Index F,
                                                               float *score) {
  for (Index r = lo; r < hi; ++r) score[r] = row_score_l2(grad + r * F, F);
}
static void convert_row_any(const float *src, uint16_t *d, Index F) {
  for (Index c = 0; c < F; ++c) d[c] = f32_to_f16(src[c]);
}
__attribute__((target("avx2,f16c"))) static void convert_row_f16c(const float *src, uint16_t *d, Index F) {
  Index c = 0;
  for (; c + 8 <= F; c += 8)
    _mm_storeu_si128((__m128i *)(d + c),
                     _mm256_cvtps_ph(_mm256_loadu_ps(src + c), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
  for (; c < F; ++c) d[c] = f32_to_f16(src[c]);
}
void mt_convert_row(const float *src, uint16_t *d, Index F, int hw) {
  if (hw && __builtin_cpu_supports("f16c") && __builtin_cpu_supports("avx2")) convert_row_f16c(src, d, F);
  else convert_row_any(src, d, F);
}
void mt_score_rows(const float *grad, Index M, Index F, float *score, int hw) {
  if (hw && __builtin_cpu_supports("fma") && __builtin_cpu_supports("avx2")) score_rows_fma(grad, 0, M, F, score);
  else score_rows_any(grad, 0, M, F, score);
}

int mt_grad_check_f16(const float *grad, const float *emb, const Index *slot, const int32_t *age,
                      const Index *sub_to_full, float thres, int32_t age_limit, uint8_t *mask_out,
                      float *score_out, uint16_t *table, Index capacity, Index *full2slot, Index *slot2full,
                      Index *checkin, Index *header, Index glb_iter, Index M, Index F, Index *rank /* [M] scratch */) {
  const int T = omp_get_max_threads();
  Index *part = (Index *)calloc((size_t)T + 1, sizeof(Index));
  if (!part) return ORC_EINVAL;
  int bad = 0;
  const Index h0 = *header;
  const int hw_fma = __builtin_cpu_supports("fma") && __builtin_cpu_supports("avx2");
  const int hw_f16c = __builtin_cpu_supports("f16c") && __builtin_cpu_supports("avx2");
#pragma omp parallel num_threads(T)
  {
    const int t = omp_get_thread_num();
    const Index lo = M * t / T, hi = M * (t + 1) / T;
    Index n = 0;
    if (hw_fma) score_rows_fma(grad, lo, hi, F, score_out);
    else score_rows_any(grad, lo, hi, F, score_out);
    for (Index r = lo; r < hi; ++r) {
      const float sc = score_out[r];
      const int admit = (sc < thres) && (slot[r] == -1 || (age && age[r] >= age_limit));
      mask_out[r] = (uint8_t)admit;
      rank[r] = n;
      n += admit;
    }
    part[t + 1] = n;
#pragma omp barrier
#pragma omp single
    {
      for (int k = 0; k < T; ++k) part[k + 1] += part[k];
      if (part[T] > capacity) bad = 1;
      else *header = (h0 + part[T]) % capacity;
    }
    if (!bad) {
      for (Index r = lo; r < hi; ++r) {                 /* un-map the previous owners of the slots taken */
        if (!mask_out[r]) continue;
        const Index s = (h0 + part[t] + rank[r]) % capacity;
        rank[r] = s;
        const Index old = slot2full[s];
        /* two slots can name the same previous owner (a stale entry); at most one of them matches */
        if (old != -1 && __atomic_load_n(&full2slot[old], __ATOMIC_RELAXED) == s)
          __atomic_store_n(&full2slot[old], (Index)-1, __ATOMIC_RELAXED);
      }
#pragma omp barrier
      for (Index r = lo; r < hi; ++r) {
        if (!mask_out[r]) continue;
        const Index s = rank[r];
        full2slot[sub_to_full[r]] = s;
        slot2full[s] = sub_to_full[r];
        if (checkin) checkin[s] = glb_iter;
        if (hw_f16c) convert_row_f16c(emb + r * F, table + s * F, F);
        else convert_row_any(emb + r * F, table + s * F, F);
      }
    }
  }
  free(part);
  return bad ? ORC_EINVAL : ORC_OK;
}
