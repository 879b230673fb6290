// Helpers shared by the two builders of the transposed view (transpose.hip: counting sort of small
// blocks and the library-sort fallback; view_sort.hip: the two-level bucket sort of large blocks).
#pragma once

#include "hc_common.h"

// largest r in [lo, hi] with ptr[r] <= e (ptr[lo] <= e is the caller's business)
template <typename P>
__device__ __forceinline__ int64_t tr_row_of(P ptr, int64_t lo, int64_t hi, int64_t e) {
  while (lo < hi) {
    const int64_t mid = (lo + hi + 1) >> 1;
    if (ptr[mid] <= e) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

// The same search by a whole wave, 64 probes per memory round trip (three round trips for 2^18 rows
// instead of eighteen): largest r in [0, R] with ptr[r] <= e, assuming ptr[0] <= e.  Every lane
// returns the result.
__device__ __forceinline__ int64_t tr_row_of_wave(const int64_t *__restrict__ ptr, int64_t R, int64_t e,
                                                  int lane) {
  int64_t lo = 0, hi = R;   // ptr[lo] <= e; the answer lies in [lo, hi]
  while (hi > lo) {
    const int64_t step = (hi - lo + HC_WAVE - 1) / HC_WAVE;
    int64_t p = lo + (int64_t)(lane + 1) * step;
    if (p > hi) p = hi;
    const unsigned long long ok = __ballot(ptr[p] <= e);   // a prefix of the lanes: ptr does not decrease
    const int k = __popcll(ok);
    int64_t nlo = lo + (int64_t)k * step;                  // the last probe that held (lo itself when k == 0)
    if (nlo > hi) nlo = hi;
    int64_t nhi = hi;
    if (k < HC_WAVE) {
      nhi = lo + (int64_t)(k + 1) * step;                  // the first probe that failed, minus one
      if (nhi > hi) nhi = hi;
      nhi -= 1;
    }
    lo = nlo;
    hi = nhi < nlo ? nlo : nhi;
  }
  return lo;
}

// ---- the bucket sort of large blocks (view_sort.hip) -------------------------------------------
// True when the bucket sort covers a block of E edge slots and n_src sources.
bool vs_supported(int64_t E, int64_t n_src);
// Workspace of the bucket sort (0 when unsupported); 256-byte aligned base expected.
size_t vs_workspace_bytes(int64_t E, int64_t n_src);
// Enqueues the bucket sort.  hmap_row / hmap_src are nullable: rows with hmap_row[r] != -1 and sources with
// hmap_src[s] != -1 are left out.  Returns an hc_status.
int vs_launch(const int64_t *ptr, const int64_t *idx, const int64_t *hmap_row, const int64_t *hmap_src,
              int64_t R, int64_t E, int64_t n_src, int64_t *ptrT, int32_t *rowT, int32_t *edgeT, char *ws,
              size_t ws_bytes, hipStream_t st);
