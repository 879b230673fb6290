// History-aware aggregation, backward, as a gather over the transposed view.
//
// Every SOURCE row s is summed by exactly one wavefront, in ascending
// destination-row order: g[r,:]/deg(r) (mean) or g[r,:]*edge_value[j]
// (weighted) over the edges that point at s.  No float atomics: each output
// element has one writer and a fixed summation order, the same order a
// sequential walk of the CSR block in row/edge order produces.
//
// Semantics follow the reference kernels gen_bwd_history_grad_v2*
// (/root/reference/src/cpp/src/history_aggr.cu:127-397): history rows route
// g[r,:] to grads_history[r,:] undivided (:144-149) and push nothing to their
// neighbours; the other rows push g/deg (:140-142,161-166) or g*edge_value
// (:209); edge_grad[j] = <g[r,:], vin[idx[j],:]> (:258-267).
#include "hc_common.h"

namespace {

// ---------------------------------------------------------------------------------------
// Fast path: mean, fp32 upstream gradient, F == 64 * VEC * CHUNKS.
//
// A wave owns BWD_SRC_PER_WAVE consecutive source rows.  Their incoming edges are one
// contiguous span of the transposed arrays, so the wave streams that span 64 edges at a time
// (one coalesced load of destination rows, one gather of their degrees) and walks it with a
// wave-uniform cursor: when the cursor passes the end of a source's segment the accumulator
// is stored (zeros for sources without edges) and reset.  Up to UNROLL gradient rows are in
// flight before the first add; adds stay in transposed-edge order.  Compared with one wave
// per source this amortises the dependent loads (segment bounds -> rows -> degrees) over
// many sources, which matters when most sources have only one or two incoming edges.
// Blocks [0, src_blocks) own source rows; blocks beyond own rows of grad_hbuf.
// ---------------------------------------------------------------------------------------
constexpr int BWD_SRC_PER_WAVE = 32;
constexpr int BWD_XCD_CHUNK = 64;  // consecutive blocks (8192 sources) that share an XCD
// With a workspace, a source with more than BWD_CHUNK incoming edges ("hub") is summed in chunks
// of BWD_CHUNK edges by independent waves; the chunk sums are then combined left to right.
constexpr int BWD_CHUNK = 512;
constexpr int W_NONE = 0, W_EDGE = 1, W_EDGE_HEAD = 2;

// Hubs need no list.  The transposed edge positions are cut into windows of BWD_CHUNK positions and
// one wave looks at each window.  A hub's chunks start at ptrT[s] + k * BWD_CHUNK, so a window holds at
// most two chunk starts: one of the hub that covers the window's first position from before (found by
// a binary search over ptrT) and the first chunk of a hub that starts inside the window (the last
// source that starts before the window's end, because a hub is longer than a window).  The wave sums
// those chunks into partial[2 * window] and partial[2 * window + 1].  A second launch, again one wave
// per window, combines the chunk sums of the hub that starts in its window, left to right.
inline int64_t bwd_windows(int64_t E) { return (E + BWD_CHUNK - 1) / BWD_CHUNK; }
inline size_t bwd_partial_sums_bytes(int64_t E, int64_t F) {
  return hc_align_up((size_t)(2 * bwd_windows(E)) * (size_t)F * sizeof(float), 256);
}
// the chunk sums, then one word per window: the hub that starts in the window, or -1
inline size_t bwd_partial_bytes(int64_t E, int64_t F) {
  return bwd_partial_sums_bytes(E, F) + hc_align_up((size_t)bwd_windows(E) * sizeof(int64_t), 256);
}

// last s in [0, n_src) with ptrT[s] <= target (ptrT[0] == 0 <= target), found by the whole wave: the lanes
// probe 64 evenly spaced entries per step, so the range shrinks 64-fold per round trip to memory (three
// dependent loads for 200 000 sources where a bisection takes eighteen).  Every lane returns the result;
// `target` must be the same in all lanes.
__device__ __forceinline__ int64_t bwd_last_source_at(const int64_t *__restrict__ ptrT, int64_t n_src,
                                                      int64_t target, int lane) {
  int64_t lo = 0, hi = n_src - 1;   // ptrT[lo] <= target, the answer lies in [lo, hi]
  while (hi - lo >= HC_WAVE) {
    const int64_t step = (hi - lo) / HC_WAVE + 1;
    const int64_t probe = lo + step * (lane + 1);
    const bool le = probe <= hi && ptrT[probe] <= target;     // true in a prefix of the lanes: ptrT does not decrease
    const int c = __popcll(__ballot(le));
    const int64_t next = lo + step * (c + 1) - 1;             // the first probe that failed, less one
    lo += step * c;
    hi = next < hi ? next : hi;
  }
  const int64_t probe = lo + 1 + lane;
  const bool le = probe <= hi && ptrT[probe] <= target;
  return lo + __popcll(__ballot(le));
}

// MASKED: the view covers the whole mini-batch CSR; transposed edges whose destination row lies outside
// the first R rows, or took its history row (hmap[row] != -1), are stepped over.
template <bool MASKED>
__device__ __forceinline__ int bwd_live_row(int row, const int64_t *__restrict__ hmap, int64_t R) {
  if constexpr (MASKED) {
    if (row >= R) return -1;
    if (hmap != nullptr && hmap[row] != -1) return -1;
  }
  return row;
}

// Sum of g[r,:]/deg(r) over transposed edges [begin, end), added to acc in order by the calling wave.
template <int VEC, int CHUNKS, int UNROLL, bool MASKED>
__device__ __forceinline__ void bwd_accumulate(const int64_t *__restrict__ ptr, const int32_t *__restrict__ rowT,
                                               const float *__restrict__ g, const int64_t *__restrict__ hmap,
                                               int64_t R, int64_t begin, int64_t end, int lane,
                                               float (&acc)[CHUNKS][VEC]) {
  constexpr int F = HC_WAVE * VEC * CHUNKS;
  for (int64_t base = begin; base < end; base += HC_WAVE) {
    const int64_t left = end - base;
    const int n = left < HC_WAVE ? (int)left : HC_WAVE;
    int my_row = 0;
    float my_deg = 1.0f;
    if (lane < n) {
      my_row = bwd_live_row<MASKED>(rowT[base + lane], hmap, R);
      if (!MASKED || my_row >= 0) my_deg = (float)(int)(ptr[my_row + 1] - ptr[my_row]);
      // a row that the layer's own offsets leave empty (a batch padded for a recorded iteration keeps the rows
      // behind a layer's real ones empty, while the batch's shared view still lists their edges) is stepped over
      if (MASKED && my_row >= 0 && my_deg == 0.0f) my_row = -1;
    }
    // the staged edges that count, lowest position first (all of them without a mask)
    unsigned long long todo = MASKED ? __ballot(lane < n && my_row >= 0)
                                     : (n == HC_WAVE ? ~0ull : ((1ull << n) - 1ull));
    while (todo != 0ull) {
      float v[UNROLL][CHUNKS][VEC];
      float d[UNROLL];
      bool on[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        d[u] = 1.0f;
        on[u] = todo != 0ull;
        if (on[u]) {
          const int j = __builtin_ctzll(todo);
          todo &= todo - 1ull;
          const int r = __builtin_amdgcn_readlane(my_row, j);
          d[u] = hc_readlane_f(my_deg, j);
          const float *p = g + (int64_t)r * F + lane * VEC;
#pragma unroll
          for (int k = 0; k < CHUNKS; ++k) hc_vec<float, VEC>::load(p + k * HC_WAVE * VEC, v[u][k]);
        }
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if (on[u]) {
#pragma unroll
          for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[k][i] += v[u][k][i] / d[u];
        }
      }
    }
  }
}

// The chunk sums of the window owned by the calling wave (see the note above bwd_windows).
template <int VEC, int CHUNKS, int UNROLL, bool MASKED>
__device__ __forceinline__ void bwd_window_partials(const int64_t *__restrict__ ptr,
                                                    const int64_t *__restrict__ ptrT,
                                                    const int32_t *__restrict__ rowT,
                                                    const float *__restrict__ g,
                                                    const int64_t *__restrict__ hmap, int64_t R,
                                                    float *__restrict__ partial,
                                                    int64_t *__restrict__ hub_of,
                                                    int64_t n_src, int64_t window, int lane) {
  constexpr int F = HC_WAVE * VEC * CHUNKS;
  const int64_t wstart = window * BWD_CHUNK;
  const int64_t wend = wstart + BWD_CHUNK;
  // hub_of[window]: the hub that starts in this window (bwd_hub_final combines its chunk sums), else -1;
  // written for every window at every call, so that the final pass needs no search of its own
  int64_t hub = -1;
  if (wstart >= ptrT[n_src]) {
    if (lane == 0) hub_of[window] = hub;
    return;
  }
  // the source that covers the window's first position, and the last source that starts inside the window
  const int64_t found[2] = {hc_uniform64(bwd_last_source_at(ptrT, n_src, wstart, lane)),
                            hc_uniform64(bwd_last_source_at(ptrT, n_src, wend - 1, lane))};
  for (int which = 0; which < 2; ++which) {
    const int64_t s = found[which];
    const int64_t seg_b = ptrT[s];
    const int64_t seg_e = ptrT[s + 1];
    if (seg_e - seg_b <= BWD_CHUNK) continue;
    int64_t begin;
    if (which == 0) {
      if (seg_b >= wstart) continue;                 // it starts inside the window: handled as `which == 1`
      begin = seg_b + (wstart - seg_b + BWD_CHUNK - 1) / BWD_CHUNK * BWD_CHUNK;
      if (begin >= wend || begin >= seg_e) continue;
    } else {
      if (seg_b < wstart) continue;
      begin = seg_b;
      hub = s;
    }
    const int64_t end = begin + BWD_CHUNK < seg_e ? begin + BWD_CHUNK : seg_e;
    float acc[CHUNKS][VEC];
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[k][i] = 0.0f;
    bwd_accumulate<VEC, CHUNKS, UNROLL, MASKED>(ptr, rowT, g, hmap, R, begin, end, lane, acc);
    float *__restrict__ o = partial + (2 * window + which) * F + lane * VEC;
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k) hc_vec<float, VEC>::store(o + k * HC_WAVE * VEC, acc[k]);
  }
  if (lane == 0) hub_of[window] = hub;
}

// One wave per window: if a hub starts in the window, its chunk sums are combined left to right into
// its output row.
template <int VEC, int CHUNKS>
__global__ __launch_bounds__(HC_BLOCK) void bwd_hub_final(const int64_t *__restrict__ ptrT,
                                                           const float *__restrict__ partial,
                                                           const int64_t *__restrict__ hub_of,
                                                           float *__restrict__ grad_vin, int64_t n_src,
                                                           int64_t windows) {
  constexpr int F = HC_WAVE * VEC * CHUNKS;
  const int lane = hc_lane();
  const int64_t window = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (window >= windows) return;
  const int64_t s = hc_uniform64(hub_of[window]);      // left by the window's wave of bwd_mean_fast
  if (s < 0 || s >= n_src) return;
  const int64_t seg_b = ptrT[s];
  const int64_t len = ptrT[s + 1] - seg_b;
  const int nch = (int)((len + BWD_CHUNK - 1) / BWD_CHUNK);
  float acc[CHUNKS][VEC];
  const float *__restrict__ p0 = partial + (2 * window + 1) * F + lane * VEC;
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) hc_vec<float, VEC>::load(p0 + k * HC_WAVE * VEC, acc[k]);
  for (int c = 1; c < nch; ++c) {
    const int64_t w = (seg_b + (int64_t)c * BWD_CHUNK) / BWD_CHUNK;
    const float *__restrict__ p = partial + (2 * w) * F + lane * VEC;
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k) {
      float v[VEC];
      hc_vec<float, VEC>::load(p + k * HC_WAVE * VEC, v);
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[k][i] += v[i];
    }
  }
  float *__restrict__ o = grad_vin + s * F + lane * VEC;
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) hc_vec<float, VEC>::store(o + k * HC_WAVE * VEC, acc[k]);
}

// WMODE W_EDGE: every transposed edge contributes g[row] * edge_value[edge] (product rounded, then
// added) instead of g[row] / deg(row); edgeT gives the edge slot of a transposed edge.
// WMODE W_EDGE_HEAD: a row is n_head heads side by side and the weight is edge_value[edge, head]; a
// lane's VEC elements of a chunk lie inside one head, whose weight the lane loads itself.  (grad_hbuf
// of such blocks is written by bwd_hist_generic.)
// MASKED (plain mean only): see bwd_live_row.  Chunks of a hub are then runs of BWD_CHUNK positions of the
// whole-batch view, of which only the live edges are added.
template <int VEC, int CHUNKS, int UNROLL, int WMODE, bool MASKED>
__global__ __launch_bounds__(HC_BLOCK) void bwd_mean_fast(
    const int64_t *__restrict__ ptr, const int64_t *__restrict__ ptrT, const int32_t *__restrict__ rowT,
    const int32_t *__restrict__ edgeT, const float *__restrict__ ev, int n_head, const float *__restrict__ g,
    const int64_t *__restrict__ hmap, float *__restrict__ grad_vin, float *__restrict__ grad_hbuf,
    int64_t hsize, int64_t R, int64_t n_src, int64_t src_blocks, int64_t hist_blocks, int64_t hub_thres,
    float *__restrict__ partial, int64_t *__restrict__ hub_of, int64_t windows) {
  constexpr int F = HC_WAVE * VEC * CHUNKS;
  constexpr bool WEIGHTED = WMODE != W_NONE;
  constexpr int S = BWD_SRC_PER_WAVE;
  const int lane = hc_lane();
  const int wave = hc_wave_in_block();
  if ((int64_t)blockIdx.x >= src_blocks + hist_blocks) {
    // blocks behind the source and history blocks: the hubs' chunk sums, one window per wave
    if constexpr (WMODE == W_NONE) {
      const int64_t window = ((int64_t)blockIdx.x - src_blocks - hist_blocks) * HC_WAVES_PER_BLOCK + wave;
      if (window < windows)
        bwd_window_partials<VEC, CHUNKS, UNROLL, MASKED>(ptr, ptrT, rowT, g, hmap, R, partial, hub_of, n_src, window,
                                                         lane);
    }
    return;
  }
  if ((int64_t)blockIdx.x >= src_blocks) {
    // grad_hbuf rows: copy g for history rows, zero otherwise
    const int64_t row = ((int64_t)blockIdx.x - src_blocks) * HC_WAVES_PER_BLOCK + wave;
    if (row >= R) return;
    const bool hit = hmap[row] != -1;
    float *__restrict__ d = grad_hbuf + row * hsize;
    const float *__restrict__ s = g + row * F;
    if (hsize == F && (reinterpret_cast<uintptr_t>(grad_hbuf) % 16) == 0) {
      // the usual shape: one 16-byte store per lane and chunk (F is a multiple of 256 bytes here)
      float *__restrict__ dv = d + lane * VEC;
      const float *__restrict__ sv = s + lane * VEC;
#pragma unroll
      for (int k = 0; k < CHUNKS; ++k) {
        float v[VEC];
        if (hit) {
          hc_vec<float, VEC>::load(sv + k * HC_WAVE * VEC, v);
        } else {
#pragma unroll
          for (int i = 0; i < VEC; ++i) v[i] = 0.0f;
        }
        hc_vec<float, VEC>::store_nt(dv + k * HC_WAVE * VEC, v);
      }
      return;
    }
    for (int64_t c = lane; c < hsize; c += HC_WAVE) d[c] = (hit && c < F) ? s[c] : 0.0f;
    return;
  }
  const int64_t s0 = (hc_xcd_block<BWD_XCD_CHUNK>((int64_t)blockIdx.x, src_blocks) * HC_WAVES_PER_BLOCK + wave) * S;
  if (s0 >= n_src) return;
  const int64_t rest = n_src - s0;
  const int ns = rest < S ? (int)rest : S;
  // lane l holds the segment bound ptrT[s0 + l], l = 0..ns
  const int64_t my_p = ptrT[s0 + (lane < ns ? lane : ns)];
  const int64_t my_p1 = ptrT[s0 + (lane + 1 < ns ? lane + 1 : ns)];
  const int64_t e_end = hc_readlane64(my_p, ns);
  // sources summed elsewhere (hub path): their segments are stepped over and not stored here
  const unsigned long long hub_mask =
      hub_thres > 0 ? __ballot(lane < ns && (my_p1 - my_p) > hub_thres) : 0ull;

  float acc[CHUNKS][VEC];
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[k][i] = 0.0f;
  int cur = 0;                                   // source (relative to s0) being accumulated
  int64_t cur_end = hc_readlane64(my_p, 1);      // end of its segment
  float *__restrict__ obase = grad_vin + s0 * F + lane * VEC;
  int64_t base = hc_readlane64(my_p, 0);
  int hd[CHUNKS];
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) hd[k] = WMODE == W_EDGE_HEAD ? ((k * HC_WAVE + lane) * VEC) / (F / n_head) : 0;

  while (true) {  // every branch below advances `cur` or `base`; all of it is wave-uniform
    // close the sources whose segment ends at or before `base` (zeros for sources without edges)
    while (cur < ns && base >= cur_end) {
      if (((hub_mask >> cur) & 1ull) == 0ull) {
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) hc_vec<float, VEC>::store_nt(obase + (int64_t)cur * F + k * HC_WAVE * VEC, acc[k]);
      }
#pragma unroll
      for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[k][i] = 0.0f;
      ++cur;
      cur_end = hc_readlane64(my_p, cur + 1 <= ns ? cur + 1 : ns);
    }
    if (cur >= ns) break;
    if ((hub_mask >> cur) & 1ull) {  // step over a hub's segment
      base = cur_end;
      continue;
    }
    // stage up to 64 edges, stopping in front of the next hub's segment
    const unsigned long long ahead = hub_mask >> cur;
    const int nh = ahead != 0ull ? cur + __builtin_ctzll(ahead) : ns;
    const int64_t stop = hc_readlane64(my_p, nh);
    const int64_t left = stop - base;
    const int n = left < HC_WAVE ? (int)left : HC_WAVE;
    int my_row = 0;
    int my_edge = 0;
    float my_deg = 1.0f;
    if (lane < n) {
      my_row = bwd_live_row<MASKED>(rowT[base + lane], hmap, R);
      if constexpr (WMODE == W_EDGE_HEAD) my_edge = edgeT[base + lane];
      else if constexpr (WMODE == W_EDGE) my_deg = ev[edgeT[base + lane]];   // the weight takes the divisor's place
      else if (!MASKED || my_row >= 0) my_deg = (float)(int)(ptr[my_row + 1] - ptr[my_row]);
      // a row that the layer's own offsets leave empty is stepped over (see bwd_accumulate)
      if (MASKED && WMODE == W_NONE && my_row >= 0 && my_deg == 0.0f) my_row = -1;
    }
    // MASKED: only the live edges of the stage are visited (lowest position first), so that UNROLL rows are
    // in flight however many edges of other layers lie between them
    unsigned long long todo = 0ull;
    if constexpr (MASKED) todo = __ballot(lane < n && my_row >= 0);
    for (int j = 0; MASKED ? todo != 0ull : j < n; j += UNROLL) {
      float v[UNROLL][CHUNKS][VEC];
      float d[UNROLL];
      bool on[UNROLL];
      int pos[UNROLL];
      float wh[WMODE == W_EDGE_HEAD ? UNROLL : 1][CHUNKS];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        d[u] = 1.0f;
        if constexpr (MASKED) {
          on[u] = todo != 0ull;
          pos[u] = on[u] ? __builtin_ctzll(todo) : 0;
          todo &= todo - 1ull;                     // 0 stays 0
        } else {
          on[u] = j + u < n;
          pos[u] = j + u;
        }
        if (on[u]) {
          const int r = __builtin_amdgcn_readlane(my_row, pos[u]);
          d[u] = hc_readlane_f(my_deg, pos[u]);
          const float *p = g + (int64_t)r * F + lane * VEC;
#pragma unroll
          for (int k = 0; k < CHUNKS; ++k) hc_vec<float, VEC>::load(p + k * HC_WAVE * VEC, v[u][k]);
          if constexpr (WMODE == W_EDGE_HEAD) {
            const int64_t e = (int64_t)__builtin_amdgcn_readlane(my_edge, pos[u]) * n_head;
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) wh[u][k] = ev[e + hd[k]];
          }
        }
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if (on[u]) {
          const int64_t e = base + pos[u];
          while (e >= cur_end) {  // close finished (possibly empty) segments; none of them is a hub
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) {
              hc_vec<float, VEC>::store_nt(obase + (int64_t)cur * F + k * HC_WAVE * VEC, acc[k]);
#pragma unroll
              for (int i = 0; i < VEC; ++i) acc[k][i] = 0.0f;
            }
            ++cur;
            cur_end = hc_readlane64(my_p, cur + 1);
          }
#pragma unroll
          for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
              if constexpr (WMODE == W_EDGE_HEAD) acc[k][i] += __fmul_rn(v[u][k][i], wh[u][k]);
              else acc[k][i] += WEIGHTED ? __fmul_rn(v[u][k][i], d[u]) : v[u][k][i] / d[u];
            }
        }
      }
    }
    base += n;
  }
  (void)e_end;
}

// ---------------------------------------------------------------------------------------
// Generic path: any F, optional weights and heads.  One wave per (source, head).
// ---------------------------------------------------------------------------------------
template <bool WEIGHTED>
__global__ __launch_bounds__(HC_BLOCK) void bwd_generic(
    const int64_t *__restrict__ ptr, const int64_t *__restrict__ ptrT, const int32_t *__restrict__ rowT,
    const int32_t *__restrict__ edgeT, const float *__restrict__ g, const float *__restrict__ ev,
    int64_t H, float *__restrict__ grad_vin, int64_t n_src, int64_t F, const int64_t *__restrict__ mask_hmap,
    int64_t mask_rows) {
  // mask_rows >= 0: the view covers the whole mini-batch CSR; edges of rows >= mask_rows and of rows with
  // mask_hmap[row] != -1 are stepped over
  constexpr int TILE_K = 4;
  const int lane = hc_lane();
  const int64_t vsrc = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (vsrc >= n_src * H) return;
  const int64_t src = vsrc / H;
  const int64_t head = vsrc - src * H;
  const int64_t begin = ptrT[src];
  const int64_t end = ptrT[src + 1];
  float *__restrict__ o = grad_vin + vsrc * F;
  for (int64_t c0 = 0; c0 < F; c0 += HC_WAVE * TILE_K) {
    float acc[TILE_K];
#pragma unroll
    for (int k = 0; k < TILE_K; ++k) acc[k] = 0.0f;
    for (int64_t base = begin; base < end; base += HC_WAVE) {
      const int64_t left = end - base;
      const int n = left < HC_WAVE ? (int)left : HC_WAVE;
      int my_row = 0;
      float my_s = 1.0f;
      if (lane < n) {
        my_row = rowT[base + lane];
        if (mask_rows >= 0 && (my_row >= mask_rows || (mask_hmap != nullptr && mask_hmap[my_row] != -1)))
          my_row = -1;
        if (my_row < 0) my_s = 1.0f;
        else if (WEIGHTED) my_s = ev[(int64_t)edgeT[base + lane] * H + head];
        else {
          my_s = (float)(int)(ptr[my_row + 1] - ptr[my_row]);
          // a row that the layer's own offsets leave empty is stepped over (see bwd_accumulate)
          if (mask_rows >= 0 && my_s == 0.0f) { my_row = -1; my_s = 1.0f; }
        }
      }
      constexpr int GEN_UNROLL = 4;  // gradient rows in flight before the first add (order kept)
      for (int j = 0; j < n; j += GEN_UNROLL) {
        float x[GEN_UNROLL][TILE_K];
        float sc[GEN_UNROLL];
        bool on[GEN_UNROLL];
#pragma unroll
        for (int u = 0; u < GEN_UNROLL; ++u) {
          sc[u] = 1.0f;
          on[u] = false;
#pragma unroll
          for (int k = 0; k < TILE_K; ++k) x[u][k] = 0.0f;
          if (j + u < n && __builtin_amdgcn_readlane(my_row, j + u) >= 0) {
            on[u] = true;
            const int r = __builtin_amdgcn_readlane(my_row, j + u);
            sc[u] = hc_readlane_f(my_s, j + u);
            const float *p = g + ((int64_t)r * H + head) * F;
#pragma unroll
            for (int k = 0; k < TILE_K; ++k) {
              const int64_t c = c0 + k * HC_WAVE + lane;
              if (c < F) x[u][k] = p[c];
            }
          }
        }
#pragma unroll
        for (int u = 0; u < GEN_UNROLL; ++u) {
          if (on[u]) {
#pragma unroll
            for (int k = 0; k < TILE_K; ++k) {
              const int64_t c = c0 + k * HC_WAVE + lane;
              if (c < F) acc[k] += WEIGHTED ? __fmul_rn(x[u][k], sc[u]) : x[u][k] / sc[u];
            }
          }
        }
      }
    }
#pragma unroll
    for (int k = 0; k < TILE_K; ++k) {
      const int64_t c = c0 + k * HC_WAVE + lane;
      if (c < F) o[c] = acc[k];
    }
  }
}

// grad_hbuf[R, hsize] for the generic path (heads summed when hsize == F, concatenated when
// hsize == F*H; columns beyond the written span are 0).
__global__ __launch_bounds__(HC_BLOCK) void bwd_hist_generic(const float *__restrict__ g,
                                                              const int64_t *__restrict__ hmap,
                                                              float *__restrict__ grad_hbuf,
                                                              int64_t hsize, int64_t R, int64_t F,
                                                              int64_t H) {
  const int lane = hc_lane();
  const int64_t row = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (row >= R) return;
  const bool hit = hmap[row] != -1;
  float *__restrict__ d = grad_hbuf + row * hsize;
  const float *__restrict__ s = g + row * H * F;
  const bool concat = (H > 1 && hsize == F * H);
  for (int64_t c = lane; c < hsize; c += HC_WAVE) {
    float v = 0.0f;
    if (hit) {
      if (concat) {
        v = s[c];
      } else if (c < F) {
        for (int64_t h = 0; h < H; ++h) v += s[h * F + c];
      }
    }
    d[c] = v;
  }
}

// edge_grad[j,h] = <g[r,h,:], vin[idx[j],h,:]> in CSR order; 0 for edges of history rows and
// for edge slots in [ptr[R], E_total).  One wave per (row, head); extra blocks clear the tail.
template <typename T>
__global__ __launch_bounds__(HC_BLOCK) void bwd_edge_grad(
    const int64_t *__restrict__ ptr, const int64_t *__restrict__ idx, const float *__restrict__ g,
    const int64_t *__restrict__ hmap, const T *__restrict__ vin, float *__restrict__ edge_grad,
    int64_t E_total, int64_t R, int64_t F, int64_t H, int64_t row_blocks) {
  const int lane = hc_lane();
  if ((int64_t)blockIdx.x >= row_blocks) {
    const int64_t nb = (int64_t)gridDim.x - row_blocks;
    const int64_t start = ptr[R] * H;
    const int64_t stop = E_total * H;
    for (int64_t i = start + ((int64_t)blockIdx.x - row_blocks) * HC_BLOCK + threadIdx.x; i < stop;
         i += nb * HC_BLOCK)
      edge_grad[i] = 0.0f;
    return;
  }
  const int64_t vrow = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (vrow >= R * H) return;
  const int64_t row = vrow / H;
  const int64_t head = vrow - row * H;
  const int64_t begin = ptr[row];
  int64_t end = ptr[row + 1];
  if (end > E_total) end = E_total;
  if (hmap != nullptr && hmap[row] != -1) {
    for (int64_t e = begin + lane; e < end; e += HC_WAVE) edge_grad[e * H + head] = 0.0f;
    return;
  }
  const float *__restrict__ gr = g + vrow * F;
  for (int64_t base = begin; base < end; base += HC_WAVE) {
    const int64_t left = end - base;
    const int n = left < HC_WAVE ? (int)left : HC_WAVE;
    int64_t my_id = 0;
    if (lane < n) my_id = idx[base + lane];
    float my_out = 0.0f;
    for (int j = 0; j < n; ++j) {
      const int64_t id = hc_readlane64(my_id, j);
      const T *__restrict__ x = vin + (id * H + head) * F;
      float part = 0.0f;
      for (int64_t c = lane; c < F; c += HC_WAVE) part = __fmaf_rn(gr[c], hc_to_f32<T>(x[c]), part);
      part = hc_wave_sum_butterfly(part);
      if (lane == j) my_out = part;
    }
    if (lane < n) edge_grad[(base + lane) * H + head] = my_out;
  }
}

// edge_grad on the fast widths, single head: one wave per 64 consecutive edge slots, whatever rows
// they belong to (a row of thousands of edges is shared by many waves).  Lane l finds the row of
// slot base + l by binary search over the row offsets between the rows of the wave's first and last
// slot; then, UNROLL edges at a time, the wave loads g[row] and vin[idx] (consecutive edges of one
// row re-read the same g row from L1), forms the 64 per-lane partial dot products with fused
// multiply-adds and sums them with the butterfly.  Slots of history rows and slots behind the last
// row get 0.
template <typename T, int VEC, int CHUNKS, int UNROLL>
__global__ __launch_bounds__(HC_BLOCK) void bwd_edge_grad_fast(
    const int64_t *__restrict__ ptr, const int64_t *__restrict__ idx, const float *__restrict__ g,
    const int64_t *__restrict__ hmap, const T *__restrict__ vin, float *__restrict__ edge_grad,
    int64_t E_total, int64_t R) {
  constexpr int F = HC_WAVE * VEC * CHUNKS;
  const int lane = hc_lane();
  const int64_t base = ((int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block()) * HC_WAVE;
  if (base >= E_total) return;
  const int64_t left = E_total - base;
  const int n = left < HC_WAVE ? (int)left : HC_WAVE;
  // rows of the first and the last slot: largest r in [0, R] with ptr[r] <= slot
  int64_t lo = 0, hi = R;
  const int64_t probe = lane == 0 ? base : base + n - 1;
  while (lo < hi) {
    const int64_t mid = (lo + hi + 1) >> 1;
    if (ptr[mid] <= probe) lo = mid;
    else hi = mid - 1;
  }
  // lanes 0 and 1 searched for the first and the last slot (every other lane repeated the last)
  int64_t a = hc_readlane64(lo, 0), b = hc_readlane64(lo, 1);
  int64_t my_row = -1, my_id = 0;
  if (lane < n) {
    const int64_t e = base + lane;
    while (a < b) {
      const int64_t mid = (a + b + 1) >> 1;
      if (ptr[mid] <= e) a = mid;
      else b = mid - 1;
    }
    if (a < R && ptr[a] <= e && (hmap == nullptr || hmap[a] == -1)) {
      my_row = a;
      my_id = idx[e];
    }
  }
  float my_out = 0.0f;
  for (int j = 0; j < n; j += UNROLL) {
    float x[UNROLL][CHUNKS][VEC], gr[UNROLL][CHUNKS][VEC];
    bool live[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      live[u] = false;
      if (j + u < n) {
        const int64_t r = hc_readlane64(my_row, j + u);
        if (r >= 0) {
          live[u] = true;
          const T *px = vin + hc_readlane64(my_id, j + u) * F + lane * VEC;
          const float *pg = g + r * F + lane * VEC;
#pragma unroll
          for (int k = 0; k < CHUNKS; ++k) {
            hc_vec<T, VEC>::load(px + k * HC_WAVE * VEC, x[u][k]);
            hc_vec<float, VEC>::load(pg + k * HC_WAVE * VEC, gr[u][k]);
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if (live[u]) {  // wave-uniform
        float part = 0.0f;
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
          for (int i = 0; i < VEC; ++i) part = __fmaf_rn(gr[u][k][i], x[u][k][i], part);
        part = hc_wave_sum_butterfly(part);
        if (lane == j + u) my_out = part;
      }
    }
  }
  if (lane < n) edge_grad[base + lane] = my_out;
}

// The same for rows of n_head heads side by side (F = n_head * fh elements): edge_grad[e, h] is the dot
// product over head h only.  A head is either a whole number of 64-lane chunks (one butterfly over the
// wave per head) or a power-of-two group of lanes inside a chunk (a butterfly inside each group); the
// first lane of a group stores its head's value.  Slots of history rows and behind the last row get 0.
template <typename T, int VEC, int CHUNKS, int UNROLL>
__global__ __launch_bounds__(HC_BLOCK) void bwd_edge_grad_fast_heads(
    const int64_t *__restrict__ ptr, const int64_t *__restrict__ idx, const float *__restrict__ g,
    const int64_t *__restrict__ hmap, const T *__restrict__ vin, float *__restrict__ edge_grad,
    int64_t E_total, int64_t R, int n_head) {
  constexpr int F = HC_WAVE * VEC * CHUNKS;
  const int lane = hc_lane();
  const int64_t base = ((int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block()) * HC_WAVE;
  if (base >= E_total) return;
  const int64_t left = E_total - base;
  const int n = left < HC_WAVE ? (int)left : HC_WAVE;
  const int lanes_per_head = (F / n_head) / VEC;
  int64_t lo = 0, hi = R;
  const int64_t probe = lane == 0 ? base : base + n - 1;
  while (lo < hi) {
    const int64_t mid = (lo + hi + 1) >> 1;
    if (ptr[mid] <= probe) lo = mid;
    else hi = mid - 1;
  }
  int64_t a = hc_readlane64(lo, 0), b = hc_readlane64(lo, 1);
  int64_t my_row = -1, my_id = 0;
  if (lane < n) {
    const int64_t e = base + lane;
    while (a < b) {
      const int64_t mid = (a + b + 1) >> 1;
      if (ptr[mid] <= e) a = mid;
      else b = mid - 1;
    }
    if (a < R && ptr[a] <= e && (hmap == nullptr || hmap[a] == -1)) {
      my_row = a;
      my_id = idx[e];
    }
  }
  for (int j = 0; j < n; j += UNROLL) {
    float x[UNROLL][CHUNKS][VEC], gr[UNROLL][CHUNKS][VEC];
    bool live[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      live[u] = false;
      if (j + u < n) {
        const int64_t r = hc_readlane64(my_row, j + u);
        if (r >= 0) {
          live[u] = true;
          const T *px = vin + hc_readlane64(my_id, j + u) * F + lane * VEC;
          const float *pg = g + r * F + lane * VEC;
#pragma unroll
          for (int k = 0; k < CHUNKS; ++k) {
            hc_vec<T, VEC>::load(px + k * HC_WAVE * VEC, x[u][k]);
            hc_vec<float, VEC>::load(pg + k * HC_WAVE * VEC, gr[u][k]);
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if (!live[u]) continue;  // wave-uniform
      float *__restrict__ o = edge_grad + (base + j + u) * n_head;
      if (lanes_per_head >= HC_WAVE) {
        const int chunks_per_head = lanes_per_head / HC_WAVE;
        for (int h = 0; h < n_head; ++h) {
          float part = 0.0f;
#pragma unroll
          for (int k = 0; k < CHUNKS; ++k)
            if (k / chunks_per_head == h) {
#pragma unroll
              for (int i = 0; i < VEC; ++i) part = __fmaf_rn(gr[u][k][i], x[u][k][i], part);
            }
          part = hc_wave_sum_butterfly(part);
          if (lane == 0) o[h] = part;
        }
      } else {
        const int heads_per_chunk = HC_WAVE / lanes_per_head;
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
          float part = 0.0f;
#pragma unroll
          for (int i = 0; i < VEC; ++i) part = __fmaf_rn(gr[u][k][i], x[u][k][i], part);
          for (int d = lanes_per_head >> 1; d >= 1; d >>= 1) part += __shfl_xor(part, d, HC_WAVE);
          if (lane % lanes_per_head == 0) o[k * heads_per_chunk + lane / lanes_per_head] = part;
        }
      }
    }
  }
  if (lane < n && my_row < 0) {
    float *__restrict__ o = edge_grad + (base + lane) * n_head;
    for (int h = 0; h < n_head; ++h) o[h] = 0.0f;
  }
}

// Can bwd_edge_grad_fast_heads<.., VEC, ..> take rows of n_head heads of fh elements?
inline bool edge_grad_heads_ok(int64_t fh, int vec) {
  if (fh % vec != 0) return false;
  const int64_t lanes = fh / vec;
  if (lanes >= HC_WAVE) return lanes % HC_WAVE == 0;
  return lanes >= 1 && (lanes & (lanes - 1)) == 0;
}

template <int VEC, int CHUNKS>
int launch_fast(const int64_t *ptr, const int64_t *ptrT, const int32_t *rowT, const int32_t *edgeT,
                const float *ev, int n_head, const float *g, const int64_t *hmap, float *grad_vin,
                float *grad_hbuf, int64_t hsize, int64_t R, int64_t n_src, int64_t E_slots, void *workspace,
                size_t workspace_bytes, bool masked, hipStream_t st) {
  constexpr int per = VEC * CHUNKS;
  constexpr int UNROLL = per >= 16 ? 4 : (per >= 4 ? 8 : 16);
  constexpr int F = HC_WAVE * VEC * CHUNKS;
  const int64_t per_block = (int64_t)HC_WAVES_PER_BLOCK * BWD_SRC_PER_WAVE;
  const int64_t sb = (n_src + per_block - 1) / per_block;
  // rows of several heads: grad_hbuf is written by bwd_hist_generic (the caller launches it)
  const int64_t hb = (grad_hbuf && hmap && n_head == 1) ? (R + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK : 0;
  if (sb + hb == 0) return HC_OK;
  int64_t hub_thres = 0;
  char *ws = static_cast<char *>(workspace);
  // weighted sums keep the strictly sequential order (no hub chunks); a block of up to BWD_CHUNK edge
  // slots cannot hold a hub
  const bool hubs = ev == nullptr && workspace != nullptr && E_slots > BWD_CHUNK && n_src > 0 &&
                    workspace_bytes >= bwd_partial_bytes(E_slots, F) && reinterpret_cast<uintptr_t>(ws) % 256 == 0;
  float *partial = reinterpret_cast<float *>(ws);
  int64_t *hub_of = hubs ? reinterpret_cast<int64_t *>(ws + bwd_partial_sums_bytes(E_slots, F)) : nullptr;
  const int64_t windows = hubs ? bwd_windows(E_slots) : 0;
  const int64_t wb = (windows + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
  if (hubs) hub_thres = BWD_CHUNK;
  if (!hc_grid_ok(sb + hb + wb)) return HC_EUNSUPPORTED;
  const dim3 grid((unsigned)(sb + hb + wb)), block(HC_BLOCK);
  if (masked && ev != nullptr) return HC_EUNSUPPORTED;
  if (masked)
    bwd_mean_fast<VEC, CHUNKS, UNROLL, W_NONE, true><<<grid, block, 0, st>>>(
        ptr, ptrT, rowT, edgeT, ev, n_head, g, hmap, grad_vin, grad_hbuf, hsize, R, n_src, sb, hb, hub_thres, partial,
        hub_of, windows);
  else if (ev != nullptr && n_head > 1)
    bwd_mean_fast<VEC, CHUNKS, UNROLL, W_EDGE_HEAD, false><<<grid, block, 0, st>>>(
        ptr, ptrT, rowT, edgeT, ev, n_head, g, hmap, grad_vin, grad_hbuf, hsize, R, n_src, sb, hb, hub_thres, partial,
        hub_of, windows);
  else if (ev != nullptr)
    bwd_mean_fast<VEC, CHUNKS, UNROLL, W_EDGE, false><<<grid, block, 0, st>>>(
        ptr, ptrT, rowT, edgeT, ev, n_head, g, hmap, grad_vin, grad_hbuf, hsize, R, n_src, sb, hb, hub_thres, partial,
        hub_of, windows);
  else
    bwd_mean_fast<VEC, CHUNKS, UNROLL, W_NONE, false><<<grid, block, 0, st>>>(
        ptr, ptrT, rowT, edgeT, ev, n_head, g, hmap, grad_vin, grad_hbuf, hsize, R, n_src, sb, hb, hub_thres, partial,
        hub_of, windows);
  if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
  if (hubs) {
    bwd_hub_final<VEC, CHUNKS><<<dim3((unsigned)wb), block, 0, st>>>(ptrT, partial, hub_of, grad_vin, n_src, windows);
  }
  return hc_launch_status();
}

// ---------------------------------------------------------------------------------------
// Relational layer over the mini-batch's shared view.  The layer's forward sums, for every (row, relation)
// group, x[src] * (1 / deg(row)) over the group's kept edges; here source s collects
// g[row * K + rel(e), :] * (1 / deg(row)) over its kept edges in ascending (row, edge slot) order: the order
// of the batch view, so that no view of the regrouped block has to be built.  An edge is kept under
// hc_typed_csr's rule: row < R, slot < E, relation in [0, K), source flagged in `used` (when given).
// One wave per source; up to UNROLL gradient rows in flight; products rounded, then added in order.
// ---------------------------------------------------------------------------------------
template <int VEC, int CHUNKS, int UNROLL>
__global__ __launch_bounds__(HC_BLOCK) void bwd_typed_batch_view(
    const int64_t *__restrict__ ptr, const int64_t *__restrict__ ptrT, const int32_t *__restrict__ rowT,
    const int32_t *__restrict__ edgeT, const int64_t *__restrict__ et, const uint8_t *__restrict__ used,
    const float *__restrict__ g, float *__restrict__ grad_vin, int64_t R, int64_t E, int K, int64_t n_src) {
  constexpr int F = HC_WAVE * VEC * CHUNKS;
  const int lane = hc_lane();
  const int64_t s = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (s >= n_src) return;
  float acc[CHUNKS][VEC];
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[k][i] = 0.0f;
  const bool src_kept = used == nullptr || used[s] != 0;
  const int64_t begin = src_kept ? ptrT[s] : 0;
  const int64_t end = src_kept ? ptrT[s + 1] : 0;
  for (int64_t base = begin; base < end; base += HC_WAVE) {
    const int64_t left = end - base;
    const int n = left < HC_WAVE ? (int)left : HC_WAVE;
    int64_t my_group = -1;
    float my_w = 0.0f;
    if (lane < n) {
      const int64_t row = rowT[base + lane];
      const int64_t e = edgeT[base + lane];
      if (row < R && e < E) {
        const int64_t rel = et[e];
        const int64_t d = ptr[row + 1] - ptr[row];      // 0: a row that the layer's own offsets leave empty
        if (rel >= 0 && rel < K && d > 0) {
          my_group = row * K + rel;
          my_w = 1.0f / (float)d;
        }
      }
    }
    unsigned long long todo = __ballot(my_group >= 0);
    while (todo != 0ull) {
      float v[UNROLL][CHUNKS][VEC];
      float w[UNROLL];
      bool on[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        w[u] = 0.0f;
        on[u] = todo != 0ull;
        if (on[u]) {
          const int j = __builtin_ctzll(todo);
          todo &= todo - 1ull;
          w[u] = hc_readlane_f(my_w, j);
          const float *p = g + hc_readlane64(my_group, j) * F + lane * VEC;
#pragma unroll
          for (int k = 0; k < CHUNKS; ++k) hc_vec<float, VEC>::load(p + k * HC_WAVE * VEC, v[u][k]);
        }
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if (on[u]) {
#pragma unroll
          for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[k][i] += __fmul_rn(v[u][k][i], w[u]);
        }
      }
    }
  }
  float *__restrict__ o = grad_vin + s * F + lane * VEC;
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) hc_vec<float, VEC>::store(o + k * HC_WAVE * VEC, acc[k]);
}

bool bwd_fast_shape(int64_t F) {
  return F == 64 || F == 128 || F == 192 || F == 256 || F == 384 || F == 512 || F == 768 || F == 1024;
}

}  // namespace

extern "C" size_t hc_aggr_bwd_workspace_bytes(int64_t E_total, int64_t F) {
  if (E_total < 0 || F <= 0) return 0;
  if (!bwd_fast_shape(F) || E_total <= BWD_CHUNK) return 0;
  return bwd_partial_bytes(E_total, F);
}

extern "C" int64_t hc_aggr_bwd_chunk_edges(int64_t F) { return bwd_fast_shape(F) ? BWD_CHUNK : 0; }

namespace {

int aggr_bwd_impl(const int64_t *ptr, const int64_t *idx, const int64_t *ptrT,
                  const int32_t *rowT, const int32_t *edgeT, const float *g,
                  const int64_t *hmap, const float *edge_value, const void *vin, int in_dtype,
                  int64_t n_head, float *grad_vin, float *grad_hbuf, int64_t hsize,
                  float *edge_grad, int64_t E_total, int64_t R, int64_t F, int64_t n_src,
                  void *workspace, size_t workspace_bytes, bool masked, void *stream) {
  HC_REQUIRE(R >= 0 && F > 0 && n_src >= 0 && n_head >= 1 && E_total >= 0);
  HC_REQUIRE(ptr && ptrT);
  HC_REQUIRE(g || R == 0);   // a layer without rows has no gradient rows to read
  HC_REQUIRE(grad_vin || n_src == 0);
  if (n_head > 1) HC_REQUIRE(edge_value != nullptr);
  if (grad_hbuf) HC_REQUIRE(hmap != nullptr && hsize >= F);
  if (grad_hbuf && n_head > 1) HC_REQUIRE(hsize == F || hsize == F * n_head);
  if (edge_grad) {
    HC_REQUIRE(edge_value && vin && idx);
    if (in_dtype < HC_F32 || in_dtype > HC_BF16) return HC_EDTYPE;
  }
  if (edge_value) HC_REQUIRE(edgeT != nullptr);
  HC_REQUIRE(rowT != nullptr || n_src == 0);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t lim = 0x7ffffffeLL;
  if (R > lim) return HC_EUNSUPPORTED;

  bool done = false;
  const bool aligned = (reinterpret_cast<uintptr_t>(g) % 16 == 0) &&
                       (reinterpret_cast<uintptr_t>(grad_vin) % 16 == 0);
  // Weighted sums share the fast kernel: a single head when the history buffer has the plain width, several
  // heads as one row of F * n_head elements whose lanes fetch their own head's weight.
  const int64_t Frow = F * n_head;
  bool fast_hist_pending = false;
  if (n_head <= 64 && aligned && (n_head > 1 || !edge_value || !grad_hbuf || hsize == F)) {
    int rc = HC_OK;
    done = true;
    const int nh = (int)n_head;
#define HC_FAST(V, C)                                                                             \
  if (Frow == 64 * (V) * (C) && F % (V) == 0)                                                     \
    rc = launch_fast<V, C>(ptr, ptrT, rowT, edgeT, edge_value, nh, g, hmap, grad_vin, grad_hbuf, hsize, R, \
                           n_src, E_total, workspace, workspace_bytes, masked, st);                 \
  else
    HC_FAST(4, 1) HC_FAST(4, 2) HC_FAST(4, 3) HC_FAST(4, 4) HC_FAST(2, 1) HC_FAST(2, 3) HC_FAST(1, 1)
    HC_FAST(1, 3) done = false;
#undef HC_FAST
    if (done && rc != HC_OK) return rc;
    fast_hist_pending = done && n_head > 1;
  }
  if (fast_hist_pending && grad_hbuf && R > 0) {
    const int64_t hb = (R + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
    if (!hc_grid_ok(hb)) return HC_EUNSUPPORTED;
    bwd_hist_generic<<<dim3((unsigned)hb), dim3(HC_BLOCK), 0, st>>>(g, hmap, grad_hbuf, hsize, R, F, n_head);
    if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
  }
  if (!done) {
    const int64_t sb = (n_src * n_head + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
    if (sb > 0) {
      if (!hc_grid_ok(sb)) return HC_EUNSUPPORTED;
      if (edge_value)
        bwd_generic<true><<<dim3((unsigned)sb), dim3(HC_BLOCK), 0, st>>>(ptr, ptrT, rowT, edgeT, g,
                                                                         edge_value, n_head, grad_vin,
                                                                         n_src, F, nullptr, -1);
      else
        bwd_generic<false><<<dim3((unsigned)sb), dim3(HC_BLOCK), 0, st>>>(ptr, ptrT, rowT, edgeT, g,
                                                                          edge_value, n_head, grad_vin,
                                                                          n_src, F, hmap, masked ? R : -1);
      if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
    }
    if (grad_hbuf && R > 0) {
      const int64_t hb = (R + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
      if (!hc_grid_ok(hb)) return HC_EUNSUPPORTED;
      bwd_hist_generic<<<dim3((unsigned)hb), dim3(HC_BLOCK), 0, st>>>(g, hmap, grad_hbuf, hsize, R, F,
                                                                      n_head);
      if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
    }
  }
  bool eg_done = false;
  if (edge_grad && E_total > 0 && n_head == 1 && (reinterpret_cast<uintptr_t>(vin) % 16 == 0) &&
      (reinterpret_cast<uintptr_t>(g) % 16 == 0)) {
    const int64_t wb = ((E_total + HC_WAVE - 1) / HC_WAVE + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
    if (!hc_grid_ok(wb)) return HC_EUNSUPPORTED;
    dim3 gr((unsigned)wb), bl(HC_BLOCK);
    eg_done = true;
#define HC_EG(T, V, C)                                                                                 \
  if (F == 64 * (V) * (C))                                                                             \
    bwd_edge_grad_fast<T, V, C, ((V) * (C) >= 16 ? 2 : ((V) * (C) >= 8 ? 4 : 8))><<<gr, bl, 0, st>>>(     \
        ptr, idx, g, hmap, static_cast<const T *>(vin), edge_grad, E_total, R);                         \
  else
    if (in_dtype == HC_F32) {
      HC_EG(float, 4, 1) HC_EG(float, 4, 2) HC_EG(float, 4, 3) HC_EG(float, 4, 4) HC_EG(float, 2, 1)
      HC_EG(float, 1, 1) eg_done = false;
    } else if (in_dtype == HC_F16) {
      HC_EG(__half, 4, 1) HC_EG(__half, 4, 2) HC_EG(__half, 4, 3) HC_EG(__half, 4, 4) HC_EG(__half, 2, 1)
      HC_EG(__half, 1, 1) eg_done = false;
    } else {
      HC_EG(__hip_bfloat16, 4, 1) HC_EG(__hip_bfloat16, 4, 2) HC_EG(__hip_bfloat16, 4, 3)
      HC_EG(__hip_bfloat16, 4, 4) HC_EG(__hip_bfloat16, 2, 1) HC_EG(__hip_bfloat16, 1, 1) eg_done = false;
    }
#undef HC_EG
    if (eg_done && hc_launch_status() != HC_OK) return HC_ELAUNCH;
  }
  if (edge_grad && E_total > 0 && !eg_done && n_head > 1 && n_head <= 64 &&
      (reinterpret_cast<uintptr_t>(vin) % 16 == 0) && (reinterpret_cast<uintptr_t>(g) % 16 == 0)) {
    const int64_t wb = ((E_total + HC_WAVE - 1) / HC_WAVE + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
    if (!hc_grid_ok(wb)) return HC_EUNSUPPORTED;
    dim3 gr((unsigned)wb), bl(HC_BLOCK);
    const int64_t Fall = F * n_head;
    const int nh = (int)n_head;
    eg_done = true;
#define HC_EGH(T, V, C)                                                                                  \
  if (Fall == 64 * (V) * (C) && edge_grad_heads_ok(F, V))                                                \
    bwd_edge_grad_fast_heads<T, V, C, ((V) * (C) >= 16 ? 2 : ((V) * (C) >= 8 ? 4 : 8))><<<gr, bl, 0, st>>>( \
        ptr, idx, g, hmap, static_cast<const T *>(vin), edge_grad, E_total, R, nh);                       \
  else
    if (in_dtype == HC_F32) {
      HC_EGH(float, 4, 1) HC_EGH(float, 4, 2) HC_EGH(float, 4, 3) HC_EGH(float, 4, 4) HC_EGH(float, 2, 1)
      HC_EGH(float, 1, 1) eg_done = false;
    } else if (in_dtype == HC_F16) {
      HC_EGH(__half, 4, 1) HC_EGH(__half, 4, 2) HC_EGH(__half, 4, 3) HC_EGH(__half, 4, 4) HC_EGH(__half, 2, 1)
      HC_EGH(__half, 1, 1) eg_done = false;
    } else {
      HC_EGH(__hip_bfloat16, 4, 1) HC_EGH(__hip_bfloat16, 4, 2) HC_EGH(__hip_bfloat16, 4, 3)
      HC_EGH(__hip_bfloat16, 4, 4) HC_EGH(__hip_bfloat16, 2, 1) HC_EGH(__hip_bfloat16, 1, 1) eg_done = false;
    }
#undef HC_EGH
    if (eg_done && hc_launch_status() != HC_OK) return HC_ELAUNCH;
  }
  if (edge_grad && E_total > 0 && !eg_done) {
    const int64_t rb = (R * n_head + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
    const int64_t tail_blocks = 64;
    if (!hc_grid_ok(rb + tail_blocks)) return HC_EUNSUPPORTED;
    dim3 gr((unsigned)(rb + tail_blocks)), bl(HC_BLOCK);
    if (in_dtype == HC_F32)
      bwd_edge_grad<float><<<gr, bl, 0, st>>>(ptr, idx, g, hmap, static_cast<const float *>(vin),
                                              edge_grad, E_total, R, F, n_head, rb);
    else if (in_dtype == HC_F16)
      bwd_edge_grad<__half><<<gr, bl, 0, st>>>(ptr, idx, g, hmap, static_cast<const __half *>(vin),
                                               edge_grad, E_total, R, F, n_head, rb);
    else
      bwd_edge_grad<__hip_bfloat16><<<gr, bl, 0, st>>>(ptr, idx, g, hmap,
                                                       static_cast<const __hip_bfloat16 *>(vin),
                                                       edge_grad, E_total, R, F, n_head, rb);
    if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
  }
  return HC_OK;
}

}  // namespace

extern "C" int hc_aggr_bwd(const int64_t *ptr, const int64_t *idx, const int64_t *ptrT,
                           const int32_t *rowT, const int32_t *edgeT, const float *g,
                           const int64_t *hmap, const float *edge_value, const void *vin, int in_dtype,
                           int64_t n_head, float *grad_vin, float *grad_hbuf, int64_t hsize,
                           float *edge_grad, int64_t E_total, int64_t R, int64_t F, int64_t n_src,
                           void *workspace, size_t workspace_bytes, void *stream) {
  return aggr_bwd_impl(ptr, idx, ptrT, rowT, edgeT, g, hmap, edge_value, vin, in_dtype, n_head, grad_vin,
                       grad_hbuf, hsize, edge_grad, E_total, R, F, n_src, workspace, workspace_bytes, false,
                       stream);
}

extern "C" int hc_aggr_bwd_batch_view(const int64_t *ptr, const int64_t *ptrT, const int32_t *rowT,
                                      const float *g, const int64_t *hmap, float *grad_vin,
                                      float *grad_hbuf, int64_t hsize, int64_t E_view, int64_t R, int64_t F,
                                      int64_t n_src, void *workspace, size_t workspace_bytes, void *stream) {
  return aggr_bwd_impl(ptr, nullptr, ptrT, rowT, nullptr, g, hmap, nullptr, nullptr, 0, 1, grad_vin, grad_hbuf,
                       hsize, nullptr, E_view, R, F, n_src, workspace, workspace_bytes, true, stream);
}

extern "C" int hc_aggr_bwd_batch_view_typed(const int64_t *ptr, const int64_t *ptrT, const int32_t *rowT,
                                            const int32_t *edgeT, const int64_t *edge_types, int64_t E,
                                            int num_rel, const uint8_t *used_mask, const float *g,
                                            float *grad_vin, int64_t R, int64_t F, int64_t n_src, void *stream) {
  HC_REQUIRE(R >= 0 && F > 0 && n_src >= 0 && E >= 0 && num_rel >= 1);
  HC_REQUIRE(ptr && ptrT && g && edge_types);
  HC_REQUIRE(grad_vin || n_src == 0);
  HC_REQUIRE((rowT && edgeT) || n_src == 0);
  if (R > 0x7ffffffeLL / num_rel) return HC_EUNSUPPORTED;
  if (!bwd_fast_shape(F)) return HC_EUNSUPPORTED;
  if (reinterpret_cast<uintptr_t>(g) % 16 != 0 || reinterpret_cast<uintptr_t>(grad_vin) % 16 != 0)
    return HC_EUNSUPPORTED;
  if (n_src == 0) return HC_OK;
  const int64_t nb = (n_src + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
  if (!hc_grid_ok(nb)) return HC_EUNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)nb), block(HC_BLOCK);
#define HC_TYPED(V, C)                                                                                  \
  if (F == 64 * (V) * (C))                                                                              \
    bwd_typed_batch_view<V, C, ((V) * (C) >= 16 ? 4 : 8)><<<grid, block, 0, st>>>(                      \
        ptr, ptrT, rowT, edgeT, edge_types, used_mask, g, grad_vin, R, E, num_rel, n_src);              \
  else
  HC_TYPED(4, 1) HC_TYPED(4, 2) HC_TYPED(4, 3) HC_TYPED(4, 4) HC_TYPED(2, 1) HC_TYPED(2, 3) HC_TYPED(1, 1)
  HC_TYPED(1, 3) return HC_EUNSUPPORTED;
#undef HC_TYPED
  return hc_launch_status();
}
