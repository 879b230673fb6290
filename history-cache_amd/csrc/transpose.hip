// Transposed (CSC) view of a CSR block, built with a stable sort so that the
// backward pass can gather instead of scattering with float atomics.
//
// The reference has no such step: its backward pushes gradients with
// atomicAdd (/root/reference/src/cpp/src/history_aggr.cu:164), which makes the
// sums depend on scheduling.  Here every source's incoming edges end up in
// ascending destination-row order, so the backward sums have one fixed order.
//
// Pipeline (all on the caller's stream):
//   1. expand    thread per edge slot: keys[e] = idx[e] and the slot's destination row (found by
//                binary search over the row offsets of the block's tile); slots outside the first R
//                rows and rows flagged by hmap_row get the sentinel key n_src
//   2. sort      rocPRIM LSD radix sort of (key, value) pairs -- stable.  When the caller wants
//                edgeT the value is the edge slot and rowT is gathered afterwards; when it does not
//                (mean aggregation) the value is the destination row and the sort writes rowT itself
//   3. finalize  ptrT[s] = first sorted position whose key is >= s
#include <cstring>

#include <rocprim/rocprim.hpp>

#include "hc_common.h"
#include "tr_shared.h"

namespace {

// Sort input for every edge slot, one thread per slot: key = source id, or the sentinel for slots
// outside the first R rows, rows flagged by hmap_row and ids outside [0, n_src); value = edge slot
// (VAL_IS_ROW false; `rows[e]` then gets the destination row) or the destination row itself (mean
// aggregation; dropped slots carry their slot number, they sort behind every real key).
// A block covers TR_TILE consecutive slots.  The rows that overlap the tile are found with two
// binary searches; their offsets are staged in LDS when they fit, and every thread then finds the
// row of its slot with a short search.  Reads and writes are coalesced whatever the degrees are.
constexpr int TR_LDS_ROWS = 2048;
// slots per thread: 8 on large blocks; 1 on small ones (sampled batches), where more, shorter blocks
// matter more than the amortised tile search
constexpr int64_t TR_SORT_MEMSET_EDGES = 1 << 20;  // rocPRIM sorts up to this many pairs by merging (kernels only)
constexpr int TR_ITEMS_LARGE = 8;
constexpr int64_t TR_SMALL_EDGES = 1 << 18;

template <bool VAL_IS_ROW, int TR_ITEMS>
__global__ __launch_bounds__(HC_BLOCK) void tr_expand_edges(const int64_t *__restrict__ ptr,
                                                             const int64_t *__restrict__ idx,
                                                             const int64_t *__restrict__ hmap_row,
                                                             const int64_t *__restrict__ hmap_src,
                                                             const uint32_t *__restrict__ src_bits,
                                                             uint32_t *__restrict__ keys,
                                                             uint32_t *__restrict__ vals,
                                                             uint32_t *__restrict__ rows, int64_t R, int64_t E,
                                                             int64_t n_src) {
  constexpr int TR_TILE = HC_BLOCK * TR_ITEMS;
  __shared__ int64_t s_ptr[TR_LDS_ROWS];
  __shared__ int64_t s_range[2];
  const int64_t e0 = (int64_t)blockIdx.x * TR_TILE;
  const int64_t e1 = e0 + TR_TILE < E ? e0 + TR_TILE : E;
  if (threadIdx.x < 2 * HC_WAVE) {       // the tile's first and last row, searched by two waves side by side
    const int lane0 = hc_lane();
    const int which = (int)(threadIdx.x >> 6);
    const int64_t r = tr_row_of_wave(ptr, R, which == 0 ? e0 : e1 - 1, lane0);
    if (lane0 == 0) s_range[which] = r;
  }
  __syncthreads();
  const int64_t r_lo = s_range[0], r_hi = s_range[1];
  const int64_t span = r_hi - r_lo + 1;  // rows r_lo..r_hi (r_hi may be R: slots behind the last row)
  const bool staged = span <= TR_LDS_ROWS;
  if (staged)
    for (int64_t i = threadIdx.x; i < span; i += HC_BLOCK) s_ptr[i] = ptr[r_lo + i];
  __syncthreads();
  const uint32_t sentinel = (uint32_t)n_src;
  // three sweeps over the thread's slots, so that the loads of each sweep are all in flight together
  int64_t row[TR_ITEMS];
  bool live[TR_ITEMS];
#pragma unroll
  for (int it = 0; it < TR_ITEMS; ++it) {
    const int64_t e = e0 + (int64_t)it * HC_BLOCK + threadIdx.x;
    live[it] = false;
    row[it] = 0;
    if (e < e1) {
      if (staged) {
        const int64_t l = tr_row_of(s_ptr, (int64_t)0, span - 1, e);
        row[it] = r_lo + l;
        live[it] = row[it] < R && s_ptr[l] <= e;  // ptr[row + 1] > e by construction when row < R
      } else {
        row[it] = tr_row_of(ptr, r_lo, r_hi, e);
        live[it] = row[it] < R && ptr[row[it]] <= e;
      }
    }
  }
  if (hmap_row != nullptr) {
    int64_t h[TR_ITEMS];
#pragma unroll
    for (int it = 0; it < TR_ITEMS; ++it) h[it] = live[it] ? hmap_row[row[it]] : -1;
#pragma unroll
    for (int it = 0; it < TR_ITEMS; ++it) live[it] = live[it] && h[it] == -1;
  }
  int64_t src[TR_ITEMS];
#pragma unroll
  for (int it = 0; it < TR_ITEMS; ++it) {
    const int64_t e = e0 + (int64_t)it * HC_BLOCK + threadIdx.x;
    src[it] = live[it] ? idx[e] : -1;
  }
  if (hmap_src != nullptr) {   // sources that were substituted in the forward pass receive no gradient
    // src_bits (one bit per source, derived from the map by tr_src_bits) answers the question without
    // touching the map, which costs a cache line per lookup when the sources are many
    bool sub[TR_ITEMS];
#pragma unroll
    for (int it = 0; it < TR_ITEMS; ++it) {
      sub[it] = false;
      if (src[it] >= 0 && src[it] < n_src)
        sub[it] = src_bits != nullptr ? ((src_bits[src[it] >> 5] >> (src[it] & 31)) & 1u) != 0u
                                      : hmap_src[src[it]] != -1;
    }
#pragma unroll
    for (int it = 0; it < TR_ITEMS; ++it)
      if (sub[it]) {
        src[it] = -1;
        live[it] = false;
      }
  }
#pragma unroll
  for (int it = 0; it < TR_ITEMS; ++it) {
    const int64_t e = e0 + (int64_t)it * HC_BLOCK + threadIdx.x;
    if (e >= e1) continue;
    keys[e] = (src[it] >= 0 && src[it] < n_src) ? (uint32_t)src[it] : sentinel;
    if (VAL_IS_ROW) {
      vals[e] = live[it] ? (uint32_t)row[it] : (uint32_t)e;
    } else {
      vals[e] = (uint32_t)e;
      if (live[it]) rows[e] = (uint32_t)row[it];
    }
  }
}

__global__ __launch_bounds__(HC_BLOCK) void tr_finalize_edges(const uint32_t *__restrict__ skeys,
                                                               const uint32_t *__restrict__ svals,
                                                               const uint32_t *__restrict__ rows,
                                                               int32_t *__restrict__ rowT,
                                                               int32_t *__restrict__ edgeT, int64_t E,
                                                               uint32_t sentinel) {
  const int64_t p = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (p >= E) return;
  const uint32_t k = skeys[p];
  const uint32_t e = svals[p];
  if (k != sentinel) {
    rowT[p] = (int32_t)rows[e];
    edgeT[p] = (int32_t)e;
  } else {
    rowT[p] = -1;
    edgeT[p] = -1;
  }
}

// ptrT from the sorted keys by boundary detection: position p owns the sources in
// (key[p-1], key[p]] and writes ptrT[s] = p for them; the last position also closes the tail.
// Short runs are written by the owning lane; a long run (many consecutive sources without edges)
// is written by the whole wave, 64 entries per step, so no single lane loops for long.
__global__ __launch_bounds__(HC_BLOCK) void tr_ptr_from_boundaries(const uint32_t *__restrict__ skeys,
                                                                    int64_t *__restrict__ ptrT, int64_t E,
                                                                    int64_t n_src) {
  const int lane = hc_lane();
  const int64_t p = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  int64_t first = 0, last = -1;  // sources [first, last] get ptrT = p
  int64_t tail_first = 0, tail_last = -1;
  if (p < E) {
    const int64_t cur = skeys[p];
    const int64_t prev = p == 0 ? -1 : (int64_t)skeys[p - 1];
    first = prev + 1;
    last = cur;
    if (p == E - 1) {
      tail_first = cur + 1;
      tail_last = n_src;
    }
  }
  constexpr int64_t SHORT_RUN = 4;
  const int64_t run = last - first + 1;
  if (run > 0 && run <= SHORT_RUN)
    for (int64_t s = first; s <= last; ++s) ptrT[s] = p;
  // long runs: one at a time, by the whole wave
  unsigned long long m = __ballot(run > SHORT_RUN);
  while (m != 0ull) {
    const int l = __builtin_ctzll(m);
    m &= m - 1ull;
    const int64_t f = hc_readlane64(first, l);
    const int64_t t = hc_readlane64(last, l);
    const int64_t v = hc_readlane64(p, l);
    for (int64_t s = f + lane; s <= t; s += HC_WAVE) ptrT[s] = v;
  }
  // the tail behind the last key (at most one lane of the grid has one)
  unsigned long long mt = __ballot(tail_last >= tail_first);
  while (mt != 0ull) {
    const int l = __builtin_ctzll(mt);
    mt &= mt - 1ull;
    const int64_t f = hc_readlane64(tail_first, l);
    const int64_t t = hc_readlane64(tail_last, l);
    for (int64_t s = f + lane; s <= t; s += HC_WAVE) ptrT[s] = E;
  }
}

// ptrT[s] = number of sorted keys strictly below s, for s in [0, n_src] (binary search; used
// when there are many more sources than edges).
__global__ __launch_bounds__(HC_BLOCK) void tr_finalize_ptr(const uint32_t *__restrict__ skeys,
                                                             int64_t *__restrict__ ptrT, int64_t E,
                                                             int64_t n_src) {
  const int64_t s = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (s > n_src) return;
  int64_t lo = 0, hi = E;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if ((int64_t)skeys[mid] < s) lo = mid + 1;
    else hi = mid;
  }
  ptrT[s] = lo;
}

// ---------------------------------------------------------------------------------------
// Small blocks (sampled mini-batches: at most TR_SMALL_EDGES edge slots and TR_SMALL_SOURCES sources):
// a counting sort in four launches of this file's own kernels instead of the library sort's dozen.
//   tr_small_clear  zero the per-source counters and the ticket
//   tr_small_count  thread per edge slot: the slot's key (source id, or the sentinel for a dropped
//                   slot) and destination row are saved and the source's counter is bumped (integer
//                   atomics: the final counts do not depend on their order); the block that finishes
//                   last turns the counters into ptrT (exclusive scan) and into per-source cursors
//   tr_small_place  thread per edge slot: takes the next free position of its source's segment
//                   (atomic: WHICH slots a segment holds is fixed, their order inside it is not yet)
//                   and writes (row, slot) there, into temporary arrays
//   tr_small_order  copies every segment to its final place in ascending slot order -- the order a
//                   stable sort gives: one-edge segments as they are, segments of up to 8 edges
//                   sorted by their lane in registers, of up to 64 edges ranked inside a wave, longer
//                   ones by the whole block through a bitmap of the segment's slots in LDS (rank =
//                   number of set bits below the slot), one window of TR_SMALL_EDGES slots at a time
// The result is bit-identical to the sorted view of the large-block path.
// The same four kernels serve hc_build_transpose_dev, where the block's sizes are read from device
// memory (TrDims) and the launches are sized by capacities of up to 2^24 edge slots / sources.
// ---------------------------------------------------------------------------------------
constexpr int TRS_BLOCK = 1024;
constexpr int64_t TR_SMALL_SOURCES = 1 << 20;
constexpr int TRS_BITMAP_WORDS = (int)(TR_SMALL_EDGES / 32);   // one bit per edge slot
constexpr int TRS_ORDER_SOURCES = HC_BLOCK;                     // sources per block of tr_small_order
constexpr int TRS_LANE_SORT = 8;                                // longest segment a single lane sorts

struct TrSmallHeader {
  unsigned ticket;
  unsigned pad[63];
};

// Sizes of the block: given by value, or -- when the host does not know them yet (a batch that the
// sampler has just drawn) -- read from device memory and clamped to the bounds the launch was sized for.
struct TrDims {
  int64_t R, E, n_src;               // by value (or the upper bounds when the pointers are set)
  const int64_t *pR, *pE, *pS;       // nullable, all three or none
  int32_t *overflow;                 // nullable: set to 1 when a size read on the device had to be clamped, else 0
  int64_t *max_count;                // nullable: receives the largest number of live edges of one source
};
__device__ __forceinline__ void tr_dims(const TrDims &d, int64_t &R, int64_t &E, int64_t &n_src) {
  R = d.R;
  E = d.E;
  n_src = d.n_src;
  if (d.pE != nullptr) {
    const int64_t r = *d.pR, e = *d.pE, s = *d.pS;
    R = r < 0 ? 0 : r;               // rows are bounded by the caller's ptr array
    E = e < 0 ? 0 : (e < d.E ? e : d.E);
    n_src = s < 0 ? 0 : (s < d.n_src ? s : d.n_src);
  }
}
// Did tr_dims clamp anything?  (A view of a truncated block is a valid view of the wrong block.)
__device__ __forceinline__ bool tr_dims_clamped(const TrDims &d) {
  if (d.pE == nullptr) return false;
  const int64_t r = *d.pR, e = *d.pE, s = *d.pS;
  return r < 0 || e < 0 || s < 0 || e > d.E || s > d.n_src;
}

// zero the ticket and the counters of sources [0, n_src] (rounded up to whole 16-byte groups)
__global__ __launch_bounds__(HC_BLOCK) void tr_small_clear(uint32_t *__restrict__ p, TrDims dims) {
  int64_t R, E, n_src;
  tr_dims(dims, R, E, n_src);
  const int64_t n = (int64_t)(sizeof(TrSmallHeader) / sizeof(uint32_t)) + (n_src + 1 + 3) / 4 * 4;
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i < n) p[i] = 0u;
  if (i == 0 && dims.overflow != nullptr) *dims.overflow = tr_dims_clamped(dims) ? 1 : 0;
}

// Read of a counter by the block that scans them.  The counters were only ever touched by atomics (which
// work in the L2) and this block reads them behind its device-scope fence, so an ordinary load sees the
// final values; ordinary loads, unlike atomic ones, are issued back to back.
__device__ __forceinline__ int trs_load(const int *p) { return *p; }

__global__ __launch_bounds__(TRS_BLOCK) void tr_small_count(
    const int64_t *__restrict__ ptr, const int64_t *__restrict__ idx, const int64_t *__restrict__ hmap_row,
    const int64_t *__restrict__ hmap_src, uint32_t *__restrict__ keys, int32_t *__restrict__ rows,
    int *__restrict__ count, TrSmallHeader *__restrict__ header, int64_t *__restrict__ ptrT, TrDims dims) {
  __shared__ int64_t s_ptr[TR_LDS_ROWS];
  __shared__ int64_t s_range[2];
  __shared__ int s_wave[TRS_BLOCK / HC_WAVE];
  __shared__ int s_last;
  int64_t R, E, n_src;
  tr_dims(dims, R, E, n_src);
  // The launch may be sized for more edge slots than the block has (sizes read on the device): only the
  // blocks that own edge slots take part, and block 0 always does, so that some block runs the scan.
  // (Every ticket is an atomic on one address; hundreds of idle blocks queueing for it cost more than
  // the work itself.)
  const int64_t with_edges = R > 0 ? (E + TRS_BLOCK - 1) / TRS_BLOCK : 0;
  const unsigned active = with_edges > 0 ? (unsigned)with_edges : 1u;
  if (blockIdx.x >= active) return;
  const int64_t e0 = (int64_t)blockIdx.x * TRS_BLOCK;
  const int64_t e1 = e0 + TRS_BLOCK < E ? e0 + TRS_BLOCK : E;
  if (e0 < E && R > 0) {                 // block-uniform (false only for block 0 of a block without edges)
    if (threadIdx.x < 2 * HC_WAVE) {       // the tile's first and last row, searched by two waves side by side
      const int lane0 = hc_lane();
      const int which = (int)(threadIdx.x >> 6);
      const int64_t r = tr_row_of_wave(ptr, R, which == 0 ? e0 : e1 - 1, lane0);
      if (lane0 == 0) s_range[which] = r;
    }
    __syncthreads();
    const int64_t r_lo = s_range[0], r_hi = s_range[1];
    const int64_t span = r_hi - r_lo + 1;
    const bool staged = span <= TR_LDS_ROWS;
    if (staged)
      for (int64_t i = threadIdx.x; i < span; i += TRS_BLOCK) s_ptr[i] = ptr[r_lo + i];
    __syncthreads();
    const int64_t e = e0 + threadIdx.x;
    if (e < e1) {
      int64_t row;
      bool live;
      if (staged) {
        const int64_t l = tr_row_of(s_ptr, (int64_t)0, span - 1, e);
        row = r_lo + l;
        live = row < R && s_ptr[l] <= e;
      } else {
        row = tr_row_of(ptr, r_lo, r_hi, e);
        live = row < R && ptr[row] <= e;
      }
      if (live && hmap_row != nullptr) live = hmap_row[row] == -1;
      int64_t src = live ? idx[e] : -1;
      if (src < 0 || src >= n_src) live = false;
      if (live && hmap_src != nullptr) live = hmap_src[src] == -1;
      keys[e] = live ? (uint32_t)src : (uint32_t)n_src;
      rows[e] = live ? (int32_t)row : -1;
      if (live) atomicAdd(count + src, 1);
    }
  }
  // The block that takes the last ticket sees every block's counts.  One device-scope release per
  // block, by the thread that takes the ticket, behind the block's barrier (which orders the other
  // waves' atomics in front of it): on this multi-die part a device-scope release writes the die's L2
  // back, and one per wave made this kernel several times longer.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (threadIdx.x == 0) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    s_last = atomicAdd(&header->ticket, 1u) == active - 1u ? 1 : 0;
  }
  __syncthreads();
  if (!s_last) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  // Exclusive scan of count[0, n_src] by this one block, TRS_SUPER entries per sweep.  Every wave owns a
  // contiguous run of 2 048 entries of the sweep and loads it with eight 16-byte loads per lane issued
  // together (entry = run + (g * 64 + lane) * 4 + j: each load instruction covers 1 KiB), scans its run
  // with shuffles alone, and the sixteen waves exchange their totals once per sweep (two barriers per
  // 32 768 entries; a block-wide scan per slab of 4 096 entries took a barrier pair per slab and made the
  // scan of 230 000 counters 80 us long).  (One thread per contiguous run of entries would issue 64
  // scattered requests per instruction from a single compute unit: measured 60 us for 26 000 sources.)
  // Entries between n_src and the end of the counter array are zero.
  constexpr int NW = TRS_BLOCK / HC_WAVE;
  constexpr int G = 8;
  constexpr int64_t WAVE_SPAN = (int64_t)HC_WAVE * 4 * G;
  constexpr int64_t TRS_SUPER = WAVE_SPAN * NW;
  const int lane = hc_lane();
  const int wave = (int)(threadIdx.x >> 6);
  const int64_t n_entries = n_src + 1;                      // ptrT has n_src + 1 entries
  const int64_t padded = (n_entries + 3) / 4 * 4;           // the counter array is zero-padded to 256 bytes
  int carry = 0;
  int longest = 0;                                          // the lane's largest counter
  for (int64_t base = 0; base < n_entries; base += TRS_SUPER) {
    const int64_t run0 = base + (int64_t)wave * WAVE_SPAN;
    int4 c[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int64_t i = run0 + ((int64_t)g * HC_WAVE + lane) * 4;
      c[g] = i < padded ? *reinterpret_cast<const int4 *>(count + i) : make_int4(0, 0, 0, 0);
      longest = max(max(longest, max(c[g].x, c[g].y)), max(c[g].z, c[g].w));
    }
    int pre[G];                                             // entries of the run in front of the lane's four
    int run = 0;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int mine = (c[g].x + c[g].y) + (c[g].z + c[g].w);
      int x = mine;                                         // inclusive scan over the wave
#pragma unroll
      for (int d = 1; d < HC_WAVE; d <<= 1) {
        const int y = __shfl_up(x, d, HC_WAVE);
        if (lane >= d) x += y;
      }
      pre[g] = run + x - mine;
      run += __builtin_amdgcn_readlane(x, HC_WAVE - 1);
    }
    if (lane == 0) s_wave[wave] = run;
    __syncthreads();
    int off = carry;
    int sweep = 0;
    for (int w = 0; w < NW; ++w) {
      const int t = s_wave[w];
      if (w < wave) off += t;
      sweep += t;
    }
    __syncthreads();
    carry += sweep;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int64_t i = run0 + ((int64_t)g * HC_WAVE + lane) * 4;
      if (i < n_entries) {
        const int p0 = off + pre[g], p1 = p0 + c[g].x, p2 = p1 + c[g].y, p3 = p2 + c[g].z;
        if (i + 3 < n_entries) {
          *reinterpret_cast<int4 *>(count + i) = make_int4(p0, p1, p2, p3);   // the segments' cursors
          ptrT[i] = p0;
          ptrT[i + 1] = p1;
          ptrT[i + 2] = p2;
          ptrT[i + 3] = p3;
        } else {
          const int p[4] = {p0, p1, p2, p3};
          for (int j = 0; j < 4 && i + j < n_entries; ++j) {
            count[i + j] = p[j];
            ptrT[i + j] = p[j];
          }
        }
      }
    }
  }
  if (dims.max_count != nullptr) {                          // (kernel argument: the whole block takes the branch)
#pragma unroll
    for (int d = HC_WAVE / 2; d > 0; d >>= 1) longest = max(longest, __shfl_xor(longest, d, HC_WAVE));
    if (lane == 0) s_wave[wave] = longest;                  // free since the last sweep's second barrier
    __syncthreads();
    if (threadIdx.x == 0) {
      int m = 0;
      for (int w = 0; w < NW; ++w) m = max(m, s_wave[w]);
      *dims.max_count = m;
    }
  }
}

__global__ __launch_bounds__(HC_BLOCK) void tr_small_place(const uint32_t *__restrict__ keys,
                                                            const int32_t *__restrict__ rows,
                                                            int *__restrict__ cursor,
                                                            int32_t *__restrict__ tmp_row,
                                                            int32_t *__restrict__ tmp_edge, TrDims dims) {
  int64_t R, E, n_src;
  tr_dims(dims, R, E, n_src);
  const int64_t e = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (e >= E || R <= 0) return;
  const uint32_t k = keys[e];
  if (k == (uint32_t)n_src) return;      // the sentinel of a dropped slot
  const int p = atomicAdd(cursor + k, 1);
  tmp_row[p] = rows[e];
  tmp_edge[p] = (int32_t)e;
}

__global__ __launch_bounds__(HC_BLOCK) void tr_small_order(const int64_t *__restrict__ ptrT,
                                                            const int32_t *__restrict__ tmp_row,
                                                            const int32_t *__restrict__ tmp_edge,
                                                            int32_t *__restrict__ rowT,
                                                            int32_t *__restrict__ edgeT, TrDims dims) {
  int64_t R_unused, E, n_src;
  tr_dims(dims, R_unused, E, n_src);
  __shared__ uint32_t bits[TRS_BITMAP_WORDS];
  __shared__ int pre8[TRS_BITMAP_WORDS / 8];
  __shared__ int long_src[TRS_ORDER_SOURCES];
  __shared__ int n_long_s;
  __shared__ int s_wave[HC_WAVES_PER_BLOCK];
  const int lane = hc_lane();
  const int wave = hc_wave_in_block();
  if (threadIdx.x == 0) n_long_s = 0;
  __syncthreads();
  const int64_t s = (int64_t)blockIdx.x * TRS_ORDER_SOURCES + threadIdx.x;
  int64_t b = 0;
  int len = 0;
  if (s < n_src) {
    b = ptrT[s];
    len = (int)(ptrT[s + 1] - b);
  }
  if (len == 1) {
    rowT[b] = tmp_row[b];
    if (edgeT != nullptr) edgeT[b] = tmp_edge[b];
  }
  if (len > HC_WAVE) long_src[atomicAdd(&n_long_s, 1)] = (int)threadIdx.x;
  // segments of 2..TRS_LANE_SORT edges (most of what is not a single edge): every lane sorts its own
  // segment in registers -- an odd-even transposition network on the slots, the rows ride along
  if (len >= 2 && len <= TRS_LANE_SORT) {
    int ve[TRS_LANE_SORT], vr[TRS_LANE_SORT];
#pragma unroll
    for (int k = 0; k < TRS_LANE_SORT; ++k) {
      ve[k] = k < len ? tmp_edge[b + k] : 0x7fffffff;
      vr[k] = k < len ? tmp_row[b + k] : 0;
    }
#pragma unroll
    for (int round = 0; round < TRS_LANE_SORT; ++round) {
#pragma unroll
      for (int k = round & 1; k + 1 < TRS_LANE_SORT; k += 2) {
        const bool sw = ve[k + 1] < ve[k];
        const int e0 = sw ? ve[k + 1] : ve[k], e1 = sw ? ve[k] : ve[k + 1];
        const int r0 = sw ? vr[k + 1] : vr[k], r1 = sw ? vr[k] : vr[k + 1];
        ve[k] = e0; ve[k + 1] = e1;
        vr[k] = r0; vr[k + 1] = r1;
      }
    }
#pragma unroll
    for (int k = 0; k < TRS_LANE_SORT; ++k) {
      if (k < len) {
        rowT[b + k] = vr[k];
        if (edgeT != nullptr) edgeT[b + k] = ve[k];
      }
    }
  }
  // segments of up to 64 edges: ranked inside the wave, one segment at a time
  unsigned long long m = __ballot(len > TRS_LANE_SORT && len <= HC_WAVE);
  while (m != 0ull) {
    const int l = __builtin_ctzll(m);
    m &= m - 1ull;
    const int64_t sb = hc_readlane64(b, l);
    const int sl = __builtin_amdgcn_readlane(len, l);
    const bool have = lane < sl;
    const int ve = have ? tmp_edge[sb + lane] : 0x7fffffff;
    const int vr = have ? tmp_row[sb + lane] : 0;
    int rank = 0;
    for (int j = 0; j < sl; ++j) rank += __builtin_amdgcn_readlane(ve, j) < ve ? 1 : 0;   // slots are distinct
    if (have) {
      rowT[sb + rank] = vr;
      if (edgeT != nullptr) edgeT[sb + rank] = ve;
    }
  }
  __syncthreads();
  // longer segments: the whole block, one segment at a time.  The segment's slots set their bits in an
  // LDS bitmap over a window of TR_SMALL_EDGES edge slots (one window covers a whole block of that size;
  // larger blocks take several); a slot's rank is the number of the segment's slots in earlier windows
  // plus the set bits below it in its own.
  const int n_long = n_long_s;
  for (int t = 0; t < n_long; ++t) {
    const int64_t src = (int64_t)blockIdx.x * TRS_ORDER_SOURCES + long_src[t];
    const int64_t sb = ptrT[src];
    const int sl = (int)(ptrT[src + 1] - sb);
    int before = 0;                                  // the segment's slots in the windows already done
    for (int64_t w0 = 0; w0 < E; w0 += TR_SMALL_EDGES) {
      const int64_t span = E - w0 < TR_SMALL_EDGES ? E - w0 : TR_SMALL_EDGES;
      const int words = (int)((span + 31) / 32);
      for (int w = threadIdx.x; w < words; w += HC_BLOCK) bits[w] = 0u;
      __syncthreads();
      for (int i = threadIdx.x; i < sl; i += HC_BLOCK) {
        const int64_t e = (int64_t)tmp_edge[sb + i] - w0;
        if (e >= 0 && e < span) atomicOr(&bits[e >> 5], 1u << (e & 31));
      }
      __syncthreads();
      // pre8[g] = set bits in front of word group g (8 words): per-thread run of groups, block scan
      const int groups = (words + 7) / 8;
      const int per = (groups + HC_BLOCK - 1) / HC_BLOCK;
      int glo = (int)threadIdx.x * per, ghi = glo + per;
      if (glo > groups) glo = groups;
      if (ghi > groups) ghi = groups;
      int sum = 0;
      for (int g = glo; g < ghi; ++g)
        for (int w = g * 8; w < g * 8 + 8 && w < words; ++w) sum += __popc(bits[w]);
      int x = sum;
#pragma unroll
      for (int d = 1; d < HC_WAVE; d <<= 1) {
        const int y = __shfl_up(x, d, HC_WAVE);
        if (lane >= d) x += y;
      }
      if (lane == HC_WAVE - 1) s_wave[wave] = x;
      __syncthreads();
      int run = before + x - sum;
      int in_window = 0;
      for (int w = 0; w < HC_WAVES_PER_BLOCK; ++w) {
        if (w < wave) run += s_wave[w];
        in_window += s_wave[w];
      }
      for (int g = glo; g < ghi; ++g) {
        pre8[g] = run;
        for (int w = g * 8; w < g * 8 + 8 && w < words; ++w) run += __popc(bits[w]);
      }
      __syncthreads();
      for (int i = threadIdx.x; i < sl; i += HC_BLOCK) {
        const int e_abs = tmp_edge[sb + i];
        const int64_t e = (int64_t)e_abs - w0;
        if (e < 0 || e >= span) continue;
        const int r = tmp_row[sb + i];
        const int w = (int)(e >> 5);
        int rank = pre8[w >> 3];
        for (int q = (w >> 3) * 8; q < w; ++q) rank += __popc(bits[q]);
        rank += __popc(bits[w] & ((1u << (e & 31)) - 1u));
        rowT[sb + rank] = r;
        if (edgeT != nullptr) edgeT[sb + rank] = e_abs;
      }
      before += in_window;
      __syncthreads();
    }
  }
}

struct SmallLayout {
  size_t count, keys, rows, tmp_row, tmp_edge, total;
};
SmallLayout small_layout(int64_t E, int64_t n_src) {
  SmallLayout L;
  const size_t arr = hc_align_up((size_t)(E > 0 ? E : 1) * sizeof(uint32_t), 256);
  L.count = sizeof(TrSmallHeader);
  L.keys = L.count + hc_align_up((size_t)(n_src + 1) * sizeof(int), 256);
  L.rows = L.keys + arr;
  L.tmp_row = L.rows + arr;
  L.tmp_edge = L.tmp_row + arr;
  L.total = L.tmp_edge + arr;
  return L;
}
inline bool small_block(int64_t E, int64_t n_src) { return E <= TR_SMALL_EDGES && n_src <= TR_SMALL_SOURCES; }
// Large blocks go to the bucket sort of view_sort.hip; what it does not cover (more than 2^28 edge slots or
// about 44 M sources) and the blocks between the two sizes stay with the library sort below.
constexpr int64_t TR_BUCKET_SORT_EDGES = (int64_t)1 << 20;
inline bool bucket_sorted(int64_t E, int64_t n_src) { return E > TR_BUCKET_SORT_EDGES && vs_supported(E, n_src); }

// The four launches of the counting sort; dims.E / dims.n_src size the grids (upper bounds when the real
// sizes are read on the device).
int small_launch(const int64_t *ptr, const int64_t *idx, const int64_t *hmap_row, const int64_t *hmap_src,
                 const TrDims &dims, int64_t *ptrT, int32_t *rowT, int32_t *edgeT, char *w, const SmallLayout &S,
                 hipStream_t st) {
  TrSmallHeader *header = reinterpret_cast<TrSmallHeader *>(w);
  int *count = reinterpret_cast<int *>(w + S.count);
  uint32_t *keys = reinterpret_cast<uint32_t *>(w + S.keys);
  int32_t *rows = reinterpret_cast<int32_t *>(w + S.rows);
  int32_t *tmp_row = reinterpret_cast<int32_t *>(w + S.tmp_row);
  int32_t *tmp_edge = reinterpret_cast<int32_t *>(w + S.tmp_edge);
  const int64_t E = dims.E > 0 ? dims.E : 1, n_src = dims.n_src;
  const int64_t clear_words = (int64_t)(S.keys / sizeof(uint32_t));   // header + counters
  const int64_t cb = (clear_words + HC_BLOCK - 1) / HC_BLOCK, eb = (E + TRS_BLOCK - 1) / TRS_BLOCK;
  const int64_t pb = (E + HC_BLOCK - 1) / HC_BLOCK, ob = (n_src + TRS_ORDER_SOURCES - 1) / TRS_ORDER_SOURCES;
  if (!hc_grid_ok(cb) || !hc_grid_ok(eb) || !hc_grid_ok(pb) || !hc_grid_ok(ob)) return HC_EUNSUPPORTED;
  tr_small_clear<<<dim3((unsigned)cb), dim3(HC_BLOCK), 0, st>>>(reinterpret_cast<uint32_t *>(w), dims);
  tr_small_count<<<dim3((unsigned)eb), dim3(TRS_BLOCK), 0, st>>>(ptr, idx, hmap_row, hmap_src, keys, rows, count,
                                                                 header, ptrT, dims);
  tr_small_place<<<dim3((unsigned)pb), dim3(HC_BLOCK), 0, st>>>(keys, rows, count, tmp_row, tmp_edge, dims);
  if (n_src > 0)
    tr_small_order<<<dim3((unsigned)ob), dim3(HC_BLOCK), 0, st>>>(ptrT, tmp_row, tmp_edge, rowT, edgeT, dims);
  return hc_launch_status();
}

// bits[s] = (hmap_src[s] != -1), 64 sources per ballot
__global__ __launch_bounds__(HC_BLOCK) void tr_src_bits(const int64_t *__restrict__ hmap, int64_t n_src,
                                                         unsigned long long *__restrict__ bits) {
  const int lane = hc_lane();
  const int64_t stride = (int64_t)gridDim.x * HC_WAVES_PER_BLOCK * HC_WAVE;
  for (int64_t base = ((int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block()) * HC_WAVE; base < n_src;
       base += stride) {
    const bool has = base + lane < n_src && hmap[base + lane] != -1;
    const unsigned long long bal = __ballot(has);
    if (lane == 0) bits[base / HC_WAVE] = bal;
  }
}

int key_bits(int64_t n_src) {
  int b = 1;
  while (b < 32 && ((int64_t)1 << b) <= n_src) ++b;
  return b;
}

struct Layout {
  size_t keys0, keys1, vals0, vals1, rows, bits, temp, total;
};

// The library's radix sort with the digit width and tile sizes chosen on this GPU: 9-bit digits (source
// ids of 19 to 27 bits take three passes instead of three to four 8-bit ones), 1024-thread blocks with 8
// keys per thread in the scatter kernel and 16 in the histogram kernel, wave-level ranking.  20 M pairs
// with 24-bit / 25-bit keys: 0.43 ms against 0.53 / 0.68 ms with the library's own choice; nine other
// combinations of digit width (8 - 11) and tile shape were slower.  Blocks below the merge-sort limit
// (2^20 pairs) are not affected.
using TrSortConfig = rocprim::radix_sort_config<
    rocprim::default_config, rocprim::default_config,
    rocprim::radix_sort_onesweep_config<rocprim::kernel_config<1024, 16>, rocprim::kernel_config<1024, 8>, 9,
                                        rocprim::block_radix_rank_algorithm::match>>;

hipError_t sort_temp_bytes(int64_t E, int bits, size_t *bytes) {
  rocprim::double_buffer<uint32_t> k(nullptr, nullptr), v(nullptr, nullptr);
  *bytes = 0;
  return rocprim::radix_sort_pairs<TrSortConfig>(nullptr, *bytes, k, v, (size_t)E, 0u, (unsigned)bits,
                                   (hipStream_t)0, false);
}

bool make_layout(int64_t E, int64_t n_src, Layout *L) {
  size_t temp = 0;
  if (E > 0 && sort_temp_bytes(E, key_bits(n_src), &temp) != hipSuccess) return false;
  const size_t arr = hc_align_up((size_t)(E > 0 ? E : 1) * sizeof(uint32_t), 256);
  L->keys0 = 0;
  L->keys1 = arr;
  L->vals0 = 2 * arr;
  L->vals1 = 3 * arr;
  L->rows = 4 * arr;
  L->bits = 5 * arr;   // one bit per source (used when a source map is given)
  L->temp = L->bits + hc_align_up((size_t)((n_src + 63) / 64) * 8 + 8, 256);
  L->total = L->temp + hc_align_up(temp > 0 ? temp : 1, 256);
  return true;
}

}  // namespace

extern "C" size_t hc_transpose_workspace_bytes(int64_t R, int64_t E, int64_t n_src) {
  (void)R;
  if (E < 0 || n_src < 0) return 0;
  if (small_block(E, n_src)) return small_layout(E, n_src).total;   // no library query on this path
  if (bucket_sorted(E, n_src)) return vs_workspace_bytes(E, n_src);
  Layout L;
  if (!make_layout(E, n_src, &L)) return 0;
  return L.total;
}

extern "C" int hc_build_transpose(const int64_t *ptr, const int64_t *idx, const int64_t *hmap_row,
                                  const int64_t *hmap_src, int64_t R, int64_t E, int64_t n_src, int64_t *ptrT,
                                  int32_t *rowT, int32_t *edgeT, void *workspace, size_t workspace_bytes,
                                  void *stream) {
  HC_REQUIRE(R >= 0 && E >= 0 && n_src >= 0 && ptrT);
  const int64_t lim = 0x7ffffffeLL;
  if (R > lim || E > lim || n_src > lim) return HC_EUNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t pblocks = (n_src + 1 + HC_BLOCK - 1) / HC_BLOCK;
  if (E == 0 || R == 0) {
    // no edges: every segment is empty (binary search over zero keys writes 0)
    tr_finalize_ptr<<<dim3((unsigned)pblocks), dim3(HC_BLOCK), 0, st>>>(nullptr, ptrT, 0, n_src);
    return hc_launch_status();
  }
  HC_REQUIRE(ptr && idx && rowT);
  if (small_block(E, n_src)) {
    const SmallLayout S = small_layout(E, n_src);
    if (!workspace || workspace_bytes < S.total) return HC_EWORKSPACE;
    char *w = static_cast<char *>(workspace);
    if (reinterpret_cast<uintptr_t>(w) % 256 != 0) return HC_EWORKSPACE;
    const TrDims dims{R, E, n_src, nullptr, nullptr, nullptr, nullptr, nullptr};
    return small_launch(ptr, idx, hmap_row, hmap_src, dims, ptrT, rowT, edgeT, w, S, st);
  }
  if (bucket_sorted(E, n_src)) {
    char *w = static_cast<char *>(workspace);
    if (!workspace || reinterpret_cast<uintptr_t>(w) % 256 != 0) return HC_EWORKSPACE;
    return vs_launch(ptr, idx, hmap_row, hmap_src, R, E, n_src, ptrT, rowT, edgeT, w, workspace_bytes, st);
  }
  if (E > TR_SORT_MEMSET_EDGES) {
    // Above this size the sort library takes its one-sweep path, which clears its counters with
    // hipMemsetAsync; a captured graph would replay those as memset nodes.  Refuse instead.
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cs) != hipSuccess) {
      (void)hipGetLastError();
    } else if (cs != hipStreamCaptureStatusNone) {
      return HC_EUNSUPPORTED;
    }
  }
  Layout L;
  if (!make_layout(E, n_src, &L)) return HC_ELAUNCH;
  if (!workspace || workspace_bytes < L.total) return HC_EWORKSPACE;
  char *ws = static_cast<char *>(workspace);
  if (reinterpret_cast<uintptr_t>(ws) % 256 != 0) return HC_EWORKSPACE;
  uint32_t *keys0 = reinterpret_cast<uint32_t *>(ws + L.keys0);
  uint32_t *keys1 = reinterpret_cast<uint32_t *>(ws + L.keys1);
  uint32_t *vals0 = reinterpret_cast<uint32_t *>(ws + L.vals0);
  uint32_t *vals1 = reinterpret_cast<uint32_t *>(ws + L.vals1);
  uint32_t *rows = reinterpret_cast<uint32_t *>(ws + L.rows);
  void *temp = ws + L.temp;
  size_t temp_bytes = L.total - L.temp;
  const uint32_t sentinel = (uint32_t)n_src;
  const uint32_t *src_bits = nullptr;
  if (hmap_src != nullptr && n_src >= ((int64_t)1 << 20)) {
    unsigned long long *bits = reinterpret_cast<unsigned long long *>(ws + L.bits);
    tr_src_bits<<<dim3(2048), dim3(HC_BLOCK), 0, st>>>(hmap_src, n_src, bits);
    src_bits = reinterpret_cast<const uint32_t *>(bits);
  }

  const int64_t eblocks = (E + HC_BLOCK - 1) / HC_BLOCK;
  const int64_t rblocks = (R + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
  if (!hc_grid_ok(eblocks) || !hc_grid_ok(rblocks) || !hc_grid_ok(pblocks)) return HC_EUNSUPPORTED;

  const bool want_edges = edgeT != nullptr;
  const unsigned bits = (unsigned)key_bits(n_src);
  const uint32_t *skeys = nullptr;
  const int items = E <= TR_SMALL_EDGES ? 1 : TR_ITEMS_LARGE;
  const int64_t tile = (int64_t)HC_BLOCK * items;
  const dim3 tgrid((unsigned)((E + tile - 1) / tile));
  if (want_edges) {
    if (items == 1)
      tr_expand_edges<false, 1><<<tgrid, dim3(HC_BLOCK), 0, st>>>(ptr, idx, hmap_row, hmap_src, src_bits, keys0, vals0, rows, R, E, n_src);
    else
      tr_expand_edges<false, TR_ITEMS_LARGE><<<tgrid, dim3(HC_BLOCK), 0, st>>>(ptr, idx, hmap_row, hmap_src, src_bits, keys0,
                                                                               vals0, rows, R, E, n_src);
    rocprim::double_buffer<uint32_t> dk(keys0, keys1), dv(vals0, vals1);
    if (rocprim::radix_sort_pairs<TrSortConfig>(temp, temp_bytes, dk, dv, (size_t)E, 0u, bits, st, false) != hipSuccess)
      return HC_ELAUNCH;
    tr_finalize_edges<<<dim3((unsigned)eblocks), dim3(HC_BLOCK), 0, st>>>(dk.current(), dv.current(), rows,
                                                                          rowT, edgeT, E, sentinel);
    skeys = dk.current();
  } else {
    // value = destination row; dropped edge slots keep the fill value and sort behind the sentinel
    if (items == 1)
      tr_expand_edges<true, 1><<<tgrid, dim3(HC_BLOCK), 0, st>>>(ptr, idx, hmap_row, hmap_src, src_bits, keys0, vals0, nullptr, R, E, n_src);
    else
      tr_expand_edges<true, TR_ITEMS_LARGE><<<tgrid, dim3(HC_BLOCK), 0, st>>>(ptr, idx, hmap_row, hmap_src, src_bits, keys0,
                                                                              vals0, nullptr, R, E, n_src);
    // rowT doubles as the sort's second value buffer; copy only if the result landed in the first
    uint32_t *rowT_u = reinterpret_cast<uint32_t *>(rowT);
    rocprim::double_buffer<uint32_t> dk(keys0, keys1), dv(vals0, rowT_u);
    if (rocprim::radix_sort_pairs<TrSortConfig>(temp, temp_bytes, dk, dv, (size_t)E, 0u, bits, st, false) != hipSuccess)
      return HC_ELAUNCH;
    if (dv.current() != rowT_u &&
        hipMemcpyAsync(rowT, dv.current(), (size_t)E * sizeof(uint32_t), hipMemcpyDeviceToDevice, st) != hipSuccess)
      return HC_ELAUNCH;
    skeys = dk.current();
  }
  if (n_src <= 4 * E) {
    tr_ptr_from_boundaries<<<dim3((unsigned)eblocks), dim3(HC_BLOCK), 0, st>>>(skeys, ptrT, E, n_src);
  } else {
    tr_finalize_ptr<<<dim3((unsigned)pblocks), dim3(HC_BLOCK), 0, st>>>(skeys, ptrT, E, n_src);
  }
  return hc_launch_status();
}

// Limits of the variant with device-resident sizes: the counters are 32-bit and one block scans them.
constexpr int64_t TR_DEV_MAX_EDGES = (int64_t)1 << 24;
constexpr int64_t TR_DEV_MAX_SOURCES = (int64_t)1 << 24;

extern "C" size_t hc_transpose_dev_workspace_bytes(int64_t max_E, int64_t max_src) {
  if (max_E < 0 || max_src < 0 || max_E > TR_DEV_MAX_EDGES || max_src > TR_DEV_MAX_SOURCES) return 0;
  return small_layout(max_E, max_src).total;
}

extern "C" int hc_build_transpose_dev(const int64_t *ptr, const int64_t *idx, const int64_t *R_dev,
                                      const int64_t *E_dev, const int64_t *n_src_dev, int64_t max_E,
                                      int64_t max_src, int64_t *ptrT, int32_t *rowT, int32_t *edgeT,
                                      int32_t *overflow, void *workspace, size_t workspace_bytes, void *stream) {
  return hc_build_transpose_dev_deg(ptr, idx, R_dev, E_dev, n_src_dev, max_E, max_src, ptrT, rowT, edgeT, overflow,
                                    nullptr, workspace, workspace_bytes, stream);
}

extern "C" int hc_build_transpose_dev_deg(const int64_t *ptr, const int64_t *idx, const int64_t *R_dev,
                                          const int64_t *E_dev, const int64_t *n_src_dev, int64_t max_E,
                                          int64_t max_src, int64_t *ptrT, int32_t *rowT, int32_t *edgeT,
                                          int32_t *overflow, int64_t *max_in_degree, void *workspace,
                                          size_t workspace_bytes, void *stream) {
  HC_REQUIRE(ptr && idx && R_dev && E_dev && n_src_dev && ptrT && max_E >= 0 && max_src >= 0);
  HC_REQUIRE(rowT != nullptr || max_E == 0);
  if (max_E > TR_DEV_MAX_EDGES || max_src > TR_DEV_MAX_SOURCES) return HC_EUNSUPPORTED;
  const SmallLayout S = small_layout(max_E, max_src);
  if (!workspace || workspace_bytes < S.total) return HC_EWORKSPACE;
  char *w = static_cast<char *>(workspace);
  if (reinterpret_cast<uintptr_t>(w) % 256 != 0) return HC_EWORKSPACE;
  const TrDims dims{0, max_E, max_src, R_dev, E_dev, n_src_dev, overflow, max_in_degree};
  return small_launch(ptr, idx, nullptr, nullptr, dims, ptrT, rowT, edgeT, w, S, static_cast<hipStream_t>(stream));
}
