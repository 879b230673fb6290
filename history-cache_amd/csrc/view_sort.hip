// Transposed (CSC) view of a LARGE CSR block: a stable two-level bucket sort of the live edge slots
// by source id, written for this GPU (no sort library, kernels only, so the call can be captured).
//
// The reference has no such step (its backward scatters with float atomicAdd,
// /root/reference/src/cpp/src/history_aggr.cu:164); the view is what lets the backward gather in a
// fixed order.  Dropped edge slots (rows that took their history row, substituted sources, slots
// behind the first R rows) never enter the sort.
//
// Source ids are split into a bucket (the high bits) and a local id (the low `lb` bits, at most 13):
//   vs_count    block per tile of 8192 edge slots: the slot's key (source id, or DEAD) is written as
//               32 bits and the tile's live slots are counted per bucket (LDS histogram)
//   vs_group_sum / vs_bucket_scan / vs_bucket_offsets
//               exclusive offsets of every (tile, bucket) pair inside its bucket, in tile order
//               (groups of 8 tiles; a wave scans one bucket's groups), and the buckets' offsets
//   vs_scatter  block per tile again: every live slot is ranked among the slots of its bucket in the
//               tile, in slot order (the four waves of the block own consecutive quarters of the
//               tile; inside a wave 64 consecutive slots are ranked at a time by matching bucket
//               ids bit by bit with ballots, the running per-wave count of a bucket lives in LDS),
//               and (local id, value) goes to its final place inside the bucket: the partition is
//               stable.  value = destination row (mean aggregation) or the edge slot
//   vs_bucket   one wave per bucket: counts the local ids (LDS), scans them -- which IS this bucket's
//               stretch of ptrT --, then ranks the bucket's pairs in order, 64 at a time with the same
//               ballot matching, and writes rowT (and edgeT) at segment start + rank
// Every (source, slot) pair therefore lands where a stable sort by source puts it; the passes move
// 8 bytes per live slot twice instead of three to four radix passes over all slots.
#include "tr_shared.h"

namespace {

constexpr int VS_WAVES = 4;
constexpr int VS_THREADS = VS_WAVES * HC_WAVE;
constexpr int VS_ITERS = 32;                             // edge slots per lane
constexpr int VS_WAVE_SLOTS = HC_WAVE * VS_ITERS;        // 2048 consecutive slots per wave
constexpr int VS_TILE = VS_WAVES * VS_WAVE_SLOTS;        // 8192 slots per block
constexpr int VS_GROUP = 8;                              // tiles per group of the offset scan
constexpr int VS_MAX_BUCKETS = 5376;                     // 12 bytes of LDS per bucket in vs_scatter: 63 KB
constexpr int VS_MAX_LOCAL_BITS = 13;                    // 4 bytes of LDS per local id in vs_bucket: 32 KB
constexpr int64_t VS_MAX_EDGES = (int64_t)1 << 28;       // the per-tile counts stay a few hundred MB
constexpr uint32_t VS_DEAD = 0xffffffffu;

// Tile of a block: workgroup i runs on XCD i % 8, and every XCD gets one contiguous eighth of the
// tiles, so that the partial lines at the write front of every bucket (runs of a few pairs per tile)
// are completed inside one L2 before they are written back.
__device__ __forceinline__ int64_t vs_tile_of_block(int64_t bid, int64_t ntiles) {
  const int64_t per = ntiles / HC_NUM_XCD;
  if (bid >= per * HC_NUM_XCD) return bid;
  return (bid % HC_NUM_XCD) * per + bid / HC_NUM_XCD;
}

__device__ __forceinline__ uint32_t vs_wave_incl_scan(uint32_t v, int lane) {
#pragma unroll
  for (int d = 1; d < HC_WAVE; d <<= 1) {
    const uint32_t y = (uint32_t)__shfl_up((int)v, d, HC_WAVE);
    if (lane >= d) v += y;
  }
  return v;
}

// The lanes of the wave whose `id` equals this lane's, among the lanes of `live` (bits [0, nbits) of id
// are compared).  A lane outside `live` gets a meaningless mask.
__device__ __forceinline__ unsigned long long vs_match(uint32_t id, int nbits, unsigned long long live) {
  unsigned long long peers = live;
  for (int bit = 0; bit < nbits; ++bit) {
    const bool one = ((id >> bit) & 1u) != 0u;
    const unsigned long long bal = __ballot(one);
    peers &= one ? bal : ~bal;
  }
  return peers;
}

// ---- destination row of an edge slot, for the slots of one tile -------------------------------
// The live slots of a tile are [a, b) (inside the first R rows).  When every row that overlaps them is
// non-empty, the rows' first slots are distinct and a bitmap of them answers "row of slot e" with two
// LDS reads (r_lo + number of row starts at or below e); a tile that overlaps empty rows searches ptr.
struct VsRowFinder {
  uint32_t bits[VS_TILE / 32];
  uint32_t pre[VS_TILE / 32];
  int64_t r_lo, r_hi;
  int dense;
};

// Block-wide (every thread of the block calls it; a < b).
__device__ __forceinline__ void vs_rows_setup(VsRowFinder &f, const int64_t *__restrict__ ptr, int64_t R,
                                              int64_t e0, int64_t a, int64_t b) {
  const int tid = (int)threadIdx.x;
  const int lane = hc_lane();
  if (tid < 2 * HC_WAVE) {
    const int which = tid >> 6;
    const int64_t r = tr_row_of_wave(ptr, R, which == 0 ? a : b - 1, lane);
    if (lane == 0) {
      if (which == 0) f.r_lo = r;
      else f.r_hi = r;
    }
  }
  for (int i = tid; i < VS_TILE / 32; i += VS_THREADS) f.bits[i] = 0u;
  __syncthreads();
  const int64_t r_lo = f.r_lo, r_hi = f.r_hi;
  int empty = 0;
  if (r_hi - r_lo <= VS_TILE) {
    for (int64_t r = r_lo + 1 + tid; r <= r_hi; r += VS_THREADS) {
      const int64_t s = ptr[r], sp = ptr[r - 1];
      if (s == sp) {
        empty = 1;                                       // row r - 1 has no edges
      } else {
        const uint32_t off = (uint32_t)(s - e0);         // a < s <= b - 1: inside the tile
        atomicOr(&f.bits[off >> 5], 1u << (off & 31u));
      }
    }
  } else {
    empty = 1;
  }
  empty = __syncthreads_or(empty);
  if (!empty && tid < HC_WAVE) {
    uint32_t c[4], sum = 0u;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      c[q] = (uint32_t)__popc(f.bits[4 * lane + q]);
      sum += c[q];
    }
    uint32_t run = vs_wave_incl_scan(sum, lane) - sum;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      f.pre[4 * lane + q] = run;
      run += c[q];
    }
  }
  if (tid == 0) f.dense = empty ? 0 : 1;
  __syncthreads();
}

__device__ __forceinline__ int64_t vs_row_of(const VsRowFinder &f, const int64_t *__restrict__ ptr, int64_t e0,
                                             int64_t e) {
  if (f.dense) {
    const uint32_t off = (uint32_t)(e - e0);
    const uint32_t w = off >> 5;
    const uint32_t below = (2u << (off & 31u)) - 1u;     // bits 0..off%32 (all 32 when off%32 == 31)
    return f.r_lo + (int64_t)(f.pre[w] + (uint32_t)__popc(f.bits[w] & below));
  }
  return tr_row_of(ptr, f.r_lo, f.r_hi, e);
}

// bits[s] = (hmap_src[s] != -1), 64 sources per ballot
__global__ __launch_bounds__(HC_BLOCK) void vs_src_bits(const int64_t *__restrict__ hmap, int64_t n_src,
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

struct VsShape {
  int64_t R, E, n_src;
  int64_t ntiles, ngroups;
  int lb;          // bits of a local id
  int bbits;       // bits of a bucket id
  int nb;          // buckets: ids 0 .. n_src (ptrT has an entry for n_src too)
  int nbp;         // row pitch of the per-tile and per-group count matrices
  int nbc;         // pitch of a wave's 16-bit counters in vs_scatter's LDS
};

template <bool ROWMAP>
__global__ __launch_bounds__(VS_THREADS) void vs_count(const int64_t *__restrict__ ptr,
                                                        const int64_t *__restrict__ idx,
                                                        const int64_t *__restrict__ hmap_row,
                                                        const uint32_t *__restrict__ src_bits,
                                                        uint32_t *__restrict__ key32,
                                                        uint16_t *__restrict__ tile_count, VsShape S) {
  __shared__ uint32_t hist[VS_MAX_BUCKETS];
  __shared__ VsRowFinder rf;
  const int tid = (int)threadIdx.x;
  const int lane = hc_lane();
  const int wave = tid >> 6;
  const int64_t tile = vs_tile_of_block(blockIdx.x, S.ntiles);
  const int64_t e0 = tile * VS_TILE;
  const int64_t e1 = e0 + VS_TILE < S.E ? e0 + VS_TILE : S.E;
  for (int b = tid; b < S.nb; b += VS_THREADS) hist[b] = 0u;
  const int64_t first = ptr[0], last = ptr[S.R];
  const int64_t a = e0 > first ? e0 : first;             // the tile's slots inside the first R rows: [a, bnd)
  const int64_t bnd = e1 < last ? e1 : last;
  if (ROWMAP && a < bnd) vs_rows_setup(rf, ptr, S.R, e0, a, bnd);   // block-uniform condition
  else __syncthreads();
  const int64_t base = e0 + (int64_t)wave * VS_WAVE_SLOTS + lane;
  int64_t src[VS_ITERS];
#pragma unroll
  for (int j = 0; j < VS_ITERS; ++j) {
    const int64_t e = base + (int64_t)j * HC_WAVE;
    src[j] = (e >= a && e < bnd) ? __builtin_nontemporal_load(idx + e) : -1;
  }
#pragma unroll
  for (int j = 0; j < VS_ITERS; ++j)
    if (src[j] >= S.n_src) src[j] = -1;
  if (ROWMAP) {
    int64_t h[VS_ITERS];
#pragma unroll
    for (int j = 0; j < VS_ITERS; ++j) {
      const int64_t e = base + (int64_t)j * HC_WAVE;
      h[j] = src[j] >= 0 ? hmap_row[vs_row_of(rf, ptr, e0, e)] : -1;
    }
#pragma unroll
    for (int j = 0; j < VS_ITERS; ++j)
      if (h[j] != -1) src[j] = -1;
  }
  if (src_bits != nullptr) {
    uint32_t w[VS_ITERS];
#pragma unroll
    for (int j = 0; j < VS_ITERS; ++j) w[j] = src[j] >= 0 ? src_bits[src[j] >> 5] : 0u;
#pragma unroll
    for (int j = 0; j < VS_ITERS; ++j)
      if (src[j] >= 0 && ((w[j] >> (src[j] & 31)) & 1u) != 0u) src[j] = -1;
  }
#pragma unroll
  for (int j = 0; j < VS_ITERS; ++j) {
    const int64_t e = base + (int64_t)j * HC_WAVE;
    const uint32_t key = src[j] >= 0 ? (uint32_t)src[j] : VS_DEAD;
    if (e < e1) key32[e] = key;
    if (src[j] >= 0) atomicAdd(&hist[key >> S.lb], 1u);
  }
  __syncthreads();
  uint16_t *row = tile_count + tile * S.nbp;
  for (int b = tid; b < S.nb; b += VS_THREADS) row[b] = (uint16_t)hist[b];   // at most VS_TILE
}

// group_count[g][b] = live slots of bucket b in the tiles of group g
__global__ __launch_bounds__(HC_BLOCK) void vs_group_sum(const uint16_t *__restrict__ tile_count,
                                                          uint32_t *__restrict__ group_count, VsShape S) {
  const int b = (int)(blockIdx.x * HC_BLOCK + threadIdx.x);
  const int64_t g = blockIdx.y;
  if (b >= S.nb) return;
  uint32_t sum = 0u;
#pragma unroll
  for (int i = 0; i < VS_GROUP; ++i) {
    const int64_t t = g * VS_GROUP + i;
    if (t < S.ntiles) sum += tile_count[t * S.nbp + b];
  }
  group_count[g * S.nbp + b] = sum;
}

// One wave per bucket: the bucket's group counts become exclusive offsets (in group order) and
// bucket_total[b] their sum.
__global__ __launch_bounds__(HC_BLOCK) void vs_bucket_scan(uint32_t *__restrict__ group_count,
                                                            uint32_t *__restrict__ bucket_total, VsShape S) {
  const int lane = hc_lane();
  const int b = (int)(blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block());
  if (b >= S.nb) return;
  uint32_t carry = 0u;
  for (int64_t g0 = 0; g0 < S.ngroups; g0 += HC_WAVE) {
    const int64_t g = g0 + lane;
    const uint32_t v = g < S.ngroups ? group_count[g * S.nbp + b] : 0u;
    const uint32_t incl = vs_wave_incl_scan(v, lane);
    if (g < S.ngroups) group_count[g * S.nbp + b] = carry + incl - v;
    carry += (uint32_t)__builtin_amdgcn_readlane((int)incl, HC_WAVE - 1);
  }
  if (lane == 0) bucket_total[b] = carry;
}

// One block: bucket_off[0 .. nb] = exclusive scan of the bucket totals (bucket_off[nb] = live slots).
constexpr int VS_OFF_THREADS = 1024;
__global__ __launch_bounds__(VS_OFF_THREADS) void vs_bucket_offsets(const uint32_t *__restrict__ bucket_total,
                                                                     uint32_t *__restrict__ bucket_off, VsShape S) {
  __shared__ uint32_t s_wave[VS_OFF_THREADS / HC_WAVE];
  constexpr int PER = (VS_MAX_BUCKETS + VS_OFF_THREADS - 1) / VS_OFF_THREADS;
  const int tid = (int)threadIdx.x;
  const int lane = hc_lane();
  const int wave = tid >> 6;
  uint32_t c[PER], sum = 0u;
#pragma unroll
  for (int q = 0; q < PER; ++q) {
    const int b = tid * PER + q;
    c[q] = b < S.nb ? bucket_total[b] : 0u;
    sum += c[q];
  }
  const uint32_t incl = vs_wave_incl_scan(sum, lane);
  if (lane == HC_WAVE - 1) s_wave[wave] = incl;
  __syncthreads();
  uint32_t run = incl - sum;
  for (int w = 0; w < wave; ++w) run += s_wave[w];
#pragma unroll
  for (int q = 0; q < PER; ++q) {
    const int b = tid * PER + q;
    if (b < S.nb) bucket_off[b] = run;
    run += c[q];
    if (b == S.nb - 1) bucket_off[S.nb] = run;
  }
}

// Dynamic LDS: uint32 base[nb] (the tile's first position in every bucket), then uint16 cnt[4][nbc].
template <bool VAL_IS_ROW>
__global__ __launch_bounds__(VS_THREADS) void vs_scatter(const int64_t *__restrict__ ptr,
                                                          const uint32_t *__restrict__ key32,
                                                          const uint16_t *__restrict__ tile_count,
                                                          const uint32_t *__restrict__ group_off,
                                                          const uint32_t *__restrict__ bucket_off,
                                                          uint2 *__restrict__ pairs, uint32_t *__restrict__ rows,
                                                          VsShape S) {
  extern __shared__ uint32_t vs_lds[];
  __shared__ VsRowFinder rf;
  uint32_t *gbase = vs_lds;
  uint16_t *cnt = reinterpret_cast<uint16_t *>(vs_lds + S.nbc);
  const int tid = (int)threadIdx.x;
  const int lane = hc_lane();
  const int wave = tid >> 6;
  const int64_t tile = vs_tile_of_block(blockIdx.x, S.ntiles);
  const int64_t e0 = tile * VS_TILE;
  const int64_t e1 = e0 + VS_TILE < S.E ? e0 + VS_TILE : S.E;
  {
    uint32_t *c32 = reinterpret_cast<uint32_t *>(cnt);
    for (int i = tid; i < VS_WAVES * S.nbc / 2; i += VS_THREADS) c32[i] = 0u;
  }
  const int64_t first = ptr[0], last = ptr[S.R];
  const int64_t a = e0 > first ? e0 : first;
  const int64_t bnd = e1 < last ? e1 : last;
  if (a < bnd) vs_rows_setup(rf, ptr, S.R, e0, a, bnd);   // block-uniform condition
  else __syncthreads();
  const int64_t base = e0 + (int64_t)wave * VS_WAVE_SLOTS + lane;
  uint32_t key[VS_ITERS];
#pragma unroll
  for (int j = 0; j < VS_ITERS; ++j) {
    const int64_t e = base + (int64_t)j * HC_WAVE;
    key[j] = e < e1 ? __builtin_nontemporal_load(key32 + e) : VS_DEAD;
  }
  // rank of every live slot among the slots of its bucket in this wave's quarter, in slot order
  uint16_t *mine = cnt + wave * S.nbc;
  const unsigned long long below = (1ull << lane) - 1ull;
  uint32_t rk[VS_ITERS];
#pragma unroll
  for (int j = 0; j < VS_ITERS; ++j) {
    const bool live = key[j] != VS_DEAD;
    const uint32_t b = key[j] >> S.lb;
    const unsigned long long peers = vs_match(b, S.bbits, __ballot(live));
    uint32_t pre = 0u;
    if (live) pre = mine[b];
    if (live && (peers >> lane) == 1ull) mine[b] = (uint16_t)(pre + (uint32_t)__popcll(peers));   // the group's last lane
    rk[j] = pre + (uint32_t)__popcll(peers & below);
  }
  __syncthreads();
  // the waves' counts become offsets of the quarters; base = the tile's first position in the bucket
  {
    const int64_t g = tile / VS_GROUP;
    const int t_in = (int)(tile - g * VS_GROUP);
    for (int b = tid; b < S.nb; b += VS_THREADS) {
      uint32_t p = bucket_off[b] + group_off[g * S.nbp + b];
      for (int i = 0; i < t_in; ++i) p += tile_count[(g * VS_GROUP + i) * S.nbp + b];
      const uint32_t c0 = cnt[b], c1 = cnt[S.nbc + b], c2 = cnt[2 * S.nbc + b];
      cnt[b] = 0;
      cnt[S.nbc + b] = (uint16_t)c0;
      cnt[2 * S.nbc + b] = (uint16_t)(c0 + c1);
      cnt[3 * S.nbc + b] = (uint16_t)(c0 + c1 + c2);
      gbase[b] = p;
    }
  }
  __syncthreads();
  const uint32_t local_mask = (1u << S.lb) - 1u;
#pragma unroll
  for (int j = 0; j < VS_ITERS; ++j) {
    if (key[j] == VS_DEAD) continue;
    const int64_t e = base + (int64_t)j * HC_WAVE;
    const uint32_t b = key[j] >> S.lb;
    const uint32_t pos = gbase[b] + mine[b] + rk[j];
    const uint32_t row = (uint32_t)vs_row_of(rf, ptr, e0, e);
    if (VAL_IS_ROW) {
      pairs[pos] = make_uint2(key[j] & local_mask, row);
    } else {
      pairs[pos] = make_uint2(key[j] & local_mask, (uint32_t)e);
      rows[e] = row;
    }
  }
}

template <bool WANT_EDGES>
__global__ __launch_bounds__(HC_WAVE) void vs_bucket(const uint2 *__restrict__ pairs,
                                                      const uint32_t *__restrict__ bucket_off,
                                                      const uint32_t *__restrict__ rows,
                                                      int64_t *__restrict__ ptrT, int32_t *__restrict__ rowT,
                                                      int32_t *__restrict__ edgeT, VsShape S) {
  extern __shared__ uint32_t cur[];                      // one cursor per local id
  const int lane = hc_lane();
  const int64_t b = blockIdx.x;
  const int n_local = 1 << S.lb;
  const uint32_t p0 = bucket_off[b];
  const uint32_t n = bucket_off[b + 1] - p0;
  const uint2 *mine = pairs + p0;
  for (int k = lane; k < n_local; k += HC_WAVE) cur[k] = 0u;
  __syncthreads();
#pragma unroll 4
  for (uint32_t i = lane; i < n; i += HC_WAVE) atomicAdd(&cur[mine[i].x], 1u);
  __syncthreads();
  // exclusive scan of the counts: the segment starts of this bucket's sources, i.e. its stretch of ptrT
  uint32_t carry = 0u;
  for (int k0 = 0; k0 < n_local; k0 += HC_WAVE) {
    const int k = k0 + lane;
    const uint32_t v = k < n_local ? cur[k] : 0u;
    const uint32_t incl = vs_wave_incl_scan(v, lane);
    const uint32_t excl = carry + incl - v;
    const int64_t id = b * n_local + k;
    if (k < n_local) {
      cur[k] = excl;
      if (id <= S.n_src) ptrT[id] = (int64_t)p0 + excl;
    }
    carry += (uint32_t)__builtin_amdgcn_readlane((int)incl, HC_WAVE - 1);
  }
  __syncthreads();
  // the pairs in order, four loads of 64 in flight: position = segment cursor + rank among equal ids
  const unsigned long long below = (1ull << lane) - 1ull;
  constexpr int DEPTH = 4;
  for (uint32_t i0 = 0; i0 < n; i0 += DEPTH * HC_WAVE) {
    uint2 pr[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const uint32_t i = i0 + d * HC_WAVE + lane;
      pr[d] = i < n ? mine[i] : make_uint2(0u, 0u);
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const uint32_t i = i0 + d * HC_WAVE + lane;
      const bool live = i < n;
      const unsigned long long all = __ballot(live);
      if (all == 0ull) break;                                       // wave-uniform
      const uint32_t k = pr[d].x;
      const uint32_t k_first = (uint32_t)__builtin_amdgcn_readfirstlane((int)k);   // lane 0 is live
      const bool uniform = __ballot(live && k != k_first) == 0ull;  // a hub's stretch: no matching needed
      const unsigned long long peers = uniform ? all : vs_match(k, S.lb, all);
      uint32_t pre = 0u;
      if (live) pre = cur[k];
      if (live && (peers >> lane) == 1ull) cur[k] = pre + (uint32_t)__popcll(peers);
      const uint32_t pos = p0 + pre + (uint32_t)__popcll(peers & below);
      if (live) {
        if (WANT_EDGES) {
          edgeT[pos] = (int32_t)pr[d].y;
          rowT[pos] = (int32_t)rows[pr[d].y];
        } else {
          rowT[pos] = (int32_t)pr[d].y;
        }
      }
    }
  }
}

struct VsLayout {
  size_t key32, tile_count, group_count, bucket_total, bucket_off, pairs, rows, bits, total;
};

bool vs_shape(int64_t R, int64_t E, int64_t n_src, VsShape *S) {
  if (E <= 0 || E > VS_MAX_EDGES || n_src < 0 || n_src > 0x7ffffffeLL) return false;
  const int64_t ids = n_src + 1;
  int tb = 0;
  while (((int64_t)1 << tb) < ids) ++tb;
  int lb = tb > 12 ? tb - 12 : 0;
  while (lb <= VS_MAX_LOCAL_BITS && ((ids + ((int64_t)1 << lb) - 1) >> lb) > VS_MAX_BUCKETS) ++lb;
  if (lb > VS_MAX_LOCAL_BITS) return false;
  S->R = R;
  S->E = E;
  S->n_src = n_src;
  S->lb = lb;
  S->nb = (int)((ids + ((int64_t)1 << lb) - 1) >> lb);
  int bb = 0;
  while ((1 << bb) < S->nb) ++bb;
  S->bbits = bb;
  S->nbp = (S->nb + 63) / 64 * 64;
  S->nbc = (S->nb + 1) / 2 * 2;
  S->ntiles = (E + VS_TILE - 1) / VS_TILE;
  S->ngroups = (S->ntiles + VS_GROUP - 1) / VS_GROUP;
  return true;
}

VsLayout vs_layout(const VsShape &S) {
  VsLayout L;
  size_t at = 0;
  auto take = [&at](size_t bytes) {
    const size_t here = at;
    at += hc_align_up(bytes > 0 ? bytes : 1, 256);
    return here;
  };
  L.key32 = take((size_t)S.ntiles * VS_TILE * sizeof(uint32_t));
  L.tile_count = take((size_t)S.ntiles * S.nbp * sizeof(uint16_t));
  L.group_count = take((size_t)S.ngroups * S.nbp * sizeof(uint32_t));
  L.bucket_total = take((size_t)S.nbp * sizeof(uint32_t));
  L.bucket_off = take((size_t)(S.nbp + 1) * sizeof(uint32_t));
  L.pairs = take((size_t)S.E * sizeof(uint2));
  L.rows = take((size_t)S.E * sizeof(uint32_t));
  L.bits = take((size_t)((S.n_src + 63) / 64) * 8 + 8);
  L.total = at;
  return L;
}

}  // namespace

bool vs_supported(int64_t E, int64_t n_src) {
  VsShape S;
  return vs_shape(0, E, n_src, &S);
}

size_t vs_workspace_bytes(int64_t E, int64_t n_src) {
  VsShape S;
  if (!vs_shape(0, E, n_src, &S)) return 0;
  return vs_layout(S).total;
}

int vs_launch(const int64_t *ptr, const int64_t *idx, const int64_t *hmap_row, const int64_t *hmap_src,
              int64_t R, int64_t E, int64_t n_src, int64_t *ptrT, int32_t *rowT, int32_t *edgeT, char *ws,
              size_t ws_bytes, hipStream_t st) {
  VsShape S;
  if (!vs_shape(R, E, n_src, &S)) return HC_EUNSUPPORTED;
  const VsLayout L = vs_layout(S);
  if (ws == nullptr || ws_bytes < L.total) return HC_EWORKSPACE;
  uint32_t *key32 = reinterpret_cast<uint32_t *>(ws + L.key32);
  uint16_t *tile_count = reinterpret_cast<uint16_t *>(ws + L.tile_count);
  uint32_t *group_count = reinterpret_cast<uint32_t *>(ws + L.group_count);
  uint32_t *bucket_total = reinterpret_cast<uint32_t *>(ws + L.bucket_total);
  uint32_t *bucket_off = reinterpret_cast<uint32_t *>(ws + L.bucket_off);
  uint2 *pairs = reinterpret_cast<uint2 *>(ws + L.pairs);
  uint32_t *rows = reinterpret_cast<uint32_t *>(ws + L.rows);
  const uint32_t *src_bits = nullptr;
  if (hmap_src != nullptr) {
    unsigned long long *bits = reinterpret_cast<unsigned long long *>(ws + L.bits);
    const int64_t words = (n_src + HC_WAVE - 1) / HC_WAVE;
    int64_t blocks = (words + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
    if (blocks > 2048) blocks = 2048;
    if (blocks > 0) vs_src_bits<<<dim3((unsigned)blocks), dim3(HC_BLOCK), 0, st>>>(hmap_src, n_src, bits);
    src_bits = reinterpret_cast<const uint32_t *>(bits);
  }
  const dim3 tgrid((unsigned)S.ntiles);
  if (hmap_row != nullptr)
    vs_count<true><<<tgrid, dim3(VS_THREADS), 0, st>>>(ptr, idx, hmap_row, src_bits, key32, tile_count, S);
  else
    vs_count<false><<<tgrid, dim3(VS_THREADS), 0, st>>>(ptr, idx, hmap_row, src_bits, key32, tile_count, S);
  vs_group_sum<<<dim3((unsigned)((S.nb + HC_BLOCK - 1) / HC_BLOCK), (unsigned)S.ngroups), dim3(HC_BLOCK), 0, st>>>(
      tile_count, group_count, S);
  vs_bucket_scan<<<dim3((unsigned)((S.nb + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK)), dim3(HC_BLOCK), 0, st>>>(
      group_count, bucket_total, S);
  vs_bucket_offsets<<<dim3(1), dim3(VS_OFF_THREADS), 0, st>>>(bucket_total, bucket_off, S);
  const size_t lds = (size_t)S.nbc * sizeof(uint32_t) + (size_t)VS_WAVES * S.nbc * sizeof(uint16_t);
  const size_t blds = ((size_t)1 << S.lb) * sizeof(uint32_t);
  if (edgeT != nullptr) {
    vs_scatter<false><<<tgrid, dim3(VS_THREADS), lds, st>>>(ptr, key32, tile_count, group_count, bucket_off, pairs,
                                                           rows, S);
    vs_bucket<true><<<dim3((unsigned)S.nb), dim3(HC_WAVE), blds, st>>>(pairs, bucket_off, rows, ptrT, rowT, edgeT, S);
  } else {
    vs_scatter<true><<<tgrid, dim3(VS_THREADS), lds, st>>>(ptr, key32, tile_count, group_count, bucket_off, pairs,
                                                          rows, S);
    vs_bucket<false><<<dim3((unsigned)S.nb), dim3(HC_WAVE), blds, st>>>(pairs, bucket_off, rows, ptrT, rowT, edgeT, S);
  }
  return hc_launch_status();
}
