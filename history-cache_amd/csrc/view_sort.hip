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
//               tile, in slot order, and (local id, value) goes to its final place inside the bucket:
//               the partition is stable.  The eight waves of the block own consecutive eighths of the
//               tile and keep a running count per bucket in LDS; a wave ranks 64 consecutive slots
//               at a time (see vs_rank_among_equal).  value = destination row (mean aggregation)
//               or the edge slot
//   vs_bucket   block per bucket: counts the local ids per wave (the four waves own consecutive
//               quarters of the bucket's pairs), scans them -- which IS this bucket's stretch of
//               ptrT --, ranks the pairs in order the same way and writes rowT (and edgeT) at segment
//               start + rank, through LDS so that the stores are whole lines
// Every (source, slot) pair therefore lands where a stable sort by source puts it.  The cost is set
// by the number of memory requests rather than by bytes: the scattered 8-byte stores of vs_scatter
// are one request per live slot, which is why there are two levels and not three, and why everything
// else is staged so that its requests are whole lines.
#include "tr_shared.h"

namespace {

constexpr int VS_WAVES = 8;                              // waves per block of vs_count / vs_scatter
constexpr int VS_THREADS = VS_WAVES * HC_WAVE;
constexpr int VS_ITERS = 16;                             // edge slots per lane
constexpr int VS_WAVE_SLOTS = HC_WAVE * VS_ITERS;        // 1024 consecutive slots per wave
constexpr int VS_TILE = VS_WAVES * VS_WAVE_SLOTS;        // 8192 slots per block
constexpr int VS_GROUP = 8;                              // tiles per group of the offset scan
constexpr int VS_MAX_BUCKETS = 5376;                     // 20 bytes of LDS per bucket in vs_scatter: 105 KB
constexpr int VS_MAX_LOCAL_BITS = 13;                    // 16 bytes of LDS per local id in vs_bucket: 128 KB
constexpr int64_t VS_MAX_EDGES = (int64_t)1 << 28;       // the per-tile counts stay a few hundred MB
constexpr uint32_t VS_DEAD = 0xffffffffu;

constexpr int VB_WAVES = 4;                              // waves per block of vs_bucket
constexpr int VB_THREADS = VB_WAVES * HC_WAVE;
constexpr int VB_ITERS = 32;                             // pairs per lane on the register path
constexpr uint32_t VB_STAGED = VB_THREADS * VB_ITERS;    // 8192: largest bucket that takes the register path

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

// Rank of this lane among the live lanes of the wave that hold the same id, in lane order.  `same` is
// the number of such lanes (this one included), which the caller reads off the id's counter: its value
// behind the wave's adds minus its value in front of them.  A lane that is alone with its id (most are)
// needs no matching; the others are matched one distinct id per round.
__device__ __forceinline__ uint32_t vs_rank_among_equal(uint32_t id, bool live, uint32_t same,
                                                        unsigned long long below) {
  uint32_t rank = 0u;
  unsigned long long dups = __ballot(live && same > 1u);
  while (dups != 0ull) {                                   // wave-uniform
    const int l = __builtin_ctzll(dups);
    const uint32_t v = (uint32_t)__builtin_amdgcn_readlane((int)id, l);
    const unsigned long long grp = __ballot(live && id == v);
    if (live && id == v) rank = (uint32_t)__popcll(grp & below);
    dups &= ~grp;
  }
  return rank;
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
  if (tid < 2 * HC_WAVE) {                               // the first and the last row, by two waves side by side
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
  int nb;          // buckets: ids 0 .. n_src (ptrT has an entry for n_src too)
  int nbp;         // row pitch of the per-tile and per-group count matrices
  int nbc;         // pitch of a wave's 16-bit counters in vs_scatter's LDS (even)
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
  const int64_t base = e0 + (int64_t)wave * VS_WAVE_SLOTS + lane;
  int64_t src[VS_ITERS];
#pragma unroll
  for (int j = 0; j < VS_ITERS; ++j) {
    const int64_t e = base + (int64_t)j * HC_WAVE;
    src[j] = (e >= a && e < bnd) ? __builtin_nontemporal_load(idx + e) : -1;
  }
  if (ROWMAP && a < bnd) vs_rows_setup(rf, ptr, S.R, e0, a, bnd);   // block-uniform condition
  else __syncthreads();
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
    if (e < e1) __builtin_nontemporal_store(key, key32 + e);
    if (src[j] >= 0) atomicAdd(&hist[key >> S.lb], 1u);
  }
  __syncthreads();
  uint16_t *row = tile_count + tile * S.nbp;
  for (int b = tid; b < S.nb; b += VS_THREADS) row[b] = (uint16_t)hist[b];   // at most VS_TILE
}

// group_count[g][b] = live slots of bucket b in the tiles of group g; the tiles' own counts become
// exclusive offsets inside their group (at most 7 * VS_TILE: 16 bits hold them).
__global__ __launch_bounds__(HC_BLOCK) void vs_group_sum(uint16_t *__restrict__ tile_count,
                                                          uint32_t *__restrict__ group_count, VsShape S) {
  const int b = (int)(blockIdx.x * HC_BLOCK + threadIdx.x);
  const int64_t g = blockIdx.y;
  if (b >= S.nb) return;
  uint32_t c[VS_GROUP];
#pragma unroll
  for (int i = 0; i < VS_GROUP; ++i) {
    const int64_t t = g * VS_GROUP + i;
    c[i] = t < S.ntiles ? tile_count[t * S.nbp + b] : 0u;
  }
  uint32_t sum = 0u;
#pragma unroll
  for (int i = 0; i < VS_GROUP; ++i) {
    const int64_t t = g * VS_GROUP + i;
    if (t < S.ntiles) tile_count[t * S.nbp + b] = (uint16_t)sum;
    sum += c[i];
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
  constexpr int Q = 4;                                    // rounds of 64 groups whose loads are in flight together
  for (int64_t g0 = 0; g0 < S.ngroups; g0 += Q * HC_WAVE) {
    uint32_t v[Q];
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      const int64_t g = g0 + q * HC_WAVE + lane;
      v[q] = g < S.ngroups ? group_count[g * S.nbp + b] : 0u;
    }
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      const int64_t g = g0 + q * HC_WAVE + lane;
      const uint32_t incl = vs_wave_incl_scan(v[q], lane);
      if (g < S.ngroups) group_count[g * S.nbp + b] = carry + incl - v[q];
      carry += (uint32_t)__builtin_amdgcn_readlane((int)incl, HC_WAVE - 1);
    }
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

// Dynamic LDS: uint32 base[nbc] (the tile's first position in every bucket), then the waves'
// 16-bit counters, cnt[VS_WAVES][nbc], two to a 32-bit word.
template <bool VAL_IS_ROW>
__global__ __launch_bounds__(VS_THREADS) void vs_scatter(const int64_t *__restrict__ ptr,
                                                          const uint32_t *__restrict__ key32,
                                                          const uint16_t *__restrict__ tile_off,
                                                          const uint32_t *__restrict__ group_off,
                                                          const uint32_t *__restrict__ bucket_off,
                                                          uint2 *__restrict__ pairs, uint32_t *__restrict__ rows,
                                                          VsShape S) {
  extern __shared__ uint32_t vs_lds[];
  __shared__ VsRowFinder rf;
  uint32_t *gbase = vs_lds;
  uint32_t *cnt32 = vs_lds + S.nbc;
  uint16_t *cnt = reinterpret_cast<uint16_t *>(cnt32);
  const int tid = (int)threadIdx.x;
  const int lane = hc_lane();
  const int wave = tid >> 6;
  const int64_t tile = vs_tile_of_block(blockIdx.x, S.ntiles);
  const int64_t e0 = tile * VS_TILE;
  const int64_t e1 = e0 + VS_TILE < S.E ? e0 + VS_TILE : S.E;
  const int64_t base = e0 + (int64_t)wave * VS_WAVE_SLOTS + lane;
  uint32_t key[VS_ITERS];                                 // in flight while the rows are set up
#pragma unroll
  for (int j = 0; j < VS_ITERS; ++j) {
    const int64_t e = base + (int64_t)j * HC_WAVE;
    key[j] = e < e1 ? __builtin_nontemporal_load(key32 + e) : VS_DEAD;
  }
  for (int i = tid; i < VS_WAVES * S.nbc / 2; i += VS_THREADS) cnt32[i] = 0u;
  const int64_t first = ptr[0], last = ptr[S.R];
  const int64_t a = e0 > first ? e0 : first;
  const int64_t bnd = e1 < last ? e1 : last;
  if (a < bnd) vs_rows_setup(rf, ptr, S.R, e0, a, bnd);   // block-uniform condition
  else __syncthreads();
  // Rank of every live slot among the slots of its bucket in this wave's eighth of the tile, in slot
  // order: the bucket's running count in front of these 64 slots plus the rank among them.
  uint32_t *mine32 = cnt32 + wave * (S.nbc / 2);
  const unsigned long long below = (1ull << lane) - 1ull;
  uint32_t rk[VS_ITERS];
#pragma unroll
  for (int j = 0; j < VS_ITERS; ++j) {
    const bool live = key[j] != VS_DEAD;
    const uint32_t b = key[j] >> S.lb;
    uint32_t before = 0u, same = 0u;
    if (live) {
      const uint32_t sh = (b & 1u) * 16u;
      const uint32_t w0 = mine32[b >> 1];
      atomicAdd(&mine32[b >> 1], 1u << sh);
      const uint32_t w1 = mine32[b >> 1];
      before = (w0 >> sh) & 0xffffu;
      same = ((w1 >> sh) & 0xffffu) - before;
    }
    rk[j] = before + vs_rank_among_equal(b, live, same, below);
  }
  __syncthreads();
  // the waves' counts become the eighths' offsets; base = the tile's first position in the bucket
  {
    const int64_t g = tile / VS_GROUP;
    const uint32_t *grow = group_off + g * S.nbp;
    const uint16_t *trow = tile_off + tile * S.nbp;
    constexpr int Q = 2;
    for (int b0 = tid; b0 < S.nb; b0 += Q * VS_THREADS) {
      uint32_t p[Q];
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        const int b = b0 + q * VS_THREADS;
        p[q] = b < S.nb ? bucket_off[b] + grow[b] + trow[b] : 0u;
      }
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        const int b = b0 + q * VS_THREADS;
        if (b < S.nb) {
          uint32_t run = 0u;
#pragma unroll
          for (int w = 0; w < VS_WAVES; ++w) {
            const uint32_t c = cnt[w * S.nbc + b];
            cnt[w * S.nbc + b] = (uint16_t)run;
            run += c;
          }
          gbase[b] = p[q];
        }
      }
    }
  }
  __syncthreads();
  const uint16_t *mine = cnt + wave * S.nbc;
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

// ---- vs_bucket -------------------------------------------------------------------------------------
// Cursor arrays in LDS, one per wave, indexed by local id.  The scan hands 16 consecutive ids to a
// thread; the swizzles spread the runs of neighbouring threads over the banks.
// 32-bit cursors (buckets of any size): word k -> vb_swz32(k).
__device__ __forceinline__ uint32_t vb_swz32(uint32_t k) { return (k & ~15u) | ((k & 15u) ^ ((k >> 5) & 15u)); }
// 16-bit cursors (buckets of at most VB_STAGED pairs), two to a word: word k / 2 -> vb_swz16w(k / 2).
__device__ __forceinline__ uint32_t vb_swz16w(uint32_t w) { return (w & ~7u) | ((w & 7u) ^ ((w >> 5) & 7u)); }

// Buckets of at most VB_STAGED pairs: the pairs are read once and stay in registers, the cursors are
// 16 bits wide and the bucket's stretch of rowT is put together in LDS and stored line by line.
// LDS: cur16[VB_WAVES][n_local] (as words), then stage[VB_STAGED].
template <bool WANT_EDGES>
__device__ __forceinline__ void vb_small(const uint2 *__restrict__ mine, uint32_t n, uint32_t p0, int64_t b,
                                         uint32_t *__restrict__ lds, uint32_t *__restrict__ s_wave,
                                         const uint32_t *__restrict__ rows, int64_t *__restrict__ ptrT,
                                         int32_t *__restrict__ rowT, int32_t *__restrict__ edgeT, const VsShape &S) {
  const int tid = (int)threadIdx.x;
  const int lane = hc_lane();
  const int wave = tid >> 6;
  const uint32_t n_local = 1u << S.lb;
  const uint32_t words = (n_local + 1u) / 2u;             // cursor words per wave
  uint32_t *stage = lds + VB_WAVES * words;
  uint32_t *my = lds + (uint32_t)wave * words;
  // the four waves own consecutive quarters of the bucket's pairs
  const uint32_t quarter = ((n + VB_WAVES - 1) / VB_WAVES + HC_WAVE - 1) / HC_WAVE * HC_WAVE;
  const uint32_t q_begin = (uint32_t)wave * quarter < n ? (uint32_t)wave * quarter : n;
  const uint32_t q_len = q_begin + quarter < n ? quarter : n - q_begin;
  uint2 pr[VB_ITERS];
#pragma unroll
  for (int j = 0; j < VB_ITERS; ++j) {
    const uint32_t i = (uint32_t)j * HC_WAVE + lane;
    pr[j] = i < q_len ? mine[q_begin + i] : make_uint2(0u, 0u);
  }
  for (uint32_t i = tid; i < VB_WAVES * words; i += VB_THREADS) lds[i] = 0u;
  __syncthreads();
#pragma unroll
  for (int j = 0; j < VB_ITERS; ++j) {
    const uint32_t i = (uint32_t)j * HC_WAVE + lane;
    if (i < q_len) atomicAdd(&my[vb_swz16w(pr[j].x >> 1)], 1u << ((pr[j].x & 1u) * 16u));
  }
  __syncthreads();
  // Counts -> cursors: local id k's segment starts at the exclusive sum over the ids below it (that is
  // this bucket's stretch of ptrT), wave w's pairs of k follow those of the waves before it.
  {
    const uint32_t per = words >= (uint32_t)VB_THREADS ? words / VB_THREADS : 1u;   // words per thread
    const uint32_t w0 = (uint32_t)tid * per;
    uint32_t sum = 0u;
    if (w0 < words)
      for (uint32_t wd = w0; wd < w0 + per; ++wd) {
        const uint32_t at = vb_swz16w(wd);
#pragma unroll
        for (int w = 0; w < VB_WAVES; ++w) {
          const uint32_t v = lds[(uint32_t)w * words + at];
          sum += (v & 0xffffu) + (v >> 16);
        }
      }
    const uint32_t incl = vs_wave_incl_scan(sum, lane);
    if (lane == HC_WAVE - 1) s_wave[wave] = incl;
    __syncthreads();
    uint32_t run = incl - sum;
    for (int w = 0; w < wave; ++w) run += s_wave[w];
    if (w0 < words)
      for (uint32_t wd = w0; wd < w0 + per; ++wd) {
        const uint32_t at = vb_swz16w(wd);
        uint32_t v[VB_WAVES];
#pragma unroll
        for (int w = 0; w < VB_WAVES; ++w) v[w] = lds[(uint32_t)w * words + at];
        uint32_t lo = run;                                 // cursors of the even id, wave by wave
#pragma unroll
        for (int w = 0; w < VB_WAVES; ++w) {
          const uint32_t c = v[w] & 0xffffu;
          v[w] = (v[w] & 0xffff0000u) | lo;
          lo += c;
        }
        uint32_t hi = lo;                                  // then the odd id's
#pragma unroll
        for (int w = 0; w < VB_WAVES; ++w) {
          const uint32_t c = v[w] >> 16;
          v[w] = (v[w] & 0xffffu) | (hi << 16);
          hi += c;
        }
        run = hi;
#pragma unroll
        for (int w = 0; w < VB_WAVES; ++w) lds[(uint32_t)w * words + at] = v[w];
      }
  }
  __syncthreads();
  for (uint32_t k = tid; k < n_local; k += VB_THREADS) {
    const int64_t id = b * (int64_t)n_local + k;
    const uint32_t v = lds[vb_swz16w(k >> 1)];            // wave 0's cursor = the segment's start
    if (id <= S.n_src) ptrT[id] = (int64_t)p0 + ((v >> ((k & 1u) * 16u)) & 0xffffu);
  }
  __syncthreads();
  // every wave ranks the pairs of its quarter in order, 64 at a time
  const unsigned long long below = (1ull << lane) - 1ull;
#pragma unroll
  for (int j = 0; j < VB_ITERS; ++j) {
    if ((uint32_t)j * HC_WAVE >= q_len) break;            // wave-uniform
    const uint32_t i = (uint32_t)j * HC_WAVE + lane;
    const bool live = i < q_len;
    const uint32_t k = pr[j].x;
    uint32_t before = 0u, same = 0u;
    if (live) {
      uint32_t *c = &my[vb_swz16w(k >> 1)];
      const uint32_t sh = (k & 1u) * 16u;
      const uint32_t v0 = *c;
      atomicAdd(c, 1u << sh);
      const uint32_t v1 = *c;
      before = (v0 >> sh) & 0xffffu;
      same = ((v1 >> sh) & 0xffffu) - before;
    }
    const uint32_t pos = before + vs_rank_among_equal(k, live, same, below);
    if (live) stage[pos] = pr[j].y;
  }
  __syncthreads();
  for (uint32_t i = tid; i < n; i += VB_THREADS) {
    const uint32_t v = stage[i];
    if (WANT_EDGES) {
      edgeT[p0 + i] = (int32_t)v;
      rowT[p0 + i] = (int32_t)rows[v];
    } else {
      rowT[p0 + i] = (int32_t)v;
    }
  }
}

// Buckets above VB_STAGED pairs (hub sources): 32-bit cursors, the pairs are read twice and the
// results stored as they come.  LDS: cur[VB_WAVES][n_local].
template <bool WANT_EDGES>
__device__ __forceinline__ void vb_large(const uint2 *__restrict__ mine, uint32_t n, uint32_t p0, int64_t b,
                                         uint32_t *__restrict__ cur, uint32_t *__restrict__ s_wave,
                                         const uint32_t *__restrict__ rows, int64_t *__restrict__ ptrT,
                                         int32_t *__restrict__ rowT, int32_t *__restrict__ edgeT, const VsShape &S) {
  const int tid = (int)threadIdx.x;
  const int lane = hc_lane();
  const int wave = tid >> 6;
  const uint32_t n_local = 1u << S.lb;
  const uint32_t quarter = ((n + VB_WAVES - 1) / VB_WAVES + HC_WAVE - 1) / HC_WAVE * HC_WAVE;
  const uint32_t q_begin = (uint32_t)wave * quarter < n ? (uint32_t)wave * quarter : n;
  const uint32_t q_end = q_begin + quarter < n ? q_begin + quarter : n;
  uint32_t *my = cur + (uint32_t)wave * n_local;
  for (uint32_t i = tid; i < VB_WAVES * n_local; i += VB_THREADS) cur[i] = 0u;
  __syncthreads();
#pragma unroll 4
  for (uint32_t i = q_begin + lane; i < q_end; i += HC_WAVE) atomicAdd(&my[vb_swz32(mine[i].x)], 1u);
  __syncthreads();
  {
    const uint32_t per = n_local >= (uint32_t)VB_THREADS ? n_local / VB_THREADS : 1u;   // ids per thread
    const uint32_t k0 = (uint32_t)tid * per;
    uint32_t sum = 0u;
    if (k0 < n_local)
      for (uint32_t k = k0; k < k0 + per; ++k) {
        const uint32_t at = vb_swz32(k);
        sum += cur[at] + cur[n_local + at] + cur[2 * n_local + at] + cur[3 * n_local + at];
      }
    const uint32_t incl = vs_wave_incl_scan(sum, lane);
    if (lane == HC_WAVE - 1) s_wave[wave] = incl;
    __syncthreads();
    uint32_t run = incl - sum;
    for (int w = 0; w < wave; ++w) run += s_wave[w];
    if (k0 < n_local)
      for (uint32_t k = k0; k < k0 + per; ++k) {
        const uint32_t at = vb_swz32(k);
        const uint32_t c0 = cur[at], c1 = cur[n_local + at], c2 = cur[2 * n_local + at], c3 = cur[3 * n_local + at];
        cur[at] = run;
        cur[n_local + at] = run + c0;
        cur[2 * n_local + at] = run + c0 + c1;
        cur[3 * n_local + at] = run + c0 + c1 + c2;
        run += c0 + c1 + c2 + c3;
      }
  }
  __syncthreads();
  for (uint32_t k = tid; k < n_local; k += VB_THREADS) {
    const int64_t id = b * (int64_t)n_local + k;
    if (id <= S.n_src) ptrT[id] = (int64_t)p0 + cur[vb_swz32(k)];    // wave 0's cursor = the segment's start
  }
  __syncthreads();
  const unsigned long long below = (1ull << lane) - 1ull;
  constexpr int DEPTH = 4;
  for (uint32_t i0 = q_begin; i0 < q_end; i0 += DEPTH * HC_WAVE) {
    uint2 pr[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const uint32_t i = i0 + d * HC_WAVE + lane;
      pr[d] = i < q_end ? mine[i] : make_uint2(0u, 0u);
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const uint32_t i = i0 + d * HC_WAVE + lane;
      const bool live = i < q_end;
      const uint32_t k = pr[d].x;
      uint32_t before = 0u, same = 0u;
      if (live) {
        uint32_t *c = &my[vb_swz32(k)];
        before = *c;
        atomicAdd(c, 1u);
        same = *c - before;
      }
      const uint32_t pos = p0 + before + vs_rank_among_equal(k, live, same, below);
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

template <bool WANT_EDGES>
__global__ __launch_bounds__(VB_THREADS) void vs_bucket(const uint2 *__restrict__ pairs,
                                                         const uint32_t *__restrict__ bucket_off,
                                                         const uint32_t *__restrict__ rows,
                                                         int64_t *__restrict__ ptrT, int32_t *__restrict__ rowT,
                                                         int32_t *__restrict__ edgeT, VsShape S) {
  extern __shared__ uint32_t vb_lds[];
  __shared__ uint32_t s_wave[VB_WAVES];
  const int64_t b = blockIdx.x;
  const uint32_t p0 = bucket_off[b];
  const uint32_t n = bucket_off[b + 1] - p0;               // block-uniform
  if (n <= VB_STAGED) vb_small<WANT_EDGES>(pairs + p0, n, p0, b, vb_lds, s_wave, rows, ptrT, rowT, edgeT, S);
  else vb_large<WANT_EDGES>(pairs + p0, n, p0, b, vb_lds, s_wave, rows, ptrT, rowT, edgeT, S);
}

struct VsLayout {
  size_t key32, tile_count, group_count, bucket_total, bucket_off, pairs, rows, bits, total;
};

bool vs_shape(int64_t R, int64_t E, int64_t n_src, VsShape *S) {
  if (E <= 0 || E > VS_MAX_EDGES || n_src < 0 || n_src > 0x7ffffffeLL) return false;
  const int64_t ids = n_src + 1;
  int tb = 0;
  while (((int64_t)1 << tb) < ids) ++tb;
  // between 1024 and 2048 buckets where the ids allow it (enough blocks for vs_bucket, few enough counters
  // per tile in vs_scatter); at most 12 local bits unless the buckets would be too many
  int lb = tb > 11 ? tb - 11 : 0;
  if (lb > 12) lb = 12;
  while (lb <= VS_MAX_LOCAL_BITS && ((ids + ((int64_t)1 << lb) - 1) >> lb) > VS_MAX_BUCKETS) ++lb;
  if (lb > VS_MAX_LOCAL_BITS) return false;
  S->R = R;
  S->E = E;
  S->n_src = n_src;
  S->lb = lb;
  S->nb = (int)((ids + ((int64_t)1 << lb) - 1) >> lb);
  S->nbp = (S->nb + 63) / 64 * 64;
  S->nbc = (S->nb + 1) / 2 * 2;
  S->ntiles = (E + VS_TILE - 1) / VS_TILE;
  S->ngroups = (S->ntiles + VS_GROUP - 1) / VS_GROUP;
  return true;
}

// Dynamic LDS of vs_scatter and vs_bucket.
size_t vs_scatter_lds(const VsShape &S) {
  return (size_t)S.nbc * sizeof(uint32_t) + (size_t)VS_WAVES * S.nbc * sizeof(uint16_t);
}
size_t vs_bucket_lds(const VsShape &S) {
  const size_t n_local = (size_t)1 << S.lb;
  const size_t small = VB_WAVES * ((n_local + 1) / 2) * sizeof(uint32_t) + (size_t)VB_STAGED * sizeof(uint32_t);
  const size_t large = VB_WAVES * n_local * sizeof(uint32_t);
  return small > large ? small : large;
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

// A launch with more dynamic LDS than the default limit (64 KB) has to be allowed once per kernel; the
// compute unit has 160 KB.  The largest size allowed so far is remembered per kernel (a benign race: two
// threads may both ask).
template <typename K>
bool vs_allow_lds(K kernel, size_t bytes) {
  static size_t allowed = 60 * 1024;
  if (bytes <= allowed) return true;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)bytes) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  allowed = bytes;
  return true;
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
  const size_t lds = vs_scatter_lds(S), blds = vs_bucket_lds(S);
  const bool lds_ok = edgeT != nullptr
                          ? vs_allow_lds(&vs_scatter<false>, lds) && vs_allow_lds(&vs_bucket<true>, blds)
                          : vs_allow_lds(&vs_scatter<true>, lds) && vs_allow_lds(&vs_bucket<false>, blds);
  if (!lds_ok) return HC_ELAUNCH;
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
  if (edgeT != nullptr) {
    vs_scatter<false><<<tgrid, dim3(VS_THREADS), lds, st>>>(ptr, key32, tile_count, group_count, bucket_off, pairs,
                                                           rows, S);
    vs_bucket<true><<<dim3((unsigned)S.nb), dim3(VB_THREADS), blds, st>>>(pairs, bucket_off, rows, ptrT, rowT, edgeT,
                                                                        S);
  } else {
    vs_scatter<true><<<tgrid, dim3(VS_THREADS), lds, st>>>(ptr, key32, tile_count, group_count, bucket_off, pairs,
                                                          rows, S);
    vs_bucket<false><<<dim3((unsigned)S.nb), dim3(VB_THREADS), blds, st>>>(pairs, bucket_off, rows, ptrT, rowT, edgeT,
                                                                         S);
  }
  return hc_launch_status();
}
