// Gradient-based cache admission ("grad_check"): row scores, the threshold /
// staleness test, the admission mask, ring-slot assignment in row order and the
// history-table scatter-update.
//
// Reference semantics: record_history_kernel_used_mask
// (/root/reference/src/cpp/src/grad_check.cu:6-46) for the ring insert and the
// predicate on precomputed scores; HistoryCache.update_history
// (/root/reference/hiscache/history_cache.py:205-254) for the L2 score, the
// strict "<" test and the append-only variant; HistoryTable.record_history
// (/root/reference/hiscache/history_table.py:161) for the L1 score.
//
// The reference takes ring slots with atomicInc in arrival order
// (grad_check.cu:25), so its slot numbering changes from run to run.  Here the
// k-th admitted row (in row order) gets slot (header + k) mod capacity:
//   pass 1  score + predicate per row, mask byte, admitted count per 64-row tile
//   pass 2  one block scans the counts of 32-tile chunks (exclusive), advances the header
//           (calls of up to 65 536 rows go without it: pass 3 adds the tile counts up itself)
//   pass 3  per tile: ballot-rank the mask, un-map old owners, map, copy rows
// Pass 1 is the only pass that touches the gradient matrix; pass 3 only touches
// admitted rows, so HBM traffic is the algorithmic minimum.
#include "hc_common.h"

#include <mutex>

namespace {

constexpr int GC_TILE = 64;                                   // rows per block (= one ballot)
constexpr int GC_ROWS_PER_WAVE = GC_TILE / HC_WAVES_PER_BLOCK;  // 16

// Scalars shared between the passes (workspace prefix).
struct GcScalars {
  int64_t header_old;  // header before this call
  int64_t admitted;    // number of admitted rows
  int64_t written;     // append mode: rows that fit below capacity
  int64_t pad[5];
};

__device__ __forceinline__ float fold(float acc, float x, int norm_kind) {
  return norm_kind == HC_NORM_L2 ? __fmaf_rn(x, x, acc) : acc + fabsf(x);
}

// Partial score of one row held by this lane: elements e with (e/4)%64 == lane, increasing e.
__device__ __forceinline__ float row_partial_generic(const float *__restrict__ row, int64_t F,
                                                     int lane, int norm_kind) {
  float acc = 0.0f;
  const bool vec_ok = (reinterpret_cast<uintptr_t>(row) % 16) == 0;
  for (int64_t b = (int64_t)lane * 4; b < F; b += HC_WAVE * 4) {
    if (vec_ok && b + 3 < F) {
      const float4 v = *reinterpret_cast<const float4 *>(row + b);
      acc = fold(acc, v.x, norm_kind);
      acc = fold(acc, v.y, norm_kind);
      acc = fold(acc, v.z, norm_kind);
      acc = fold(acc, v.w, norm_kind);
    } else {
      for (int i = 0; i < 4; ++i)
        if (b + i < F) acc = fold(acc, row[b + i], norm_kind);
    }
  }
  return acc;
}

__device__ __forceinline__ float finish_score(float partial, int norm_kind) {
  const float tot = hc_wave_sum_butterfly(partial);
  return norm_kind == HC_NORM_L2 ? sqrtf(tot) : tot;  // correctly rounded (-fhip-fp32-correctly-rounded-divide-sqrt)
}

// Scores of the GC_ROWS_PER_WAVE rows owned by this wave; lane i ends up holding row i's score.
// CH > 0: F == 256*CH, 16-byte aligned rows, 8 rows of loads in flight.  CH == 0: any F.
template <int CH>
__device__ __forceinline__ float wave_scores(const float *__restrict__ grad, int64_t row0, int64_t M,
                                             int64_t F, int lane, int norm_kind) {
  float mine = 0.0f;
  if constexpr (CH > 0) {
    constexpr int RB = (CH <= 2) ? 8 : 4;
    for (int i0 = 0; i0 < GC_ROWS_PER_WAVE; i0 += RB) {
      float4 v[RB][CH];
#pragma unroll
      for (int i = 0; i < RB; ++i) {
        const int64_t r = row0 + i0 + i;
        if (r < M) {
          const float4 *p = reinterpret_cast<const float4 *>(grad + r * (256 * CH)) + lane;
#pragma unroll
          for (int k = 0; k < CH; ++k) {
            float t[4];
            hc_vec<float, 4>::load_nt(reinterpret_cast<const float *>(p + k * HC_WAVE), t);
            v[i][k] = make_float4(t[0], t[1], t[2], t[3]);
          }
        } else {
#pragma unroll
          for (int k = 0; k < CH; ++k) v[i][k] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
      }
#pragma unroll
      for (int i = 0; i < RB; ++i) {
        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < CH; ++k) {
          acc = fold(acc, v[i][k].x, norm_kind);
          acc = fold(acc, v[i][k].y, norm_kind);
          acc = fold(acc, v[i][k].z, norm_kind);
          acc = fold(acc, v[i][k].w, norm_kind);
        }
        const float s = finish_score(acc, norm_kind);
        if (lane == i0 + i) mine = s;
      }
    }
  } else if (F <= 256 && F % 4 == 0 && (reinterpret_cast<uintptr_t>(grad) % 16) == 0) {
    // narrow rows (one 16-byte piece per lane at most): the loads of 8 rows are in flight before the first
    // reduction, instead of a load and a reduction per row one after the other; same sums in the same order
    constexpr int RB = 8;
    const bool has = (int64_t)lane * 4 < F;
    for (int i0 = 0; i0 < GC_ROWS_PER_WAVE; i0 += RB) {
      float4 v[RB];
#pragma unroll
      for (int i = 0; i < RB; ++i) {
        const int64_t r = row0 + i0 + i;
        v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (r < M && has) v[i] = *(reinterpret_cast<const float4 *>(grad + r * F) + lane);
      }
#pragma unroll
      for (int i = 0; i < RB; ++i) {
        float acc = 0.0f;
        if (has) {
          acc = fold(acc, v[i].x, norm_kind);
          acc = fold(acc, v[i].y, norm_kind);
          acc = fold(acc, v[i].z, norm_kind);
          acc = fold(acc, v[i].w, norm_kind);
        }
        const float s = finish_score(acc, norm_kind);
        if (lane == i0 + i) mine = s;
      }
    }
  } else {
    for (int i = 0; i < GC_ROWS_PER_WAVE; ++i) {
      const int64_t r = row0 + i;
      float acc = 0.0f;
      if (r < M) acc = row_partial_generic(grad + r * F, F, lane, norm_kind);
      const float s = finish_score(acc, norm_kind);
      if (lane == i) mine = s;
    }
  }
  return mine;
}

// ---------------------------------------------------------------------------------------
// Pass 1.  PRED == false: scores only (counts untouched).
// ---------------------------------------------------------------------------------------
template <int CH, bool PRED>
__global__ __launch_bounds__(HC_BLOCK) void gc_pass1(
    const float *__restrict__ grad, const float *__restrict__ score_in, const int64_t *__restrict__ slot,
    const int32_t *__restrict__ age, const uint8_t *__restrict__ used, const float *__restrict__ thres_p,
    int32_t age_limit, int norm_kind, int cmp_kind, uint8_t *__restrict__ mask_out,
    float *__restrict__ score_out, uint8_t *__restrict__ tile_counts, int64_t M, int64_t F,
    const int64_t *__restrict__ header, GcScalars *__restrict__ scalars) {
  __shared__ int wave_cnt[HC_WAVES_PER_BLOCK];
  // without a pass 2 (small calls) pass 3 takes the header from here: nothing changes it in between
  if (PRED && scalars != nullptr && blockIdx.x == 0 && threadIdx.x == 0) scalars->header_old = header[0];
  const int lane = hc_lane();
  const int wave = hc_wave_in_block();
  const int64_t row0 = (int64_t)blockIdx.x * GC_TILE + wave * GC_ROWS_PER_WAVE;
  const int64_t r = row0 + lane;
  const bool owner = lane < GC_ROWS_PER_WAVE && r < M;

  float sc = 0.0f;
  if (grad != nullptr) sc = wave_scores<CH>(grad, row0, M, F, lane, norm_kind);
  else if (owner) sc = score_in[r];
  if (owner && score_out != nullptr) score_out[r] = sc;
  if (!PRED) return;

  bool admit = false;
  if (owner) {
    const float thres = thres_p[0];
    const bool pass = (cmp_kind == HC_CMP_LT) ? (sc < thres) : !(thres != 0.0f && sc > thres);
    const bool fresh = (slot[r] == -1) || (age != nullptr && age[r] >= age_limit);
    const bool use = (used == nullptr) || (used[r] != 0);
    admit = pass && fresh && use;
    mask_out[r] = admit ? 1 : 0;
  }
  const unsigned long long bal = __ballot(admit);
  if (lane == 0) wave_cnt[wave] = __popcll(bal);
  __syncthreads();
  if (threadIdx.x == 0) {
    int t = 0;
#pragma unroll
    for (int w = 0; w < HC_WAVES_PER_BLOCK; ++w) t += wave_cnt[w];
    tile_counts[blockIdx.x] = (uint8_t)t;   // at most GC_TILE = 64
  }
}

// ---------------------------------------------------------------------------------------
// Pass 2: header bookkeeping and the exclusive scan of the admitted counts, by one block.  Pass 1
// leaves one BYTE per tile (a count is at most 64); a thread takes a chunk of GC_CHUNK = 32
// consecutive tiles with two 16-byte loads and the block scans the chunk sums.  Pass 3 adds the
// counts of the tiles before its own inside the chunk (the same two loads, masked).  Scanning 32
// times fewer values than one 8-byte count per tile takes the pass from 27 to a few microseconds
// for 2 M rows; writing one offset per tile from this single block would cost most of that again.
// ring != 0: header = (header + A) mod capacity.   ring == 0 (append): rows beyond capacity
// are dropped, header += written, *overflow = dropped.
// ---------------------------------------------------------------------------------------
constexpr int GC_SCAN_THREADS = 1024;
constexpr int GC_CHUNK = 32;  // tiles per thread and sweep

__global__ __launch_bounds__(GC_SCAN_THREADS) void gc_pass2(const uint8_t *__restrict__ tile_counts,
                                                             int64_t n_tiles, int64_t *__restrict__ chunk_prefix,
                                                             GcScalars *__restrict__ sc,
                                                             int64_t *__restrict__ header,
                                                             int64_t capacity, int ring,
                                                             int64_t *__restrict__ overflow) {
  __shared__ int wave_tot[GC_SCAN_THREADS / HC_WAVE];
  __shared__ int64_t carry_s;
  const int lane = hc_lane();
  const int wave = (int)(threadIdx.x >> 6);
  if (threadIdx.x == 0) carry_s = 0;
  __syncthreads();
  const int64_t n_chunks = (n_tiles + GC_CHUNK - 1) / GC_CHUNK;
  for (int64_t base = 0; base < n_chunks; base += GC_SCAN_THREADS) {
    const int64_t t0 = (base + threadIdx.x) * GC_CHUNK;
    uint32_t w[GC_CHUNK / 4];
#pragma unroll
    for (int k = 0; k < GC_CHUNK / 4; ++k) w[k] = 0u;
    if (t0 + GC_CHUNK <= n_tiles) {        // tile_counts is 16-byte aligned
      const uint4 a = *reinterpret_cast<const uint4 *>(tile_counts + t0);
      const uint4 b = *reinterpret_cast<const uint4 *>(tile_counts + t0 + 16);
      w[0] = a.x; w[1] = a.y; w[2] = a.z; w[3] = a.w;
      w[4] = b.x; w[5] = b.y; w[6] = b.z; w[7] = b.w;
    } else {
#pragma unroll
      for (int k = 0; k < GC_CHUNK; ++k)
        if (t0 + k < n_tiles) w[k / 4] |= (uint32_t)tile_counts[t0 + k] << (8 * (k % 4));
    }
    int mine = 0;
#pragma unroll
    for (int k = 0; k < GC_CHUNK / 4; ++k) {
      const uint32_t s2 = (w[k] & 0x00ff00ffu) + ((w[k] >> 8) & 0x00ff00ffu);
      mine += (int)((s2 & 0xffffu) + (s2 >> 16));
    }
    // inclusive scan of the per-thread sums inside the wave (a sweep's total is below 2^22)
    int x = mine;
#pragma unroll
    for (int d = 1; d < HC_WAVE; d <<= 1) {
      const int y = __shfl_up(x, d, HC_WAVE);
      if (lane >= d) x += y;
    }
    if (lane == HC_WAVE - 1) wave_tot[wave] = x;
    __syncthreads();
    int wave_off = 0, sweep_total = 0;
    for (int wv = 0; wv < GC_SCAN_THREADS / HC_WAVE; ++wv) {
      const int t = wave_tot[wv];
      if (wv < wave) wave_off += t;
      sweep_total += t;
    }
    const int64_t carry = carry_s;
    if (base + threadIdx.x < n_chunks) chunk_prefix[base + threadIdx.x] = carry + wave_off + x - mine;
    __syncthreads();
    if (threadIdx.x == 0) carry_s = carry + sweep_total;
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const int64_t A = carry_s;
    const int64_t h = header[0];
    sc->header_old = h;
    sc->admitted = A;
    if (ring) {
      sc->written = A;
      header[0] = capacity > 0 ? (h + A) % capacity : 0;
    } else {
      int64_t room = capacity - h;
      if (room < 0) room = 0;
      const int64_t w = A < room ? A : room;
      sc->written = w;
      header[0] = h + w;
      if (overflow != nullptr) overflow[0] = A - w;
    }
  }
}

// Wave-cooperative row store with conversion to the table dtype.
template <typename TT>
__device__ __forceinline__ void store_row(const float *__restrict__ src, TT *__restrict__ dst, int64_t F,
                                          int lane) {
  const bool vec_ok = (F % 4 == 0) && (reinterpret_cast<uintptr_t>(src) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(dst) % (4 * sizeof(TT)) == 0);
  if (vec_ok) {
    for (int64_t c = (int64_t)lane * 4; c < F; c += HC_WAVE * 4) {
      float v[4];
      hc_vec<float, 4>::load_nt(src + c, v);
      hc_vec<TT, 4>::store_nt(dst + c, v);
    }
  } else {
    for (int64_t c = lane; c < F; c += HC_WAVE) dst[c] = hc_from_f32<TT>(src[c]);
  }
}

__device__ __forceinline__ void store_row_any(const float *src, void *table, int table_dtype,
                                              int64_t elem_off, int64_t F, int lane) {
  if (table_dtype == HC_F32) store_row<float>(src, static_cast<float *>(table) + elem_off, F, lane);
  else if (table_dtype == HC_F16) store_row<__half>(src, static_cast<__half *>(table) + elem_off, F, lane);
  else store_row<__hip_bfloat16>(src, static_cast<__hip_bfloat16 *>(table) + elem_off, F, lane);
}

__device__ __forceinline__ void store_relaxed(int64_t *p, int64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Rank of a tile's first admitted row among all admitted rows: its chunk's prefix plus the counts of
// the tiles before it inside the chunk.  Every thread of the block computes the same value from the
// same 40 bytes.  (The count array is padded to whole chunks; bytes of tiles that do not exist are
// never added, because they lie behind every existing tile of their chunk.)
__device__ __forceinline__ int64_t tile_offset(const uint8_t *__restrict__ tile_counts,
                                               const int64_t *__restrict__ chunk_prefix, int64_t tile) {
  const int64_t chunk = tile / GC_CHUNK;
  const int within = (int)(tile - chunk * GC_CHUNK);
  const uint4 a = *reinterpret_cast<const uint4 *>(tile_counts + chunk * GC_CHUNK);
  const uint4 b = *reinterpret_cast<const uint4 *>(tile_counts + chunk * GC_CHUNK + 16);
  const uint32_t w[GC_CHUNK / 4] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
  int sum = 0;
#pragma unroll
  for (int k = 0; k < GC_CHUNK / 4; ++k) {
    const int nb = within - 4 * k;   // bytes of this word that belong to earlier tiles
    const uint32_t m = nb >= 4 ? 0xffffffffu : (nb <= 0 ? 0u : ((1u << (8 * nb)) - 1u));
    const uint32_t v = w[k] & m;
    const uint32_t s2 = (v & 0x00ff00ffu) + ((v >> 8) & 0x00ff00ffu);
    sum += (int)((s2 & 0xffffu) + (s2 >> 16));
  }
  return chunk_prefix[chunk] + sum;
}

// ---------------------------------------------------------------------------------------
// Pass 3 (ring): per tile, rank the admitted rows, un-map old owners, map, copy.
// The map work of a tile is done by the lanes of wave 0 side by side (one row per lane): the
// slots of a tile's admitted rows are consecutive, so their previous owners are one coalesced
// read, and the un-map compare-and-swaps of the whole tile are in flight together instead of
// one dependent chain per row in front of its copy.  The four waves then copy the admitted
// rows, GC_COPY_ROWS rows in flight per wave.
// SMALL: there was no pass 2 (at most GC_SMALL_TILES tiles): every block adds up the tile counts in
// front of its own tile itself, and block 0 advances the header.
// ---------------------------------------------------------------------------------------
constexpr int GC_COPY_ROWS = 4;
constexpr int GC_SMALL_TILES = 1024;   // 65 536 rows

// Sum of the four bytes of every word of v.
__device__ __forceinline__ int byte_sum4(uint4 v) {
  int t = 0;
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const uint32_t s2 = (w[k] & 0x00ff00ffu) + ((w[k] >> 8) & 0x00ff00ffu);
    t += (int)((s2 & 0xffffu) + (s2 >> 16));
  }
  return t;
}

// Rows of the tile copied by the calling wave: admitted rows of rank q0, q0+1, ... (GC_COPY_ROWS at a
// time, all loads in front of the stores); src_lane[j] (held by lane j) is the tile row of rank j.
template <typename TT, int CH>
__device__ __forceinline__ void copy_rows_fast(const float *__restrict__ emb, TT *__restrict__ table,
                                               int src_lane, int64_t tile0, int64_t slot0, int64_t capacity,
                                               int first_rank, int n_adm, int wave, int lane) {
  constexpr int F = 256 * CH;
  for (int q0 = first_rank + wave * GC_COPY_ROWS; q0 < n_adm; q0 += HC_WAVES_PER_BLOCK * GC_COPY_ROWS) {
    float v[GC_COPY_ROWS][CH][4];
#pragma unroll
    for (int u = 0; u < GC_COPY_ROWS; ++u) {
      if (q0 + u < n_adm) {
        const int rl = __builtin_amdgcn_readlane(src_lane, q0 + u);
        const float *p = emb + (tile0 + rl) * F + lane * 4;
#pragma unroll
        for (int k = 0; k < CH; ++k) hc_vec<float, 4>::load_nt(p + k * 256, v[u][k]);
      }
    }
#pragma unroll
    for (int u = 0; u < GC_COPY_ROWS; ++u) {
      if (q0 + u < n_adm) {
        const int64_t s = (slot0 + q0 + u) % capacity;
        TT *d = table + s * F + lane * 4;
#pragma unroll
        for (int k = 0; k < CH; ++k) hc_vec<TT, 4>::store_nt(d + k * 256, v[u][k]);
      }
    }
  }
}

// No barrier and no LDS: every wave of the block reads the tile's 64 mask bytes and offsets itself, so
// its first row loads are issued one memory round trip after the wave starts.
template <bool SMALL>
__global__ __launch_bounds__(HC_BLOCK) void gc_pass3_ring(
    const uint8_t *__restrict__ mask, const uint8_t *__restrict__ tile_counts,
    const int64_t *__restrict__ chunk_prefix, const GcScalars *__restrict__ sc, const float *__restrict__ emb,
    const int64_t *__restrict__ sub_to_full, void *__restrict__ table, int table_dtype, int64_t capacity,
    int64_t *__restrict__ full2slot, int64_t *__restrict__ slot2full, int64_t *__restrict__ checkin,
    int64_t *__restrict__ slot_out, int64_t *__restrict__ header, int64_t glb_iter_value,
    const int64_t *__restrict__ glb_iter_dev, int64_t M, int64_t F, int64_t n_tiles) {
  const int lane = hc_lane();
  const int wave = hc_wave_in_block();
  // the iteration number that admitted rows are stamped with: by value, or read from device memory by
  // callers whose launches are recorded once and replayed
  const int64_t glb_iter = glb_iter_dev != nullptr ? *glb_iter_dev : glb_iter_value;
  const int64_t tile0 = (int64_t)blockIdx.x * GC_TILE;
  const int64_t r = tile0 + lane;
  // everything that does not depend on anything else is requested first
  const bool m = r < M && mask[r] != 0;
  const int64_t full = (wave == 0 && r < M) ? sub_to_full[r] : 0;
  const int64_t header_old = sc->header_old;
  int64_t A, tile_off;
  if constexpr (SMALL) {
    // at most 1 024 tile counts of one byte: 16 per lane, summed over the wave
    const int64_t t0 = (int64_t)lane * 16;
    uint4 c = make_uint4(0u, 0u, 0u, 0u);
    if (t0 + 16 <= n_tiles) {
      c = *reinterpret_cast<const uint4 *>(tile_counts + t0);   // the count array is 16-byte aligned and padded
    } else {
      uint32_t w[4] = {0u, 0u, 0u, 0u};
      for (int k = 0; k < 16; ++k)
        if (t0 + k < n_tiles) w[k / 4] |= (uint32_t)tile_counts[t0 + k] << (8 * (k % 4));
      c = make_uint4(w[0], w[1], w[2], w[3]);
    }
    int all = byte_sum4(c);
    // counts of the tiles in front of this block's tile
    const int64_t mine = (int64_t)blockIdx.x;
    int before = 0;
    if (t0 + 16 <= mine) {
      before = all;
    } else if (t0 < mine) {
      const int nb = (int)(mine - t0);   // 1..15 leading bytes
      const uint32_t w[4] = {c.x, c.y, c.z, c.w};
      for (int k = 0; k < 4; ++k) {
        const int n = nb - 4 * k;
        const uint32_t msk = n >= 4 ? 0xffffffffu : (n <= 0 ? 0u : ((1u << (8 * n)) - 1u));
        const uint32_t v = w[k] & msk;
        const uint32_t s2 = (v & 0x00ff00ffu) + ((v >> 8) & 0x00ff00ffu);
        before += (int)((s2 & 0xffffu) + (s2 >> 16));
      }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
      before += __shfl_xor(before, d, HC_WAVE);
      all += __shfl_xor(all, d, HC_WAVE);
    }
    tile_off = before;
    A = all;
    // nobody reads the header in this launch (pass 1 left its value in sc->header_old)
    if (blockIdx.x == 0 && threadIdx.x == 0) header[0] = (header_old + A) % capacity;
  } else {
    A = sc->admitted;
    tile_off = tile_offset(tile_counts, chunk_prefix, (int64_t)blockIdx.x);
  }
  const unsigned long long bal = __ballot(m);
  const int n_adm = __popcll(bal);
  if (n_adm == 0 && slot_out == nullptr) return;
  const unsigned long long below = (1ull << lane) - 1ull;
  const int rank = __popcll(bal & below);
  const int64_t first_live = A > capacity ? A - capacity : 0;   // ranks below are overwritten later in this call
  // ranks of this tile that are dead on arrival: a prefix of the tile's ranks
  const int64_t dead64 = first_live - tile_off;
  const int first_rank = dead64 <= 0 ? 0 : (dead64 >= n_adm ? n_adm : (int)dead64);
  const int64_t slot0 = header_old + tile_off;                   // slot of rank q is (slot0 + q) % capacity

  if (wave == 0) {
    // the tile's map work, one row per lane: consecutive slots, so the previous owners are one
    // coalesced read and the un-map compare-and-swaps of the whole tile are in flight together
    if (m) {
      if (rank < first_rank) {
        // inserted and evicted again within this call: net effect is "not cached"
        store_relaxed(full2slot + full, -1);
      } else {
        const int64_t s = (slot0 + rank) % capacity;
        const int64_t old = slot2full[s];
        if (old != -1) {
          unsigned long long expect = (unsigned long long)s;
          __hip_atomic_compare_exchange_strong(reinterpret_cast<unsigned long long *>(full2slot + old),
                                               &expect, (unsigned long long)(int64_t)-1, __ATOMIC_RELAXED,
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // The un-map above and this store may land in either order when `old` is this call's own node of
        // another row: the compare-and-swap only clears an entry that still names the slot, so the new
        // mapping survives both orders.  This row's own node and slot are touched by this lane only.
        store_relaxed(full2slot + full, s);
        slot2full[s] = full;
        if (checkin != nullptr) checkin[s] = glb_iter;
      }
    }
    if (slot_out != nullptr && r < M) slot_out[r] = m ? (slot0 + rank) % capacity : -1;
  }
  if (n_adm == 0) return;
  // lane j learns which tile row has rank j: admitted lanes push their lane number to lane `rank`,
  // the others to the lanes behind the admitted ones (a permutation of the 64 lanes)
  const int target = m ? rank : n_adm + (lane - rank);
  const int src_lane = __builtin_amdgcn_ds_permute(target << 2, lane);
  const bool fast = (F % 256 == 0) && (F / 256 <= 4) && (reinterpret_cast<uintptr_t>(emb) % 16 == 0) &&
                    (reinterpret_cast<uintptr_t>(table) % 16 == 0);
  if (fast) {
#define HC_COPY(TT)                                                                                              \
  switch (F / 256) {                                                                                             \
    case 1: copy_rows_fast<TT, 1>(emb, static_cast<TT *>(table), src_lane, tile0, slot0, capacity, first_rank, n_adm, wave, lane); break; \
    case 2: copy_rows_fast<TT, 2>(emb, static_cast<TT *>(table), src_lane, tile0, slot0, capacity, first_rank, n_adm, wave, lane); break; \
    case 3: copy_rows_fast<TT, 3>(emb, static_cast<TT *>(table), src_lane, tile0, slot0, capacity, first_rank, n_adm, wave, lane); break; \
    default: copy_rows_fast<TT, 4>(emb, static_cast<TT *>(table), src_lane, tile0, slot0, capacity, first_rank, n_adm, wave, lane); break; \
  }
    if (table_dtype == HC_F32) { HC_COPY(float) }
    else if (table_dtype == HC_F16) { HC_COPY(__half) }
    else { HC_COPY(__hip_bfloat16) }
#undef HC_COPY
    return;
  }
  for (int q = first_rank + wave; q < n_adm; q += HC_WAVES_PER_BLOCK) {
    const int rl = __builtin_amdgcn_readlane(src_lane, q);
    const int64_t s = (slot0 + q) % capacity;
    store_row_any(emb + (tile0 + rl) * F, table, table_dtype, s * F, F, lane);
  }
}

// ---------------------------------------------------------------------------------------
// Append mode (HistoryCache.update_history): invalidation, then copy + map.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(HC_BLOCK) void gc_append_invalidate(
    const GcScalars *__restrict__ sc, int64_t H, int64_t F_in, int64_t *__restrict__ full2embed,
    const int64_t *__restrict__ embed2full, const int64_t *__restrict__ feat2full, int64_t n_feat,
    int64_t max_feat_span, int64_t M) {
  const int64_t h = sc->header_old;
  const int64_t w = sc->written;
  const int64_t t = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  // (a) feature slots overlapped by [h, h+w) embedding rows (history_cache.py:223-226)
  if (t < max_feat_span && feat2full != nullptr && w >= 0) {
    const int64_t b = h * H / F_in;
    int64_t e = ((h + w) * H + F_in - 1) / F_in;
    if (e > n_feat) e = n_feat;
    const int64_t i = b + t;
    if (i < e) {
      const int64_t f = feat2full[i];
      if (f >= 0) full2embed[f] = -1;
    }
  }
  // (b) previous owners of the overwritten embedding slots (history_cache.py:230-240)
  if (t < M && t < w) {
    const int64_t f = embed2full[h + t];
    if (f >= 0) {
      const int64_t v = full2embed[f];
      if (v >= h && v < h + w) full2embed[f] = -1;
    }
  }
}

__global__ __launch_bounds__(HC_BLOCK) void gc_pass3_append(
    const uint8_t *__restrict__ mask, const uint8_t *__restrict__ tile_counts,
    const int64_t *__restrict__ chunk_prefix, const GcScalars *__restrict__ sc, const float *__restrict__ emb,
    const int64_t *__restrict__ sub_to_full, float *__restrict__ buffer, int64_t H,
    int64_t *__restrict__ full2embed, int64_t *__restrict__ embed2full, int64_t M) {
  __shared__ int local_rows[GC_TILE];
  __shared__ int n_admitted_s;
  const int lane = hc_lane();
  const int wave = hc_wave_in_block();
  const int64_t tile0 = (int64_t)blockIdx.x * GC_TILE;
  const int64_t header_old = sc->header_old;
  const int64_t written = sc->written;
  const int64_t tile_off = tile_offset(tile_counts, chunk_prefix, (int64_t)blockIdx.x);
  if (wave == 0) {
    const int64_t r = tile0 + lane;
    const bool m = r < M && mask[r] != 0;
    const unsigned long long bal = __ballot(m);
    const int rank = __popcll(bal & ((1ull << lane) - 1ull));
    if (m) local_rows[rank] = lane;
    if (lane == 0) n_admitted_s = __popcll(bal);
  }
  __syncthreads();
  const int n_adm = n_admitted_s;
  for (int q = wave; q < n_adm; q += HC_WAVES_PER_BLOCK) {
    const int64_t k = tile_off + q;
    if (k >= written) continue;  // would land beyond the buffer
    const int64_t r = tile0 + local_rows[q];
    const int64_t s = header_old + k;
    store_row<float>(emb + r * H, buffer + s * H, H, lane);
    if (lane == 0) {
      const int64_t full = sub_to_full[r];
      full2embed[full] = s;
      embed2full[s] = full;
    }
  }
}

// Workspace: GcScalars | chunk_prefix[chunks] int64 | tile_counts[chunks * 32] uint8 (16-byte aligned).
struct GcLayout {
  size_t prefix, counts, total;
};
GcLayout gc_layout(int64_t M) {
  const int64_t tiles = M > 0 ? (M + GC_TILE - 1) / GC_TILE : 1;
  const int64_t chunks = (tiles + GC_CHUNK - 1) / GC_CHUNK;
  GcLayout L;
  L.prefix = sizeof(GcScalars);
  L.counts = hc_align_up(L.prefix + (size_t)chunks * sizeof(int64_t), 16);
  L.total = hc_align_up(L.counts + (size_t)chunks * GC_CHUNK, 256);
  return L;
}
size_t ws_bytes(int64_t M) { return gc_layout(M).total; }

template <bool PRED>
int launch_pass1(const float *grad, const float *score_in, const int64_t *slot, const int32_t *age,
                 const uint8_t *used, const float *thres, int32_t age_limit, int norm_kind, int cmp_kind,
                 uint8_t *mask_out, float *score_out, uint8_t *tile_counts, int64_t M, int64_t F,
                 hipStream_t st, const int64_t *header = nullptr, GcScalars *sc = nullptr) {
  const int64_t tiles = (M + GC_TILE - 1) / GC_TILE;
  if (!hc_grid_ok(tiles)) return HC_EUNSUPPORTED;
  dim3 g((unsigned)tiles), b(HC_BLOCK);
  const bool fast = grad != nullptr && (F % 256 == 0) && (F / 256 <= 4) &&
                    (reinterpret_cast<uintptr_t>(grad) % 16 == 0);
#define HC_P1(CH)                                                                                    \
  gc_pass1<CH, PRED><<<g, b, 0, st>>>(grad, score_in, slot, age, used, thres, age_limit, norm_kind,  \
                                      cmp_kind, mask_out, score_out, tile_counts, M, F, header, sc)
  if (fast && F == 256) HC_P1(1);
  else if (fast && F == 512) HC_P1(2);
  else if (fast && F == 768) HC_P1(3);
  else if (fast && F == 1024) HC_P1(4);
  else HC_P1(0);
#undef HC_P1
  return hc_launch_status();
}

}  // namespace

extern "C" size_t hc_grad_check_workspace_bytes(int64_t M) { return M < 0 ? 0 : ws_bytes(M); }

extern "C" int hc_row_scores(const float *grad, float *score, int64_t M, int64_t F, int norm_kind,
                             void *stream) {
  HC_REQUIRE(M >= 0 && F > 0);
  HC_REQUIRE(norm_kind == HC_NORM_L2 || norm_kind == HC_NORM_L1);
  if (M == 0) return HC_OK;
  HC_REQUIRE(grad && score);
  return launch_pass1<false>(grad, nullptr, nullptr, nullptr, nullptr, nullptr, 0, norm_kind, 0, nullptr,
                             score, nullptr, M, F, static_cast<hipStream_t>(stream));
}

namespace {
int grad_check_launch(const float *grad, const float *score_in, const float *emb, const int64_t *slot,
                      const int32_t *age, const uint8_t *used, const int64_t *sub_to_full, const float *thres,
                      int32_t age_limit, int norm_kind, int cmp_kind, uint8_t *mask_out, float *score_out,
                      int64_t *slot_out, void *table, int table_dtype, int64_t capacity, int64_t *full2slot,
                      int64_t *slot2full, int64_t *checkin, int64_t *header, int64_t glb_iter,
                      const int64_t *glb_iter_dev, int64_t M, int64_t F, void *workspace, size_t workspace_bytes,
                      void *stream) {
  HC_REQUIRE(M >= 0 && F > 0 && capacity > 0);
  HC_REQUIRE(norm_kind == HC_NORM_L2 || norm_kind == HC_NORM_L1);
  HC_REQUIRE(cmp_kind == HC_CMP_LT || cmp_kind == HC_CMP_NOT_GT);
  if (table_dtype < HC_F32 || table_dtype > HC_BF16) return HC_EDTYPE;
  HC_REQUIRE(header != nullptr);
  if (M == 0) return HC_OK;
  HC_REQUIRE((grad || score_in) && emb && slot && sub_to_full && thres && mask_out && table &&
             full2slot && slot2full);
  if (!workspace || workspace_bytes < ws_bytes(M) || reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
    return HC_EWORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  GcScalars *sc = static_cast<GcScalars *>(workspace);
  const GcLayout L = gc_layout(M);
  int64_t *chunk_prefix = reinterpret_cast<int64_t *>(static_cast<char *>(workspace) + L.prefix);
  uint8_t *tiles_buf = reinterpret_cast<uint8_t *>(workspace) + L.counts;
  const int64_t tiles = (M + GC_TILE - 1) / GC_TILE;

  const bool small = tiles <= GC_SMALL_TILES;
  int rc = launch_pass1<true>(grad, score_in, slot, age, used, thres, age_limit, norm_kind, cmp_kind,
                              mask_out, score_out, tiles_buf, M, F, st, header, small ? sc : nullptr);
  if (rc != HC_OK) return rc;
  if (small) {
    // two launches: every pass-3 block adds up the (at most 1 024) tile counts in front of it itself
    gc_pass3_ring<true><<<dim3((unsigned)tiles), dim3(HC_BLOCK), 0, st>>>(
        mask_out, tiles_buf, chunk_prefix, sc, emb, sub_to_full, table, table_dtype, capacity, full2slot, slot2full,
        checkin, slot_out, header, glb_iter, glb_iter_dev, M, F, tiles);
    return hc_launch_status();
  }
  gc_pass2<<<dim3(1), dim3(GC_SCAN_THREADS), 0, st>>>(tiles_buf, tiles, chunk_prefix, sc, header, capacity, 1,
                                                      nullptr);
  if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
  gc_pass3_ring<false><<<dim3((unsigned)tiles), dim3(HC_BLOCK), 0, st>>>(
      mask_out, tiles_buf, chunk_prefix, sc, emb, sub_to_full, table, table_dtype, capacity, full2slot, slot2full,
      checkin, slot_out, header, glb_iter, glb_iter_dev, M, F, tiles);
  return hc_launch_status();
}
}  // namespace

extern "C" int hc_grad_check(const float *grad, const float *score_in, const float *emb,
                             const int64_t *slot, const int32_t *age, const uint8_t *used,
                             const int64_t *sub_to_full, const float *thres, int32_t age_limit,
                             int norm_kind, int cmp_kind, uint8_t *mask_out, float *score_out,
                             int64_t *slot_out, void *table, int table_dtype, int64_t capacity,
                             int64_t *full2slot, int64_t *slot2full, int64_t *checkin, int64_t *header,
                             int64_t glb_iter, int64_t M, int64_t F, void *workspace,
                             size_t workspace_bytes, void *stream) {
  return grad_check_launch(grad, score_in, emb, slot, age, used, sub_to_full, thres, age_limit, norm_kind, cmp_kind,
                           mask_out, score_out, slot_out, table, table_dtype, capacity, full2slot, slot2full, checkin,
                           header, glb_iter, nullptr, M, F, workspace, workspace_bytes, stream);
}

extern "C" int hc_grad_check_dev(const float *grad, const float *score_in, const float *emb,
                                 const int64_t *slot, const int32_t *age, const uint8_t *used,
                                 const int64_t *sub_to_full, const float *thres, int32_t age_limit,
                                 int norm_kind, int cmp_kind, uint8_t *mask_out, float *score_out,
                                 int64_t *slot_out, void *table, int table_dtype, int64_t capacity,
                                 int64_t *full2slot, int64_t *slot2full, int64_t *checkin, int64_t *header,
                                 const int64_t *glb_iter_dev, int64_t M, int64_t F, void *workspace,
                                 size_t workspace_bytes, void *stream) {
  HC_REQUIRE(glb_iter_dev != nullptr);
  return grad_check_launch(grad, score_in, emb, slot, age, used, sub_to_full, thres, age_limit, norm_kind, cmp_kind,
                           mask_out, score_out, slot_out, table, table_dtype, capacity, full2slot, slot2full, checkin,
                           header, 0, glb_iter_dev, M, F, workspace, workspace_bytes, stream);
}

// ---------------------------------------------------------------------------------------
// hc_grad_check_static: the fused admission pass for callers that cannot allocate (code under
// stream capture, serving loops, harnesses that forbid hipMalloc).  Its scratch (the scalars, the
// chunk prefixes and the tile counts of gc_layout) lives in a file-scope device array instead of a
// caller workspace.  In host code the array's name is only a handle: its device address is
// looked up once per device with hipGetSymbolAddress and kept; the kernels take that address.
// Every GPU holds its own copy of the array until the process ends.  Nothing in it has to start at
// zero: pass 1 writes every tile count pass 2 and pass 3 read, pass 2 writes the scalars and the
// chunk prefixes pass 3 reads, so a call is not disturbed by what the previous one left behind.
// ---------------------------------------------------------------------------------------
namespace {

constexpr int64_t GC_STATIC_MAX_ROWS = HC_GRAD_CHECK_STATIC_MAX_ROWS;   // rows per call
constexpr int64_t GC_STATIC_TILES = GC_STATIC_MAX_ROWS / GC_TILE;
constexpr int64_t GC_STATIC_CHUNKS = GC_STATIC_TILES / GC_CHUNK;
// GcScalars | chunk_prefix | tile_counts, rounded up as gc_layout rounds (checked at run time)
constexpr size_t GC_STATIC_BYTES =
    (sizeof(GcScalars) + (size_t)GC_STATIC_CHUNKS * sizeof(int64_t) + (size_t)GC_STATIC_CHUNKS * GC_CHUNK + 255) /
    256 * 256;

static __device__ __align__(256) unsigned char scratch[GC_STATIC_BYTES];

constexpr int GC_MAX_DEVICES = 64;
void *g_scratch_ptr[GC_MAX_DEVICES];   // device address of `scratch`, per device (nullptr: not looked up yet)
std::mutex g_scratch_mutex;

// Device address of this device's copy of `scratch`; nullptr on failure.
void *static_scratch(int *status) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) { *status = HC_ENODEVICE; return nullptr; }
  if (dev < 0 || dev >= GC_MAX_DEVICES) { *status = HC_EUNSUPPORTED; return nullptr; }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void *p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      *status = HC_ELAUNCH;
      return nullptr;
    }
    g_scratch_ptr[dev] = p;
  }
  *status = HC_OK;
  return g_scratch_ptr[dev];
}

}  // namespace

extern "C" int hc_grad_check_static(const float *grad, const float *score_in, const float *emb,
                                    const int64_t *slot, const int32_t *age, const uint8_t *used,
                                    const int64_t *sub_to_full, const float *thres, int32_t age_limit,
                                    int norm_kind, int cmp_kind, uint8_t *mask_out, float *score_out,
                                    int64_t *slot_out, void *table, int table_dtype, int64_t capacity,
                                    int64_t *full2slot, int64_t *slot2full, int64_t *checkin,
                                    int64_t *header, int64_t glb_iter, int64_t M, int64_t F, void *stream) {
  HC_REQUIRE(M >= 0);
  if (M > GC_STATIC_MAX_ROWS || ws_bytes(M) > GC_STATIC_BYTES) return HC_EUNSUPPORTED;
  int rc = HC_OK;
  void *ws = static_scratch(&rc);
  if (ws == nullptr) return rc;
  return hc_grad_check(grad, score_in, emb, slot, age, used, sub_to_full, thres, age_limit, norm_kind,
                       cmp_kind, mask_out, score_out, slot_out, table, table_dtype, capacity, full2slot,
                       slot2full, checkin, header, glb_iter, M, F, ws, GC_STATIC_BYTES, stream);
}

extern "C" int hc_record_history(const float *buffer_new, float *buffer_all, const uint8_t *used_mask,
                                 const int64_t *sub_to_full, const int64_t *sub_to_history,
                                 int64_t *history_to_full, int64_t *full_to_history, int64_t *header,
                                 const float *score, const float *thres, int64_t *checkin_iter,
                                 int64_t glb_iter, int64_t M, int64_t history_num, int64_t history_size,
                                 void *workspace, size_t workspace_bytes, void *stream) {
  HC_REQUIRE(M >= 0 && history_size > 0 && history_num >= 0);
  if (M == 0 || history_num == 0) return HC_OK;
  HC_REQUIRE(score != nullptr);
  // mask lives behind the tile array in the workspace: the reference has no mask output
  const size_t base = ws_bytes(M);
  const size_t need = base + hc_align_up((size_t)M, 256);
  if (!workspace || workspace_bytes < need) return HC_EWORKSPACE;
  uint8_t *mask = static_cast<uint8_t *>(workspace) + base;
  return hc_grad_check(nullptr, score, buffer_new, sub_to_history, nullptr, used_mask, sub_to_full, thres,
                       0, HC_NORM_L2, HC_CMP_NOT_GT, mask, nullptr, nullptr, buffer_all, HC_F32,
                       history_num, full_to_history, history_to_full, checkin_iter, header, glb_iter, M,
                       history_size, workspace, base, stream);
}

extern "C" int hc_cache_append(const float *score, const float *thres, const float *emb,
                               const int64_t *sub2embed, const int64_t *sub_to_full, uint8_t *mask_out,
                               float *buffer, int64_t capacity, int64_t H, int64_t F_in,
                               int64_t *full2embed, int64_t *embed2full, const int64_t *feat2full,
                               int64_t n_feat, int64_t *header, int64_t *overflow, int64_t M,
                               void *workspace, size_t workspace_bytes, void *stream) {
  HC_REQUIRE(M >= 0 && H > 0 && F_in > 0 && capacity >= 0 && n_feat >= 0);
  HC_REQUIRE(header != nullptr);
  if (M == 0) return HC_OK;
  HC_REQUIRE(score && thres && emb && sub2embed && sub_to_full && mask_out && buffer && full2embed &&
             embed2full);
  HC_REQUIRE(feat2full != nullptr || n_feat == 0);
  if (!workspace || workspace_bytes < ws_bytes(M) || reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
    return HC_EWORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  GcScalars *sc = static_cast<GcScalars *>(workspace);
  const GcLayout L = gc_layout(M);
  int64_t *chunk_prefix = reinterpret_cast<int64_t *>(static_cast<char *>(workspace) + L.prefix);
  uint8_t *tiles_buf = reinterpret_cast<uint8_t *>(workspace) + L.counts;
  const int64_t tiles = (M + GC_TILE - 1) / GC_TILE;

  int rc = launch_pass1<true>(nullptr, score, sub2embed, nullptr, nullptr, thres, 0, HC_NORM_L2,
                              HC_CMP_LT, mask_out, nullptr, tiles_buf, M, H, st);
  if (rc != HC_OK) return rc;
  gc_pass2<<<dim3(1), dim3(GC_SCAN_THREADS), 0, st>>>(tiles_buf, tiles, chunk_prefix, sc, header, capacity, 0,
                                                      overflow);
  if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
  // worst-case span of feature slots covered by M embedding rows
  const int64_t max_feat_span = (M * H + F_in - 1) / F_in + 2;
  const int64_t span = max_feat_span > M ? max_feat_span : M;
  const int64_t iblocks = (span + HC_BLOCK - 1) / HC_BLOCK;
  if (!hc_grid_ok(iblocks)) return HC_EUNSUPPORTED;
  gc_append_invalidate<<<dim3((unsigned)iblocks), dim3(HC_BLOCK), 0, st>>>(
      sc, H, F_in, full2embed, embed2full, feat2full, n_feat, max_feat_span, M);
  if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
  gc_pass3_append<<<dim3((unsigned)tiles), dim3(HC_BLOCK), 0, st>>>(mask_out, tiles_buf, chunk_prefix, sc, emb,
                                                                    sub_to_full, buffer, H, full2embed,
                                                                    embed2full, M);
  return hc_launch_status();
}

// ---------------------------------------------------------------------------------------
// Eviction (HistoryTable.evict_by_staleness / evict_by_both,
// /root/reference/hiscache/history_table.py:189-251) as one launch.  Threads [0, M) handle the
// batch rows: a row with a slot and score >= *thres gives its slot up.  Threads [M, M + capacity)
// handle the slots: a slot with -1 < checkin <= stale_iter is given up.  Giving a slot up writes
// -1 into the owner's map entry, the slot's owner and its check-in; a slot reached from both
// sides gets the same three stores twice, so the result does not depend on the interleaving.
// ---------------------------------------------------------------------------------------
namespace {

__device__ __forceinline__ void evict_slot(int64_t s, int64_t *__restrict__ checkin,
                                           int64_t *__restrict__ slot2full, int64_t *__restrict__ full2slot,
                                           int64_t n_full) {
  const int64_t owner = slot2full[s];
  if (owner >= 0 && owner < n_full) full2slot[owner] = -1;
  slot2full[s] = -1;
  checkin[s] = -1;
}

__global__ __launch_bounds__(HC_BLOCK) void evict_kernel(const int64_t *__restrict__ sub2slot,
                                                          const float *__restrict__ score,
                                                          const float *__restrict__ thres, int64_t M,
                                                          int64_t stale_iter, int64_t *__restrict__ checkin,
                                                          int64_t *__restrict__ slot2full,
                                                          int64_t *__restrict__ full2slot, int64_t capacity,
                                                          int64_t n_full) {
  const int64_t t = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (t < M) {
    const int64_t s = sub2slot[t];
    if (s >= 0 && s < capacity && score[t] >= *thres) evict_slot(s, checkin, slot2full, full2slot, n_full);
    return;
  }
  const int64_t s = t - M;
  if (s >= capacity) return;
  const int64_t c = checkin[s];
  if (c > -1 && c <= stale_iter) evict_slot(s, checkin, slot2full, full2slot, n_full);
}

}  // namespace

extern "C" int hc_evict(const int64_t *sub2slot, const float *score, const float *thres, int64_t M,
                        int64_t stale_iter, int64_t *checkin, int64_t *slot2full, int64_t *full2slot,
                        int64_t capacity, int64_t n_full, void *stream) {
  HC_REQUIRE(M >= 0 && capacity >= 0 && n_full >= 0);
  if (M > 0) HC_REQUIRE(sub2slot && score && thres);
  if (M + capacity == 0) return HC_OK;
  HC_REQUIRE(checkin && slot2full && full2slot);
  const int64_t blocks = (M + capacity + HC_BLOCK - 1) / HC_BLOCK;
  if (!hc_grid_ok(blocks)) return HC_EUNSUPPORTED;
  evict_kernel<<<dim3((unsigned)blocks), dim3(HC_BLOCK), 0, static_cast<hipStream_t>(stream)>>>(
      sub2slot, score, thres, M, stale_iter, checkin, slot2full, full2slot, capacity, n_full);
  return hc_launch_status();
}


// ---------------------------------------------------------------------------------------
// Admission threshold as a quantile of the scores: the two order statistics that
// torch.quantile's linear interpolation reads (/root/reference/hiscache/history_cache.py:211,
// history_table.py:173), found by a radix select instead of a sort, and the interpolation in
// separately rounded fp32 steps.  One block, over keys that order like the floats (sign flipped
// for non-negative values, all bits for negative ones): the bits that all keys share are skipped,
// 8-bit digit passes below them narrow the keys down to at most 128, which are ranked against
// each other; that finds the lower statistic, one more pass the upper one where it is another
// key.  Up to 16 384 scores are read once and kept in registers (a sampled batch's 1-hop nodes
// are a few thousand); up to QT_MAX_N are read again in every pass.
// ---------------------------------------------------------------------------------------
namespace {

constexpr int QT_BLOCK = 1024;
constexpr int64_t QT_MAX_N = 1 << 17;

__device__ __forceinline__ uint32_t qt_key(float v) {
  const uint32_t b = __float_as_uint(v);
  if (v != v) return 0xffffffffu;        // NaN of either sign ranks last, as a sort places it
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float qt_value(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

constexpr int QT_WAVES = QT_BLOCK / HC_WAVE;
constexpr int QT_REG = 16;   // keys a thread keeps in registers: up to QT_BLOCK * QT_REG scores are read once
constexpr int QT_CAND = 128;   // this many keys or fewer are ranked against each other (m * m comparisons) instead of counted by digit

struct QtShared {
  int hist[QT_WAVES][256];   // one histogram per wave: lanes of different waves never meet on a counter
  int total[256];
  int pick[3];               // the bin that holds the rank, the keys in front of it, the keys inside it
  uint32_t next;             // smallest key above the selected one
  uint32_t range[2][QT_WAVES];   // the waves' smallest and largest keys
  alignas(16) uint32_t cand[QT_CAND];    // the keys that are left, padded with 0xffffffff (no key: NaN ends the kernel earlier)
  int n_cand;
  uint32_t result[3];        // the selected key, the rank's position among the keys equal to it, their number
};

// f(key) for every key of the thread: from its registers (REG) or from `score`.
template <bool REG, class F>
__device__ __forceinline__ void qt_for_each(const float *__restrict__ score, int64_t n, const uint32_t (&rk)[QT_REG],
                                            int nk, F f) {
  if constexpr (REG) {
#pragma unroll
    for (int j = 0; j < QT_REG; ++j)
      if (j < nk) f(rk[j]);
  } else {
    // eight loads issued together (a load per iteration would wait out the memory latency every time)
    constexpr int U = 8;
    for (int64_t base = threadIdx.x; base < n; base += (int64_t)QT_BLOCK * U) {
      float v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t i = base + (int64_t)u * QT_BLOCK;
        v[u] = score[i < n ? i : n - 1];
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (base + (int64_t)u * QT_BLOCK < n) f(qt_key(v[u]));
    }
  }
}

// The key of rank k (0-based) among the n scores; every thread returns it.  REG: the keys sit in the
// thread's registers (rk[0, nk)), otherwise they are read from `score` in every pass.  *k_in_bin and *n_equal
// return the rank's position among the keys equal to the result and how many those are.
// The smallest and the largest key fix the bits that all keys share (scores of one batch lie within a few
// octaves: a pass over the leading byte would tell nothing apart); digit passes of up to 8 bits below them go on
// only while more than QT_CAND keys are left, then the rest is ranked directly: a thread per key counts the
// smaller and the equal ones.  Ten thousand scores take one digit pass instead of four.
template <bool REG>
__device__ uint32_t qt_select(const float *__restrict__ score, int64_t n, const uint32_t (&rk)[QT_REG], int nk,
                              int64_t k, QtShared &sh, int64_t *k_in_bin, int *n_equal) {
  const int wave = (int)(threadIdx.x / HC_WAVE);
  const int lane = hc_lane();
  uint32_t mn = 0xffffffffu, mx = 0u;
  qt_for_each<REG>(score, n, rk, nk, [&](uint32_t key) {
    mn = key < mn ? key : mn;
    mx = key > mx ? key : mx;
  });
#pragma unroll
  for (int d = HC_WAVE / 2; d > 0; d >>= 1) {
    const uint32_t a = (uint32_t)__shfl_xor((int)mn, d, HC_WAVE), b = (uint32_t)__shfl_xor((int)mx, d, HC_WAVE);
    mn = a < mn ? a : mn;
    mx = b > mx ? b : mx;
  }
  if (lane == 0) {
    sh.range[0][wave] = mn;
    sh.range[1][wave] = mx;
  }
  if (threadIdx.x < QT_CAND) sh.cand[threadIdx.x] = 0xffffffffu;
  if (threadIdx.x == 0) sh.n_cand = 0;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < QT_WAVES; ++w) {
    const uint32_t a = sh.range[0][w], b = sh.range[1][w];
    mn = a < mn ? a : mn;
    mx = b > mx ? b : mx;
  }
  if (mn == mx) {                        // block-uniform: every score is the same
    *k_in_bin = k;
    *n_equal = (int)n;
    return mn;
  }
  const int top = 31 - __clz((int)(mn ^ mx));              // the highest bit in which two keys differ
  uint32_t mask = top == 31 ? 0u : ~((2u << top) - 1u);   // the bits above it are the same for all
  uint32_t prefix = mn & mask;
  int remaining = top + 1;                                 // undecided low bits
  int64_t left = n;                                        // keys that agree with the prefix
  while (remaining > 0 && left > QT_CAND) {                // block-uniform
    const int bits = remaining < 8 ? remaining : 8;
    const int shift = remaining - bits;
    const uint32_t digit_mask = (1u << bits) - 1u;
    for (int b = threadIdx.x; b < QT_WAVES * 256; b += QT_BLOCK) (&sh.hist[0][0])[b] = 0;
    __syncthreads();
    qt_for_each<REG>(score, n, rk, nk, [&](uint32_t key) {
      if ((key & mask) == prefix) atomicAdd(&sh.hist[wave][(key >> shift) & digit_mask], 1);
    });
    __syncthreads();
    if (threadIdx.x < 256) {
      int t = 0;
#pragma unroll
      for (int w = 0; w < QT_WAVES; ++w) t += sh.hist[w][threadIdx.x];
      sh.total[threadIdx.x] = t;
    }
    __syncthreads();
    if (threadIdx.x < HC_WAVE) {
      // the bin that holds rank k: the first wave scans the 256 counts, four bins per lane
      const int l = (int)threadIdx.x;
      const int c[4] = {sh.total[4 * l], sh.total[4 * l + 1], sh.total[4 * l + 2], sh.total[4 * l + 3]};
      const int mine = (c[0] + c[1]) + (c[2] + c[3]);
      int x = mine;
#pragma unroll
      for (int d = 1; d < HC_WAVE; d <<= 1) {
        const int y = __shfl_up(x, d, HC_WAVE);
        if (l >= d) x += y;
      }
      const unsigned long long reached = __ballot((int64_t)x > k);
      const int owner = reached != 0ull ? __builtin_ctzll(reached) : HC_WAVE - 1;
      if (l == owner) {
        // (indices known at compile time: an array indexed by a variable lives in scratch memory, and a kernel
        // with scratch memory starts more slowly)
        int before = x - mine, b = 0, inside = c[0];
#pragma unroll
        for (int t = 0; t < 3; ++t)
          if (b == t && (int64_t)before + c[t] <= k) {
            before += c[t];
            b = t + 1;
            inside = c[t + 1];
          }
        sh.pick[0] = 4 * l + b;
        sh.pick[1] = before;           // at most n < 2^31
        sh.pick[2] = inside;
      }
    }
    __syncthreads();
    prefix |= (uint32_t)sh.pick[0] << shift;
    mask |= digit_mask << shift;
    k -= sh.pick[1];
    left = sh.pick[2];
    remaining = shift;
    __syncthreads();
  }
  if (remaining == 0) {                  // every bit decided: the keys that are left are equal
    *k_in_bin = k;
    *n_equal = (int)left;
    return prefix;
  }
  // at most QT_CAND keys left: side by side in LDS (in any order), every one ranked by its own thread
  qt_for_each<REG>(score, n, rk, nk, [&](uint32_t key) {
    if ((key & mask) == prefix) sh.cand[atomicAdd(&sh.n_cand, 1)] = key;
  });
  __syncthreads();
  const int m = sh.n_cand;               // == left
  if ((int)threadIdx.x < m) {
    const uint32_t c = sh.cand[threadIdx.x];
    int less = 0, equal = 0;
    for (int j = 0; j < m; j += 4) {     // (the padding ranks above every key)
      const uint4 x = *reinterpret_cast<const uint4 *>(&sh.cand[j]);
      less += (int)(x.x < c) + (int)(x.y < c) + (int)(x.z < c) + (int)(x.w < c);
      equal += (int)(x.x == c) + (int)(x.y == c) + (int)(x.z == c) + (int)(x.w == c);
    }
    if ((int64_t)less <= k && k < (int64_t)less + equal) {   // threads with equal keys write the same words
      sh.result[0] = c;
      sh.result[1] = (uint32_t)(k - less);
      sh.result[2] = (uint32_t)equal;
    }
  }
  __syncthreads();
  *k_in_bin = (int64_t)sh.result[1];
  *n_equal = (int)sh.result[2];
  return sh.result[0];
}

// The smallest key above `key`; every thread returns it (0xffffffff when there is none).
template <bool REG>
__device__ uint32_t qt_next_above(const float *__restrict__ score, int64_t n, const uint32_t (&rk)[QT_REG], int nk,
                                  uint32_t key, QtShared &sh) {
  if (threadIdx.x == 0) sh.next = 0xffffffffu;
  __syncthreads();
  uint32_t m = 0xffffffffu;
  qt_for_each<REG>(score, n, rk, nk, [&](uint32_t x) {
    if (x > key && x < m) m = x;
  });
#pragma unroll
  for (int d = HC_WAVE / 2; d > 0; d >>= 1) {
    const uint32_t y = (uint32_t)__shfl_xor((int)m, d, HC_WAVE);
    m = y < m ? y : m;
  }
  if (hc_lane() == 0 && m != 0xffffffffu) atomicMin(&sh.next, m);
  __syncthreads();
  return sh.next;
}

// One block.  The order statistic of rank lo by four 8-bit passes; the one of rank hi = lo + 1 is the same key
// when the rank stays among the keys equal to it, else the smallest key above it (one more pass).
template <bool REG>
__device__ __forceinline__ void qt_block(const float *__restrict__ score, int64_t n, int64_t lo, int64_t hi, float w,
                                         float one_minus_w, float *__restrict__ out, QtShared &sh) {
  uint32_t rk[QT_REG];
  int nk = 0;
  int nan_seen = 0;                    // torch.quantile answers NaN when any score is NaN: so does this kernel
  if constexpr (REG) {
    // every load issued before the first use (behind a bounds branch each would wait for the one in front:
    // 0.5 us apiece); a load beyond the scores reads the last one again and is dropped
    float v[QT_REG];
#pragma unroll
    for (int j = 0; j < QT_REG; ++j) {
      const int64_t i = (int64_t)j * QT_BLOCK + threadIdx.x;
      v[j] = score[i < n ? i : n - 1];
    }
#pragma unroll
    for (int j = 0; j < QT_REG; ++j) {
      const int64_t i = (int64_t)j * QT_BLOCK + threadIdx.x;
      rk[j] = 0u;
      if (i < n) {
        rk[j] = qt_key(v[j]);
        nk = j + 1;
        if (rk[j] == 0xffffffffu) nan_seen = 1;
      }
    }
  } else {
    qt_for_each<false>(score, n, rk, 0, [&](uint32_t key) {
      if (key == 0xffffffffu) nan_seen = 1;
    });
  }
  nan_seen = __syncthreads_or(nan_seen);
  if (nan_seen) {                      // block-uniform
    if (threadIdx.x == 0) out[0] = __uint_as_float(0x7fc00000u);
    return;
  }
  int64_t k_in_bin = 0;
  int n_equal = 0;
  const uint32_t ka = qt_select<REG>(score, n, rk, nk, lo, sh, &k_in_bin, &n_equal);
  uint32_t kb = ka;
  if (hi != lo && k_in_bin + 1 >= (int64_t)n_equal) kb = qt_next_above<REG>(score, n, rk, nk, ka, sh);
  if (threadIdx.x == 0) {
    const float a = qt_value(ka), b = qt_value(kb);
    const float d = __fsub_rn(b, a);
    out[0] = w < 0.5f ? __fadd_rn(a, __fmul_rn(d, w)) : __fsub_rn(b, __fmul_rn(d, one_minus_w));
  }
}

template <bool REG>
__global__ __launch_bounds__(QT_BLOCK) __attribute__((amdgpu_waves_per_eu(4, 4))) void quantile_kernel(const float *__restrict__ score, int64_t n, int64_t lo,
                                                             int64_t hi, float w, float one_minus_w,
                                                             float *__restrict__ out) {
  __shared__ QtShared sh;
  qt_block<REG>(score, n, lo, hi, w, one_minus_w, out, sh);
}

// The same with the number of scores read from device memory (kept inside [1, n_max]) and the rank worked
// out here as the host works it out: pos = fp32(rate) * fp32(n - 1), lo = floor(pos), w = pos - lo, each
// step rounded to fp32.
template <bool REG>
__global__ __launch_bounds__(QT_BLOCK) __attribute__((amdgpu_waves_per_eu(4, 4))) void quantile_kernel_dev(const float *__restrict__ score,
                                                                 const int64_t *__restrict__ n_dev, int64_t n_max,
                                                                 float rate, float *__restrict__ out) {
  __shared__ QtShared sh;
  int64_t n = *n_dev;
  n = n < 1 ? 1 : (n < n_max ? n : n_max);
  const float pos = __fmul_rn(rate, (float)(n - 1));
  int64_t lo = (int64_t)floorf(pos);
  lo = lo < 0 ? 0 : (lo < n - 1 ? lo : n - 1);
  const int64_t hi = lo + 1 < n - 1 ? lo + 1 : n - 1;
  const float w = __fsub_rn(pos, (float)lo);
  qt_block<REG>(score, n, lo, hi, w, __fsub_rn(1.0f, w), out, sh);
}

// ---- more scores than one block takes: the same select by the whole chip ------------------------
// Four launches, one 8-bit digit each: every block replays the picks of the digits in front from the
// histograms of the earlier launches (256 counters each, one wave), counts its share of the scores whose key
// has that prefix in LDS and adds its 256 counts to the launch's histogram.  A lane keeps the count of the digit
// it saw last in a register and touches LDS when the digit changes: the keys of gradient norms share their
// leading digits, and a counter that every lane of a wave wants would serialise them.  A fifth launch finds
// the smallest key above the selected one when the upper order statistic is another key, a sixth writes the
// interpolation.  Workspace: QL_WORDS 32-bit words, cleared by a launch in front.
constexpr int QL_BLOCK = 1024;
constexpr int QL_MAX_BLOCKS = 256;    // every block ends with one atomic per counter: those on one address queue up
constexpr int QL_NAN = 4 * 256;       // workspace word: number of NaN scores
constexpr int QL_NEXT = 4 * 256 + 1;  // workspace word: smallest key above the selected one
constexpr int QL_WORDS = 4 * 256 + 2;
constexpr int64_t QL_FROM_N = 1 << 15;   // fewer scores go to the one block: its passes cost less than seven launches

struct QlPick {
  uint32_t prefix;    // the digits picked so far, in place
  int64_t k;          // the rank among the keys with that prefix
  uint32_t n_equal;   // how many keys have that prefix
};

// By one whole wave: the first `passes` digits of the key of rank k, from the launches' histograms.
__device__ QlPick ql_replay(const uint32_t *__restrict__ hist, int passes, int64_t k, int lane) {
  QlPick r{0u, k, 0u};
  for (int p = 0; p < passes; ++p) {
    const uint32_t *h = hist + p * 256;
    const uint32_t c[4] = {h[4 * lane], h[4 * lane + 1], h[4 * lane + 2], h[4 * lane + 3]};
    const long long mine = ((long long)c[0] + c[1]) + ((long long)c[2] + c[3]);
    long long x = mine;
#pragma unroll
    for (int d = 1; d < HC_WAVE; d <<= 1) {
      const long long y = __shfl_up(x, d, HC_WAVE);
      if (lane >= d) x += y;
    }
    const unsigned long long reached = __ballot(x > (long long)r.k);
    const int owner = reached != 0ull ? __builtin_ctzll(reached) : HC_WAVE - 1;
    long long before = x - mine;
    int b = 0;
    auto in_bin = c[0];                  // (indices known at compile time keep c out of scratch memory)
#pragma unroll
    for (int t = 0; t < 3; ++t)
      if (b == t && before + (long long)c[t] <= (long long)r.k) {
        before += c[t];
        b = t + 1;
        in_bin = c[t + 1];
      }
    const int bin = __shfl(4 * lane + b, owner, HC_WAVE);
    const long long front = __shfl(before, owner, HC_WAVE);
    const uint32_t inside = (uint32_t)__shfl((int)in_bin, owner, HC_WAVE);
    r.prefix |= (uint32_t)bin << (24 - 8 * p);
    r.k -= front;
    r.n_equal = inside;
  }
  return r;
}

__global__ void ql_clear(uint32_t *__restrict__ ws) {
  for (int i = threadIdx.x; i < QL_WORDS; i += blockDim.x) ws[i] = i == QL_NEXT ? 0xffffffffu : 0u;
}

// Calls f(key) for this thread's share of the scores.  VEC4 (score 16-byte aligned): four scores per load and
// two loads in flight; the last n % 4 scores go to the first threads of block 0.
template <bool VEC4, typename Fn>
__device__ __forceinline__ void ql_for_each_key(const float *__restrict__ score, int64_t n, Fn f) {
  const int64_t stride = (int64_t)gridDim.x * QL_BLOCK;
  const int64_t t = (int64_t)blockIdx.x * QL_BLOCK + threadIdx.x;
  if constexpr (VEC4) {
    const float4 *__restrict__ s4 = reinterpret_cast<const float4 *>(score);
    const int64_t n4 = n >> 2;
    for (int64_t i = t; i < n4; i += 2 * stride) {
      const float4 a = s4[i];
      const bool two = i + stride < n4;
      const float4 b = two ? s4[i + stride] : a;
      f(qt_key(a.x)); f(qt_key(a.y)); f(qt_key(a.z)); f(qt_key(a.w));
      if (two) { f(qt_key(b.x)); f(qt_key(b.y)); f(qt_key(b.z)); f(qt_key(b.w)); }
    }
    if (t < (n & 3)) f(qt_key(score[(n4 << 2) + t]));
  } else {
    for (int64_t i = t; i < n; i += stride) f(qt_key(score[i]));
  }
}

template <int PASS, bool VEC4>
__global__ __launch_bounds__(QL_BLOCK) void ql_pass(const float *__restrict__ score, int64_t n, int64_t k,
                                                     uint32_t *__restrict__ ws) {
  __shared__ uint32_t lh[256];
  __shared__ uint32_t s_prefix;
  if (threadIdx.x < HC_WAVE) {
    const QlPick pk = ql_replay(ws, PASS, k, (int)threadIdx.x);
    if (threadIdx.x == 0) s_prefix = pk.prefix;
  }
  if (threadIdx.x < 256) lh[threadIdx.x] = 0u;
  __syncthreads();
  const uint32_t prefix = s_prefix;
  constexpr int shift = 24 - 8 * PASS;
  constexpr uint32_t mask = PASS == 0 ? 0u : 0xffffffffu << (shift + 8);
  uint32_t cur = 0u, cnt = 0u, nan = 0u;
  ql_for_each_key<VEC4>(score, n, [&](uint32_t key) {
    if (PASS == 0 && key == 0xffffffffu) ++nan;
    if ((key & mask) == prefix) {
      const uint32_t d = (key >> shift) & 0xffu;
      if (d != cur) {
        if (cnt) atomicAdd(&lh[cur], cnt);
        cur = d;
        cnt = 0u;
      }
      ++cnt;
    }
  });
  if (cnt) atomicAdd(&lh[cur], cnt);
  if (PASS == 0 && nan) atomicAdd(&ws[QL_NAN], nan);
  __syncthreads();
  if (threadIdx.x < 256) {
    const uint32_t v = lh[threadIdx.x];
    if (v) atomicAdd(&ws[PASS * 256 + threadIdx.x], v);
  }
}

// The smallest key above the one of rank lo, when rank hi is not among the keys equal to it.
template <bool VEC4>
__global__ __launch_bounds__(QL_BLOCK) void ql_next(const float *__restrict__ score, int64_t n, int64_t lo,
                                                     int64_t hi, uint32_t *__restrict__ ws) {
  __shared__ uint32_t s_key, s_min;
  __shared__ int s_need;
  if (threadIdx.x < HC_WAVE) {
    const QlPick pk = ql_replay(ws, 4, lo, (int)threadIdx.x);
    if (threadIdx.x == 0) {
      s_key = pk.prefix;
      s_min = 0xffffffffu;
      s_need = hi != lo && pk.k + 1 >= (int64_t)pk.n_equal;
    }
  }
  __syncthreads();
  if (!s_need) return;                  // block-uniform
  const uint32_t key = s_key;
  uint32_t m = 0xffffffffu;
  ql_for_each_key<VEC4>(score, n, [&](uint32_t x) {
    if (x > key && x < m) m = x;
  });
#pragma unroll
  for (int d = HC_WAVE / 2; d > 0; d >>= 1) {
    const uint32_t y = (uint32_t)__shfl_xor((int)m, d, HC_WAVE);
    m = y < m ? y : m;
  }
  if (hc_lane() == 0 && m != 0xffffffffu) atomicMin(&s_min, m);
  __syncthreads();
  if (threadIdx.x == 0 && s_min != 0xffffffffu) atomicMin(&ws[QL_NEXT], s_min);
}

__global__ __launch_bounds__(HC_WAVE) void ql_final(int64_t lo, int64_t hi, float w, float one_minus_w,
                                                     const uint32_t *__restrict__ ws, float *__restrict__ out) {
  const QlPick pk = ql_replay(ws, 4, lo, (int)threadIdx.x);
  if (threadIdx.x != 0) return;
  if (ws[QL_NAN] != 0u) {
    out[0] = __uint_as_float(0x7fc00000u);
    return;
  }
  const uint32_t ka = pk.prefix;
  const uint32_t kb = (hi != lo && pk.k + 1 >= (int64_t)pk.n_equal) ? ws[QL_NEXT] : ka;
  const float a = qt_value(ka), b = qt_value(kb);
  const float d = __fsub_rn(b, a);
  out[0] = w < 0.5f ? __fadd_rn(a, __fmul_rn(d, w)) : __fsub_rn(b, __fmul_rn(d, one_minus_w));
}

}  // namespace

extern "C" int64_t hc_quantile_max_scores(void) { return QT_MAX_N; }

extern "C" int hc_quantile_threshold(const float *score, int64_t n, int64_t lo, int64_t hi, float w,
                                     float one_minus_w, float *out, void *stream) {
  HC_REQUIRE(score && out && n >= 1 && lo >= 0 && hi >= lo && hi < n && hi <= lo + 1);
  if (n > QT_MAX_N) return HC_EUNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (n <= (int64_t)QT_BLOCK * QT_REG)
    quantile_kernel<true><<<dim3(1), dim3(QT_BLOCK), 0, st>>>(score, n, lo, hi, w, one_minus_w, out);
  else
    quantile_kernel<false><<<dim3(1), dim3(QT_BLOCK), 0, st>>>(score, n, lo, hi, w, one_minus_w, out);
  return hc_launch_status();
}

extern "C" int hc_quantile_threshold_dev(const float *score, const int64_t *n_dev, int64_t n_max, float rate,
                                         float *out, void *stream) {
  HC_REQUIRE(score && n_dev && out && n_max >= 1 && rate >= 0.0f && rate <= 1.0f);
  if (n_max > QT_MAX_N) return HC_EUNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (n_max <= (int64_t)QT_BLOCK * QT_REG)
    quantile_kernel_dev<true><<<dim3(1), dim3(QT_BLOCK), 0, st>>>(score, n_dev, n_max, rate, out);
  else
    quantile_kernel_dev<false><<<dim3(1), dim3(QT_BLOCK), 0, st>>>(score, n_dev, n_max, rate, out);
  return hc_launch_status();
}

extern "C" size_t hc_quantile_workspace_bytes(int64_t n) {
  return n > QL_FROM_N ? (size_t)QL_WORDS * sizeof(uint32_t) : 0;
}

extern "C" int hc_quantile_threshold_ws(const float *score, int64_t n, int64_t lo, int64_t hi, float w,
                                        float one_minus_w, float *out, void *workspace, size_t workspace_bytes,
                                        void *stream) {
  if (n <= QL_FROM_N) return hc_quantile_threshold(score, n, lo, hi, w, one_minus_w, out, stream);
  HC_REQUIRE(score && out && lo >= 0 && hi >= lo && hi < n && hi <= lo + 1 && n <= (int64_t)0x7fffffff);
  HC_REQUIRE(workspace && workspace_bytes >= hc_quantile_workspace_bytes(n) &&
             (reinterpret_cast<uintptr_t>(workspace) & 3u) == 0);
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint32_t *ws = static_cast<uint32_t *>(workspace);
  int64_t blocks = (n + (int64_t)QL_BLOCK * 8 - 1) / ((int64_t)QL_BLOCK * 8);
  if (blocks > QL_MAX_BLOCKS) blocks = QL_MAX_BLOCKS;
  const dim3 grid((unsigned)blocks), block(QL_BLOCK);
  ql_clear<<<dim3(1), dim3(256), 0, st>>>(ws);
  if ((reinterpret_cast<uintptr_t>(score) & 15u) == 0) {
    ql_pass<0, true><<<grid, block, 0, st>>>(score, n, lo, ws);
    ql_pass<1, true><<<grid, block, 0, st>>>(score, n, lo, ws);
    ql_pass<2, true><<<grid, block, 0, st>>>(score, n, lo, ws);
    ql_pass<3, true><<<grid, block, 0, st>>>(score, n, lo, ws);
    ql_next<true><<<grid, block, 0, st>>>(score, n, lo, hi, ws);
  } else {
    ql_pass<0, false><<<grid, block, 0, st>>>(score, n, lo, ws);
    ql_pass<1, false><<<grid, block, 0, st>>>(score, n, lo, ws);
    ql_pass<2, false><<<grid, block, 0, st>>>(score, n, lo, ws);
    ql_pass<3, false><<<grid, block, 0, st>>>(score, n, lo, ws);
    ql_next<false><<<grid, block, 0, st>>>(score, n, lo, hi, ws);
  }
  ql_final<<<dim3(1), dim3(HC_WAVE), 0, st>>>(lo, hi, w, one_minus_w, ws, out);
  return hc_launch_status();
}
