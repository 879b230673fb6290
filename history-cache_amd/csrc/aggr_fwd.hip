// History-aware CSR gather-reduce, forward.
//
// One wavefront owns one destination row.  The row's neighbour ids are staged
// 64 at a time with one coalesced load (one id per lane); each id is then
// broadcast with v_readlane so the neighbour row's base address is
// wave-uniform and the 64 lanes read one contiguous span of the row with
// vector loads (16 bytes per lane when the row length allows).  Up to UNROLL
// neighbour rows are in flight per wave before the first add; the adds run in
// CSR order in fp32.  Rows of up to 256 edges are therefore summed in exactly
// the order a sequential CPU loop would use; longer rows (fast path only) are
// summed as four contiguous quarters combined left to right -- a fixed order,
// so results stay bit-reproducible.
//
// Semantics follow the reference kernels gen_fwd_history_v2,
// gen_fwd_history_v2_edge_value and gen_fwd_history_v2_edge_value_multi_head
// (/root/reference/src/cpp/src/history_aggr.cu:7-125); offsets are 64-bit
// (the reference truncates neighbour ids and offsets to 32-bit int, :19,34-35).
#include "hc_common.h"

#include <type_traits>

namespace {

// Rows with more edges than this are summed by the four waves of their block (quarter split).
// The CPU checker applies the same rule; the header documents it.
constexpr int64_t HC_LONG_ROW_EDGES = 256;

// Wave-cooperative copy of one row of a history buffer into an fp32 output row.
template <typename TH>
__device__ __forceinline__ void copy_row_typed(const TH *__restrict__ src, float *__restrict__ dst,
                                               int64_t F, int lane) {
  constexpr int V = 4;
  const bool vec_ok = (F % V == 0) && ((reinterpret_cast<uintptr_t>(src) % (sizeof(TH) * V)) == 0) &&
                      ((reinterpret_cast<uintptr_t>(dst) % 16) == 0);
  if (vec_ok) {
    for (int64_t c = (int64_t)lane * V; c < F; c += HC_WAVE * V) {
      float v[V];
      hc_vec<TH, V>::load(src + c, v);
      *reinterpret_cast<float4 *>(dst + c) = make_float4(v[0], v[1], v[2], v[3]);
    }
  } else {
    for (int64_t c = lane; c < F; c += HC_WAVE) dst[c] = hc_to_f32<TH>(src[c]);
  }
}

__device__ __forceinline__ void copy_row_any(const void *hbuf, int hist_dtype, int64_t elem_off,
                                             float *dst, int64_t F, int lane) {
  if (hist_dtype == HC_F32) {
    copy_row_typed<float>(static_cast<const float *>(hbuf) + elem_off, dst, F, lane);
  } else if (hist_dtype == HC_F16) {
    copy_row_typed<__half>(static_cast<const __half *>(hbuf) + elem_off, dst, F, lane);
  } else {
    copy_row_typed<__hip_bfloat16>(static_cast<const __hip_bfloat16 *>(hbuf) + elem_off, dst, F, lane);
  }
}

// ---------------------------------------------------------------------------------------
// Fast path: mean aggregation, row length F == 64 * VEC * CHUNKS elements exactly.
// src_mode == 0: per-destination-row substitution (hbuf row-aligned, any dtype).
// src_mode == 1: per-source substitution (hbuf is a table of the same dtype as vin).
// ---------------------------------------------------------------------------------------
// Sum of the neighbour rows of edges [begin, end), added to acc in edge order by the calling wave.
// STREAM: neighbour rows and ids are loaded with the non-temporal hint.  With per-source
// substitution every edge also looks its source up in the map, and the map (not the rows, which
// are too many to be reused) is what is worth keeping in the caches.
// WMODE 0: acc += row.  WMODE 1: acc = fma(row, edge_value[edge], acc).  WMODE 2: the row holds
// n_head heads side by side and every head has its own weight, edge_value[edge, head]; a lane's VEC
// elements of a chunk lie inside one head (hd[chunk]), whose weight the lane loads itself.
constexpr int W_NONE = 0, W_EDGE = 1, W_EDGE_HEAD = 2;
// Per-source substitution.  `bits` (nullable) holds one bit per source, set when the source has an entry in
// the map: a source whose bit is clear never touches the map, which costs a whole cache line per lookup.
// TH is the element type of the history table; when it differs from T the staged address carries a tag in
// its lowest bit (rows are at least 8-byte aligned) and the load of a neighbour row picks the element type
// from it -- the branch is wave-uniform, as the row address is.
struct FwdSrc {
  const int64_t *hmap;    // nullptr: no substitution
  const void *htab;
  int64_t hsize;
  const uint32_t *bits;
};
template <typename T, typename TH, int VEC, int CHUNKS, int UNROLL, bool STREAM, int WMODE>
__device__ __forceinline__ void fwd_accumulate(const int64_t *__restrict__ idx, const T *__restrict__ vin,
                                               const FwdSrc src, const float *__restrict__ ev,
                                               int n_head, const int (&hd)[CHUNKS],
                                               int64_t begin, int64_t end, int lane,
                                               float (&acc)[CHUNKS][VEC]) {
  constexpr int F = HC_WAVE * VEC * CHUNKS;
  constexpr bool WEIGHTED = WMODE != W_NONE;
  constexpr bool MIXED = !std::is_same<T, TH>::value;
  const TH *__restrict__ htab = static_cast<const TH *>(src.htab);
  for (int64_t base = begin; base < end; base += HC_WAVE) {
    const int64_t left = end - base;
    const int n = left < HC_WAVE ? (int)left : HC_WAVE;
    // Stage: lane l resolves the address of neighbour base+l.
    int64_t my_addr = 0;
    float my_w = 0.0f;
    if (lane < n) {
      const int64_t id = STREAM ? __builtin_nontemporal_load(idx + base + lane) : idx[base + lane];
      my_addr = reinterpret_cast<int64_t>(vin + id * F);
      if (src.hmap != nullptr) {
        const bool maybe = src.bits == nullptr || ((src.bits[id >> 5] >> (id & 31)) & 1u) != 0u;
        if (maybe) {
          const int64_t slot = src.hmap[id];
          if (slot != -1) my_addr = reinterpret_cast<int64_t>(htab + slot * src.hsize) | (MIXED ? 1 : 0);
        }
      }
      if constexpr (WMODE == W_EDGE) my_w = ev[base + lane];
    }
    for (int j = 0; j < n; j += UNROLL) {
      float v[UNROLL][CHUNKS][VEC];
      float wh[WMODE == W_EDGE_HEAD ? UNROLL : 1][CHUNKS];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if (j + u < n) {
          const int64_t a = hc_readlane64(my_addr, j + u);
          if (MIXED && (a & 1) != 0) {      // a row of the history table, in its own element type
            const TH *p = reinterpret_cast<const TH *>(a - 1) + lane * VEC;
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) {
              if constexpr (STREAM) hc_vec<TH, VEC>::load_nt(p + k * HC_WAVE * VEC, v[u][k]);
              else hc_vec<TH, VEC>::load(p + k * HC_WAVE * VEC, v[u][k]);
            }
          } else {
          const T *p = reinterpret_cast<const T *>(a) + lane * VEC;
#pragma unroll
          for (int k = 0; k < CHUNKS; ++k) {
            if constexpr (STREAM) hc_vec<T, VEC>::load_nt(p + k * HC_WAVE * VEC, v[u][k]);
            else hc_vec<T, VEC>::load(p + k * HC_WAVE * VEC, v[u][k]);
            if constexpr (WMODE == W_EDGE_HEAD) wh[u][k] = ev[(base + j + u) * n_head + hd[k]];
          }
          }
        } else {
#pragma unroll
          for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
            for (int i = 0; i < VEC; ++i) v[u][k][i] = 0.0f;
        }
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if constexpr (WMODE == W_EDGE_HEAD) {
          if (j + u < n) {
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
              for (int i = 0; i < VEC; ++i) acc[k][i] = __fmaf_rn(v[u][k][i], wh[u][k], acc[k][i]);
          }
        } else if constexpr (WEIGHTED) {
          // lanes past the row's end hold zero rows and a zero weight: fma(0, 0, acc) == acc
          const float w = j + u < n ? hc_readlane_f(my_w, j + u) : 0.0f;
          if (j + u < n) {
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
              for (int i = 0; i < VEC; ++i) acc[k][i] = __fmaf_rn(v[u][k][i], w, acc[k][i]);
          }
        } else {
#pragma unroll
          for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[k][i] += v[u][k][i];
        }
      }
    }
  }
}

// A block owns four consecutive destination rows, one per wave.  Rows of up to `long_thres`
// edges are summed by their wave, in CSR order.  Longer rows are then summed by the whole block:
// wave w takes the w-th contiguous quarter of the row's edges (quarter length ceil(deg/4)), sums
// it in CSR order, and wave 0 combines the four partial sums left to right,
// ((q0 + q1) + q2) + q3, before the division.  Without this a power-law block ends with a few
// waves grinding through multi-thousand-edge rows at one wave's memory parallelism.
// long_thres == 0 disables the split (every row is then summed strictly in CSR order).
constexpr int FWD_ROWS_PER_BLOCK = HC_WAVES_PER_BLOCK;
constexpr int FWD_XCD_CHUNK = 256;  // consecutive blocks (1024 rows) that share an XCD

// List of the long rows of a launch (optional, in caller-provided scratch): a pre-pass notes every
// row with more than `long_thres` edges, and the first `front` blocks of the grid sum those rows
// before anything else is scheduled, so that a multi-thousand-edge row overlaps with the bulk of
// the launch instead of finishing alone at its end.  Each listed row is summed exactly as an
// unlisted long row would be (same quarters, same order); the order of the list does not matter.
struct FwdLongList {
  int count;  // rows noted (may exceed cap: then the list is ignored)
  int cap;
  int pad[62];
};

struct FwdSched {
  FwdLongList *head;  // nullptr: no list
  int *rows;
  int front;          // blocks at the start of the grid that work through the list
};

__global__ void fwd_long_clear(FwdLongList *h, int cap) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    h->count = 0;
    h->cap = cap;
  }
}

// A block scans FWD_FIND_TILE rows, collects its long rows in LDS and takes one run of list slots
// with a single global atomic (one atomic per long row would serialise on the counter).
constexpr int FWD_FIND_ITEMS = 8;
constexpr int FWD_FIND_TILE = HC_BLOCK * FWD_FIND_ITEMS;

__global__ __launch_bounds__(HC_BLOCK) void fwd_long_find(const int64_t *__restrict__ ptr,
                                                           const int64_t *__restrict__ hmap_row, int64_t R,
                                                           int64_t long_thres, FwdLongList *__restrict__ h,
                                                           int *__restrict__ rows) {
  __shared__ int found[FWD_FIND_TILE];
  __shared__ int n_found;
  __shared__ int base;
  if (threadIdx.x == 0) n_found = 0;
  __syncthreads();
  const int64_t r0 = (int64_t)blockIdx.x * FWD_FIND_TILE;
#pragma unroll
  for (int it = 0; it < FWD_FIND_ITEMS; ++it) {
    const int64_t r = r0 + (int64_t)it * HC_BLOCK + threadIdx.x;
    if (r < R && ptr[r + 1] - ptr[r] > long_thres && (hmap_row == nullptr || hmap_row[r] == -1))
      found[atomicAdd(&n_found, 1)] = (int)r;
  }
  __syncthreads();
  const int n = n_found;
  if (n == 0) return;
  if (threadIdx.x == 0) base = atomicAdd(&h->count, n);
  __syncthreads();
  const int cap = h->cap;
  for (int i = threadIdx.x; i < n; i += HC_BLOCK)
    if (base + i < cap) rows[base + i] = found[i];
}

// One long row summed by the four waves of the calling block (all of them must call this).
template <typename T, typename TH, int VEC, int CHUNKS, int UNROLL, bool STREAM, int WMODE>
__device__ __forceinline__ void fwd_long_row(const int64_t *__restrict__ ptr, const int64_t *__restrict__ idx,
                                             const T *__restrict__ vin, const FwdSrc src,
                                             const float *__restrict__ ev, float *__restrict__ vout,
                                             int64_t lrow, int lane, int wave,
                                             float (*part)[HC_WAVE * VEC * CHUNKS]) {
  constexpr int F = HC_WAVE * VEC * CHUNKS;
  constexpr bool WEIGHTED = WMODE != W_NONE;
  static_assert(WMODE != W_EDGE_HEAD, "rows of several heads are never split");
  const int no_heads[CHUNKS] = {};
  const int64_t lb = ptr[lrow];
  const int64_t le = ptr[lrow + 1];
  const int64_t deg = le - lb;
  const int64_t q = (deg + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
  int64_t sb = lb + wave * q;
  int64_t se = sb + q;
  if (sb > le) sb = le;
  if (se > le) se = le;
  float acc[CHUNKS][VEC];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[c][i] = 0.0f;
  fwd_accumulate<T, TH, VEC, CHUNKS, UNROLL, STREAM, WMODE>(idx, vin, src, ev, 1, no_heads, sb, se, lane, acc);
  if (wave > 0) {
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
      for (int i = 0; i < VEC; ++i) part[wave - 1][(c * HC_WAVE + lane) * VEC + i] = acc[c][i];
  }
  __syncthreads();
  if (wave == 0) {
    const float fdeg = (float)(int)deg;
    float *__restrict__ orow = vout + lrow * F;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      float o[VEC];
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        float t2 = acc[c][i];
#pragma unroll
        for (int pw = 0; pw < HC_WAVES_PER_BLOCK - 1; ++pw) t2 += part[pw][(c * HC_WAVE + lane) * VEC + i];
        o[i] = WEIGHTED ? t2 : (deg > 0 ? t2 / fdeg : 0.0f);
      }
      if constexpr (STREAM) hc_store_f32_nt<VEC>(orow + c * HC_WAVE * VEC + lane * VEC, o);
      else hc_store_f32<VEC>(orow + c * HC_WAVE * VEC + lane * VEC, o);
    }
  }
  __syncthreads();
}

// WMODE == W_EDGE_HEAD: a row is n_head heads of F / n_head elements side by side (vin[n_src, n_head, F/n_head],
// edge_value[E, n_head]); such launches come with long_thres == 0 and no list, so every row is summed
// strictly in CSR order by its wave, and a history row copies hbuf[r, :hsize] once (hsize == F) or once
// per head (hsize == F / n_head).
template <typename T, typename TH, int VEC, int CHUNKS, int UNROLL, bool STREAM, int WMODE>
__global__ __launch_bounds__(HC_BLOCK) void fwd_mean_fast(
    const int64_t *__restrict__ ptr, const int64_t *__restrict__ idx, const T *__restrict__ vin,
    const int64_t *__restrict__ hmap, const void *__restrict__ hbuf, int hist_dtype, int64_t hsize,
    int src_mode, const uint32_t *__restrict__ src_bits, const float *__restrict__ ev, int n_head,
    float *__restrict__ vout, int64_t R, int64_t long_thres, FwdSched sched) {
  constexpr int F = HC_WAVE * VEC * CHUNKS;
  constexpr bool WEIGHTED = WMODE != W_NONE;
  // without heads the rows may be split: the split code is compiled for those modes only
  constexpr int LMODE = WMODE == W_EDGE_HEAD ? W_EDGE : WMODE;
  __shared__ float part[HC_WAVES_PER_BLOCK - 1][F];
  __shared__ int long_rows[FWD_ROWS_PER_BLOCK];
  __shared__ int n_long_s;
  const int lane = hc_lane();
  const int wave = hc_wave_in_block();
  const FwdSrc src{src_mode ? hmap : nullptr, hbuf, hsize, src_bits};
  // every thread of the grid reads the same two words, so the decision is uniform
  const int n_listed = sched.head != nullptr ? sched.head->count : 0;
  const bool listed = sched.head != nullptr && n_listed <= sched.head->cap;
  if ((int)blockIdx.x < sched.front) {
    if (!listed) return;
    for (int t = (int)blockIdx.x; t < n_listed; t += sched.front)
      fwd_long_row<T, TH, VEC, CHUNKS, UNROLL, STREAM, LMODE>(ptr, idx, vin, src, ev, vout,
                                                              (int64_t)sched.rows[t], lane, wave, part);
    return;
  }
  const int64_t row0 = hc_xcd_block<FWD_XCD_CHUNK>((int64_t)blockIdx.x - sched.front,
                                                   (int64_t)gridDim.x - sched.front) * FWD_ROWS_PER_BLOCK;
  const int64_t rest = R - row0;
  const int nrows = rest < FWD_ROWS_PER_BLOCK ? (int)rest : FWD_ROWS_PER_BLOCK;

  if (long_thres > 0) {
    if (threadIdx.x == 0) n_long_s = 0;
    __syncthreads();
  }

  float acc[CHUNKS][VEC];
  const int k = wave;
  if (k < nrows) {
    const int64_t row = row0 + k;
    float *__restrict__ orow = vout + row * F;
    bool hist = false;
    if (!src_mode && hmap != nullptr) hist = hmap[row] != -1;
    if (hist) {
      if (WMODE == W_EDGE_HEAD && hsize != F) {      // one history row shared by the heads
        const int64_t fh = F / n_head;
        for (int h = 0; h < n_head; ++h) copy_row_any(hbuf, hist_dtype, row * hsize, orow + h * fh, fh, lane);
      } else {
        copy_row_any(hbuf, hist_dtype, row * hsize, orow, F, lane);
      }
    } else {
      const int64_t begin = ptr[row];
      const int64_t end = ptr[row + 1];
      const int64_t deg = end - begin;
      if (long_thres > 0 && deg > long_thres) {
        // a listed row is summed by the front blocks
        if (!listed && lane == 0) long_rows[atomicAdd(&n_long_s, 1)] = k;
      } else {
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
          for (int i = 0; i < VEC; ++i) acc[c][i] = 0.0f;
        int hd[CHUNKS];
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) hd[c] = WMODE == W_EDGE_HEAD ? ((c * HC_WAVE + lane) * VEC) / (F / n_head) : 0;
        fwd_accumulate<T, TH, VEC, CHUNKS, UNROLL, STREAM, WMODE>(idx, vin, src, ev, n_head, hd, begin, end, lane,
                                                                  acc);
        const float fdeg = (float)(int)deg;
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
          float o[VEC];
#pragma unroll
          for (int i = 0; i < VEC; ++i) o[i] = WEIGHTED ? acc[c][i] : (deg > 0 ? acc[c][i] / fdeg : 0.0f);
          if constexpr (STREAM) hc_store_f32_nt<VEC>(orow + c * HC_WAVE * VEC + lane * VEC, o);
          else hc_store_f32<VEC>(orow + c * HC_WAVE * VEC + lane * VEC, o);
        }
      }
    }
  }
  if (long_thres <= 0 || listed) return;  // the whole grid takes the same branch
  __syncthreads();
  const int n_long = n_long_s;
  // The order in which long rows were noted does not matter: each is summed on its own.
  for (int t = 0; t < n_long; ++t)
    fwd_long_row<T, TH, VEC, CHUNKS, UNROLL, STREAM, LMODE>(ptr, idx, vin, src, ev, vout, row0 + long_rows[t], lane,
                                                            wave, part);
}

// ---------------------------------------------------------------------------------------
// Generic path: any F, optional per-edge weights, optional heads.  One wave per
// (row, head); columns are walked in tiles of 256; the neighbour list is re-read per tile.
// ---------------------------------------------------------------------------------------
template <typename T, bool WEIGHTED>
__global__ __launch_bounds__(HC_BLOCK) void fwd_generic(
    const int64_t *__restrict__ ptr, const int64_t *__restrict__ idx, const T *__restrict__ vin,
    const int64_t *__restrict__ hmap, const void *__restrict__ hbuf, int hist_dtype, int64_t hsize,
    int src_mode, const float *__restrict__ ev, int64_t H, float *__restrict__ vout, int64_t R,
    int64_t F) {
  constexpr int TILE_K = 4;
  const int lane = hc_lane();
  const int64_t vrow = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (vrow >= R * H) return;
  const int64_t row = vrow / H;
  const int64_t head = vrow - row * H;
  float *__restrict__ orow = vout + vrow * F;

  if (!src_mode && hmap != nullptr) {
    if (hmap[row] != -1) {
      const int64_t off = row * hsize + (hsize == F ? 0 : head * F);
      copy_row_any(hbuf, hist_dtype, off, orow, F, lane);
      return;
    }
  }
  const int64_t begin = ptr[row];
  const int64_t end = ptr[row + 1];
  const int64_t deg = end - begin;
  const float fdeg = (float)(int)deg;
  // per-source substitution may read a table of another element type than vin (hist_dtype)
  const bool same_type = hist_dtype == (std::is_same<T, float>::value ? HC_F32 : (std::is_same<T, __half>::value ? HC_F16 : HC_BF16));
  const size_t hesz = hist_dtype == HC_F32 ? 4 : 2;

  for (int64_t c0 = 0; c0 < F; c0 += HC_WAVE * TILE_K) {
    float acc[TILE_K];
#pragma unroll
    for (int k = 0; k < TILE_K; ++k) acc[k] = 0.0f;
    for (int64_t base = begin; base < end; base += HC_WAVE) {
      const int64_t left = end - base;
      const int n = left < HC_WAVE ? (int)left : HC_WAVE;
      int64_t my_addr = 0;
      int my_hist = 0;   // 1: the address is a row of the history table in another element type
      float my_w = 0.0f;
      if (lane < n) {
        const int64_t id = idx[base + lane];
        my_addr = reinterpret_cast<int64_t>(vin + (id * H + head) * F);
        if (src_mode && hmap != nullptr) {
          const int64_t slot = hmap[id];
          if (slot != -1) {
            my_addr = reinterpret_cast<int64_t>(static_cast<const char *>(hbuf) + slot * hsize * hesz);
            my_hist = same_type ? 0 : 1;
          }
        }
        if (WEIGHTED) my_w = ev[(base + lane) * H + head];
      }
      // GEN_UNROLL neighbour rows are loaded before the first add; the adds keep the edge order
      constexpr int GEN_UNROLL = 4;
      for (int j = 0; j < n; j += GEN_UNROLL) {
        float x[GEN_UNROLL][TILE_K];
        float w[GEN_UNROLL];
#pragma unroll
        for (int u = 0; u < GEN_UNROLL; ++u) {
          w[u] = 0.0f;
#pragma unroll
          for (int k = 0; k < TILE_K; ++k) x[u][k] = 0.0f;
          if (j + u < n) {
            const int64_t a = hc_readlane64(my_addr, j + u);
            const int other = __builtin_amdgcn_readlane(my_hist, j + u);
            w[u] = WEIGHTED ? hc_readlane_f(my_w, j + u) : 1.0f;
#pragma unroll
            for (int k = 0; k < TILE_K; ++k) {
              const int64_t c = c0 + k * HC_WAVE + lane;
              if (c >= F) continue;
              if (!other) x[u][k] = hc_to_f32<T>(reinterpret_cast<const T *>(a)[c]);
              else if (hist_dtype == HC_F32) x[u][k] = reinterpret_cast<const float *>(a)[c];
              else if (hist_dtype == HC_F16) x[u][k] = __half2float(reinterpret_cast<const __half *>(a)[c]);
              else x[u][k] = __bfloat162float(reinterpret_cast<const __hip_bfloat16 *>(a)[c]);
            }
          }
        }
#pragma unroll
        for (int u = 0; u < GEN_UNROLL; ++u) {
          if (j + u < n) {
#pragma unroll
            for (int k = 0; k < TILE_K; ++k) acc[k] = WEIGHTED ? __fmaf_rn(x[u][k], w[u], acc[k]) : acc[k] + x[u][k];
          }
        }
      }
    }
#pragma unroll
    for (int k = 0; k < TILE_K; ++k) {
      const int64_t c = c0 + k * HC_WAVE + lane;
      if (c < F) orow[c] = WEIGHTED ? acc[k] : (deg > 0 ? acc[k] / fdeg : 0.0f);
    }
  }
}

// Rows below this count are launched without the long-row list even when scratch is given: the two
// extra launches cost more than the list saves.
constexpr int64_t FWD_LIST_MIN_ROWS = 65536;
constexpr int FWD_FRONT_BLOCKS = 2048;
// Source tables below this size go without the one-bit-per-source filter in front of the map lookup:
// their map (8 bytes per source) stays in the L2s anyway.
constexpr int64_t FWD_BITS_MIN_SRC = (int64_t)1 << 20;

struct FwdScratch {
  void *ptr;
  size_t bytes;
};

// Workspace of a forward launch: the long-row list (large blocks), then one bit per source (per-source
// substitution over many sources).  Either part may be absent (0 bytes).
struct FwdWsLayout {
  size_t list_bytes, bits_off, bits_bytes, total;
};
FwdWsLayout fwd_ws_layout(int mode, int64_t R, int64_t E, int64_t n_src) {
  FwdWsLayout L{0, 0, 0, 0};
  if (R >= FWD_LIST_MIN_ROWS && E > HC_LONG_ROW_EDGES) {
    // at most E / (HC_LONG_ROW_EDGES + 1) rows can be long
    int64_t cap = E / (HC_LONG_ROW_EDGES + 1) + 1;
    if (cap > R) cap = R;
    L.list_bytes = hc_align_up(sizeof(FwdLongList) + (size_t)cap * sizeof(int), 256);
  }
  L.bits_off = L.list_bytes;
  if (mode == HC_SUBST_SRC && n_src >= FWD_BITS_MIN_SRC) L.bits_bytes = hc_align_up((size_t)((n_src + 63) / 64) * 8, 256);
  L.total = L.bits_off + L.bits_bytes;
  return L;
}

// bits[s] = (hmap[s] != -1), 64 sources per ballot.  The map is read with ordinary loads: this pass also
// brings it into the last-level cache in front of the launch that looks sources up in it.
__global__ __launch_bounds__(HC_BLOCK) void fwd_src_bits(const int64_t *__restrict__ hmap, int64_t n_src,
                                                          unsigned long long *__restrict__ bits) {
  const int lane = hc_lane();
  const int64_t stride = (int64_t)gridDim.x * HC_WAVES_PER_BLOCK * HC_WAVE;
  for (int64_t base = ((int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block()) * HC_WAVE; base < n_src;
       base += stride) {
    const bool has = base + lane < n_src && hmap[base + lane] != -1;
    const unsigned long long b = __ballot(has);
    if (lane == 0) bits[base / HC_WAVE] = b;
  }
}

template <typename T, int VEC, int CHUNKS>
int launch_fast(const int64_t *ptr, const int64_t *idx, const void *vin, const int64_t *hmap,
                const void *hbuf, int hist_dtype, int64_t hsize, int src_mode, const float *ev, int n_head,
                float *vout, int64_t R, int64_t n_src, FwdScratch ws, hipStream_t st) {
  constexpr int per = VEC * CHUNKS;
  constexpr int UNROLL = per >= 16 ? 4 : (per >= 4 ? 8 : 16);
  int64_t blocks = (R + FWD_ROWS_PER_BLOCK - 1) / FWD_ROWS_PER_BLOCK;
  FwdSched sched{nullptr, nullptr, 0};
  int64_t cap = 0;
  const int64_t long_thres = n_head > 1 ? 0 : (int64_t)HC_LONG_ROW_EDGES;   // rows of several heads are never split
  // the caller sized the workspace with hc_aggr_fwd_workspace_bytes(mode, R, E, n_src): the bitmap, when
  // there is one, takes the last bits_bytes bytes and the list what lies in front of it
  const uint32_t *src_bits = nullptr;
  const bool ws_ok = ws.ptr != nullptr && reinterpret_cast<uintptr_t>(ws.ptr) % 256 == 0;
  size_t list_room = ws_ok ? ws.bytes : 0;
  if (ws_ok && src_mode && hmap != nullptr && n_src >= FWD_BITS_MIN_SRC) {
    const size_t bb = hc_align_up((size_t)((n_src + 63) / 64) * 8, 256);
    if (ws.bytes >= bb) {
      list_room = (ws.bytes - bb) / 256 * 256;
      unsigned long long *bits = reinterpret_cast<unsigned long long *>(static_cast<char *>(ws.ptr) + list_room);
      fwd_src_bits<<<dim3(2048), dim3(HC_BLOCK), 0, st>>>(hmap, n_src, bits);
      src_bits = reinterpret_cast<const uint32_t *>(bits);
    }
  }
  if (n_head == 1 && list_room >= sizeof(FwdLongList) + sizeof(int) && R >= FWD_LIST_MIN_ROWS &&
      R <= 0x7fffffffLL) {
    cap = (int64_t)((list_room - sizeof(FwdLongList)) / sizeof(int));
    if (cap > R) cap = R;
    sched.head = static_cast<FwdLongList *>(ws.ptr);
    sched.rows = reinterpret_cast<int *>(static_cast<char *>(ws.ptr) + sizeof(FwdLongList));
    sched.front = (int)(cap < FWD_FRONT_BLOCKS ? cap : FWD_FRONT_BLOCKS);
    blocks += sched.front;
  }
  if (!hc_grid_ok(blocks)) return HC_EUNSUPPORTED;
  if (sched.head != nullptr) {
    fwd_long_clear<<<dim3(1), dim3(HC_WAVE), 0, st>>>(sched.head, (int)cap);
    fwd_long_find<<<dim3((unsigned)((R + FWD_FIND_TILE - 1) / FWD_FIND_TILE)), dim3(HC_BLOCK), 0, st>>>(
        ptr, src_mode ? nullptr : hmap, R, (int64_t)HC_LONG_ROW_EDGES, sched.head, sched.rows);
  }
#define HC_FWD_LAUNCH(TH, STREAM, WMODE)                                                                   \
  fwd_mean_fast<T, TH, VEC, CHUNKS, UNROLL, STREAM, WMODE><<<dim3((unsigned)blocks), dim3(HC_BLOCK), 0, st>>>( \
      ptr, idx, static_cast<const T *>(vin), hmap, hbuf, hist_dtype, hsize, src_mode, src_bits, ev, n_head, vout, R, \
      long_thres, sched)
  if (ev != nullptr && n_head > 1) HC_FWD_LAUNCH(T, false, W_EDGE_HEAD);
  else if (ev != nullptr) HC_FWD_LAUNCH(T, false, W_EDGE);
  else if (src_mode && hmap != nullptr) {
    // the table of a per-source substitution may be narrower than fp32 features
    if (std::is_same<T, float>::value && hist_dtype == HC_F16) HC_FWD_LAUNCH(__half, true, W_NONE);
    else if (std::is_same<T, float>::value && hist_dtype == HC_BF16) HC_FWD_LAUNCH(__hip_bfloat16, true, W_NONE);
    else HC_FWD_LAUNCH(T, true, W_NONE);
  } else HC_FWD_LAUNCH(T, false, W_NONE);
#undef HC_FWD_LAUNCH
  return hc_launch_status();
}

// Pick (VEC, CHUNKS) with F == 64*VEC*CHUNKS, VEC as wide as 16 bytes allows, CHUNKS <= 4.
template <typename T>
int dispatch_fast(int64_t F, const int64_t *ptr, const int64_t *idx, const void *vin,
                  const int64_t *hmap, const void *hbuf, int hist_dtype, int64_t hsize, int src_mode,
                  const float *ev, int n_head, float *vout, int64_t R, int64_t n_src, FwdScratch ws,
                  hipStream_t st, bool *handled) {
  // F is the whole row (all heads); with several heads a lane's vector must not straddle two of them
  *handled = true;
#define HC_FAST(V, C)                                                                              \
  if (F == 64 * (V) * (C) && (F / n_head) % (V) == 0)                                              \
    return launch_fast<T, V, C>(ptr, idx, vin, hmap, hbuf, hist_dtype, hsize, src_mode, ev, n_head, vout, R, n_src, \
                                ws, st);
  constexpr int VMAX = 16 / (int)sizeof(T);
  if constexpr (VMAX == 8) {
    HC_FAST(8, 1) HC_FAST(8, 2) HC_FAST(8, 3) HC_FAST(8, 4)
  }
  HC_FAST(4, 1) HC_FAST(4, 3)
  if constexpr (VMAX == 4) { HC_FAST(4, 2) HC_FAST(4, 4) }
  HC_FAST(2, 1) HC_FAST(2, 3)
  HC_FAST(1, 1) HC_FAST(1, 3)
#undef HC_FAST
  *handled = false;
  return HC_OK;
}

template <typename T>
int launch_generic(const int64_t *ptr, const int64_t *idx, const void *vin, const int64_t *hmap,
                   const void *hbuf, int hist_dtype, int64_t hsize, int src_mode, const float *ev,
                   int64_t H, float *vout, int64_t R, int64_t F, hipStream_t st) {
  const int64_t blocks = (R * H + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
  if (!hc_grid_ok(blocks)) return HC_EUNSUPPORTED;
  dim3 g((unsigned)blocks), b(HC_BLOCK);
  if (ev)
    fwd_generic<T, true><<<g, b, 0, st>>>(ptr, idx, static_cast<const T *>(vin), hmap, hbuf, hist_dtype,
                                          hsize, src_mode, ev, H, vout, R, F);
  else
    fwd_generic<T, false><<<g, b, 0, st>>>(ptr, idx, static_cast<const T *>(vin), hmap, hbuf,
                                           hist_dtype, hsize, src_mode, ev, H, vout, R, F);
  return hc_launch_status();
}

}  // namespace

namespace {
bool fast_shape(int64_t F, int in_dtype) {
  if (F <= 0 || F % 64 != 0) return false;
  const int vmax = in_dtype == HC_F32 ? 4 : 8;
  for (int v = vmax; v >= 1; v /= 2) {
    if (F % (64 * v) != 0) continue;
    const int64_t c = F / (64 * v);
    if (v == vmax) return c >= 1 && c <= 4;
    return c == 1 || c == 3;
  }
  return false;
}
}  // namespace

extern "C" int64_t hc_aggr_fwd_long_row_edges(int64_t F, int in_dtype) {
  if (in_dtype < HC_F32 || in_dtype > HC_BF16) return 0;
  return fast_shape(F, in_dtype) ? HC_LONG_ROW_EDGES : 0;
}

extern "C" size_t hc_aggr_fwd_workspace_bytes(int mode, int64_t R, int64_t E, int64_t n_src) {
  if (R < 0 || E < 0 || n_src < 0) return 0;
  return fwd_ws_layout(mode, R, E, n_src).total;
}

extern "C" int hc_aggr_fwd(int mode, const int64_t *ptr, const int64_t *idx, const void *vin,
                           int in_dtype, const int64_t *hmap, const void *hbuf, int hist_dtype,
                           int64_t hsize, const float *edge_value, int64_t n_head, float *vout,
                           int64_t R, int64_t F, int64_t n_src, void *workspace,
                           size_t workspace_bytes, void *stream) {
  const FwdScratch ws{workspace, workspace ? workspace_bytes : 0};
  HC_REQUIRE(R >= 0 && F > 0 && n_src >= 0 && n_head >= 1);
  if (R == 0) return HC_OK;
  HC_REQUIRE(ptr && vout);
  HC_REQUIRE(mode == HC_SUBST_ROW || mode == HC_SUBST_SRC);
  if (in_dtype < HC_F32 || in_dtype > HC_BF16) return HC_EDTYPE;
  if (hmap && (hist_dtype < HC_F32 || hist_dtype > HC_BF16)) return HC_EDTYPE;
  if (hmap) HC_REQUIRE(hbuf != nullptr && hsize > 0);
  if (n_head > 1) HC_REQUIRE(edge_value != nullptr);
  const int src_mode = (mode == HC_SUBST_SRC) ? 1 : 0;
  if (src_mode) {
    if (edge_value) return HC_EUNSUPPORTED;
    if (hmap) {
      HC_REQUIRE(hsize >= F);
      // the table has the features' element type, or the features are fp32 and the table is narrower
      if (hist_dtype != in_dtype && in_dtype != HC_F32) return HC_EUNSUPPORTED;
    }
  } else if (hmap) {
    HC_REQUIRE(hsize == F * n_head || (hsize >= F && n_head == 1) || hsize == F);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);

  const size_t hesz = hist_dtype == HC_F32 ? 4 : 2;
  const bool aligned = (reinterpret_cast<uintptr_t>(vin) % 16 == 0) &&
                       (reinterpret_cast<uintptr_t>(vout) % 16 == 0) &&
                       (!src_mode || !hmap ||
                        ((reinterpret_cast<uintptr_t>(hbuf) % 16 == 0) && ((hsize * hesz) % 16 == 0)));
  // weighted sums share the fast path; a history row of a weighted block copies hbuf[r, :F].  With several
  // heads the row of the fast path is all heads side by side (F * n_head elements).
  const bool weighted_ok = !edge_value || (!src_mode && (!hmap || hsize >= F));
  const int64_t Frow = F * n_head;
  if (n_head <= 64 && weighted_ok && aligned && vin != nullptr) {
    bool handled = false;
    int rc;
    const int nh = (int)n_head;
    if (in_dtype == HC_F32)
      rc = dispatch_fast<float>(Frow, ptr, idx, vin, hmap, hbuf, hist_dtype, hsize, src_mode, edge_value, nh, vout, R,
                                n_src, ws, st, &handled);
    else if (in_dtype == HC_F16)
      rc = dispatch_fast<__half>(Frow, ptr, idx, vin, hmap, hbuf, hist_dtype, hsize, src_mode, edge_value, nh, vout,
                                 R, n_src, ws, st, &handled);
    else
      rc = dispatch_fast<__hip_bfloat16>(Frow, ptr, idx, vin, hmap, hbuf, hist_dtype, hsize, src_mode,
                                         edge_value, nh, vout, R, n_src, ws, st, &handled);
    if (handled) return rc;
  }
  if (in_dtype == HC_F32)
    return launch_generic<float>(ptr, idx, vin, hmap, hbuf, hist_dtype, hsize, src_mode, edge_value,
                                 n_head, vout, R, F, st);
  if (in_dtype == HC_F16)
    return launch_generic<__half>(ptr, idx, vin, hmap, hbuf, hist_dtype, hsize, src_mode, edge_value,
                                  n_head, vout, R, F, st);
  return launch_generic<__hip_bfloat16>(ptr, idx, vin, hmap, hbuf, hist_dtype, hsize, src_mode,
                                        edge_value, n_head, vout, R, F, st);
}
