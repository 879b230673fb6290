// Typed CSR: the edges of every row regrouped by relation, so that one mean-aggregation launch
// over (row, relation) groups feeds the relational convolution
// (/root/reference/hiscache/history_model.py:248-270 does the grouping with a per-call sort inside
// cxgnncomp's RGCNOP_sorted; here it is two wave-per-row passes and one scan, no sort).
//
//   1. count   wave per row: lane k counts the row's kept edges of relation k
//   2. scan    group offsets: for up to 2^20 groups (sampled batches) the count kernel's last block (a
//              ticket the caller provides, left at zero) scans the row totals and the place kernel fills in
//              the offsets inside a row; otherwise the library's inclusive scan of all group sizes
//   3. place   wave per row: every kept edge goes to its group's next slot, in edge order
//
// An edge is kept when its relation is in [0, K), its source id is in [0, n_src) and, when a used
// mask is given, the mask holds for its source.
#include <cstring>

#include <rocprim/rocprim.hpp>

#include "hc_common.h"

namespace {

constexpr int TC_MAX_REL = HC_WAVE;  // one lane per relation
constexpr int64_t TC_SMALL_GROUPS = 1 << 20;   // (row, relation) groups that one block scans

struct TcEdge {
  int64_t src;
  int rel;
  bool ok;
};

__device__ __forceinline__ TcEdge tc_load(const int64_t *__restrict__ idx, const int64_t *__restrict__ et,
                                          const uint8_t *__restrict__ used, int64_t e, int64_t end, int K,
                                          int64_t n_src) {
  TcEdge r;
  r.src = -1;
  r.rel = -1;
  r.ok = false;
  if (e < end) {
    r.src = idx[e];
    const int64_t t = et[e];
    if (t >= 0 && t < K && r.src >= 0 && r.src < n_src) {
      r.rel = (int)t;
      r.ok = used == nullptr || used[r.src] != 0;
    }
  }
  return r;
}

__global__ __launch_bounds__(HC_BLOCK) void tc_count(const int64_t *__restrict__ ptr,
                                                      const int64_t *__restrict__ idx,
                                                      const int64_t *__restrict__ et,
                                                      const uint8_t *__restrict__ used,
                                                      int64_t *__restrict__ cnt, int64_t *__restrict__ deg,
                                                      int64_t *__restrict__ ptr2, int64_t R, int64_t E, int K,
                                                      int64_t n_src) {
  const int lane = hc_lane();
  const int64_t row = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (row == 0 && lane == 0) ptr2[0] = 0;
  if (row >= R) return;
  const int64_t begin = ptr[row];
  const int64_t full_end = ptr[row + 1];
  const int64_t end = full_end < E ? full_end : E;
  int c = 0;
  for (int64_t base = begin; base < end; base += HC_WAVE) {
    const TcEdge ed = tc_load(idx, et, used, base + lane, end, K, n_src);
    for (int k = 0; k < K; ++k) {
      const unsigned long long b = __ballot(ed.ok && ed.rel == k);
      if (lane == k) c += __popcll(b);
    }
  }
  if (lane < K) cnt[row * K + lane] = c;
  if (lane == 0) deg[row] = full_end - begin;
}

__device__ __forceinline__ int64_t tc_shfl_up64(int64_t v, int d) {
  const int lo = __shfl_up((int)(uint32_t)(uint64_t)v, d, HC_WAVE);
  const int hi = __shfl_up((int)(uint32_t)((uint64_t)v >> 32), d, HC_WAVE);
  return (int64_t)(((uint64_t)(uint32_t)hi << 32) | (uint64_t)(uint32_t)lo);
}

// Small blocks: only the ROW totals need a scan across the grid -- inside a row the K group offsets are a
// prefix over the lanes of the wave that owns the row.  The count kernel leaves row r's total in
// ptr2[(r + 1) * K]; the block that finishes last turns these R entries into their inclusive scan in place,
// which is their final value (the end of row r's last group); the place kernel derives the other K - 1
// offsets of its row from ptr2[r * K] and the row's counts and writes them.
constexpr int TCS_BLOCK = 1024;
constexpr int TCS_WAVES = TCS_BLOCK / HC_WAVE;

// p[(i + 1) * K] <- p[K] + ... + p[(i + 1) * K] for i < R, by one block of TCS_BLOCK threads; up to eight
// slabs of TCS_BLOCK entries are loaded together, then scanned one after the other.
__device__ __forceinline__ void tc_scan_row_totals(int64_t *__restrict__ p, int64_t R, int K, int64_t *s_wave) {
  constexpr int G = 8;
  const int lane = hc_lane();
  const int wave = (int)(threadIdx.x >> 6);
  int64_t carry = 0;
  for (int64_t base = 0; base < R; base += (int64_t)TCS_BLOCK * G) {
    int64_t c[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int64_t i = base + (int64_t)g * TCS_BLOCK + threadIdx.x;
      c[g] = i < R ? p[(i + 1) * K] : 0;
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (base + (int64_t)g * TCS_BLOCK >= R) break;          // uniform over the block
      const int64_t i = base + (int64_t)g * TCS_BLOCK + threadIdx.x;
      int64_t x = c[g];
#pragma unroll
      for (int d = 1; d < HC_WAVE; d <<= 1) {
        const int64_t y = tc_shfl_up64(x, d);
        if (lane >= d) x += y;
      }
      if (lane == HC_WAVE - 1) s_wave[wave] = x;
      __syncthreads();
      int64_t off = carry + x;
      int64_t slab = 0;
      for (int w = 0; w < TCS_WAVES; ++w) {
        const int64_t t = s_wave[w];
        if (w < wave) off += t;
        slab += t;
      }
      __syncthreads();
      carry += slab;
      if (i < R) p[(i + 1) * K] = off;
    }
  }
}

// tc_count for small blocks (row totals into ptr2, see above), and the scan of the totals by the block that
// arrives last (one device-scope release per block, by the thread that takes the ticket, behind the block's
// barrier; the ticket is zero again when the kernel ends)
__global__ __launch_bounds__(TCS_BLOCK) void tc_count_scan(const int64_t *__restrict__ ptr,
                                                            const int64_t *__restrict__ idx,
                                                            const int64_t *__restrict__ et,
                                                            const uint8_t *__restrict__ used,
                                                            int64_t *__restrict__ cnt, int64_t *__restrict__ deg,
                                                            int64_t *__restrict__ ptr2, int64_t R, int64_t E, int K,
                                                            int64_t n_src, unsigned *__restrict__ ticket) {
  __shared__ int64_t s_wave[TCS_WAVES];
  __shared__ int s_last;
  const int lane = hc_lane();
  const int64_t row = (int64_t)blockIdx.x * TCS_WAVES + hc_wave_in_block();
  if (row < R) {
    const int64_t begin = ptr[row];
    const int64_t full_end = ptr[row + 1];
    const int64_t end = full_end < E ? full_end : E;
    int c = 0, total = 0;
    for (int64_t base = begin; base < end; base += HC_WAVE) {
      const TcEdge ed = tc_load(idx, et, used, base + lane, end, K, n_src);
      total += __popcll(__ballot(ed.ok));
      for (int k = 0; k < K; ++k) {
        const unsigned long long b = __ballot(ed.ok && ed.rel == k);
        if (lane == k) c += __popcll(b);
      }
    }
    if (lane < K) cnt[row * K + lane] = c;
    if (lane == 0) {
      deg[row] = full_end - begin;
      ptr2[(row + 1) * K] = total;
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (threadIdx.x == 0) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    const unsigned t = atomicAdd(ticket, 1u);
    s_last = t == gridDim.x - 1 ? 1 : 0;
    if (t == gridDim.x - 1) atomicExch(ticket, 0u);
  }
  __syncthreads();
  if (!s_last) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  if (threadIdx.x == 0) ptr2[0] = 0;
  tc_scan_row_totals(ptr2, R, K, s_wave);
}

// ROW_BASE: ptr2 holds only the rows' end offsets (entries at multiples of K) and cnt the group sizes; the
// wave derives its row's other offsets and writes them.
template <bool ROW_BASE>
__global__ __launch_bounds__(HC_BLOCK) void tc_place(const int64_t *__restrict__ ptr,
                                                      const int64_t *__restrict__ idx,
                                                      const int64_t *__restrict__ et,
                                                      const uint8_t *__restrict__ used,
                                                      const int64_t *__restrict__ cnt,
                                                      int64_t *__restrict__ ptr2,
                                                      int64_t *__restrict__ idx2,
                                                      float *__restrict__ edge_weight, int64_t R, int64_t E,
                                                      int K, int64_t n_src) {
  const int lane = hc_lane();
  const int64_t row = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (row >= R) return;
  const int64_t begin = ptr[row];
  const int64_t full_end = ptr[row + 1];
  const int64_t end = full_end < E ? full_end : E;
  // what an edge of this row weighs in the row's mean over ALL its edges (kept or dropped)
  const float w = 1.0f / (float)(full_end - begin > 0 ? full_end - begin : 1);
  // lane k: next free slot of group (row, k)
  int64_t next;
  if constexpr (ROW_BASE) {
    const int64_t mine = lane < K ? cnt[row * K + lane] : 0;
    int64_t x = mine;                                          // inclusive prefix over the lanes
#pragma unroll
    for (int d = 1; d < HC_WAVE; d <<= 1) {
      const int64_t y = tc_shfl_up64(x, d);
      if (lane >= d) x += y;
    }
    next = ptr2[row * K] + x - mine;
    if (lane >= 1 && lane < K) ptr2[row * K + lane] = next;
  } else {
    next = lane < K ? ptr2[row * K + lane] : 0;
  }
  const unsigned long long below = lane == 0 ? 0ull : (~0ull >> (HC_WAVE - lane));
  for (int64_t base = begin; base < end; base += HC_WAVE) {
    const TcEdge ed = tc_load(idx, et, used, base + lane, end, K, n_src);
    int rank = 0, add = 0;
    for (int k = 0; k < K; ++k) {
      const unsigned long long b = __ballot(ed.ok && ed.rel == k);
      if (ed.ok && ed.rel == k) rank = __popcll(b & below);
      if (lane == k) add = __popcll(b);
    }
    const int from = ed.ok ? ed.rel : 0;
    const uint32_t lo = (uint32_t)__shfl((int)(uint32_t)(uint64_t)next, from, HC_WAVE);
    const uint32_t hi = (uint32_t)__shfl((int)(uint32_t)((uint64_t)next >> 32), from, HC_WAVE);
    const int64_t start = (int64_t)(((uint64_t)hi << 32) | lo);
    if (ed.ok && start + rank < E) {
      idx2[start + rank] = ed.src;
      if (edge_weight != nullptr) edge_weight[start + rank] = w;
    }
    next += add;
  }
}

__global__ void tc_zero_first(int64_t *ptr2) {
  if (threadIdx.x == 0 && blockIdx.x == 0) ptr2[0] = 0;
}

size_t tc_scan_bytes(int64_t n) {
  size_t bytes = 0;
  int64_t *none = nullptr;
  if (rocprim::inclusive_scan(nullptr, bytes, none, none, (size_t)n, rocprim::plus<int64_t>()) != hipSuccess)
    return 0;
  return bytes;
}

}  // namespace

extern "C" size_t hc_typed_csr_workspace_bytes(int64_t R, int num_rel) {
  if (R <= 0 || num_rel <= 0) return 256;
  return hc_align_up(tc_scan_bytes(R * (int64_t)num_rel), 256) + 256;
}

extern "C" int hc_typed_csr(const int64_t *ptr, const int64_t *idx, const int64_t *edge_types,
                            const uint8_t *used_mask, int64_t R, int64_t E, int64_t n_src, int num_rel,
                            int64_t *ptr2, int64_t *idx2, int64_t *cnt, int64_t *deg, float *edge_weight,
                            void *workspace, size_t workspace_bytes, unsigned *ticket, void *stream) {
  HC_REQUIRE(R >= 0 && E >= 0 && n_src >= 0 && num_rel > 0 && ptr2);
  if (num_rel > TC_MAX_REL) return HC_EUNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (R == 0) {
    tc_zero_first<<<dim3(1), dim3(HC_WAVE), 0, st>>>(ptr2);
    return hc_launch_status();
  }
  HC_REQUIRE(ptr && cnt && deg && (E == 0 || (idx && edge_types && idx2)));
  const int64_t groups = R * (int64_t)num_rel;
  const int64_t blocks = (R + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
  if (!hc_grid_ok(blocks)) return HC_EUNSUPPORTED;
  if (ticket != nullptr && groups <= TC_SMALL_GROUPS) {
    // sampled batches: count + scan in one launch, no library call (and no size query on the host)
    tc_count_scan<<<dim3((unsigned)((R + TCS_WAVES - 1) / TCS_WAVES)), dim3(TCS_BLOCK), 0, st>>>(
        ptr, idx, edge_types, used_mask, cnt, deg, ptr2, R, E, num_rel, n_src, ticket);
    tc_place<true><<<dim3((unsigned)blocks), dim3(HC_BLOCK), 0, st>>>(ptr, idx, edge_types, used_mask, cnt, ptr2,
                                                                     idx2, edge_weight, R, E, num_rel, n_src);
    return hc_launch_status();
  }
  if (workspace_bytes < hc_typed_csr_workspace_bytes(R, num_rel) || !workspace) return HC_EWORKSPACE;
  tc_count<<<dim3((unsigned)blocks), dim3(HC_BLOCK), 0, st>>>(ptr, idx, edge_types, used_mask, cnt, deg, ptr2,
                                                             R, E, num_rel, n_src);
  if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
  size_t scan_bytes = tc_scan_bytes(groups);
  if (rocprim::inclusive_scan(workspace, scan_bytes, cnt, ptr2 + 1, (size_t)groups, rocprim::plus<int64_t>(),
                              st) != hipSuccess)
    return HC_ELAUNCH;
  tc_place<false><<<dim3((unsigned)blocks), dim3(HC_BLOCK), 0, st>>>(ptr, idx, edge_types, used_mask, cnt, ptr2,
                                                                    idx2, edge_weight, R, E, num_rel, n_src);
  return hc_launch_status();
}

// ---------------------------------------------------------------------------------------------
// Relation of every edge from the node types of its two ends; a node's type is the number of
// bounds its full id has reached (bounds ascending).  Wave per row: the row's type is found once,
// every lane classifies one source.
namespace {

constexpr int TC_MAX_BOUNDS = 64;

__device__ __forceinline__ int tc_type_of(int64_t full, const int64_t *__restrict__ bounds, int n_bounds) {
  int t = 0;
  for (int b = 0; b < n_bounds; ++b) t += full >= bounds[b] ? 1 : 0;
  return t;
}

__global__ __launch_bounds__(HC_BLOCK) void tc_edge_types(const int64_t *__restrict__ ptr,
                                                           const int64_t *__restrict__ idx,
                                                           const int64_t *__restrict__ sub_to_full,
                                                           const int64_t *__restrict__ bounds, int n_bounds,
                                                           const int64_t *__restrict__ pair_to_rel,
                                                           int64_t *__restrict__ out, int64_t R, int64_t E,
                                                           int64_t n_all, int64_t row_blocks) {
  const int lane = hc_lane();
  if ((int64_t)blockIdx.x >= row_blocks) {
    // the blocks behind the rows' blocks: edge slots that no row of the block owns get -1
    const int64_t nb = (int64_t)gridDim.x - row_blocks;
    const int64_t start = R > 0 ? ptr[R] : 0;
    for (int64_t e = start + ((int64_t)blockIdx.x - row_blocks) * HC_BLOCK + threadIdx.x; e < E; e += nb * HC_BLOCK)
      out[e] = -1;
    return;
  }
  const int64_t row = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (row >= R) return;
  const int64_t begin = ptr[row];
  const int64_t full_end = ptr[row + 1];
  const int64_t end = full_end < E ? full_end : E;
  const int n_types = n_bounds + 1;
  const int t_dst = row < n_all ? tc_type_of(sub_to_full[row], bounds, n_bounds) : 0;
  for (int64_t e = begin + lane; e < end; e += HC_WAVE) {
    const int64_t s = idx[e];
    int64_t rel = -1;
    if (s >= 0 && s < n_all) rel = pair_to_rel[t_dst * n_types + tc_type_of(sub_to_full[s], bounds, n_bounds)];
    out[e] = rel;
  }
}

}  // namespace

extern "C" int hc_edge_types_by_ranges(const int64_t *ptr, const int64_t *idx, const int64_t *sub_to_full,
                                       int64_t n_all, const int64_t *bounds, int n_bounds,
                                       const int64_t *pair_to_rel, int64_t *out, int64_t R, int64_t E,
                                       void *stream) {
  HC_REQUIRE(R >= 0 && E >= 0 && n_all >= 0 && n_bounds >= 0);
  if (n_bounds > TC_MAX_BOUNDS) return HC_EUNSUPPORTED;
  if (E == 0) return HC_OK;
  HC_REQUIRE(out != nullptr);
  if (R > 0) HC_REQUIRE(ptr && idx && sub_to_full && pair_to_rel && (n_bounds == 0 || bounds));
  const int64_t blocks = (R + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
  const int64_t tail_blocks = 32;   // grid-stride over the slots behind the last row (usually none)
  if (!hc_grid_ok(blocks + tail_blocks)) return HC_EUNSUPPORTED;
  tc_edge_types<<<dim3((unsigned)(blocks + tail_blocks)), dim3(HC_BLOCK), 0, static_cast<hipStream_t>(stream)>>>(
      ptr, idx, sub_to_full, bounds, n_bounds, pair_to_rel, out, R, E, n_all, blocks);
  return hc_launch_status();
}
