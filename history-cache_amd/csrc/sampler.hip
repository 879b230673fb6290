// Layered neighbour sampling on the device: produces the mini-batch wire format the model and the
// cache consume (/root/reference/hiscache/history_model.py:120-153, history_cache.py:307-324 read
// ptr / idx / sub_to_full / num_node_in_layer from the loader; the reference gets them from the
// external cxgnndl loader).  Sub-graph nodes are numbered seeds first, then every hop's new nodes in
// first-seen order; one shared CSR holds the sampled neighbours of all but the last hop's nodes.
//
// Per hop, for the frontier rows [lo, hi):
//   count    c(u) = min(deg(u), fanout)
//   scan     row offsets
//   pick     neighbour j of row u is position perm_u(j) of u's adjacency list (all of them, in
//            list order, when deg <= fanout); its full id goes to idx, and an integer atomicMin
//            leaves the first edge slot that mentions an unseen node in the node map
//   flag     an edge owns its node when the map holds its own slot
//   scan     owners before every slot -> new local ids in first-seen order
//            (count and flag stay launches of their own: read through a functor inside the scans, their
//            random reads of the graph and of the node map made a batch a third slower)
//   relabel  idx <- local ids; owners append to sub_to_full
//   commit   node map <- local ids of the new nodes; its first thread writes the next hop's state
//            (lo, hi, edges): every hop has a state of its own, so nothing it reads changes under it
// perm_u is a keyed bijection of [0, deg): four Feistel rounds on the next even power of two with
// cycle walking, so the picks of a row are distinct (sampling without replacement) at O(fanout)
// work whatever the degree.  Everything is integer work with one well-defined result.
#include <cstring>

#include <rocprim/rocprim.hpp>

#include "hc_common.h"

namespace {

constexpr int32_t SP_UNSEEN = 0x7fffffff;
constexpr int32_t SP_PROV = 0x40000000;  // map values at or above this are edge slots, below are ids
constexpr int SP_GROUP = 16;             // lanes that share one row in the pick kernel

struct SpState {
  int64_t lo, hi;   // frontier rows of the current hop
  int64_t edges;    // edges written by earlier hops
  uint64_t key;     // the batch's sampling key
};

__host__ __device__ __forceinline__ uint64_t sp_mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// Keyed bijection of [0, d), d >= 2.
__device__ __forceinline__ uint64_t sp_perm(uint64_t j, uint64_t d, uint64_t key) {
  const int bits = 64 - __builtin_clzll(d - 1);  // d - 1 >= 1
  const int h = (bits + 1) >> 1;
  const uint64_t mask = (1ull << h) - 1ull;
  uint64_t x = j;
  do {
    uint64_t l = x >> h, r = x & mask;
#pragma unroll
    for (int round = 0; round < 4; ++round) {
      const uint64_t f = sp_mix64(r ^ key ^ ((uint64_t)round << 56)) & mask;
      const uint64_t t = l ^ f;
      l = r;
      r = t;
    }
    x = (l << h) | r;
  } while (x >= d);  // the walk stays inside x's cycle, which contains the start value < d
  return x;
}

__global__ __launch_bounds__(HC_BLOCK) void sp_fill_map(int32_t *__restrict__ loc, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i < n) loc[i] = SP_UNSEEN;
}

__global__ __launch_bounds__(HC_BLOCK) void sp_init(const int64_t *__restrict__ seeds, int64_t n_seed,
                                                     int64_t num_nodes, int32_t *__restrict__ loc,
                                                     int64_t *__restrict__ sub_to_full, int64_t *__restrict__ ptr,
                                                     int64_t *__restrict__ counts, SpState *__restrict__ st,
                                                     uint64_t rng_seed, const uint64_t *__restrict__ rng_seed_at) {
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i == 0) {
    st->lo = 0;
    st->hi = n_seed;
    st->edges = 0;
    st->key = rng_seed_at ? *rng_seed_at : rng_seed;
    ptr[0] = 0;
    counts[0] = n_seed;
  }
  if (i >= n_seed) return;
  const int64_t s = seeds[i];
  sub_to_full[i] = s;
  if (s >= 0 && s < num_nodes) loc[s] = (int32_t)i;
}

__global__ __launch_bounds__(HC_BLOCK) void sp_count(const int64_t *__restrict__ indptr,
                                                      const int64_t *__restrict__ sub_to_full,
                                                      const SpState *__restrict__ st, int64_t fanout,
                                                      int64_t num_nodes, int32_t *__restrict__ cnt, int64_t cap) {
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i >= cap) return;
  const int64_t u = st->lo + i;
  int32_t c = 0;
  if (u < st->hi) {
    const int64_t full = sub_to_full[u];
    if (full >= 0 && full < num_nodes) {
      const int64_t d = indptr[full + 1] - indptr[full];
      c = (int32_t)(d < fanout ? (d < 0 ? 0 : d) : fanout);
    }
  }
  cnt[i] = c;
}

__global__ __launch_bounds__(HC_BLOCK) void sp_pick(const int64_t *__restrict__ indptr,
                                                     const int64_t *__restrict__ indices,
                                                     const int64_t *__restrict__ sub_to_full,
                                                     const SpState *__restrict__ st, int64_t fanout,
                                                     int64_t num_nodes, int hop,
                                                     const int32_t *__restrict__ incl, int32_t *__restrict__ loc,
                                                     int64_t *__restrict__ ptr, int64_t *__restrict__ idx,
                                                     int64_t cap) {
  const int64_t t = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  const int64_t i = t / SP_GROUP;
  const int sub = (int)(t % SP_GROUP);
  if (i >= cap) return;
  const int64_t u = st->lo + i;
  if (u >= st->hi) return;
  const int64_t begin = i > 0 ? (int64_t)incl[i - 1] : 0;  // slot of the row's first pick inside this hop
  const int32_t c = (int32_t)((int64_t)incl[i] - begin);
  const int64_t base = st->edges;
  if (sub == 0) ptr[u + 1] = base + incl[i];
  if (c == 0) return;
  const int64_t full = sub_to_full[u];
  const int64_t first = indptr[full];
  const uint64_t d = (uint64_t)(indptr[full + 1] - first);
  const uint64_t key = sp_mix64(sp_mix64(st->key + (uint64_t)hop) ^ (uint64_t)full);
  for (int64_t j = sub; j < c; j += SP_GROUP) {
    const uint64_t pos = d > (uint64_t)fanout ? sp_perm((uint64_t)j, d, key) : (uint64_t)j;
    const int64_t v = indices[first + (int64_t)pos];
    idx[base + begin + j] = v;
    if (v >= 0 && v < num_nodes) atomicMin(loc + v, SP_PROV + (int32_t)(begin + j));
  }
}

__global__ __launch_bounds__(HC_BLOCK) void sp_flag(const int64_t *__restrict__ idx,
                                                     const int32_t *__restrict__ loc,
                                                     const SpState *__restrict__ st,
                                                     const int32_t *__restrict__ incl, int64_t cap,
                                                     int64_t num_nodes, int32_t *__restrict__ flag,
                                                     int64_t edge_cap) {
  const int64_t p = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (p >= edge_cap) return;
  const int64_t hop_edges = incl[cap - 1];
  int32_t f = 0;
  if (p < hop_edges) {
    const int64_t v = idx[st->edges + p];
    f = (v >= 0 && v < num_nodes && loc[v] == SP_PROV + (int32_t)p) ? 1 : 0;
  }
  flag[p] = f;
}

__global__ __launch_bounds__(HC_BLOCK) void sp_relabel(int64_t *__restrict__ idx,
                                                        const int32_t *__restrict__ loc,
                                                        const SpState *__restrict__ st,
                                                        const int32_t *__restrict__ incl, int64_t cap,
                                                        int64_t num_nodes, const int32_t *__restrict__ rank_incl,
                                                        int64_t *__restrict__ sub_to_full, int64_t edge_cap) {
  const int64_t p = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (p >= edge_cap) return;
  const int64_t hop_edges = incl[cap - 1];
  if (p >= hop_edges) return;
  const int64_t e = st->edges + p;
  const int64_t v = idx[e];
  int64_t id = -1;
  if (v >= 0 && v < num_nodes) {
    const int32_t t = loc[v];
    if (t >= SP_PROV) {
      const int32_t q = t - SP_PROV;  // the owning edge slot of this hop
      id = st->hi + rank_incl[q] - 1;
      if (q == (int32_t)p) sub_to_full[id] = v;
    } else {
      id = t;
    }
  }
  idx[e] = id;
}

__global__ __launch_bounds__(HC_BLOCK) void sp_commit(const int64_t *__restrict__ sub_to_full,
                                                       const SpState *__restrict__ st, SpState *__restrict__ next,
                                                       const int32_t *__restrict__ incl, int64_t cap,
                                                       const int32_t *__restrict__ rank_incl,
                                                       int32_t *__restrict__ loc, int64_t *__restrict__ counts,
                                                       int hop, int num_hops, int64_t edge_cap) {
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i >= edge_cap) return;
  const int64_t hop_edges = incl[cap - 1];
  const int64_t fresh = hop_edges > 0 ? rank_incl[hop_edges - 1] : 0;
  if (i == 0) {  // the next hop's state (this hop's is read by the other threads and stays as it is)
    next->lo = st->hi;
    next->hi = st->hi + fresh;
    next->edges = st->edges + hop_edges;
    next->key = st->key;
    counts[hop + 1] = st->hi + fresh;
    counts[num_hops + 1 + hop] = st->edges + hop_edges;
  }
  if (i >= fresh) return;
  const int64_t id = st->hi + i;
  loc[sub_to_full[id]] = (int32_t)id;
}

__global__ __launch_bounds__(HC_BLOCK) void sp_reset(const int64_t *__restrict__ sub_to_full,
                                                      const SpState *__restrict__ st, int64_t num_nodes,
                                                      int32_t *__restrict__ loc, int64_t node_cap) {
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i >= node_cap || i >= st->hi) return;
  const int64_t v = sub_to_full[i];
  if (v >= 0 && v < num_nodes) loc[v] = SP_UNSEEN;
}

struct SpCaps {
  int64_t rows[HC_SAMPLE_MAX_HOPS];   // frontier bound per hop
  int64_t edges[HC_SAMPLE_MAX_HOPS];  // edge bound per hop
  int64_t max_rows, max_edges, total_rows, total_edges, total_nodes;
  bool ok;
};

SpCaps sp_caps(int64_t n_seed, const int64_t *fanout, int num_hops, int64_t num_nodes) {
  SpCaps c{};
  c.ok = num_hops >= 1 && num_hops <= HC_SAMPLE_MAX_HOPS && n_seed >= 0 && fanout != nullptr;
  if (!c.ok) return c;
  int64_t rows = n_seed;
  c.total_nodes = n_seed;
  for (int k = 0; k < num_hops; ++k) {
    if (fanout[k] < 1 || fanout[k] > (1 << 20)) {
      c.ok = false;
      return c;
    }
    c.rows[k] = rows;
    c.edges[k] = rows * fanout[k];
    if (c.edges[k] >= (int64_t)SP_PROV - 1) {
      c.ok = false;
      return c;
    }
    c.total_rows += rows;
    c.total_edges += c.edges[k];
    if (rows > c.max_rows) c.max_rows = rows;
    if (c.edges[k] > c.max_edges) c.max_edges = c.edges[k];
    // new nodes of a hop: at most its edges, and at most the graph
    rows = c.edges[k];
    if (num_nodes > 0 && rows > num_nodes) rows = num_nodes;
    c.total_nodes += rows;
  }
  if (num_nodes > 0 && c.total_nodes > num_nodes) c.total_nodes = num_nodes > n_seed ? num_nodes : n_seed;
  if (c.total_nodes >= (int64_t)SP_PROV) c.ok = false;
  return c;
}

size_t sp_scan_bytes(int64_t n) {
  size_t bytes = 0;
  int32_t *none = nullptr;
  if (rocprim::inclusive_scan(nullptr, bytes, none, none, (size_t)(n > 0 ? n : 1), rocprim::plus<int32_t>()) !=
      hipSuccess)
    return 0;
  return bytes;
}

struct SpLayout {
  size_t state, cnt, incl, flag, rank, scan, total;
};

SpLayout sp_layout(const SpCaps &c) {
  SpLayout l{};
  size_t off = 0;
  l.state = off;                                   // one state per hop and the final one
  off += hc_align_up(sizeof(SpState) * (HC_SAMPLE_MAX_HOPS + 1), 256);
  l.cnt = off;
  off += hc_align_up((size_t)(c.max_rows + 1) * 4, 256);
  l.incl = off;
  off += hc_align_up((size_t)(c.max_rows + 1) * 4, 256);
  l.flag = off;
  off += hc_align_up((size_t)(c.max_edges + 1) * 4, 256);
  l.rank = off;
  off += hc_align_up((size_t)(c.max_edges + 1) * 4, 256);
  l.scan = off;
  size_t a = sp_scan_bytes(c.max_rows), b = sp_scan_bytes(c.max_edges);
  off += hc_align_up(a > b ? a : b, 256) + 256;
  l.total = off;
  return l;
}

inline unsigned sp_blocks(int64_t n) { return (unsigned)((n + HC_BLOCK - 1) / HC_BLOCK); }

}  // namespace

extern "C" int hc_sample_capacity(int64_t n_seed, const int64_t *fanout, int num_hops, int64_t num_nodes,
                                  int64_t *max_rows, int64_t *max_edges, int64_t *max_nodes) {
  const SpCaps c = sp_caps(n_seed, fanout, num_hops, num_nodes);
  if (!c.ok) return HC_EINVAL;
  if (max_rows) *max_rows = c.total_rows;
  if (max_edges) *max_edges = c.total_edges;
  if (max_nodes) *max_nodes = c.total_nodes;
  return HC_OK;
}

extern "C" size_t hc_sample_workspace_bytes(int64_t n_seed, const int64_t *fanout, int num_hops,
                                            int64_t num_nodes) {
  const SpCaps c = sp_caps(n_seed, fanout, num_hops, num_nodes);
  if (!c.ok) return 0;
  return sp_layout(c).total;
}

extern "C" int hc_sample_map_init(int32_t *node_map, int64_t num_nodes, void *stream) {
  HC_REQUIRE(num_nodes >= 0);
  if (num_nodes == 0) return HC_OK;
  HC_REQUIRE(node_map != nullptr);
  if (!hc_grid_ok(sp_blocks(num_nodes))) return HC_EUNSUPPORTED;
  sp_fill_map<<<dim3(sp_blocks(num_nodes)), dim3(HC_BLOCK), 0, static_cast<hipStream_t>(stream)>>>(node_map,
                                                                                                  num_nodes);
  return hc_launch_status();
}

namespace {

int sample_layers_impl(const int64_t *indptr, const int64_t *indices, int64_t num_nodes, const int64_t *seeds,
                       int64_t n_seed, const int64_t *fanout, int num_hops, uint64_t rng_seed,
                       const uint64_t *rng_seed_at, int32_t *node_map, int64_t *ptr, int64_t *idx,
                       int64_t *sub_to_full, int64_t *counts, void *workspace, size_t workspace_bytes,
                       void *stream) {
  HC_REQUIRE(num_nodes > 0 && n_seed > 0);
  HC_REQUIRE(indptr && indices && seeds && node_map && ptr && idx && sub_to_full && counts);
  const SpCaps c = sp_caps(n_seed, fanout, num_hops, num_nodes);
  if (!c.ok) return HC_EUNSUPPORTED;
  const SpLayout l = sp_layout(c);
  if (!workspace || workspace_bytes < l.total) return HC_EWORKSPACE;
  if (!hc_grid_ok(sp_blocks(c.max_edges)) || !hc_grid_ok(sp_blocks(c.max_rows * SP_GROUP)) ||
      !hc_grid_ok(sp_blocks(c.total_nodes)))
    return HC_EUNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  char *w = static_cast<char *>(workspace);
  SpState *states = reinterpret_cast<SpState *>(w + l.state);
  int32_t *cnt = reinterpret_cast<int32_t *>(w + l.cnt);
  int32_t *incl = reinterpret_cast<int32_t *>(w + l.incl);
  int32_t *flag = reinterpret_cast<int32_t *>(w + l.flag);
  int32_t *rank = reinterpret_cast<int32_t *>(w + l.rank);
  void *scan_ws = w + l.scan;
  const dim3 bl(HC_BLOCK);

  sp_init<<<dim3(sp_blocks(n_seed)), bl, 0, s>>>(seeds, n_seed, num_nodes, node_map, sub_to_full, ptr, counts, states,
                                                 rng_seed, rng_seed_at);
  for (int k = 0; k < num_hops; ++k) {
    const int64_t cap = c.rows[k], ecap = c.edges[k];
    const SpState *st = states + k;
    sp_count<<<dim3(sp_blocks(cap)), bl, 0, s>>>(indptr, sub_to_full, st, fanout[k], num_nodes, cnt, cap);
    size_t bytes = sp_scan_bytes(cap);
    if (rocprim::inclusive_scan(scan_ws, bytes, cnt, incl, (size_t)cap, rocprim::plus<int32_t>(), s) != hipSuccess)
      return HC_ELAUNCH;
    sp_pick<<<dim3(sp_blocks(cap * SP_GROUP)), bl, 0, s>>>(indptr, indices, sub_to_full, st, fanout[k], num_nodes,
                                                          k, incl, node_map, ptr, idx, cap);
    sp_flag<<<dim3(sp_blocks(ecap)), bl, 0, s>>>(idx, node_map, st, incl, cap, num_nodes, flag, ecap);
    bytes = sp_scan_bytes(ecap);
    if (rocprim::inclusive_scan(scan_ws, bytes, flag, rank, (size_t)ecap, rocprim::plus<int32_t>(), s) !=
        hipSuccess)
      return HC_ELAUNCH;
    sp_relabel<<<dim3(sp_blocks(ecap)), bl, 0, s>>>(idx, node_map, st, incl, cap, num_nodes, rank, sub_to_full,
                                                   ecap);
    sp_commit<<<dim3(sp_blocks(ecap)), bl, 0, s>>>(sub_to_full, st, states + k + 1, incl, cap, rank, node_map,
                                                  counts, k, num_hops, ecap);
    if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
  }
  const SpState *st = states + num_hops;
  sp_reset<<<dim3(sp_blocks(c.total_nodes)), bl, 0, s>>>(sub_to_full, st, num_nodes, node_map, c.total_nodes);
  return hc_launch_status();
}

}  // namespace

extern "C" int hc_sample_layers(const int64_t *indptr, const int64_t *indices, int64_t num_nodes,
                                const int64_t *seeds, int64_t n_seed, const int64_t *fanout, int num_hops,
                                uint64_t rng_seed, int32_t *node_map, int64_t *ptr, int64_t *idx,
                                int64_t *sub_to_full, int64_t *counts, void *workspace, size_t workspace_bytes,
                                void *stream) {
  return sample_layers_impl(indptr, indices, num_nodes, seeds, n_seed, fanout, num_hops, rng_seed, nullptr, node_map,
                            ptr, idx, sub_to_full, counts, workspace, workspace_bytes, stream);
}

extern "C" int hc_sample_layers_seed_at(const int64_t *indptr, const int64_t *indices, int64_t num_nodes,
                                        const int64_t *seeds, int64_t n_seed, const int64_t *fanout, int num_hops,
                                        const uint64_t *rng_seed_at, int32_t *node_map, int64_t *ptr,
                                        int64_t *idx, int64_t *sub_to_full, int64_t *counts, void *workspace,
                                        size_t workspace_bytes, void *stream) {
  HC_REQUIRE(rng_seed_at != nullptr);
  return sample_layers_impl(indptr, indices, num_nodes, seeds, n_seed, fanout, num_hops, 0, rng_seed_at, node_map,
                            ptr, idx, sub_to_full, counts, workspace, workspace_bytes, stream);
}
