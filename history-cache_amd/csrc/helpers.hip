// Used-mask reconstruction, small graph helpers, row gathers and library metadata.
#include "hc_common.h"

namespace {

__global__ __launch_bounds__(HC_BLOCK) void fill_u8(uint8_t *__restrict__ p, int64_t n, uint8_t v) {
  // 16 bytes per thread where possible
  const int64_t i = ((int64_t)blockIdx.x * HC_BLOCK + threadIdx.x) * 16;
  if (i + 16 <= n && (reinterpret_cast<uintptr_t>(p) % 16) == 0) {
    const uint32_t w = 0x01010101u * v;
    *reinterpret_cast<uint4 *>(p + i) = make_uint4(w, w, w, w);
  } else {
    for (int64_t k = i; k < n && k < i + 16; ++k) p[k] = v;
  }
}

__global__ __launch_bounds__(HC_BLOCK) void fill_i64(int64_t *__restrict__ p, int64_t n, int64_t v) {
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i < n) p[i] = v;
}

__global__ __launch_bounds__(HC_BLOCK) void fill_i32(int32_t *__restrict__ p, int64_t n, int32_t v) {
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i < n) p[i] = v;
}

// One pass of the used-mask rule (/root/reference/src/cpp/src/grad_check.cu:70-101).
// Wave per row.  A row is active if it is a seed on the first pass (:79-82) or use_in[row]
// is set (:83-84); an active row with history stops (:87-90); otherwise it marks itself
// (:92-94) and its neighbours (:97-100).  Every store writes the constant 1.
__global__ __launch_bounds__(HC_BLOCK) void count_history_pass(
    const int64_t *__restrict__ ptr, const int64_t *__restrict__ idx, const int64_t *__restrict__ hmap,
    int64_t hmap_len, uint8_t *__restrict__ use_in, uint8_t *__restrict__ use_out, int64_t ptr_rows,
    int64_t n_all, int64_t n_seed, int first_pass) {
  const int lane = hc_lane();
  const int64_t row = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (row >= ptr_rows || row >= n_all) return;
  if (first_pass && row < n_seed) {
    if (lane == 0) use_in[row] = 1;
  } else if (use_in[row] != 1) {
    return;
  }
  if (hmap != nullptr && row < hmap_len && hmap[row] != -1) return;
  if (lane == 0) use_out[row] = 1;
  const int64_t begin = ptr[row];
  const int64_t end = ptr[row + 1];
  for (int64_t e = begin + lane; e < end; e += HC_WAVE) {
    const int64_t n = idx[e];
    if (n >= 0 && n < n_all) use_out[n] = 1;
  }
}

// Histogram that skips value 0 (/root/reference/src/cpp/src/grad_check.cu:165-172).
__global__ __launch_bounds__(HC_BLOCK) void count_num_kernel(const int64_t *__restrict__ arr,
                                                              int32_t *__restrict__ out, int64_t n,
                                                              int64_t mmax) {
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i >= n) return;
  const int64_t a = arr[i];
  if (a > 0 && a <= mmax) atomicAdd(out + a, 1);
}

// Same histogram for few bins (relation ids): every block counts its slice in LDS and adds its
// non-zero bins to the result once, instead of one contended global atomic per element.
constexpr int CN_LDS_BINS = 4096;
__global__ __launch_bounds__(HC_BLOCK) void count_num_lds_kernel(const int64_t *__restrict__ arr,
                                                                  int32_t *__restrict__ out, int64_t n,
                                                                  int mmax, int64_t per_block) {
  __shared__ int hist[CN_LDS_BINS];
  const int bins = mmax + 1;
  for (int b = threadIdx.x; b < bins; b += HC_BLOCK) hist[b] = 0;
  __syncthreads();
  const int64_t begin = (int64_t)blockIdx.x * per_block;
  const int64_t end = begin + per_block < n ? begin + per_block : n;
  for (int64_t i = begin + threadIdx.x; i < end; i += HC_BLOCK) {
    const int64_t a = arr[i];
    if (a > 0 && a <= mmax) atomicAdd(&hist[(int)a], 1);
  }
  __syncthreads();
  for (int b = threadIdx.x; b < bins; b += HC_BLOCK) {
    const int c = hist[b];
    if (c != 0) atomicAdd(out + b, c);
  }
}

// One level-synchronous pass of the structure score: rows with prev != 0 offer prev*deg to
// neighbours whose prev is 0; the smallest offer wins (unsigned min over a 0 = "unset" encoding).
__global__ __launch_bounds__(HC_BLOCK) void structure_pass(const int64_t *__restrict__ ptr,
                                                            const int64_t *__restrict__ idx,
                                                            const int64_t *__restrict__ prev,
                                                            unsigned long long *__restrict__ next,
                                                            int64_t ptr_rows, int64_t n_all) {
  const int lane = hc_lane();
  const int64_t row = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (row >= ptr_rows || row >= n_all) return;
  const int64_t pv = prev[row];
  if (pv == 0) return;
  const int64_t begin = ptr[row];
  const int64_t end = ptr[row + 1];
  const int64_t offer = pv * (end - begin);
  for (int64_t e = begin + lane; e < end; e += HC_WAVE) {
    const int64_t n = idx[e];
    if (n < 0 || n >= n_all || prev[n] != 0) continue;
    // "unset" is stored as 0; offer-1 in unsigned space keeps 0 (from deg 0 rows) representable
    atomicMin(next + n, (unsigned long long)offer - 1ull);
  }
}

// Reset the offer array to "unset" (all ones) before a pass.
__global__ __launch_bounds__(HC_BLOCK) void structure_stage(unsigned long long *__restrict__ next,
                                                             int64_t n_all) {
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i < n_all) next[i] = ~0ull;
}

__global__ __launch_bounds__(HC_BLOCK) void structure_commit(int64_t *__restrict__ out,
                                                              const unsigned long long *__restrict__ next,
                                                              int64_t n_all) {
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i >= n_all) return;
  const unsigned long long v = next[i];
  if (out[i] == 0 && v != ~0ull) out[i] = (int64_t)(v + 1ull);
}

__global__ __launch_bounds__(HC_BLOCK) void structure_seed(int64_t *__restrict__ out, int64_t n_seed,
                                                            int64_t n_all) {
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i < n_seed && i < n_all) out[i] = 1;
}

// dst[i,:] = (mask == NULL || mask[i]) ? src[ids[i],:] : 0  (optionally accumulated).
// Wave per output row; 4 elements per lane per step when the row allows.  src may be mapped host
// memory.  TS / TD are the element types of the source table and of the destination.
template <typename TS, typename TD>
__global__ __launch_bounds__(HC_BLOCK) void gather_rows_kernel(const TS *__restrict__ src, int64_t n_rows,
                                                                const int64_t *__restrict__ ids,
                                                                const uint8_t *__restrict__ mask,
                                                                TD *__restrict__ dst, int accumulate,
                                                                int64_t n, int64_t F) {
  constexpr int V = 4;
  const int lane = hc_lane();
  const int64_t stride = (int64_t)gridDim.x * HC_WAVES_PER_BLOCK;
  for (int64_t i = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block(); i < n; i += stride) {
  TD *__restrict__ o = dst + i * F;
  bool take = mask == nullptr || mask[i] != 0;
  int64_t id = 0;
  if (take) {
    id = ids[i];
    if (id < 0) id += n_rows;
    if (id < 0 || id >= n_rows) take = false;
  }
  const TS *__restrict__ s = src + id * F;
  const bool vec_ok = (F % V == 0) && (reinterpret_cast<uintptr_t>(s) % (sizeof(TS) * V) == 0) &&
                      (reinterpret_cast<uintptr_t>(o) % (sizeof(TD) * V) == 0);
  if (vec_ok) {
    for (int64_t c = (int64_t)lane * V; c < F; c += HC_WAVE * V) {
      float v[V];
      if (take) {
        hc_vec<TS, V>::load(s + c, v);
      } else {
#pragma unroll
        for (int k = 0; k < V; ++k) v[k] = 0.0f;
      }
      if (accumulate) {
        float old[V];
        hc_vec<TD, V>::load(o + c, old);
#pragma unroll
        for (int k = 0; k < V; ++k) v[k] = old[k] + v[k];
      }
      hc_vec<TD, V>::store(o + c, v);
    }
  } else {
    for (int64_t c = lane; c < F; c += HC_WAVE) {
      float v = take ? hc_to_f32<TS>(s[c]) : 0.0f;
      if (accumulate) v = hc_to_f32<TD>(o[c]) + v;
      o[c] = hc_from_f32<TD>(v);
    }
  }
  }
}

__global__ __launch_bounds__(HC_BLOCK) void lookup_kernel(const int64_t *__restrict__ map,
                                                           int64_t map_len,
                                                           const int64_t *__restrict__ ids,
                                                           int64_t offset, int64_t *__restrict__ out,
                                                           int64_t n, const int64_t *__restrict__ n_valid_dev) {
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i >= n) return;
  if (n_valid_dev != nullptr && i >= *n_valid_dev) {     // padding behind the entries in use finds nothing
    out[i] = -1;
    return;
  }
  int64_t k = ids[i] + offset;
  if (k < 0) k += map_len;  // -1 addresses the last entry, as Python indexing does
  out[i] = (k >= 0 && k < map_len) ? map[k] : -1;
}

// Ring-table lookup: slot of every id, entries at least age_limit iterations old count as absent,
// and the table row of every hit widened to fp32 (zeros for the others).  Wave per id.
template <typename TT>
__global__ __launch_bounds__(HC_BLOCK) void ring_lookup_kernel(
    const int64_t *__restrict__ full2slot, int64_t n_full, const int64_t *__restrict__ ids,
    const int64_t *__restrict__ checkin, int64_t now_value, int64_t age_limit, const TT *__restrict__ table,
    int64_t capacity, int64_t F, int64_t *__restrict__ slot_out, float *__restrict__ rows_out, int64_t n,
    const int64_t *__restrict__ now_dev, const int64_t *__restrict__ n_valid_dev) {
  constexpr int V = 4;
  const int lane = hc_lane();
  const int64_t i = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (i >= n) return;
  // callers whose launches are recorded once and replayed keep the iteration number and the number of ids
  // in use in device memory: ids behind that number are padding and find nothing
  const int64_t now = now_dev != nullptr ? *now_dev : now_value;
  const bool padding = n_valid_dev != nullptr && i >= *n_valid_dev;
  const int64_t id = padding ? -1 : ids[i];
  int64_t slot = (id >= 0 && id < n_full) ? full2slot[id] : -1;
  if (slot < 0 || slot >= capacity) slot = -1;
  if (slot >= 0 && checkin != nullptr && now - checkin[slot] >= age_limit) slot = -1;
  if (lane == 0) slot_out[i] = slot;
  if (rows_out == nullptr) return;
  float *__restrict__ o = rows_out + i * F;
  const TT *__restrict__ s = table + (slot >= 0 ? slot : 0) * F;
  const bool vec_ok = (F % V == 0) && (reinterpret_cast<uintptr_t>(table) % (sizeof(TT) * V) == 0) &&
                      (reinterpret_cast<uintptr_t>(rows_out) % 16 == 0);
  if (vec_ok) {
    for (int64_t c = (int64_t)lane * V; c < F; c += HC_WAVE * V) {
      float v[V] = {0.0f, 0.0f, 0.0f, 0.0f};
      if (slot >= 0) hc_vec<TT, V>::load(s + c, v);
      hc_vec<float, V>::store(o + c, v);
    }
  } else {
    for (int64_t c = lane; c < F; c += HC_WAVE) o[c] = slot >= 0 ? hc_to_f32<TT>(s[c]) : 0.0f;
  }
}

inline unsigned blocks_for(int64_t n) { return (unsigned)((n + HC_BLOCK - 1) / HC_BLOCK); }

// Staging of a batch into arrays of fixed size: dst[i] = i < n_copy ? src[i] : fill for up to sixteen arrays
// of 8-, 4-, 2- or 1-byte elements (integers; rows of floats go through as their bit patterns with fill 0), and
// a handful of 64-bit scalars (the batch's sizes, the iteration number) written to device memory, all in one
// launch.
constexpr int STAGE_MAX_ARRAYS = 16;
constexpr int STAGE_MAX_SCALARS = 16;
struct StagePlan {
  const void *src[STAGE_MAX_ARRAYS];
  void *dst[STAGE_MAX_ARRAYS];
  int64_t n_copy[STAGE_MAX_ARRAYS];
  int64_t n_total[STAGE_MAX_ARRAYS];
  int64_t fill[STAGE_MAX_ARRAYS];
  int elem[STAGE_MAX_ARRAYS];          // bytes per element: 8, 4, 2 or 1
  int64_t *scalars_dst;
  int64_t scalars[STAGE_MAX_SCALARS];
  int n_scalars;
};

template <typename T>
__device__ __forceinline__ void stage_one(const void *src_, void *dst_, int64_t m, int64_t n, int64_t fill) {
  const T *__restrict__ src = static_cast<const T *>(src_);
  T *__restrict__ dst = static_cast<T *>(dst_);
  const int64_t stride = (int64_t)gridDim.x * HC_BLOCK;
  for (int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x; i < n; i += stride) dst[i] = i < m ? src[i] : (T)fill;
}

__global__ __launch_bounds__(HC_BLOCK) void stage_kernel(StagePlan p) {
  const int a = (int)blockIdx.y;
  if (a == 0 && blockIdx.x == 0 && (int)threadIdx.x < p.n_scalars) p.scalars_dst[threadIdx.x] = p.scalars[threadIdx.x];
  const int64_t n = p.n_total[a], m = p.n_copy[a];
  switch (p.elem[a]) {                 // block-uniform
    case 8: stage_one<int64_t>(p.src[a], p.dst[a], m, n, p.fill[a]); break;
    case 4: stage_one<int32_t>(p.src[a], p.dst[a], m, n, p.fill[a]); break;
    case 2: stage_one<int16_t>(p.src[a], p.dst[a], m, n, p.fill[a]); break;
    case 1: stage_one<int8_t>(p.src[a], p.dst[a], m, n, p.fill[a]); break;
    default: break;
  }
}

inline unsigned blocks_for_stage(int64_t longest) {
  int64_t bx = (longest + (int64_t)HC_BLOCK * 4 - 1) / ((int64_t)HC_BLOCK * 4);
  return (unsigned)(bx > 2048 ? 2048 : (bx < 1 ? 1 : bx));
}

}  // namespace

extern "C" const char *hc_version(void) { return "hiscache_hip 0.1 (gfx950)"; }

extern "C" const char *hc_strerror(int status) {
  switch (status) {
    case HC_OK: return "ok";
    case HC_EINVAL: return "invalid argument (null pointer, negative size or inconsistent shapes)";
    case HC_EDTYPE: return "unknown dtype";
    case HC_ELAUNCH: return "HIP launch error";
    case HC_EWORKSPACE: return "workspace missing, misaligned or too small";
    case HC_EUNSUPPORTED: return "request outside what the kernels cover";
    case HC_ENODEVICE: return "no usable GPU";
    default: return "unknown status";
  }
}

extern "C" int hc_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

extern "C" int hc_count_history(const int64_t *ptr, const int64_t *idx, const int64_t *hmap,
                                int64_t hmap_len, uint8_t *masks, int64_t ptr_rows, int64_t n_all,
                                int64_t n_seed, int num_layer, void *stream) {
  HC_REQUIRE(ptr_rows >= 0 && n_all >= 0 && n_seed >= 0 && num_layer >= 0 && hmap_len >= 0);
  if (n_all == 0) return HC_OK;
  HC_REQUIRE(masks != nullptr);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t total = (int64_t)(num_layer + 1) * n_all;
  const int64_t fb = (total + HC_BLOCK * 16 - 1) / (HC_BLOCK * 16);
  if (!hc_grid_ok(fb)) return HC_EUNSUPPORTED;
  fill_u8<<<dim3((unsigned)fb), dim3(HC_BLOCK), 0, st>>>(masks, total, 0);
  if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
  if (ptr_rows == 0 || num_layer == 0) return HC_OK;
  HC_REQUIRE(ptr != nullptr);
  const int64_t rb = (ptr_rows + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
  if (!hc_grid_ok(rb)) return HC_EUNSUPPORTED;
  const int L = num_layer;
  for (int i = 0; i < L; ++i) {
    // history prunes on the second pass only (grad_check.cu:122-124)
    const int64_t *hm = (i == 1) ? hmap : nullptr;
    count_history_pass<<<dim3((unsigned)rb), dim3(HC_BLOCK), 0, st>>>(
        ptr, idx, hm, hmap_len, masks + (int64_t)(L - i) * n_all, masks + (int64_t)(L - 1 - i) * n_all,
        ptr_rows, n_all, n_seed, i == 0 ? 1 : 0);
    if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
  }
  return HC_OK;
}

// Input check for a CSR block: thread t < R looks at row t's bounds, thread R + e at edge slot e.
// report[0] rows whose end lies before their start, report[1] offsets outside [0, E],
// report[2] neighbour ids outside [0, n_src) among the slots the rows cover.
namespace {
__global__ __launch_bounds__(HC_BLOCK) void check_csr_kernel(const int64_t *__restrict__ ptr,
                                                              const int64_t *__restrict__ idx, int64_t R,
                                                              int64_t E, int64_t n_src,
                                                              unsigned long long *__restrict__ report) {
  const int64_t t = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (t < R) {
    const int64_t b = ptr[t], e = ptr[t + 1];
    if (e < b) atomicAdd(report + 0, 1ull);
    if (b < 0 || b > E || e < 0 || e > E) atomicAdd(report + 1, 1ull);
    return;
  }
  const int64_t slot = t - R;
  if (slot >= E) return;
  const int64_t first = ptr[0], last = ptr[R];
  if (slot < first || slot >= last) return;
  const int64_t s = idx[slot];
  if (s < 0 || s >= n_src) atomicAdd(report + 2, 1ull);
}

__global__ void clear_report(unsigned long long *report) {
  if (threadIdx.x < 4 && blockIdx.x == 0) report[threadIdx.x] = 0ull;
}
}  // namespace

extern "C" int hc_check_csr(const int64_t *ptr, const int64_t *idx, int64_t R, int64_t E, int64_t n_src,
                            int64_t *report, void *stream) {
  HC_REQUIRE(R >= 0 && E >= 0 && n_src >= 0 && report);
  hipStream_t st = static_cast<hipStream_t>(stream);
  unsigned long long *rep = reinterpret_cast<unsigned long long *>(report);
  clear_report<<<dim3(1), dim3(HC_WAVE), 0, st>>>(rep);
  if (R == 0) return hc_launch_status();
  HC_REQUIRE(ptr && (E == 0 || idx));
  if (!hc_grid_ok((R + E + HC_BLOCK - 1) / HC_BLOCK)) return HC_EUNSUPPORTED;
  check_csr_kernel<<<dim3(blocks_for(R + E)), dim3(HC_BLOCK), 0, st>>>(ptr, idx, R, E, n_src, rep);
  return hc_launch_status();
}

extern "C" int hc_count_num(const int64_t *arr, int64_t n, int64_t mmax, int32_t *out, void *stream) {
  HC_REQUIRE(n >= 0 && mmax >= 0 && out);
  hipStream_t st = static_cast<hipStream_t>(stream);
  fill_i32<<<dim3(blocks_for(mmax + 1)), dim3(HC_BLOCK), 0, st>>>(out, mmax + 1, 0);
  if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
  if (n == 0) return HC_OK;
  HC_REQUIRE(arr);
  if (!hc_grid_ok((n + HC_BLOCK - 1) / HC_BLOCK)) return HC_EUNSUPPORTED;
  if (mmax < CN_LDS_BINS) {
    // at most 2048 blocks, at least 16 elements per thread
    int64_t per_block = (n + 2047) / 2048;
    if (per_block < 16 * HC_BLOCK) per_block = 16 * HC_BLOCK;
    const int64_t blocks = (n + per_block - 1) / per_block;
    count_num_lds_kernel<<<dim3((unsigned)blocks), dim3(HC_BLOCK), 0, st>>>(arr, out, n, (int)mmax, per_block);
  } else {
    count_num_kernel<<<dim3(blocks_for(n)), dim3(HC_BLOCK), 0, st>>>(arr, out, n, mmax);
  }
  return hc_launch_status();
}

extern "C" int hc_structure_score(const int64_t *ptr, const int64_t *idx, int64_t ptr_rows,
                                  int64_t n_all, int64_t n_seed, int num_layer, int64_t *out,
                                  int64_t *scratch, void *stream) {
  HC_REQUIRE(ptr_rows >= 0 && n_all >= 0 && n_seed >= 0 && num_layer >= 0);
  if (n_all == 0) return HC_OK;
  HC_REQUIRE(out && scratch);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!hc_grid_ok((n_all + HC_BLOCK - 1) / HC_BLOCK)) return HC_EUNSUPPORTED;
  fill_i64<<<dim3(blocks_for(n_all)), dim3(HC_BLOCK), 0, st>>>(out, n_all, 0);
  unsigned long long *next = reinterpret_cast<unsigned long long *>(scratch);
  const int64_t rb = (ptr_rows + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
  for (int p = 0; p < num_layer; ++p) {
    structure_seed<<<dim3(blocks_for(n_all)), dim3(HC_BLOCK), 0, st>>>(out, n_seed, n_all);
    structure_stage<<<dim3(blocks_for(n_all)), dim3(HC_BLOCK), 0, st>>>(next, n_all);
    if (rb > 0) {
      HC_REQUIRE(ptr != nullptr);
      if (!hc_grid_ok(rb)) return HC_EUNSUPPORTED;
      structure_pass<<<dim3((unsigned)rb), dim3(HC_BLOCK), 0, st>>>(ptr, idx, out, next, ptr_rows, n_all);
    }
    structure_commit<<<dim3(blocks_for(n_all)), dim3(HC_BLOCK), 0, st>>>(out, next, n_all);
    if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
  }
  return HC_OK;
}

template <typename TS>
int launch_gather(const void *src, int64_t n_rows, const int64_t *ids, const uint8_t *mask, void *dst,
                  int dst_dtype, int accumulate, int64_t n, int64_t F, dim3 g, dim3 bl, hipStream_t st) {
  const TS *s = static_cast<const TS *>(src);
  if (dst_dtype == HC_F32)
    gather_rows_kernel<TS, float><<<g, bl, 0, st>>>(s, n_rows, ids, mask, static_cast<float *>(dst), accumulate, n, F);
  else if (dst_dtype == HC_F16)
    gather_rows_kernel<TS, __half><<<g, bl, 0, st>>>(s, n_rows, ids, mask, static_cast<__half *>(dst), accumulate, n, F);
  else
    gather_rows_kernel<TS, __hip_bfloat16><<<g, bl, 0, st>>>(s, n_rows, ids, mask, static_cast<__hip_bfloat16 *>(dst),
                                                             accumulate, n, F);
  return hc_launch_status();
}

extern "C" int hc_gather_rows(const void *src, int src_dtype, int64_t n_rows, const int64_t *ids,
                              const uint8_t *mask, void *dst, int dst_dtype, int accumulate, int64_t n,
                              int64_t F, void *stream) {
  HC_REQUIRE(n >= 0 && F > 0 && n_rows >= 0);
  if (src_dtype < HC_F32 || src_dtype > HC_BF16 || dst_dtype < HC_F32 || dst_dtype > HC_BF16) return HC_EDTYPE;
  if (n == 0) return HC_OK;
  HC_REQUIRE(ids && dst && (src || n_rows == 0));
  hipStream_t st = static_cast<hipStream_t>(stream);
  int64_t b = (n + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
  if (!hc_grid_ok(b)) return HC_EUNSUPPORTED;
  // A table in host memory is read over the host link: a few hundred waves keep the link busy, and a
  // launch of one wave per row would park tens of thousands of waiting waves on the compute units,
  // in the way of whatever runs beside it on other streams.
  // (256 blocks = 1 024 waves read 56 - 57 GB/s, the same as 22 000 blocks).
  // A table in device memory takes the launch that serves several rows per wave.
  constexpr int64_t HOST_GATHER_BLOCKS = 256;
  constexpr int64_t CHUNKED_FROM_ROWS = 256;
  if (b > HOST_GATHER_BLOCKS || (n >= CHUNKED_FROM_ROWS && !accumulate)) {
    hipPointerAttribute_t attr;
    bool in_host_memory = false;
    if (hipPointerGetAttributes(&attr, src) == hipSuccess) {
      in_host_memory = attr.type == hipMemoryTypeHost;
    } else {
      (void)hipGetLastError();   // an address the runtime does not know: treat it as device memory
    }
    if (in_host_memory) {
      if (b > HOST_GATHER_BLOCKS) b = HOST_GATHER_BLOCKS;
    } else if (n >= CHUNKED_FROM_ROWS && !accumulate) {
      return hc_gather_rows_device(src, src_dtype, n_rows, ids, mask, dst, dst_dtype, n, F, st);
    }
  }
  dim3 g((unsigned)b), bl(HC_BLOCK);
  if (src_dtype == HC_F32) return launch_gather<float>(src, n_rows, ids, mask, dst, dst_dtype, accumulate, n, F, g, bl, st);
  if (src_dtype == HC_F16) return launch_gather<__half>(src, n_rows, ids, mask, dst, dst_dtype, accumulate, n, F, g, bl, st);
  return launch_gather<__hip_bfloat16>(src, n_rows, ids, mask, dst, dst_dtype, accumulate, n, F, g, bl, st);
}

extern "C" int hc_stream_create_cu_limited(int n_cus, void **stream) {
  HC_REQUIRE(stream != nullptr && n_cus >= 1);
  *stream = nullptr;
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
    (void)hipGetLastError();
    return HC_ELAUNCH;
  }
  const int total = prop.multiProcessorCount;
  if (total < 1) return HC_ELAUNCH;
  if (n_cus > total) n_cus = total;
  // consecutive mask bits are dealt out over the chip's dies and shader engines by the driver, so the first
  // n bits are n compute units spread evenly; default priority, like every stream of this library
  uint32_t words[32] = {0};
  const int n_words = (total + 31) / 32;
  if (n_words > 32) return HC_EUNSUPPORTED;
  for (int c = 0; c < n_cus; ++c) words[c / 32] |= 1u << (c % 32);
  hipStream_t st = nullptr;
  if (hipExtStreamCreateWithCUMask(&st, (uint32_t)n_words, words) != hipSuccess) {
    (void)hipGetLastError();
    return HC_ELAUNCH;
  }
  *stream = st;
  return HC_OK;
}

extern "C" int hc_stream_destroy(void *stream) {
  if (stream == nullptr) return HC_OK;
  if (hipStreamDestroy(static_cast<hipStream_t>(stream)) != hipSuccess) {
    (void)hipGetLastError();
    return HC_ELAUNCH;
  }
  return HC_OK;
}

extern "C" int hc_fixup_rows(const void *src, int src_dtype, int64_t n_rows, const int64_t *ids,
                             const uint8_t *need, const uint8_t *have, void *dst, int dst_dtype, int64_t n,
                             int64_t F, void *stream) {
  HC_REQUIRE(n >= 0 && F > 0 && n_rows >= 0);
  if (src_dtype < HC_F32 || src_dtype > HC_BF16 || dst_dtype < HC_F32 || dst_dtype > HC_BF16) return HC_EDTYPE;
  if (n == 0) return HC_OK;
  HC_REQUIRE(ids && dst && need && have && (src || n_rows == 0));
  // rows that were gathered ahead of time under a guess of which are needed (have), brought to the exact
  // answer (need): the few rows that differ do the work
  return hc_fixup_rows_chunked(src, src_dtype, n_rows, ids, need, have, dst, dst_dtype, n, F,
                               static_cast<hipStream_t>(stream));
}

namespace {
int lookup_launch(const int64_t *map, int64_t map_len, const int64_t *ids, int64_t offset, const int64_t *n_valid_dev,
                  int64_t *out, int64_t n, void *stream) {
  HC_REQUIRE(n >= 0 && map_len >= 0);
  if (n == 0) return HC_OK;
  HC_REQUIRE(map && ids && out);
  if (!hc_grid_ok((n + HC_BLOCK - 1) / HC_BLOCK)) return HC_EUNSUPPORTED;
  lookup_kernel<<<dim3(blocks_for(n)), dim3(HC_BLOCK), 0, static_cast<hipStream_t>(stream)>>>(
      map, map_len, ids, offset, out, n, n_valid_dev);
  return hc_launch_status();
}
}  // namespace

extern "C" int hc_lookup(const int64_t *map, int64_t map_len, const int64_t *ids, int64_t offset,
                         int64_t *out, int64_t n, void *stream) {
  return lookup_launch(map, map_len, ids, offset, nullptr, out, n, stream);
}

extern "C" int hc_lookup_dev(const int64_t *map, int64_t map_len, const int64_t *ids, int64_t offset,
                             const int64_t *n_valid_dev, int64_t *out, int64_t n, void *stream) {
  HC_REQUIRE(n_valid_dev != nullptr);
  return lookup_launch(map, map_len, ids, offset, n_valid_dev, out, n, stream);
}

namespace {
int ring_lookup_launch(const int64_t *full2slot, int64_t n_full, const int64_t *ids, const int64_t *checkin,
                       int64_t now, const int64_t *now_dev, const int64_t *n_valid_dev, int64_t age_limit,
                       const void *table, int table_dtype, int64_t capacity, int64_t F, int64_t *slot_out,
                       float *rows_out, int64_t n, void *stream) {
  HC_REQUIRE(n >= 0 && n_full >= 0 && capacity >= 0 && F > 0);
  if (table_dtype < HC_F32 || table_dtype > HC_BF16) return HC_EDTYPE;
  if (n == 0) return HC_OK;
  HC_REQUIRE(full2slot && ids && slot_out);
  HC_REQUIRE(rows_out == nullptr || table != nullptr);
  const int64_t b = (n + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
  if (!hc_grid_ok(b)) return HC_EUNSUPPORTED;
  dim3 g((unsigned)b), bl(HC_BLOCK);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (table_dtype == HC_F32)
    ring_lookup_kernel<float><<<g, bl, 0, st>>>(full2slot, n_full, ids, checkin, now, age_limit,
                                                static_cast<const float *>(table), capacity, F, slot_out, rows_out, n,
                                                now_dev, n_valid_dev);
  else if (table_dtype == HC_F16)
    ring_lookup_kernel<__half><<<g, bl, 0, st>>>(full2slot, n_full, ids, checkin, now, age_limit,
                                                 static_cast<const __half *>(table), capacity, F, slot_out, rows_out, n,
                                                 now_dev, n_valid_dev);
  else
    ring_lookup_kernel<__hip_bfloat16><<<g, bl, 0, st>>>(full2slot, n_full, ids, checkin, now, age_limit,
                                                         static_cast<const __hip_bfloat16 *>(table), capacity, F,
                                                         slot_out, rows_out, n, now_dev, n_valid_dev);
  return hc_launch_status();
}
}  // namespace

extern "C" int hc_ring_lookup(const int64_t *full2slot, int64_t n_full, const int64_t *ids,
                              const int64_t *checkin, int64_t now, int64_t age_limit, const void *table,
                              int table_dtype, int64_t capacity, int64_t F, int64_t *slot_out,
                              float *rows_out, int64_t n, void *stream) {
  return ring_lookup_launch(full2slot, n_full, ids, checkin, now, nullptr, nullptr, age_limit, table, table_dtype,
                            capacity, F, slot_out, rows_out, n, stream);
}

extern "C" int hc_ring_lookup_dev(const int64_t *full2slot, int64_t n_full, const int64_t *ids,
                                  const int64_t *checkin, const int64_t *now_dev, const int64_t *n_valid_dev,
                                  int64_t age_limit, const void *table, int table_dtype, int64_t capacity,
                                  int64_t F, int64_t *slot_out, float *rows_out, int64_t n, void *stream) {
  HC_REQUIRE(now_dev != nullptr && n_valid_dev != nullptr);
  return ring_lookup_launch(full2slot, n_full, ids, checkin, 0, now_dev, n_valid_dev, age_limit, table, table_dtype,
                            capacity, F, slot_out, rows_out, n, stream);
}

extern "C" int hc_stage_arrays(const void *const *src, void *const *dst, const int64_t *n_copy,
                               const int64_t *n_total, const int64_t *fill, const int *elem_bytes, int n_arrays,
                               int64_t *scalars_dst, const int64_t *scalars, int n_scalars, void *stream) {
  HC_REQUIRE(n_arrays >= 0 && n_arrays <= STAGE_MAX_ARRAYS && n_scalars >= 0 && n_scalars <= STAGE_MAX_SCALARS);
  HC_REQUIRE(n_arrays == 0 || (src && dst && n_copy && n_total && fill && elem_bytes));
  HC_REQUIRE(n_scalars == 0 || (scalars_dst && scalars));
  if (n_arrays == 0 && n_scalars == 0) return HC_OK;
  StagePlan p{};
  int64_t longest = 1;
  for (int a = 0; a < n_arrays; ++a) {
    HC_REQUIRE(n_total[a] >= 0 && n_copy[a] >= 0 && n_copy[a] <= n_total[a]);
    HC_REQUIRE(elem_bytes[a] == 8 || elem_bytes[a] == 4 || elem_bytes[a] == 2 || elem_bytes[a] == 1);
    HC_REQUIRE(n_total[a] == 0 || dst[a] != nullptr);
    HC_REQUIRE(n_copy[a] == 0 || src[a] != nullptr);
    p.src[a] = src[a];
    p.dst[a] = dst[a];
    p.n_copy[a] = n_copy[a];
    p.n_total[a] = n_total[a];
    p.fill[a] = fill[a];
    p.elem[a] = elem_bytes[a];
    if (n_total[a] > longest) longest = n_total[a];
  }
  p.scalars_dst = scalars_dst;
  p.n_scalars = n_scalars;
  for (int k = 0; k < n_scalars; ++k) p.scalars[k] = scalars[k];
  stage_kernel<<<dim3(blocks_for_stage(longest), (unsigned)(n_arrays > 0 ? n_arrays : 1)), dim3(HC_BLOCK), 0,
                 static_cast<hipStream_t>(stream)>>>(p);
  return hc_launch_status();
}

// ---------------------------------------------------------------------------------------
// hc_load_mask: which rows of a batch must be read from the feature store, and the cache's
// hit counters, in one launch (the reference spells the mask with three tensor operators and
// prints the same counts from a debug branch, hiscache/history_cache.py:327-341).
// ---------------------------------------------------------------------------------------
namespace {
constexpr int LM_COUNTERS = 8;

__global__ __launch_bounds__(HC_BLOCK) void load_mask_kernel(const uint8_t *__restrict__ used,
                                                              const int64_t *__restrict__ sub2feat,
                                                              const int64_t *__restrict__ sub2embed,
                                                              const uint8_t *__restrict__ prev_mask,
                                                              int64_t n_all, int64_t n1, int64_t n_prev,
                                                              uint8_t *__restrict__ hit_feat,
                                                              uint8_t *__restrict__ load_mask,
                                                              unsigned long long *__restrict__ counters) {
  __shared__ unsigned int s_cnt[LM_COUNTERS];
  if (threadIdx.x < LM_COUNTERS) s_cnt[threadIdx.x] = 0u;
  __syncthreads();
  // A block walks the elements with the grid's stride and adds its counts to the totals once: every block's
  // adds land on one cache line, where they are served one after the other (hundreds of blocks with one element
  // per thread spent most of the kernel queueing there).
  unsigned int c_pruned = 0u, c_hit = 0u, c_load = 0u, c_emb = 0u, c_adm = 0u;
  int64_t n_max = n_all > n1 ? n_all : n1;
  if (n_prev > n_max) n_max = n_prev;
  const int64_t stride = (int64_t)gridDim.x * HC_BLOCK;
  for (int64_t base = (int64_t)blockIdx.x * HC_BLOCK; base < n_max; base += stride) {   // block-uniform trip count
    const int64_t i = base + threadIdx.x;
    bool u = false, hit = false, load = false, emb = false, adm = false;
    if (i < n_all) {
      u = used[i] != 0;
      hit = sub2feat != nullptr && sub2feat[i] != -1;
      load = u && !hit;
      if (hit_feat != nullptr) hit_feat[i] = hit ? 1 : 0;
      if (load_mask != nullptr) load_mask[i] = load ? 1 : 0;
    }
    if (counters == nullptr) continue;
    if (sub2embed != nullptr && i < n1) emb = sub2embed[i] != -1;
    if (prev_mask != nullptr && i < n_prev) adm = prev_mask[i] != 0;
    c_pruned += (unsigned int)__popcll(__ballot(i < n_all && !u));
    c_hit += (unsigned int)__popcll(__ballot(hit));
    c_load += (unsigned int)__popcll(__ballot(load));
    c_emb += (unsigned int)__popcll(__ballot(emb));
    c_adm += (unsigned int)__popcll(__ballot(adm));
  }
  if (counters == nullptr) return;
  if (hc_lane() == 0) {                      // the ballots gave every lane of a wave the wave's counts
    if (c_emb) atomicAdd(&s_cnt[3], c_emb);
    if (c_pruned) atomicAdd(&s_cnt[4], c_pruned);
    if (c_hit) atomicAdd(&s_cnt[5], c_hit);
    if (c_load) atomicAdd(&s_cnt[6], c_load);
    if (c_adm) atomicAdd(&s_cnt[7], c_adm);
  }
  __syncthreads();
  if (threadIdx.x >= 3 && threadIdx.x < LM_COUNTERS && s_cnt[threadIdx.x] != 0u)
    atomicAdd(&counters[threadIdx.x], (unsigned long long)s_cnt[threadIdx.x]);
  if (blockIdx.x == 0 && threadIdx.x < 3) {
    const unsigned long long add = threadIdx.x == 0 ? 1ull : (threadIdx.x == 1 ? (unsigned long long)n_all
                                                                                : (unsigned long long)n1);
    atomicAdd(&counters[threadIdx.x], add);
  }
}
}  // namespace

extern "C" int hc_load_mask(const uint8_t *used, const int64_t *sub2feat, const int64_t *sub2embed,
                            const uint8_t *prev_mask, int64_t n_all, int64_t n1, int64_t n_prev,
                            uint8_t *hit_feat, uint8_t *load_mask, int64_t *counters, void *stream) {
  HC_REQUIRE(n_all >= 0 && n1 >= 0 && n_prev >= 0);
  HC_REQUIRE(used != nullptr || n_all == 0);
  HC_REQUIRE(sub2embed != nullptr || n1 == 0);
  HC_REQUIRE(prev_mask != nullptr || n_prev == 0);
  int64_t n = n_all > n1 ? n_all : n1;
  if (n_prev > n) n = n_prev;
  if (n == 0) n = 1;                               // the call is still counted
  int64_t b = (n + HC_BLOCK - 1) / HC_BLOCK;
  if (!hc_grid_ok(b)) return HC_EUNSUPPORTED;
  // with counters: few blocks, each walking its share (one add per block and counter); without: a thread per element
  const int64_t cap = counters != nullptr ? 128 : 4096;
  if (b > cap) b = cap;
  load_mask_kernel<<<dim3((unsigned)b), dim3(HC_BLOCK), 0, static_cast<hipStream_t>(stream)>>>(
      used, sub2feat, sub2embed, prev_mask, n_all, n1, n_prev, hit_feat, load_mask,
      reinterpret_cast<unsigned long long *>(counters));
  return hc_launch_status();
}
