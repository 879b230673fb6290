// Two-tier feature rows: copies of the most requested rows of a feature matrix live in device memory, the
// whole matrix stays in pinned host memory.  A batch's rows are fetched in two launches that write disjoint
// rows of the same output:
//   hc_gather_rows_hot      at full width: rows that have a device copy are copied from it, rows that are not
//                           asked for are cleared, the others are flagged;
//   hc_gather_rows_flagged  the flagged rows, from the host matrix over the host link.  A wave examines 64
//                           rows at a time (one flag and one id per lane), then walks the flagged ones two at
//                           a time, so that a few hundred waves keep the link busy and no wave spends its
//                           time stepping over rows it has nothing to do for.
// The role of the feature half of the reference's cache (hotness-ordered rows kept in GPU memory,
// /root/reference/hiscache/history_cache.py:121-142, merged with the rows read through UVM, :345-350).
#include "hc_common.h"

namespace {

constexpr int TV = 4;   // elements per lane per step when rows allow

template <typename TS, typename TD>
__device__ __forceinline__ bool tier_vec_ok(const TS *src, const TD *dst, int64_t F) {
  return (F % TV == 0) && (reinterpret_cast<uintptr_t>(src) % (sizeof(TS) * TV) == 0) &&
         (reinterpret_cast<uintptr_t>(dst) % (sizeof(TD) * TV) == 0);
}

// o[0..F) = s ? s[0..F) : 0 by the whole wave.
template <typename TS, typename TD>
__device__ __forceinline__ void tier_copy_row(const TS *__restrict__ s, TD *__restrict__ o, int64_t F, int lane,
                                              bool vec_ok) {
  if (vec_ok) {
    for (int64_t c = (int64_t)lane * TV; c < F; c += HC_WAVE * TV) {
      float v[TV];
      if (s != nullptr) {
        hc_vec<TS, TV>::load(s + c, v);
      } else {
#pragma unroll
        for (int k = 0; k < TV; ++k) v[k] = 0.0f;
      }
      hc_vec<TD, TV>::store(o + c, v);
    }
  } else {
    for (int64_t c = lane; c < F; c += HC_WAVE) o[c] = hc_from_f32<TD>(s != nullptr ? hc_to_f32<TS>(s[c]) : 0.0f);
  }
}

// A wave serves HOT_ROWS consecutive requested rows: one lane per row reads the row's mask byte, id and slot (three
// dependent reads for all rows at once instead of once per row), then the wave copies the rows HOT_INFLIGHT at a
// time, every row's load issued before the first store.  With a wave per row the launch is a chain of four round
// trips per 512-byte row and runs at a fraction of the memory rate.
constexpr int HOT_ROWS = 16;
constexpr int HOT_INFLIGHT = 4;
constexpr int ROW_ZERO = 0, ROW_COPY = 1, ROW_SKIP = 2;

// TIERED = false: the plain gather of a matrix in device memory (hot is the matrix, a node's row is its id, no row
// is left to another launch).
template <typename TS, typename TD, bool TIERED>
__global__ __launch_bounds__(HC_BLOCK) void tier_hot_kernel(const TS *__restrict__ hot, int64_t n_hot,
                                                             const int32_t *__restrict__ slot_map, int64_t n_map,
                                                             const int64_t *__restrict__ ids,
                                                             const uint8_t *__restrict__ mask,
                                                             TD *__restrict__ dst, uint8_t *__restrict__ cold,
                                                             int64_t n, int64_t F) {
  const int lane = hc_lane();
  const int64_t base = ((int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block()) * HOT_ROWS;
  if (base >= n) return;
  const int64_t i = base + lane;
  int state = ROW_SKIP;
  int64_t slot = 0;
  if (lane < HOT_ROWS && i < n) {
    bool take = mask == nullptr || mask[i] != 0;
    int64_t id = 0;
    if (take) {
      id = ids[i];
      if (id < 0) id += n_map;
      if (id < 0 || id >= n_map) take = false;
    }
    if constexpr (TIERED) slot = take ? (int64_t)slot_map[id] : -1;
    else slot = id;
    const bool is_cold = TIERED && take && (slot < 0 || slot >= n_hot);
    if constexpr (TIERED) cold[i] = is_cold ? 1 : 0;
    state = is_cold ? ROW_SKIP : (take ? ROW_COPY : ROW_ZERO);     // a cold row is written by the other launch
  }
  const bool vec_ok = tier_vec_ok(hot, dst, F);
#pragma unroll
  for (int r0 = 0; r0 < HOT_ROWS; r0 += HOT_INFLIGHT) {
    int st[HOT_INFLIGHT];
    const TS *s[HOT_INFLIGHT];
    bool any = false;
#pragma unroll
    for (int k = 0; k < HOT_INFLIGHT; ++k) {
      st[k] = __builtin_amdgcn_readlane(state, r0 + k);
      s[k] = hot + hc_readlane64(slot, r0 + k) * F;
      any = any || st[k] != ROW_SKIP;
    }
    if (!any) continue;                                            // wave-uniform
    TD *o = dst + (base + r0) * F;
    if (vec_ok) {
      for (int64_t c = (int64_t)lane * TV; c < F; c += HC_WAVE * TV) {
        float v[HOT_INFLIGHT][TV];
#pragma unroll
        for (int k = 0; k < HOT_INFLIGHT; ++k) {
#pragma unroll
          for (int e = 0; e < TV; ++e) v[k][e] = 0.0f;
          if (st[k] == ROW_COPY) hc_vec<TS, TV>::load(s[k] + c, v[k]);
        }
#pragma unroll
        for (int k = 0; k < HOT_INFLIGHT; ++k)
          if (st[k] != ROW_SKIP) hc_vec<TD, TV>::store(o + k * F + c, v[k]);
      }
    } else {
      for (int64_t c = lane; c < F; c += HC_WAVE) {
        float v[HOT_INFLIGHT];
#pragma unroll
        for (int k = 0; k < HOT_INFLIGHT; ++k) v[k] = st[k] == ROW_COPY ? hc_to_f32<TS>(s[k][c]) : 0.0f;
#pragma unroll
        for (int k = 0; k < HOT_INFLIGHT; ++k)
          if (st[k] != ROW_SKIP) o[k * F + c] = hc_from_f32<TD>(v[k]);
      }
    }
  }
}

// FIXUP = true: rows that were gathered under a guess (have) brought to the exact answer (flag = need): the rows
// where the two differ are the flagged ones, read if needed and cleared if not.
template <typename TS, typename TD, bool FIXUP>
__global__ __launch_bounds__(HC_BLOCK) void gather_flagged_kernel(const TS *__restrict__ src, int64_t n_rows,
                                                                   const int64_t *__restrict__ ids,
                                                                   const uint8_t *__restrict__ flag,
                                                                   const uint8_t *__restrict__ have,
                                                                   TD *__restrict__ dst, int64_t n, int64_t F) {
  const int lane = hc_lane();
  const bool vec_ok = tier_vec_ok(src, dst, F);
  const int64_t n_chunks = (n + HC_WAVE - 1) / HC_WAVE;
  const int64_t stride = (int64_t)gridDim.x * HC_WAVES_PER_BLOCK;
  for (int64_t chunk = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block(); chunk < n_chunks;
       chunk += stride) {
    const int64_t i = chunk * HC_WAVE + lane;
    bool flagged = i < n && flag[i] != 0;
    bool read = flagged;
    if constexpr (FIXUP) {
      const bool hv = i < n && have[i] != 0;
      read = flagged && !hv;                 // needed, not read yet
      flagged = i < n && flagged != hv;      // (read, not needed any more: cleared)
    }
    int64_t id = -1;
    if (read) {
      id = ids[i];
      if (id < 0) id += n_rows;
      if (id < 0 || id >= n_rows) id = -1;   // a flagged row without a source row is cleared
    }
    unsigned long long todo = __ballot(flagged);
    while (todo != 0ull) {
      const int b0 = __ffsll((long long)todo) - 1;
      todo &= todo - 1ull;
      int b1 = -1;
      if (todo != 0ull) {
        b1 = __ffsll((long long)todo) - 1;
        todo &= todo - 1ull;
      }
      const int64_t id0 = __shfl(id, b0, HC_WAVE);
      const int64_t id1 = b1 >= 0 ? __shfl(id, b1, HC_WAVE) : -1;
      const int64_t r0 = chunk * HC_WAVE + b0, r1 = chunk * HC_WAVE + (b1 >= 0 ? b1 : b0);
      const TS *s0 = id0 >= 0 ? src + id0 * F : nullptr;
      const TS *s1 = id1 >= 0 ? src + id1 * F : nullptr;
      TD *o0 = dst + r0 * F, *o1 = dst + r1 * F;
      if (vec_ok) {
        // both rows' loads are issued before either row is stored: two reads in flight per wave
        for (int64_t c = (int64_t)lane * TV; c < F; c += HC_WAVE * TV) {
          float v0[TV], v1[TV];
#pragma unroll
          for (int k = 0; k < TV; ++k) v0[k] = v1[k] = 0.0f;
          if (s0 != nullptr) hc_vec<TS, TV>::load(s0 + c, v0);
          if (s1 != nullptr) hc_vec<TS, TV>::load(s1 + c, v1);
          hc_vec<TD, TV>::store(o0 + c, v0);
          if (b1 >= 0) hc_vec<TD, TV>::store(o1 + c, v1);
        }
      } else {
        tier_copy_row<TS, TD>(s0, o0, F, lane, false);
        if (b1 >= 0) tier_copy_row<TS, TD>(s1, o1, F, lane, false);
      }
    }
  }
}

template <typename TS, bool TIERED>
int launch_hot(const void *hot, int64_t n_hot, const int32_t *slot_map, int64_t n_map, const int64_t *ids,
               const uint8_t *mask, void *dst, int dst_dtype, uint8_t *cold, int64_t n, int64_t F, dim3 g,
               hipStream_t st) {
  const TS *h = static_cast<const TS *>(hot);
  const dim3 bl(HC_BLOCK);
  if (dst_dtype == HC_F32)
    tier_hot_kernel<TS, float, TIERED><<<g, bl, 0, st>>>(h, n_hot, slot_map, n_map, ids, mask,
                                                         static_cast<float *>(dst), cold, n, F);
  else if (dst_dtype == HC_F16)
    tier_hot_kernel<TS, __half, TIERED><<<g, bl, 0, st>>>(h, n_hot, slot_map, n_map, ids, mask,
                                                          static_cast<__half *>(dst), cold, n, F);
  else
    tier_hot_kernel<TS, __hip_bfloat16, TIERED><<<g, bl, 0, st>>>(h, n_hot, slot_map, n_map, ids, mask,
                                                                  static_cast<__hip_bfloat16 *>(dst), cold, n, F);
  return hc_launch_status();
}

template <bool TIERED>
int dispatch_hot(const void *hot, int hot_dtype, int64_t n_hot, const int32_t *slot_map, int64_t n_map,
                 const int64_t *ids, const uint8_t *mask, void *dst, int dst_dtype, uint8_t *cold, int64_t n,
                 int64_t F, hipStream_t st) {
  const int64_t waves = (n + HOT_ROWS - 1) / HOT_ROWS;
  const int64_t b = (waves + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
  if (!hc_grid_ok(b)) return HC_EUNSUPPORTED;
  const dim3 g((unsigned)b);
  if (hot_dtype == HC_F32)
    return launch_hot<float, TIERED>(hot, n_hot, slot_map, n_map, ids, mask, dst, dst_dtype, cold, n, F, g, st);
  if (hot_dtype == HC_F16)
    return launch_hot<__half, TIERED>(hot, n_hot, slot_map, n_map, ids, mask, dst, dst_dtype, cold, n, F, g, st);
  return launch_hot<__hip_bfloat16, TIERED>(hot, n_hot, slot_map, n_map, ids, mask, dst, dst_dtype, cold, n, F, g, st);
}

template <typename TS, bool FIXUP>
int launch_flagged(const void *src, int64_t n_rows, const int64_t *ids, const uint8_t *flag, const uint8_t *have,
                   void *dst, int dst_dtype, int64_t n, int64_t F, dim3 g, hipStream_t st) {
  const TS *s = static_cast<const TS *>(src);
  const dim3 bl(HC_BLOCK);
  if (dst_dtype == HC_F32)
    gather_flagged_kernel<TS, float, FIXUP><<<g, bl, 0, st>>>(s, n_rows, ids, flag, have, static_cast<float *>(dst), n, F);
  else if (dst_dtype == HC_F16)
    gather_flagged_kernel<TS, __half, FIXUP><<<g, bl, 0, st>>>(s, n_rows, ids, flag, have, static_cast<__half *>(dst), n, F);
  else
    gather_flagged_kernel<TS, __hip_bfloat16, FIXUP><<<g, bl, 0, st>>>(s, n_rows, ids, flag, have,
                                                                       static_cast<__hip_bfloat16 *>(dst), n, F);
  return hc_launch_status();
}

template <bool FIXUP>
int dispatch_flagged(const void *src, int src_dtype, int64_t n_rows, const int64_t *ids, const uint8_t *flag,
                     const uint8_t *have, void *dst, int dst_dtype, int64_t n, int64_t F, int64_t max_blocks,
                     hipStream_t st) {
  const int64_t chunks = (n + HC_WAVE - 1) / HC_WAVE;
  int64_t b = (chunks + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
  if (b > max_blocks) b = max_blocks;
  const dim3 g((unsigned)b);
  if (src_dtype == HC_F32) return launch_flagged<float, FIXUP>(src, n_rows, ids, flag, have, dst, dst_dtype, n, F, g, st);
  if (src_dtype == HC_F16) return launch_flagged<__half, FIXUP>(src, n_rows, ids, flag, have, dst, dst_dtype, n, F, g, st);
  return launch_flagged<__hip_bfloat16, FIXUP>(src, n_rows, ids, flag, have, dst, dst_dtype, n, F, g, st);
}

bool dtype_ok(int d) { return d >= HC_F32 && d <= HC_BF16; }

}  // namespace

extern "C" int hc_gather_rows_hot(const void *hot, int hot_dtype, int64_t n_hot, const int32_t *slot_map,
                                  int64_t n_map, const int64_t *ids, const uint8_t *mask, void *dst,
                                  int dst_dtype, uint8_t *cold, int64_t n, int64_t F, void *stream) {
  HC_REQUIRE(n >= 0 && F > 0 && n_hot >= 0 && n_map >= 0);
  if (!dtype_ok(hot_dtype) || !dtype_ok(dst_dtype)) return HC_EDTYPE;
  if (n == 0) return HC_OK;
  HC_REQUIRE(ids && dst && cold && (slot_map || n_map == 0) && (hot || n_hot == 0));
  return dispatch_hot<true>(hot, hot_dtype, n_hot, slot_map, n_map, ids, mask, dst, dst_dtype, cold, n, F,
                            static_cast<hipStream_t>(stream));
}

// The plain gather (hc_gather_rows without accumulation) of a matrix in device memory; arguments checked by the caller.
int hc_gather_rows_device(const void *src, int src_dtype, int64_t n_rows, const int64_t *ids, const uint8_t *mask,
                          void *dst, int dst_dtype, int64_t n, int64_t F, hipStream_t st) {
  return dispatch_hot<false>(src, src_dtype, n_rows, nullptr, n_rows, ids, mask, dst, dst_dtype, nullptr, n, F, st);
}

extern "C" int hc_gather_rows_flagged(const void *src, int src_dtype, int64_t n_rows, const int64_t *ids,
                                      const uint8_t *flag, void *dst, int dst_dtype, int64_t n, int64_t F,
                                      void *stream) {
  HC_REQUIRE(n >= 0 && F > 0 && n_rows >= 0);
  if (!dtype_ok(src_dtype) || !dtype_ok(dst_dtype)) return HC_EDTYPE;
  if (n == 0) return HC_OK;
  HC_REQUIRE(ids && dst && flag && (src || n_rows == 0));
  // a matrix in host memory: a few hundred waves keep the link busy, more only stand in the way of the
  // kernels that run beside this one; a matrix in device memory: enough waves to fill the chip
  int64_t cap = 4096;
  hipPointerAttribute_t attr;
  if (src != nullptr && hipPointerGetAttributes(&attr, src) == hipSuccess) {
    if (attr.type == hipMemoryTypeHost) cap = 256;
  } else {
    (void)hipGetLastError();
  }
  return dispatch_flagged<false>(src, src_dtype, n_rows, ids, flag, nullptr, dst, dst_dtype, n, F, cap,
                                 static_cast<hipStream_t>(stream));
}

// hc_fixup_rows: the rows where need and have differ are few, whatever memory the matrix lies in.
int hc_fixup_rows_chunked(const void *src, int src_dtype, int64_t n_rows, const int64_t *ids, const uint8_t *need,
                          const uint8_t *have, void *dst, int dst_dtype, int64_t n, int64_t F, hipStream_t st) {
  return dispatch_flagged<true>(src, src_dtype, n_rows, ids, need, have, dst, dst_dtype, n, F, 4096, st);
}
