// Shared device/host helpers for the gfx950 kernels (wave64 only).
#pragma once

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hiscache_hip.h"

#define HC_WAVE 64
#define HC_BLOCK 256
#define HC_WAVES_PER_BLOCK (HC_BLOCK / HC_WAVE)

#define HC_REQUIRE(cond) \
  do {                   \
    if (!(cond)) return HC_EINVAL; \
  } while (0)

static inline int hc_launch_status() {
  return hipGetLastError() == hipSuccess ? HC_OK : HC_ELAUNCH;
}

static inline size_t hc_align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Grid limit for a 1-D launch: gridDim.x * blockDim.x must stay below 2^32 (blocks of up to
// 1024 threads are used by the scan kernel, so the bound is taken for those).
static inline bool hc_grid_ok(int64_t blocks) { return blocks > 0 && blocks <= 0xffffffffLL / HC_BLOCK; }

// feature_tiers.hip: the plain row gather of a matrix in device memory, several rows per wave
// (hc_gather_rows hands such calls over; arguments are checked there).
__attribute__((visibility("hidden"))) int hc_gather_rows_device(const void *src, int src_dtype, int64_t n_rows, const int64_t *ids, const uint8_t *mask,
                          void *dst, int dst_dtype, int64_t n, int64_t F, hipStream_t st);

// feature_tiers.hip: hc_fixup_rows' launch (64 rows examined per wave, the few that differ read or cleared).
__attribute__((visibility("hidden"))) int hc_fixup_rows_chunked(const void *src, int src_dtype, int64_t n_rows,
                                                                const int64_t *ids, const uint8_t *need,
                                                                const uint8_t *have, void *dst, int dst_dtype,
                                                                int64_t n, int64_t F, hipStream_t st);

#ifdef __HIPCC__

__device__ __forceinline__ int hc_lane() { return (int)(threadIdx.x & (HC_WAVE - 1)); }

// Index of this wave inside its block, forced into a scalar register so that
// everything derived from it (row id, row bounds) is wave-uniform.
__device__ __forceinline__ int hc_wave_in_block() {
  return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
}

__device__ __forceinline__ int64_t hc_readlane64(int64_t v, int lane) {
  int lo = __builtin_amdgcn_readlane((int)(uint32_t)(uint64_t)v, lane);
  int hi = __builtin_amdgcn_readlane((int)(uint32_t)((uint64_t)v >> 32), lane);
  return (int64_t)(((uint64_t)(uint32_t)hi << 32) | (uint64_t)(uint32_t)lo);
}

__device__ __forceinline__ int64_t hc_uniform64(int64_t v) {
  int lo = __builtin_amdgcn_readfirstlane((int)(uint32_t)(uint64_t)v);
  int hi = __builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)(uint32_t)hi << 32) | (uint64_t)(uint32_t)lo);
}

__device__ __forceinline__ float hc_readlane_f(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// Workgroups are handed to the 8 XCDs round-robin (workgroup i runs on XCD i % 8) and every XCD
// has its own L2.  This maps the hardware block index to a logical one so that an XCD works on
// runs of CHUNK consecutive logical blocks: neighbouring rows or sources, which tend to touch the
// same index lines and the same data, then share an L2.  The runs of the 8 XCDs are interleaved
// (XCD x takes run x of every group of 8 runs), so that work whose cost drifts along the block
// range -- rows sorted by degree, layers with different fan-outs -- stays balanced over the XCDs.
// A bijection of [0, n); blocks behind the last full group keep their index.
#define HC_NUM_XCD 8
template <int CHUNK>
__device__ __forceinline__ int64_t hc_xcd_block(int64_t bid, int64_t n) {
  constexpr int64_t GROUP = (int64_t)HC_NUM_XCD * CHUNK;
  const int64_t g = bid / GROUP;
  if ((g + 1) * GROUP > n) return bid;
  const int64_t in = bid - g * GROUP;
  return g * GROUP + (in % HC_NUM_XCD) * CHUNK + in / HC_NUM_XCD;
}

// Butterfly sum over the 64 lanes, partner distance 32,16,8,4,2,1.  Every lane
// ends with the same bits (fp add is commutative), and the order is the one
// the CPU checker reproduces.
__device__ __forceinline__ float hc_wave_sum_butterfly(float v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v = v + __shfl_xor(v, d, HC_WAVE);
  return v;
}

// ---- element conversion ----------------------------------------------------
template <typename T>
__device__ __forceinline__ float hc_to_f32(T v);
template <>
__device__ __forceinline__ float hc_to_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ float hc_to_f32<__half>(__half v) { return __half2float(v); }
template <>
__device__ __forceinline__ float hc_to_f32<__hip_bfloat16>(__hip_bfloat16 v) {
  return __bfloat162float(v);
}

template <typename T>
__device__ __forceinline__ T hc_from_f32(float v);
template <>
__device__ __forceinline__ float hc_from_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ __half hc_from_f32<__half>(float v) { return __float2half_rn(v); }
template <>
__device__ __forceinline__ __hip_bfloat16 hc_from_f32<__hip_bfloat16>(float v) {
  return __float2bfloat16(v);
}

// ---- vector load of VEC consecutive elements, widened to fp32 ---------------
template <int BYTES>
struct hc_raw;
template <>
struct hc_raw<2> { typedef uint16_t type; };
template <>
struct hc_raw<4> { typedef uint32_t type; };
template <>
struct hc_raw<8> { typedef uint2 type; };
template <>
struct hc_raw<16> { typedef uint4 type; };

template <typename T, int VEC>
struct hc_vec {
  typedef typename hc_raw<sizeof(T) * VEC>::type raw_t;
  union U {
    raw_t raw;
    T e[VEC];
    __device__ U() {}
  };
  // p must be aligned to sizeof(T) * VEC
  __device__ __forceinline__ static void load(const T *p, float (&out)[VEC]) {
    U u;
    u.raw = *reinterpret_cast<const raw_t *>(p);
#pragma unroll
    for (int i = 0; i < VEC; ++i) out[i] = hc_to_f32<T>(u.e[i]);
  }
  __device__ __forceinline__ static void store(T *p, const float (&in)[VEC]) {
    U u;
#pragma unroll
    for (int i = 0; i < VEC; ++i) u.e[i] = hc_from_f32<T>(in[i]);
    *reinterpret_cast<raw_t *>(p) = u.raw;
  }
  // Same load / store with the non-temporal hint: rows that are read or written once should not
  // displace the index and map lines that are reused.
  typedef uint32_t nt_t __attribute__((ext_vector_type(sizeof(T) * VEC >= 4 ? sizeof(T) * VEC / 4 : 1)));
  __device__ __forceinline__ static void load_nt(const T *p, float (&out)[VEC]) {
    if constexpr (sizeof(T) * VEC >= 4) {
      union N {
        nt_t raw;
        T e[VEC];
        __device__ N() {}
      } u;
      u.raw = __builtin_nontemporal_load(reinterpret_cast<const nt_t *>(p));
#pragma unroll
      for (int i = 0; i < VEC; ++i) out[i] = hc_to_f32<T>(u.e[i]);
    } else {
      load(p, out);
    }
  }
  __device__ __forceinline__ static void store_nt(T *p, const float (&in)[VEC]) {
    if constexpr (sizeof(T) * VEC >= 4) {
      union N {
        nt_t raw;
        T e[VEC];
        __device__ N() {}
      } u;
#pragma unroll
      for (int i = 0; i < VEC; ++i) u.e[i] = hc_from_f32<T>(in[i]);
      __builtin_nontemporal_store(u.raw, reinterpret_cast<nt_t *>(p));
    } else {
      store(p, in);
    }
  }
};

// Store VEC consecutive fp32 values (VEC may exceed one 16-byte store).
template <int VEC>
__device__ __forceinline__ void hc_store_f32(float *p, const float (&in)[VEC]) {
  if constexpr (VEC <= 4) {
    hc_vec<float, VEC>::store(p, in);
  } else {
#pragma unroll
    for (int q = 0; q < VEC / 4; ++q) {
      const float t[4] = {in[4 * q], in[4 * q + 1], in[4 * q + 2], in[4 * q + 3]};
      hc_vec<float, 4>::store(p + 4 * q, t);
    }
  }
}

// Same with the non-temporal hint (output rows that this launch does not read again).
template <int VEC>
__device__ __forceinline__ void hc_store_f32_nt(float *p, const float (&in)[VEC]) {
  if constexpr (VEC <= 4) {
    hc_vec<float, VEC>::store_nt(p, in);
  } else {
#pragma unroll
    for (int q = 0; q < VEC / 4; ++q) {
      const float t[4] = {in[4 * q], in[4 * q + 1], in[4 * q + 2], in[4 * q + 3]};
      hc_vec<float, 4>::store_nt(p + 4 * q, t);
    }
  }
}

#endif  // __HIPCC__
