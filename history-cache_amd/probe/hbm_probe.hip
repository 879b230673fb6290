// hbm_probe: what this GPU's memory system delivers for the access patterns of the aggregation kernels,
// measured with bare kernels that do nothing else.  A calibration tool beside the library (it links
// nothing of it): `bench.py --workload ceilings` runs it and prints its table.
//
//   stream read      every lane reads consecutive 16-byte words of one large array
//   fill             every lane writes consecutive 16-byte words
//   stream copy      out[i] = in[i] + 1
//   row gather       one wave per output row sums K random rows of ROW_BYTES each from a table of the
//                    given footprint, U rows in flight per wave (loads issued before the first add), row
//                    ids staged 64 at a time and broadcast lane by lane -- the forward kernel's inner loop
//                    without maps, means or long-row handling
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#define CK(x)                                                                      \
  do {                                                                             \
    hipError_t e_ = (x);                                                           \
    if (e_ != hipSuccess) {                                                        \
      std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);   \
      std::exit(1);                                                                \
    }                                                                              \
  } while (0)

typedef float f4 __attribute__((ext_vector_type(4)));

// VPR = 16-byte words per lane and row (1: 1 KiB rows, 2: 2 KiB, 4: 4 KiB)
template <int U, int VPR, bool NT>
__global__ __launch_bounds__(256) void row_gather(const f4 *__restrict__ tab, const int *__restrict__ ids,
                                                  f4 *__restrict__ out, int K, int64_t n_out) {
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  if (w >= n_out) return;
  f4 acc[VPR];
#pragma unroll
  for (int c = 0; c < VPR; ++c) acc[c] = f4{0, 0, 0, 0};
  for (int b = 0; b < K; b += 64) {
    const int n = K - b < 64 ? K - b : 64;
    const int my = lane < n ? ids[w * K + b + lane] : 0;
    for (int j = 0; j < n; j += U) {
      f4 v[U][VPR];
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int c = 0; c < VPR; ++c) v[u][c] = f4{0, 0, 0, 0};
        if (j + u < n) {
          const int id = __builtin_amdgcn_readlane(my, j + u);
          const f4 *p = tab + (int64_t)id * (64 * VPR) + lane;
#pragma unroll
          for (int c = 0; c < VPR; ++c) v[u][c] = NT ? __builtin_nontemporal_load(p + 64 * c) : p[64 * c];
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int c = 0; c < VPR; ++c) acc[c] += v[u][c];
    }
  }
#pragma unroll
  for (int c = 0; c < VPR; ++c) out[w * (64 * VPR) + 64 * c + lane] = acc[c];
}

__global__ __launch_bounds__(256) void stream_read(const f4 *__restrict__ in, f4 *__restrict__ out, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  f4 acc = f4{0, 0, 0, 0};
  for (; i + 3 * stride < n; i += 4 * stride) {
    const f4 a = in[i], b = in[i + stride], c = in[i + 2 * stride], d = in[i + 3 * stride];
    acc += (a + b) + (c + d);
  }
  for (; i < n; i += stride) acc += in[i];
  if (acc.x == 1234.5f) out[0] = acc;   // never true for a zero-filled array: keeps the loads alive
}

// fill and copy: one block per contiguous 16 KiB tile (4 words of 16 bytes per lane), the shape of a
// library elementwise kernel; NT = non-temporal stores
template <bool NT>
__global__ __launch_bounds__(256) void fill(f4 *__restrict__ out, int64_t n) {
  const int64_t base = (int64_t)blockIdx.x * 1024 + threadIdx.x;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int64_t i = base + 256 * k;
    if (i < n) {
      if (NT) __builtin_nontemporal_store(f4{1, 2, 3, 4}, out + i);
      else out[i] = f4{1, 2, 3, 4};
    }
  }
}

template <bool NT>
__global__ __launch_bounds__(256) void stream_copy(const f4 *__restrict__ in, f4 *__restrict__ out, int64_t n) {
  const int64_t base = (int64_t)blockIdx.x * 1024 + threadIdx.x;
  f4 v[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int64_t i = base + 256 * k;
    v[k] = i < n ? (NT ? __builtin_nontemporal_load(in + i) : in[i]) : f4{0, 0, 0, 0};
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int64_t i = base + 256 * k;
    if (i < n) {
      if (NT) __builtin_nontemporal_store(v[k] + 1.0f, out + i);
      else out[i] = v[k] + 1.0f;
    }
  }
}

template <typename F>
static float timed_ms(F launch, int warm, int reps) {
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  for (int i = 0; i < warm; ++i) launch();
  CK(hipEventRecord(a));
  for (int i = 0; i < reps; ++i) launch();
  CK(hipEventRecord(b));
  CK(hipEventSynchronize(b));
  CK(hipGetLastError());
  float ms = 0;
  CK(hipEventElapsedTime(&ms, a, b));
  CK(hipEventDestroy(a));
  CK(hipEventDestroy(b));
  return ms / reps;
}

template <int U, int VPR, bool NT>
static double gather_gbps(const f4 *tab, const int *ids, f4 *out, int K, int64_t n_out) {
  const unsigned grid = (unsigned)((n_out + 3) / 4);
  const float ms = timed_ms([&] { row_gather<U, VPR, NT><<<grid, 256>>>(tab, ids, out, K, n_out); }, 2, 5);
  return (double)n_out * K * (1024.0 * VPR) / ms / 1e6;
}

// `hbm_probe <GB> gather <pattern>`: only the 1 KiB row gather (8 rows in flight, ordinary loads), with the
// row ids drawn by one of these patterns -- short enough for a counter pass of its own:
//   uniform     every row id uniform over the table (the pattern of the table above)
//   page        the 20 rows of one output row lie in one 2 MiB-aligned window (windows uniform): random DRAM
//               rows, but one address translation per wave
//   block       the same with one window per block of 4 waves
//   sequential  row id = position: the gather kernel reading the table front to back
static int gather_only(double table_gb, const char *pattern) {
  const int K = 20;
  const int64_t table_bytes = (int64_t)(table_gb * 1e9) / (2 << 20) * (2 << 20);
  const int64_t rows = table_bytes / 1024, E = 20000000, n_out = E / K;
  const int64_t win_rows = (2 << 20) / 1024, n_win = rows / win_rows;
  if (n_win < 1) return 2;
  f4 *tab = nullptr, *dst = nullptr;
  int *ids = nullptr;
  CK(hipMalloc(&tab, (size_t)table_bytes));
  CK(hipMalloc(&dst, (size_t)n_out * 1024));
  CK(hipMalloc(&ids, (size_t)E * sizeof(int)));
  CK(hipMemset(tab, 0, (size_t)table_bytes));
  std::vector<int> h((size_t)E);
  uint64_t s = 0x9E3779B97F4A7C15ull;
  auto next = [&](uint64_t m) {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    return (int64_t)((s >> 33) % m);
  };
  const std::string pat(pattern);
  int64_t win = 0;
  for (int64_t i = 0; i < E; ++i) {
    if (pat == "uniform") h[(size_t)i] = (int)next((uint64_t)rows);
    else if (pat == "sequential") h[(size_t)i] = (int)(i % rows);
    else if (pat == "page" || pat == "block") {
      const int64_t group = pat == "page" ? K : 4 * K;
      if (i % group == 0) win = next((uint64_t)n_win);
      h[(size_t)i] = (int)(win * win_rows + next((uint64_t)win_rows));
    } else {
      std::printf("unknown pattern %s\n", pattern);
      return 2;
    }
  }
  CK(hipMemcpy(ids, h.data(), (size_t)E * sizeof(int), hipMemcpyHostToDevice));
  const double gbps = gather_gbps<8, 1, false>(tab, ids, dst, K, n_out);
  std::printf("row gather 1 KiB, pattern %-10s over %6.2f GB: %6.0f GB/s\n", pattern, table_bytes / 1e9, gbps);
  CK(hipFree(ids));
  CK(hipFree(dst));
  CK(hipFree(tab));
  return 0;
}

int main(int argc, char **argv) {
  const double table_gb = argc > 1 ? std::atof(argv[1]) : 20.0;   // footprint of the gathered table
  if (!(table_gb >= 0.01 && table_gb <= 64.0)) {
    std::printf("usage: hbm_probe [table GB in 0.01..64] [gather uniform|page|block|sequential]\n");
    return 2;
  }
  if (argc > 3 && std::string(argv[2]) == "gather") return gather_only(table_gb, argv[3]);
  const int K = 20;                                               // rows summed per output row
  const int64_t table_bytes = (int64_t)(table_gb * 1e9) / 4096 * 4096;
  const int64_t n16 = table_bytes / 16;
  f4 *tab = nullptr, *dst = nullptr;
  int *ids = nullptr;
  CK(hipMalloc(&tab, (size_t)table_bytes));
  const int64_t E = 20000000;                                     // gathered rows per launch for 1 KiB rows
  const int64_t gather_out_bytes = E / K * 1024;                  // the same for every row size below
  const int64_t dst_bytes = table_bytes / 2 > gather_out_bytes ? table_bytes / 2 : gather_out_bytes;
  CK(hipMalloc(&dst, (size_t)dst_bytes));                         // copy target and gather output
  CK(hipMemset(tab, 0, (size_t)table_bytes));
  const unsigned sgrid = 256 * 32;

  float ms = timed_ms([&] { stream_read<<<sgrid, 256>>>(tab, dst, n16); }, 1, 3);
  std::printf("stream read   %6.1f GB            : %8.3f ms  %6.0f GB/s\n", table_bytes / 1e9, ms, (double)table_bytes / ms / 1e6);
  const unsigned fgrid = (unsigned)((n16 + 1023) / 1024), cgrid = (unsigned)((n16 / 2 + 1023) / 1024);
  ms = timed_ms([&] { fill<false><<<fgrid, 256>>>(tab, n16); }, 1, 3);
  std::printf("fill          %6.1f GB            : %8.3f ms  %6.0f GB/s\n", table_bytes / 1e9, ms, (double)table_bytes / ms / 1e6);
  ms = timed_ms([&] { fill<true><<<fgrid, 256>>>(tab, n16); }, 1, 3);
  std::printf("fill nt       %6.1f GB            : %8.3f ms  %6.0f GB/s\n", table_bytes / 1e9, ms, (double)table_bytes / ms / 1e6);
  ms = timed_ms([&] { stream_copy<false><<<cgrid, 256>>>(tab, dst, n16 / 2); }, 1, 3);
  std::printf("stream copy   %6.1f GB in + out   : %8.3f ms  %6.0f GB/s (read + write)\n", table_bytes / 2e9, ms,
              (double)table_bytes / ms / 1e6);
  ms = timed_ms([&] { stream_copy<true><<<cgrid, 256>>>(tab, dst, n16 / 2); }, 1, 3);
  std::printf("stream copy nt%6.1f GB in + out   : %8.3f ms  %6.0f GB/s (read + write)\n", table_bytes / 2e9, ms,
              (double)table_bytes / ms / 1e6);
  CK(hipMemset(tab, 0, (size_t)table_bytes));

  // random row ids (a 64-bit LCG on the host; each row size gets ids in its own range)
  std::vector<int> h((size_t)E);
  CK(hipMalloc(&ids, (size_t)E * sizeof(int)));
  auto make_ids = [&](int64_t rows, int64_t count) {
    uint64_t s = 0x9E3779B97F4A7C15ull;
    for (int64_t i = 0; i < count; ++i) {
      s = s * 6364136223846793005ull + 1442695040888963407ull;
      h[(size_t)i] = (int)((s >> 33) % (uint64_t)rows);
    }
    CK(hipMemcpy(ids, h.data(), (size_t)count * sizeof(int), hipMemcpyHostToDevice));
  };
  {
    const int64_t rows = table_bytes / 1024, n_out = E / K;
    make_ids(rows, E);
    std::printf("row gather, 1 KiB rows, %lld rows per launch over %.1f GB, GB/s by rows in flight per wave:\n",
                (long long)E, table_bytes / 1e9);
    std::printf("   ordinary loads     U=4 %6.0f   U=8 %6.0f   U=16 %6.0f\n", gather_gbps<4, 1, false>(tab, ids, dst, K, n_out),
                gather_gbps<8, 1, false>(tab, ids, dst, K, n_out), gather_gbps<16, 1, false>(tab, ids, dst, K, n_out));
    std::printf("   non-temporal loads U=4 %6.0f   U=8 %6.0f   U=16 %6.0f\n", gather_gbps<4, 1, true>(tab, ids, dst, K, n_out),
                gather_gbps<8, 1, true>(tab, ids, dst, K, n_out), gather_gbps<16, 1, true>(tab, ids, dst, K, n_out));
  }
  {
    const int64_t rows = table_bytes / 2048, n_out = E / 2 / K;
    make_ids(rows, n_out * K);
    std::printf("row gather, 2 KiB rows, U=8: %6.0f GB/s\n", gather_gbps<8, 2, false>(tab, ids, dst, K, n_out));
  }
  {
    const int64_t rows = table_bytes / 4096, n_out = E / 4 / K;
    make_ids(rows, n_out * K);
    std::printf("row gather, 4 KiB rows, U=4: %6.0f GB/s\n", gather_gbps<4, 4, false>(tab, ids, dst, K, n_out));
  }
  CK(hipFree(ids));
  CK(hipFree(dst));
  CK(hipFree(tab));
  return 0;
}
