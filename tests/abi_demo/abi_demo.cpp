// A caller of the C ABI with no Python and no torch: device memory from hipMalloc, raw pointers in,
// status codes out.  Builds a 4-row block, runs the forward, the transposed view and the backward (over a
// view built for the call and over one shared view of the block), and checks the numbers it can work out by hand.  Prints "abi_demo: ok" and returns 0 on success.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <vector>

#include "hiscache_hip.h"

#define HIP_OK(x)                                                                   \
  do {                                                                              \
    hipError_t e_ = (x);                                                            \
    if (e_ != hipSuccess) {                                                         \
      std::printf("abi_demo: %s failed: %s\n", #x, hipGetErrorString(e_));          \
      return 2;                                                                     \
    }                                                                               \
  } while (0)
#define HC_OK_(x)                                                                   \
  do {                                                                              \
    int rc_ = (x);                                                                  \
    if (rc_ != HC_OK) {                                                             \
      std::printf("abi_demo: %s -> %s\n", #x, hc_strerror(rc_));                    \
      return 3;                                                                     \
    }                                                                               \
  } while (0)

template <typename T>
static T *to_device(const std::vector<T> &v) {
  T *d = nullptr;
  if (hipMalloc(&d, v.size() * sizeof(T) + 256) != hipSuccess) return nullptr;
  if (hipMemcpy(d, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
  return d;
}

int main() {
  if (hc_device_count() < 1) {
    std::printf("abi_demo: no GPU\n");
    return 1;
  }
  const int64_t R = 4, N = 5, F = 64, E = 6;
  // rows: 0 <- {1,2}, 1 <- {} , 2 <- {0,3,4}, 3 <- {4}; row 3 carries a history embedding
  std::vector<int64_t> ptr = {0, 2, 2, 5, 6}, idx = {1, 2, 0, 3, 4, 4}, hmap = {-1, -1, -1, 0};
  std::vector<float> x(N * F), hbuf(R * F, 0.0f), g(R * F);
  for (int64_t n = 0; n < N; ++n)
    for (int64_t c = 0; c < F; ++c) x[n * F + c] = (float)(n + 1) + 0.01f * (float)c;
  for (int64_t c = 0; c < F; ++c) hbuf[3 * F + c] = -7.0f;
  for (int64_t r = 0; r < R; ++r)
    for (int64_t c = 0; c < F; ++c) g[r * F + c] = (float)(r + 1);
  int64_t *d_ptr = to_device(ptr), *d_idx = to_device(idx), *d_hmap = to_device(hmap);
  float *d_x = to_device(x), *d_h = to_device(hbuf), *d_g = to_device(g);
  float *d_out = nullptr, *d_gx = nullptr, *d_gh = nullptr;
  int64_t *d_ptrT = nullptr;
  int32_t *d_rowT = nullptr;
  void *d_ws = nullptr;
  const size_t ws_bytes = hc_transpose_workspace_bytes(R, E, N);
  HIP_OK(hipMalloc(&d_out, R * F * sizeof(float)));
  HIP_OK(hipMalloc(&d_gx, N * F * sizeof(float)));
  HIP_OK(hipMalloc(&d_gh, R * F * sizeof(float)));
  HIP_OK(hipMalloc(&d_ptrT, (N + 1) * sizeof(int64_t)));
  HIP_OK(hipMalloc(&d_rowT, E * sizeof(int32_t)));
  HIP_OK(hipMalloc(&d_ws, ws_bytes));
  if (!d_ptr || !d_idx || !d_hmap || !d_x || !d_h || !d_g) return 2;
  hipStream_t st;
  HIP_OK(hipStreamCreate(&st));

  HC_OK_(hc_aggr_fwd(HC_SUBST_ROW, d_ptr, d_idx, d_x, HC_F32, d_hmap, d_h, HC_F32, F, nullptr, 1, d_out, R, F, N,
                     nullptr, 0, st));
  HC_OK_(hc_build_transpose(d_ptr, d_idx, d_hmap, nullptr, R, E, N, d_ptrT, d_rowT, nullptr, d_ws, ws_bytes, st));
  HC_OK_(hc_aggr_bwd(d_ptr, d_idx, d_ptrT, d_rowT, nullptr, d_g, d_hmap, nullptr, nullptr, HC_F32, 1, d_gx, d_gh, F,
                     nullptr, E, R, F, N, nullptr, 0, st));
  HIP_OK(hipStreamSynchronize(st));

  std::vector<float> out(R * F), gx(N * F), gh(R * F);
  HIP_OK(hipMemcpy(out.data(), d_out, out.size() * sizeof(float), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(gx.data(), d_gx, gx.size() * sizeof(float), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(gh.data(), d_gh, gh.size() * sizeof(float), hipMemcpyDeviceToHost));
  int bad = 0;
  for (int64_t c = 0; c < F; ++c) {
    const float o0 = (x[1 * F + c] + x[2 * F + c]) / 2.0f;
    const float o2 = ((x[0 * F + c] + x[3 * F + c]) + x[4 * F + c]) / 3.0f;
    bad += out[0 * F + c] != o0;
    bad += out[1 * F + c] != 0.0f;   // no neighbours
    bad += out[2 * F + c] != o2;
    bad += out[3 * F + c] != -7.0f;  // history row
    // sources: 0 <- row 2; 1, 2 <- row 0; 3 <- row 2; 4 <- row 2 only (row 3 is a history row)
    bad += gx[0 * F + c] != 3.0f / 3.0f;
    bad += gx[1 * F + c] != 1.0f / 2.0f;
    bad += gx[2 * F + c] != 1.0f / 2.0f;
    bad += gx[3 * F + c] != 3.0f / 3.0f;
    bad += gx[4 * F + c] != 3.0f / 3.0f;
    bad += gh[3 * F + c] != 4.0f;    // the history buffer takes the row's gradient undivided
    bad += gh[0 * F + c] != 0.0f;
  }
  // The same backward over ONE view of the whole block with nothing left out (what a loader emits with a
  // batch): the history row is stepped over inside the kernel; a layer that owns only rows 0 and 1 reads
  // the same view.
  HC_OK_(hc_build_transpose(d_ptr, d_idx, nullptr, nullptr, R, E, N, d_ptrT, d_rowT, nullptr, d_ws, ws_bytes, st));
  HC_OK_(hc_aggr_bwd_batch_view(d_ptr, d_ptrT, d_rowT, d_g, d_hmap, d_gx, d_gh, F, E, R, F, N, nullptr, 0, st));
  HIP_OK(hipStreamSynchronize(st));
  std::vector<float> gx2(N * F), gh2(R * F);
  HIP_OK(hipMemcpy(gx2.data(), d_gx, gx2.size() * sizeof(float), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(gh2.data(), d_gh, gh2.size() * sizeof(float), hipMemcpyDeviceToHost));
  for (size_t i = 0; i < gx.size(); ++i) bad += gx2[i] != gx[i];
  for (size_t i = 0; i < gh.size(); ++i) bad += gh2[i] != gh[i];
  HC_OK_(hc_aggr_bwd_batch_view(d_ptr, d_ptrT, d_rowT, d_g, nullptr, d_gx, nullptr, 0, E, 2, F, N, nullptr, 0, st));
  HIP_OK(hipStreamSynchronize(st));
  HIP_OK(hipMemcpy(gx2.data(), d_gx, gx2.size() * sizeof(float), hipMemcpyDeviceToHost));
  for (int64_t c = 0; c < F; ++c) {
    bad += gx2[0 * F + c] != 0.0f;
    bad += gx2[1 * F + c] != 1.0f / 2.0f;
    bad += gx2[2 * F + c] != 1.0f / 2.0f;
    bad += gx2[3 * F + c] != 0.0f;
    bad += gx2[4 * F + c] != 0.0f;
  }
  if (bad) {
    std::printf("abi_demo: %d wrong values\n", bad);
    return 4;
  }
  std::printf("abi_demo: ok (%s)\n", hc_version());
  return 0;
}
