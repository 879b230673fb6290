// Bias + batch normalisation (training mode) + ReLU of a layer's output, forward and backward:
// what /root/reference/hiscache/history_model.py:139-140 and :386-387 spell as
// `x = self.bns[i](x); x = F.relu(x)` behind a convolution whose linear layer adds a bias.
// Rows are nodes of a sampled batch (a few thousand to a few ten thousand), columns are hidden
// channels: every kernel is a column reduction or an elementwise pass over an [n, C] fp32 matrix and
// is bound by HBM bandwidth.
//
//   bn_stats       per slab of rows and per column: sums of (x - s) and (x - s)^2, s = the matrix' first
//                  row (a shift within a few standard deviations of the mean keeps S2 - S1^2/n harmless);
//                  the block that finishes last adds the slabs in a fixed order into mean and
//                  1/sqrt(var + eps) and updates the running statistics
//   bn_apply       y = max(0, (x - mean) * invstd * gamma + beta)
//   bn_bwd_reduce  per slab and column: sums of dy' and dy' * xhat, dy' = dy where y > 0; the block that
//                  finishes last adds the slabs in the same fixed order into dbeta and dgamma
//   bn_bwd_apply   dx = gamma * invstd * (dy' - dbeta/n - xhat * dgamma/n)
//
// A bias added in front of the normalisation cancels in y; it only shifts the mean that the running
// statistics see, and its gradient is zero.  Nothing here depends on scheduling: slabs are fixed by
// (n, C) and added in a fixed order.  The reducing kernels run 1024-thread blocks over at most 128
// slabs: the block that adds the slabs reads all partial sums through one compute unit, so their
// number is kept small and the sixteen waves split them.
#include "hc_common.h"

namespace {

constexpr int BN_MAX_SLABS = 128;
constexpr int BN_MAX_C = 1024;
constexpr int BN_BLOCK = 1024;   // threads per block of the two reducing kernels
constexpr int BN_FLIGHT = 8;     // rows a thread has in flight

struct BnShape {
  int groups;          // float4 groups per row: C / 4
  int rows_per_pass;   // rows a reducing block reads per sweep: BN_BLOCK / groups
  int64_t slab_rows;   // rows per slab (a multiple of rows_per_pass)
  int64_t slabs;
};

static bool bn_shape(int64_t n, int64_t C, BnShape *s) {
  if (n < 1 || C < 4 || C > BN_MAX_C || C % 4 != 0) return false;
  s->groups = (int)(C / 4);
  s->rows_per_pass = BN_BLOCK / s->groups;
  const int64_t p = s->rows_per_pass;
  int64_t rows = (n + BN_MAX_SLABS - 1) / BN_MAX_SLABS;
  if (rows < 2 * p) rows = 2 * p;
  rows = (rows + p - 1) / p * p;
  s->slab_rows = rows;
  s->slabs = (n + rows - 1) / rows;
  return true;
}

// Rows that count: all n, or -- when the caller's matrix is padded to a fixed capacity and the number of rows
// in use is only known on the device -- *n_dev, kept inside [1, n].  Rows behind it are neither counted nor
// changed by a gradient: the forward writes zeros there, the backward a zero gradient.
__device__ __forceinline__ int64_t bn_rows(int64_t n, const int64_t *__restrict__ n_dev) {
  if (n_dev == nullptr) return n;
  const int64_t m = *n_dev;
  return m < 1 ? 1 : (m < n ? m : n);
}

// pre-activation; the same expression decides y > 0 in forward and in backward
__device__ __forceinline__ float bn_pre(float x, float mean, float invstd, float g, float b) {
  return ((x - mean) * invstd) * g + b;
}

__device__ __forceinline__ float4 bn_ld4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ void bn_add4(float4 &a, const float4 &b) {
  a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
}

// One ticket per launch: true in the block that arrives last.  The counter is zero again when the
// kernel ends.  One device-scope release per block, by the thread that takes the ticket, behind the
// block's barrier.
__device__ __forceinline__ bool bn_last_block(unsigned *ticket, int *s_flag) {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (threadIdx.x == 0) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    const unsigned t = atomicAdd(ticket, 1u);
    *s_flag = t == gridDim.x - 1 ? 1 : 0;
    if (t == gridDim.x - 1) atomicExch(ticket, 0u);
  }
  __syncthreads();
  if (!*s_flag) return false;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  return true;
}

// Sum over the slabs of the two partial sums of column group g, by the block that arrived last:
// part[slab][2][C].  Thread (g, p) adds slabs p, p + P, ... in that order, thread (g, 0) then adds the
// P results in order of p.  Ends with the totals in the threads with p == 0.
__device__ __forceinline__ void bn_sum_slabs(const float *__restrict__ part, int64_t slabs, int C, int G, int P,
                                             int g, int p, float4 (*s_red)[BN_BLOCK], float4 &t1, float4 &t2) {
  t1 = make_float4(0.f, 0.f, 0.f, 0.f);
  t2 = t1;
  __syncthreads();      // s_red is free again
  if (p < P) {
    int64_t k = p;
    for (; k + 3 * (int64_t)P < slabs; k += 4 * (int64_t)P) {
      float4 a[4], b[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        a[j] = bn_ld4(part + (k + (int64_t)j * P) * 2 * C + 4 * g);
        b[j] = bn_ld4(part + (k + (int64_t)j * P) * 2 * C + C + 4 * g);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        bn_add4(t1, a[j]);
        bn_add4(t2, b[j]);
      }
    }
    for (; k < slabs; k += P) {
      bn_add4(t1, bn_ld4(part + k * 2 * C + 4 * g));
      bn_add4(t2, bn_ld4(part + k * 2 * C + C + 4 * g));
    }
  }
  s_red[0][threadIdx.x] = t1;
  s_red[1][threadIdx.x] = t2;
  __syncthreads();
  if (p == 0)
    for (int q = 1; q < P; ++q) {
      bn_add4(t1, s_red[0][q * G + g]);
      bn_add4(t2, s_red[1][q * G + g]);
    }
}

// part[slab][2][C]: S1 = sum (x - s), S2 = sum (x - s)^2 with s = x[0, :]
__global__ __launch_bounds__(BN_BLOCK) void bn_stats(
    const float *__restrict__ x, const float *__restrict__ bias, float *__restrict__ part,
    float *__restrict__ save_mean, float *__restrict__ save_invstd, float *__restrict__ running_mean,
    float *__restrict__ running_var, int64_t *__restrict__ batches_tracked, float momentum, float eps,
    int64_t n_cap, const int64_t *__restrict__ n_dev, int C, BnShape sh, unsigned *__restrict__ ticket) {
  __shared__ float4 s_red[2][BN_BLOCK];
  __shared__ int s_flag;
  const int64_t n = bn_rows(n_cap, n_dev);
  const int G = sh.groups, P = sh.rows_per_pass;
  const int g = (int)threadIdx.x % G, p = (int)threadIdx.x / G;
  const int64_t lo = (int64_t)blockIdx.x * sh.slab_rows;
  const int64_t hi = lo + sh.slab_rows < n ? lo + sh.slab_rows : n;
  float4 s1 = make_float4(0.f, 0.f, 0.f, 0.f), s2 = s1, sft = s1;
  if (p < P) {
    sft = bn_ld4(x + 4 * g);
    int64_t r = lo + p;
    for (; r + (BN_FLIGHT - 1) * (int64_t)P < hi; r += BN_FLIGHT * (int64_t)P) {
      float4 v[BN_FLIGHT];
#pragma unroll
      for (int k = 0; k < BN_FLIGHT; ++k) v[k] = bn_ld4(x + (r + (int64_t)k * P) * C + 4 * g);
#pragma unroll
      for (int k = 0; k < BN_FLIGHT; ++k) {
        const float a = v[k].x - sft.x, b = v[k].y - sft.y, c = v[k].z - sft.z, d = v[k].w - sft.w;
        s1.x += a; s1.y += b; s1.z += c; s1.w += d;
        s2.x += a * a; s2.y += b * b; s2.z += c * c; s2.w += d * d;
      }
    }
    for (; r < hi; r += P) {
      const float4 v = bn_ld4(x + r * C + 4 * g);
      const float a = v.x - sft.x, b = v.y - sft.y, c = v.z - sft.z, d = v.w - sft.w;
      s1.x += a; s1.y += b; s1.z += c; s1.w += d;
      s2.x += a * a; s2.y += b * b; s2.z += c * c; s2.w += d * d;
    }
  }
  s_red[0][threadIdx.x] = s1;
  s_red[1][threadIdx.x] = s2;
  __syncthreads();
  if (p == 0) {
    for (int q = 1; q < P; ++q) {
      bn_add4(s1, s_red[0][q * G + g]);
      bn_add4(s2, s_red[1][q * G + g]);
    }
    float *o = part + (int64_t)blockIdx.x * 2 * C + 4 * g;
    *reinterpret_cast<float4 *>(o) = s1;
    *reinterpret_cast<float4 *>(o + C) = s2;
  }
  if (!bn_last_block(ticket, &s_flag)) return;
  if (threadIdx.x == 0 && batches_tracked != nullptr) *batches_tracked += 1;   // BatchNorm1d's batch counter
  float4 t1, t2;
  bn_sum_slabs(part, sh.slabs, C, G, P, g, p, s_red, t1, t2);
  if (p != 0) return;
  const float cnt = (float)n;
  const float a1[4] = {t1.x, t1.y, t1.z, t1.w}, a2[4] = {t2.x, t2.y, t2.z, t2.w};
  const float sf[4] = {sft.x, sft.y, sft.z, sft.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = 4 * g + j;
    const float d = a1[j] / cnt;            // mean - shift
    float m2 = a2[j] - a1[j] * d;           // sum of squared deviations from the mean
    if (m2 < 0.f) m2 = 0.f;
    const float mean = sf[j] + d;
    const float var = m2 / cnt;
    save_mean[c] = mean;
    save_invstd[c] = 1.0f / sqrtf(var + eps);
    if (running_mean != nullptr) {
      const float shift = bias != nullptr ? bias[c] : 0.f;
      running_mean[c] = (1.0f - momentum) * running_mean[c] + momentum * (mean + shift);
    }
    if (running_var != nullptr) {
      const float unb = n > 1 ? m2 / (cnt - 1.f) : var;
      running_var[c] = (1.0f - momentum) * running_var[c] + momentum * unb;
    }
  }
}

__global__ __launch_bounds__(HC_BLOCK) void bn_apply(
    const float *__restrict__ x, const float *__restrict__ mean, const float *__restrict__ invstd,
    const float *__restrict__ gamma, const float *__restrict__ beta, float *__restrict__ y, int64_t n4,
    int G, int64_t n_cap, const int64_t *__restrict__ n_dev) {
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i >= n4) return;
  if (n_dev != nullptr && i >= bn_rows(n_cap, n_dev) * G) {     // a padding row
    *reinterpret_cast<float4 *>(y + 4 * i) = make_float4(0.f, 0.f, 0.f, 0.f);
    return;
  }
  const int c = (int)(i % G) * 4;
  const float4 v = bn_ld4(x + 4 * i), m = bn_ld4(mean + c), s = bn_ld4(invstd + c);
  const float4 ga = gamma ? bn_ld4(gamma + c) : make_float4(1.f, 1.f, 1.f, 1.f);
  const float4 be = beta ? bn_ld4(beta + c) : make_float4(0.f, 0.f, 0.f, 0.f);
  float4 o;
  o.x = fmaxf(bn_pre(v.x, m.x, s.x, ga.x, be.x), 0.f);
  o.y = fmaxf(bn_pre(v.y, m.y, s.y, ga.y, be.y), 0.f);
  o.z = fmaxf(bn_pre(v.z, m.z, s.z, ga.z, be.z), 0.f);
  o.w = fmaxf(bn_pre(v.w, m.w, s.w, ga.w, be.w), 0.f);
  *reinterpret_cast<float4 *>(y + 4 * i) = o;
}

// part[slab][2][C]: sum dy', sum dy' * xhat
__global__ __launch_bounds__(BN_BLOCK) void bn_bwd_reduce(
    const float *__restrict__ dy, const float *__restrict__ x, const float *__restrict__ mean,
    const float *__restrict__ invstd, const float *__restrict__ gamma, const float *__restrict__ beta,
    float *__restrict__ part, float *__restrict__ dgamma, float *__restrict__ dbeta,
    float *__restrict__ dbias, int64_t n_cap, const int64_t *__restrict__ n_dev, int C, BnShape sh,
    unsigned *__restrict__ ticket) {
  __shared__ float4 s_red[2][BN_BLOCK];
  __shared__ int s_flag;
  const int64_t n = bn_rows(n_cap, n_dev);
  const int G = sh.groups, P = sh.rows_per_pass;
  const int g = (int)threadIdx.x % G, p = (int)threadIdx.x / G;
  const int64_t lo = (int64_t)blockIdx.x * sh.slab_rows;
  const int64_t hi = lo + sh.slab_rows < n ? lo + sh.slab_rows : n;
  float4 s1 = make_float4(0.f, 0.f, 0.f, 0.f), s2 = s1;
  if (p < P) {
    const int c = 4 * g;
    const float4 m = bn_ld4(mean + c), s = bn_ld4(invstd + c);
    const float4 ga = gamma ? bn_ld4(gamma + c) : make_float4(1.f, 1.f, 1.f, 1.f);
    const float4 be = beta ? bn_ld4(beta + c) : make_float4(0.f, 0.f, 0.f, 0.f);
#define BN_ACC(V, D, F)                                                    \
  {                                                                        \
    const float xh = (V.F - m.F) * s.F;                                    \
    const float dd = bn_pre(V.F, m.F, s.F, ga.F, be.F) > 0.f ? D.F : 0.f;  \
    s1.F += dd;                                                            \
    s2.F += dd * xh;                                                       \
  }
    constexpr int FL = BN_FLIGHT / 2;
    int64_t r = lo + p;
    for (; r + (FL - 1) * (int64_t)P < hi; r += FL * (int64_t)P) {
      float4 v[FL], d[FL];
#pragma unroll
      for (int k = 0; k < FL; ++k) {
        v[k] = bn_ld4(x + (r + (int64_t)k * P) * C + c);
        d[k] = bn_ld4(dy + (r + (int64_t)k * P) * C + c);
      }
#pragma unroll
      for (int k = 0; k < FL; ++k) {
        BN_ACC(v[k], d[k], x) BN_ACC(v[k], d[k], y) BN_ACC(v[k], d[k], z) BN_ACC(v[k], d[k], w)
      }
    }
    for (; r < hi; r += P) {
      const float4 v0 = bn_ld4(x + r * C + c), d0 = bn_ld4(dy + r * C + c);
      BN_ACC(v0, d0, x) BN_ACC(v0, d0, y) BN_ACC(v0, d0, z) BN_ACC(v0, d0, w)
    }
#undef BN_ACC
  }
  s_red[0][threadIdx.x] = s1;
  s_red[1][threadIdx.x] = s2;
  __syncthreads();
  if (p == 0) {
    for (int q = 1; q < P; ++q) {
      bn_add4(s1, s_red[0][q * G + g]);
      bn_add4(s2, s_red[1][q * G + g]);
    }
    float *o = part + (int64_t)blockIdx.x * 2 * C + 4 * g;
    *reinterpret_cast<float4 *>(o) = s1;
    *reinterpret_cast<float4 *>(o + C) = s2;
  }
  if (!bn_last_block(ticket, &s_flag)) return;
  float4 t1, t2;
  bn_sum_slabs(part, sh.slabs, C, G, P, g, p, s_red, t1, t2);
  if (p != 0) return;
  *reinterpret_cast<float4 *>(dbeta + 4 * g) = t1;
  *reinterpret_cast<float4 *>(dgamma + 4 * g) = t2;
  if (dbias != nullptr) *reinterpret_cast<float4 *>(dbias + 4 * g) = make_float4(0.f, 0.f, 0.f, 0.f);
}

__global__ __launch_bounds__(HC_BLOCK) void bn_bwd_apply(
    const float *__restrict__ dy, const float *__restrict__ x, const float *__restrict__ mean,
    const float *__restrict__ invstd, const float *__restrict__ gamma, const float *__restrict__ beta,
    const float *__restrict__ dgamma, const float *__restrict__ dbeta, float *__restrict__ dx, int64_t n4,
    int G, int64_t n_cap, const int64_t *__restrict__ n_dev) {
  const int64_t i = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (i >= n4) return;
  const int64_t n = bn_rows(n_cap, n_dev);
  if (i >= n * G) {                                              // a padding row
    *reinterpret_cast<float4 *>(dx + 4 * i) = make_float4(0.f, 0.f, 0.f, 0.f);
    return;
  }
  const float inv_n = 1.0f / (float)n;
  const int c = (int)(i % G) * 4;
  const float4 v = bn_ld4(x + 4 * i), d = bn_ld4(dy + 4 * i);
  const float4 m = bn_ld4(mean + c), s = bn_ld4(invstd + c);
  const float4 ga = gamma ? bn_ld4(gamma + c) : make_float4(1.f, 1.f, 1.f, 1.f);
  const float4 be = beta ? bn_ld4(beta + c) : make_float4(0.f, 0.f, 0.f, 0.f);
  const float4 dg = bn_ld4(dgamma + c), db = bn_ld4(dbeta + c);
  float4 o;
#define BN_DX(F)                                                          \
  {                                                                       \
    const float xh = (v.F - m.F) * s.F;                                   \
    const float dd = bn_pre(v.F, m.F, s.F, ga.F, be.F) > 0.f ? d.F : 0.f; \
    o.F = (ga.F * s.F) * ((dd - db.F * inv_n) - xh * (dg.F * inv_n));     \
  }
  BN_DX(x) BN_DX(y) BN_DX(z) BN_DX(w)
#undef BN_DX
  *reinterpret_cast<float4 *>(dx + 4 * i) = o;
}

}  // namespace

extern "C" size_t hc_bn_relu_workspace_bytes(int64_t n, int64_t C) {
  BnShape sh;
  if (!bn_shape(n, C, &sh)) return 0;
  return hc_align_up((size_t)sh.slabs * 2 * (size_t)C * sizeof(float), 256);
}

extern "C" int hc_bn_relu_fwd_dev(const float *x, const float *bias, const float *gamma, const float *beta,
                                  float *running_mean, float *running_var, int64_t *num_batches_tracked,
                                  float momentum, float eps, float *y, float *save_mean, float *save_invstd,
                                  int64_t n, int64_t C, const int64_t *n_dev, void *workspace,
                                  size_t workspace_bytes, unsigned *ticket, void *stream) {
  HC_REQUIRE(x && y && save_mean && save_invstd && ticket);
  BnShape sh;
  if (!bn_shape(n, C, &sh)) return n >= 1 && C >= 1 ? HC_EUNSUPPORTED : HC_EINVAL;
  if (!workspace || workspace_bytes < (size_t)sh.slabs * 2 * (size_t)C * sizeof(float)) return HC_EWORKSPACE;
  if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0) return HC_EWORKSPACE;
  const int64_t n4 = n * (C / 4);
  const int64_t blocks = (n4 + HC_BLOCK - 1) / HC_BLOCK;
  if (!hc_grid_ok(blocks)) return HC_ELAUNCH;
  hipStream_t st = static_cast<hipStream_t>(stream);
  bn_stats<<<dim3((unsigned)sh.slabs), dim3(BN_BLOCK), 0, st>>>(
      x, bias, static_cast<float *>(workspace), save_mean, save_invstd, running_mean, running_var,
      num_batches_tracked, momentum, eps, n, n_dev, (int)C, sh, ticket);
  bn_apply<<<dim3((unsigned)blocks), dim3(HC_BLOCK), 0, st>>>(x, save_mean, save_invstd, gamma, beta, y, n4,
                                                              sh.groups, n, n_dev);
  return hc_launch_status();
}

extern "C" int hc_bn_relu_fwd(const float *x, const float *bias, const float *gamma, const float *beta,
                              float *running_mean, float *running_var, int64_t *num_batches_tracked,
                              float momentum, float eps, float *y, float *save_mean, float *save_invstd,
                              int64_t n, int64_t C, void *workspace, size_t workspace_bytes, unsigned *ticket,
                              void *stream) {
  return hc_bn_relu_fwd_dev(x, bias, gamma, beta, running_mean, running_var, num_batches_tracked, momentum, eps, y,
                            save_mean, save_invstd, n, C, nullptr, workspace, workspace_bytes, ticket, stream);
}

extern "C" int hc_bn_relu_bwd_dev(const float *dy, const float *x, const float *gamma, const float *beta,
                                  const float *save_mean, const float *save_invstd, float *dx, float *dgamma,
                                  float *dbeta, float *dbias, int64_t n, int64_t C, const int64_t *n_dev,
                                  void *workspace, size_t workspace_bytes, unsigned *ticket, void *stream) {
  HC_REQUIRE(dy && x && save_mean && save_invstd && dx && dgamma && dbeta && ticket);
  BnShape sh;
  if (!bn_shape(n, C, &sh)) return n >= 1 && C >= 1 ? HC_EUNSUPPORTED : HC_EINVAL;
  if (!workspace || workspace_bytes < (size_t)sh.slabs * 2 * (size_t)C * sizeof(float)) return HC_EWORKSPACE;
  if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0) return HC_EWORKSPACE;
  const int64_t n4 = n * (C / 4);
  const int64_t blocks = (n4 + HC_BLOCK - 1) / HC_BLOCK;
  if (!hc_grid_ok(blocks)) return HC_ELAUNCH;
  hipStream_t st = static_cast<hipStream_t>(stream);
  bn_bwd_reduce<<<dim3((unsigned)sh.slabs), dim3(BN_BLOCK), 0, st>>>(
      dy, x, save_mean, save_invstd, gamma, beta, static_cast<float *>(workspace), dgamma, dbeta, dbias, n, n_dev,
      (int)C, sh, ticket);
  bn_bwd_apply<<<dim3((unsigned)blocks), dim3(HC_BLOCK), 0, st>>>(
      dy, x, save_mean, save_invstd, gamma, beta, dgamma, dbeta, dx, n4, sh.groups, n, n_dev);
  return hc_launch_status();
}

extern "C" int hc_bn_relu_bwd(const float *dy, const float *x, const float *gamma, const float *beta,
                              const float *save_mean, const float *save_invstd, float *dx, float *dgamma,
                              float *dbeta, float *dbias, int64_t n, int64_t C, void *workspace,
                              size_t workspace_bytes, unsigned *ticket, void *stream) {
  return hc_bn_relu_bwd_dev(dy, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta, dbias, n, C, nullptr,
                            workspace, workspace_bytes, ticket, stream);
}
