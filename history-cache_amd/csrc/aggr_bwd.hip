// History-aware aggregation, backward, as a gather over the transposed view.
//
// Every SOURCE row s is summed by exactly one wavefront, in ascending
// destination-row order: g[r,:]/deg(r) (mean) or g[r,:]*edge_value[j]
// (weighted) over the edges that point at s.  No float atomics: each output
// element has one writer and a fixed summation order, the same order a
// sequential walk of the CSR block in row/edge order produces.
//
// Semantics follow the reference kernels gen_bwd_history_grad_v2*
// (/root/reference/src/cpp/src/history_aggr.cu:127-397): history rows route
// g[r,:] to grads_history[r,:] undivided (:144-149) and push nothing to their
// neighbours; the other rows push g/deg (:140-142,161-166) or g*edge_value
// (:209); edge_grad[j] = <g[r,:], vin[idx[j],:]> (:258-267).
#include "hc_common.h"

namespace {

// ---------------------------------------------------------------------------------------
// Fast path: mean, fp32 upstream gradient, F == 64 * VEC * CHUNKS.
//
// A wave owns BWD_SRC_PER_WAVE consecutive source rows.  Their incoming edges are one
// contiguous span of the transposed arrays, so the wave streams that span 64 edges at a time
// (one coalesced load of destination rows, one gather of their degrees) and walks it with a
// wave-uniform cursor: when the cursor passes the end of a source's segment the accumulator
// is stored (zeros for sources without edges) and reset.  Up to UNROLL gradient rows are in
// flight before the first add; adds stay in transposed-edge order.  Compared with one wave
// per source this amortises the dependent loads (segment bounds -> rows -> degrees) over
// many sources, which matters when most sources have only one or two incoming edges.
// Blocks [0, src_blocks) own source rows; blocks beyond own rows of grad_hbuf.
// ---------------------------------------------------------------------------------------
constexpr int BWD_SRC_PER_WAVE = 32;

template <int VEC, int CHUNKS, int UNROLL>
__global__ __launch_bounds__(HC_BLOCK) void bwd_mean_fast(
    const int64_t *__restrict__ ptr, const int64_t *__restrict__ ptrT, const int32_t *__restrict__ rowT,
    const float *__restrict__ g, const int64_t *__restrict__ hmap, float *__restrict__ grad_vin,
    float *__restrict__ grad_hbuf, int64_t hsize, int64_t R, int64_t n_src, int64_t src_blocks) {
  constexpr int F = HC_WAVE * VEC * CHUNKS;
  constexpr int S = BWD_SRC_PER_WAVE;
  const int lane = hc_lane();
  const int wave = hc_wave_in_block();
  if ((int64_t)blockIdx.x >= src_blocks) {
    // grad_hbuf rows: copy g for history rows, zero otherwise
    const int64_t row = ((int64_t)blockIdx.x - src_blocks) * HC_WAVES_PER_BLOCK + wave;
    if (row >= R) return;
    const bool hit = hmap[row] != -1;
    float *__restrict__ d = grad_hbuf + row * hsize;
    const float *__restrict__ s = g + row * F;
    for (int64_t c = lane; c < hsize; c += HC_WAVE) d[c] = (hit && c < F) ? s[c] : 0.0f;
    return;
  }
  const int64_t s0 = ((int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + wave) * S;
  if (s0 >= n_src) return;
  const int64_t rest = n_src - s0;
  const int ns = rest < S ? (int)rest : S;
  // lane l holds the segment bound ptrT[s0 + l], l = 0..ns
  const int64_t my_p = ptrT[s0 + (lane < ns ? lane : ns)];
  const int64_t e_begin = hc_readlane64(my_p, 0);
  const int64_t e_end = hc_readlane64(my_p, ns);

  float acc[CHUNKS][VEC];
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[k][i] = 0.0f;
  int cur = 0;                                   // source (relative to s0) being accumulated
  int64_t cur_end = hc_readlane64(my_p, 1);      // end of its segment
  float *__restrict__ obase = grad_vin + s0 * F + lane * VEC;

  for (int64_t base = e_begin; base < e_end; base += HC_WAVE) {
    const int64_t left = e_end - base;
    const int n = left < HC_WAVE ? (int)left : HC_WAVE;
    int my_row = 0;
    float my_deg = 1.0f;
    if (lane < n) {
      my_row = rowT[base + lane];
      my_deg = (float)(int)(ptr[my_row + 1] - ptr[my_row]);
    }
    for (int j = 0; j < n; j += UNROLL) {
      float v[UNROLL][CHUNKS][VEC];
      float d[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if (j + u < n) {
          const int r = __builtin_amdgcn_readlane(my_row, j + u);
          d[u] = hc_readlane_f(my_deg, j + u);
          const float *p = g + (int64_t)r * F + lane * VEC;
#pragma unroll
          for (int k = 0; k < CHUNKS; ++k) hc_vec<float, VEC>::load(p + k * HC_WAVE * VEC, v[u][k]);
        }
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if (j + u < n) {
          const int64_t e = base + j + u;
          while (e >= cur_end) {  // wave-uniform: close finished (possibly empty) segments
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) {
              hc_vec<float, VEC>::store(obase + (int64_t)cur * F + k * HC_WAVE * VEC, acc[k]);
#pragma unroll
              for (int i = 0; i < VEC; ++i) acc[k][i] = 0.0f;
            }
            ++cur;
            cur_end = hc_readlane64(my_p, cur + 1);
          }
#pragma unroll
          for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[k][i] += v[u][k][i] / d[u];
        }
      }
    }
  }
  // flush the open segment and the trailing sources without edges
  for (; cur < ns; ++cur) {
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k) {
      hc_vec<float, VEC>::store(obase + (int64_t)cur * F + k * HC_WAVE * VEC, acc[k]);
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[k][i] = 0.0f;
    }
  }
}

// ---------------------------------------------------------------------------------------
// Generic path: any F, optional weights and heads.  One wave per (source, head).
// ---------------------------------------------------------------------------------------
template <bool WEIGHTED>
__global__ __launch_bounds__(HC_BLOCK) void bwd_generic(
    const int64_t *__restrict__ ptr, const int64_t *__restrict__ ptrT, const int32_t *__restrict__ rowT,
    const int32_t *__restrict__ edgeT, const float *__restrict__ g, const float *__restrict__ ev,
    int64_t H, float *__restrict__ grad_vin, int64_t n_src, int64_t F) {
  constexpr int TILE_K = 4;
  const int lane = hc_lane();
  const int64_t vsrc = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (vsrc >= n_src * H) return;
  const int64_t src = vsrc / H;
  const int64_t head = vsrc - src * H;
  const int64_t begin = ptrT[src];
  const int64_t end = ptrT[src + 1];
  float *__restrict__ o = grad_vin + vsrc * F;
  for (int64_t c0 = 0; c0 < F; c0 += HC_WAVE * TILE_K) {
    float acc[TILE_K];
#pragma unroll
    for (int k = 0; k < TILE_K; ++k) acc[k] = 0.0f;
    for (int64_t base = begin; base < end; base += HC_WAVE) {
      const int64_t left = end - base;
      const int n = left < HC_WAVE ? (int)left : HC_WAVE;
      int my_row = 0;
      float my_s = 1.0f;
      if (lane < n) {
        my_row = rowT[base + lane];
        if (WEIGHTED) my_s = ev[(int64_t)edgeT[base + lane] * H + head];
        else my_s = (float)(int)(ptr[my_row + 1] - ptr[my_row]);
      }
      for (int j = 0; j < n; ++j) {
        const int r = __builtin_amdgcn_readlane(my_row, j);
        const float s = hc_readlane_f(my_s, j);
        const float *p = g + ((int64_t)r * H + head) * F;
#pragma unroll
        for (int k = 0; k < TILE_K; ++k) {
          const int64_t c = c0 + k * HC_WAVE + lane;
          if (c < F) {
            const float x = p[c];
            acc[k] += WEIGHTED ? __fmul_rn(x, s) : x / s;
          }
        }
      }
    }
#pragma unroll
    for (int k = 0; k < TILE_K; ++k) {
      const int64_t c = c0 + k * HC_WAVE + lane;
      if (c < F) o[c] = acc[k];
    }
  }
}

// grad_hbuf[R, hsize] for the generic path (heads summed when hsize == F, concatenated when
// hsize == F*H; columns beyond the written span are 0).
__global__ __launch_bounds__(HC_BLOCK) void bwd_hist_generic(const float *__restrict__ g,
                                                              const int64_t *__restrict__ hmap,
                                                              float *__restrict__ grad_hbuf,
                                                              int64_t hsize, int64_t R, int64_t F,
                                                              int64_t H) {
  const int lane = hc_lane();
  const int64_t row = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (row >= R) return;
  const bool hit = hmap[row] != -1;
  float *__restrict__ d = grad_hbuf + row * hsize;
  const float *__restrict__ s = g + row * H * F;
  const bool concat = (H > 1 && hsize == F * H);
  for (int64_t c = lane; c < hsize; c += HC_WAVE) {
    float v = 0.0f;
    if (hit) {
      if (concat) {
        v = s[c];
      } else if (c < F) {
        for (int64_t h = 0; h < H; ++h) v += s[h * F + c];
      }
    }
    d[c] = v;
  }
}

// edge_grad[j,h] = <g[r,h,:], vin[idx[j],h,:]> in CSR order; 0 for edges of history rows and
// for edge slots in [ptr[R], E_total).  One wave per (row, head); extra blocks clear the tail.
template <typename T>
__global__ __launch_bounds__(HC_BLOCK) void bwd_edge_grad(
    const int64_t *__restrict__ ptr, const int64_t *__restrict__ idx, const float *__restrict__ g,
    const int64_t *__restrict__ hmap, const T *__restrict__ vin, float *__restrict__ edge_grad,
    int64_t E_total, int64_t R, int64_t F, int64_t H, int64_t row_blocks) {
  const int lane = hc_lane();
  if ((int64_t)blockIdx.x >= row_blocks) {
    const int64_t nb = (int64_t)gridDim.x - row_blocks;
    const int64_t start = ptr[R] * H;
    const int64_t stop = E_total * H;
    for (int64_t i = start + ((int64_t)blockIdx.x - row_blocks) * HC_BLOCK + threadIdx.x; i < stop;
         i += nb * HC_BLOCK)
      edge_grad[i] = 0.0f;
    return;
  }
  const int64_t vrow = (int64_t)blockIdx.x * HC_WAVES_PER_BLOCK + hc_wave_in_block();
  if (vrow >= R * H) return;
  const int64_t row = vrow / H;
  const int64_t head = vrow - row * H;
  const int64_t begin = ptr[row];
  int64_t end = ptr[row + 1];
  if (end > E_total) end = E_total;
  if (hmap != nullptr && hmap[row] != -1) {
    for (int64_t e = begin + lane; e < end; e += HC_WAVE) edge_grad[e * H + head] = 0.0f;
    return;
  }
  const float *__restrict__ gr = g + vrow * F;
  for (int64_t base = begin; base < end; base += HC_WAVE) {
    const int64_t left = end - base;
    const int n = left < HC_WAVE ? (int)left : HC_WAVE;
    int64_t my_id = 0;
    if (lane < n) my_id = idx[base + lane];
    float my_out = 0.0f;
    for (int j = 0; j < n; ++j) {
      const int64_t id = hc_readlane64(my_id, j);
      const T *__restrict__ x = vin + (id * H + head) * F;
      float part = 0.0f;
      for (int64_t c = lane; c < F; c += HC_WAVE) part = __fmaf_rn(gr[c], hc_to_f32<T>(x[c]), part);
      part = hc_wave_sum_butterfly(part);
      if (lane == j) my_out = part;
    }
    if (lane < n) edge_grad[(base + lane) * H + head] = my_out;
  }
}

template <int VEC, int CHUNKS>
int launch_fast(const int64_t *ptr, const int64_t *ptrT, const int32_t *rowT, const float *g,
                const int64_t *hmap, float *grad_vin, float *grad_hbuf, int64_t hsize, int64_t R,
                int64_t n_src, hipStream_t st) {
  constexpr int per = VEC * CHUNKS;
  constexpr int UNROLL = per >= 16 ? 4 : (per >= 4 ? 8 : 16);
  const int64_t per_block = (int64_t)HC_WAVES_PER_BLOCK * BWD_SRC_PER_WAVE;
  const int64_t sb = (n_src + per_block - 1) / per_block;
  const int64_t hb = (grad_hbuf && hmap) ? (R + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK : 0;
  if (sb + hb == 0) return HC_OK;
  if (!hc_grid_ok(sb + hb)) return HC_EUNSUPPORTED;
  bwd_mean_fast<VEC, CHUNKS, UNROLL><<<dim3((unsigned)(sb + hb)), dim3(HC_BLOCK), 0, st>>>(
      ptr, ptrT, rowT, g, hmap, grad_vin, grad_hbuf, hsize, R, n_src, sb);
  return hc_launch_status();
}

}  // namespace

extern "C" int hc_aggr_bwd(const int64_t *ptr, const int64_t *idx, const int64_t *ptrT,
                           const int32_t *rowT, const int32_t *edgeT, const float *g,
                           const int64_t *hmap, const float *edge_value, const void *vin, int in_dtype,
                           int64_t n_head, float *grad_vin, float *grad_hbuf, int64_t hsize,
                           float *edge_grad, int64_t E_total, int64_t R, int64_t F, int64_t n_src,
                           void *stream) {
  HC_REQUIRE(R >= 0 && F > 0 && n_src >= 0 && n_head >= 1 && E_total >= 0);
  HC_REQUIRE(ptr && ptrT && g);
  HC_REQUIRE(grad_vin || n_src == 0);
  if (n_head > 1) HC_REQUIRE(edge_value != nullptr);
  if (grad_hbuf) HC_REQUIRE(hmap != nullptr && hsize >= F);
  if (grad_hbuf && n_head > 1) HC_REQUIRE(hsize == F || hsize == F * n_head);
  if (edge_grad) {
    HC_REQUIRE(edge_value && vin && idx);
    if (in_dtype < HC_F32 || in_dtype > HC_BF16) return HC_EDTYPE;
  }
  if (edge_value) HC_REQUIRE(edgeT != nullptr);
  HC_REQUIRE(rowT != nullptr || n_src == 0);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t lim = 0x7ffffffeLL;
  if (R > lim) return HC_EUNSUPPORTED;

  bool done = false;
  const bool aligned = (reinterpret_cast<uintptr_t>(g) % 16 == 0) &&
                       (reinterpret_cast<uintptr_t>(grad_vin) % 16 == 0);
  if (!edge_value && n_head == 1 && aligned) {
    int rc = HC_OK;
    done = true;
#define HC_FAST(V, C)                                                                             \
  if (F == 64 * (V) * (C))                                                                        \
    rc = launch_fast<V, C>(ptr, ptrT, rowT, g, hmap, grad_vin, grad_hbuf, hsize, R, n_src, st);   \
  else
    HC_FAST(4, 1) HC_FAST(4, 2) HC_FAST(4, 3) HC_FAST(4, 4) HC_FAST(2, 1) HC_FAST(2, 3) HC_FAST(1, 1)
    HC_FAST(1, 3) done = false;
#undef HC_FAST
    if (done && rc != HC_OK) return rc;
  }
  if (!done) {
    const int64_t sb = (n_src * n_head + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
    if (sb > 0) {
      if (!hc_grid_ok(sb)) return HC_EUNSUPPORTED;
      if (edge_value)
        bwd_generic<true><<<dim3((unsigned)sb), dim3(HC_BLOCK), 0, st>>>(ptr, ptrT, rowT, edgeT, g,
                                                                         edge_value, n_head, grad_vin,
                                                                         n_src, F);
      else
        bwd_generic<false><<<dim3((unsigned)sb), dim3(HC_BLOCK), 0, st>>>(ptr, ptrT, rowT, edgeT, g,
                                                                          edge_value, n_head, grad_vin,
                                                                          n_src, F);
      if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
    }
    if (grad_hbuf && R > 0) {
      const int64_t hb = (R + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
      if (!hc_grid_ok(hb)) return HC_EUNSUPPORTED;
      bwd_hist_generic<<<dim3((unsigned)hb), dim3(HC_BLOCK), 0, st>>>(g, hmap, grad_hbuf, hsize, R, F,
                                                                      n_head);
      if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
    }
  }
  if (edge_grad && E_total > 0) {
    const int64_t rb = (R * n_head + HC_WAVES_PER_BLOCK - 1) / HC_WAVES_PER_BLOCK;
    const int64_t tail_blocks = 64;
    if (!hc_grid_ok(rb + tail_blocks)) return HC_EUNSUPPORTED;
    dim3 gr((unsigned)(rb + tail_blocks)), bl(HC_BLOCK);
    if (in_dtype == HC_F32)
      bwd_edge_grad<float><<<gr, bl, 0, st>>>(ptr, idx, g, hmap, static_cast<const float *>(vin),
                                              edge_grad, E_total, R, F, n_head, rb);
    else if (in_dtype == HC_F16)
      bwd_edge_grad<__half><<<gr, bl, 0, st>>>(ptr, idx, g, hmap, static_cast<const __half *>(vin),
                                               edge_grad, E_total, R, F, n_head, rb);
    else
      bwd_edge_grad<__hip_bfloat16><<<gr, bl, 0, st>>>(ptr, idx, g, hmap,
                                                       static_cast<const __hip_bfloat16 *>(vin),
                                                       edge_grad, E_total, R, F, n_head, rb);
    if (hc_launch_status() != HC_OK) return HC_ELAUNCH;
  }
  return HC_OK;
}
