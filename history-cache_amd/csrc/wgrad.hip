// Weight gradient of a layer's linear maps: dW[H, F] = g^T x for g [n, H], x [n, F] (fp32), n = rows of a
// sampled layer (thousands to a hundred thousand), H and F a few hundred.  What torch's autograd computes
// for `self.lin_l(out)` and `self.lin_r(x[:num_node])` (/root/reference/hiscache/history_model.py:94-98)
// as one GEMM each.  A short, wide product with a very long inner dimension: the work is split over the
// rows, every block multiplies its slab of rows on the matrix cores into a partial [256, 64] tile
// (v_mfma_f32_32x32x2_f32, fp32 in and out), and a second launch adds the slabs' tiles in slab order.
// Two operands that share g (the aggregated rows and the root rows) go through the same launches.
// No atomics: the result does not depend on scheduling.
//
//   A operand of the instruction (32 x 2): A[i][k] = g[row0 + k][h0 + i]   lane l holds i = l % 32, k = l / 32
//   B operand (2 x 32):                    B[k][j] = x[row0 + k][f0 + j]   lane l holds j = l % 32, k = l / 32
//   D (32 x 32, 16 values per lane):       D[8 * (v / 4) + 4 * (l / 32) + v % 4][l % 32], v = 0..15
// so a lane's loads are one element of row (row0 + l / 32) of g and of x: two 128-byte runs per wave.
#include "hc_common.h"

namespace {

typedef float wg_acc __attribute__((ext_vector_type(16)));

constexpr int WG_TILE_H = 256;      // output rows per block: 64 per wave
constexpr int WG_TILE_F = 64;       // output columns per block
constexpr int WG_STAGE = 16;        // k-steps (pairs of rows) whose loads are in flight ahead of the matrix instructions
// One block per compute unit: with 512 or 1024 blocks the partial tiles' traffic grows faster than the
// matrix pipes gain (n = 25 800, F = 128, two operands: 48 us with 256 blocks, 57 with 512, 70 with 1024);
// 16 k-steps in flight against 8: 98 against 90 TFLOP/s at n = 89 000.
constexpr int WG_TARGET_BLOCKS = 256;
constexpr int WG_MIN_SLAB_ROWS = 64;

struct WgShape {
  int tiles_h, tiles_f;
  int64_t slab_rows, slabs;
};

static bool wg_shape(int64_t n, int64_t H, int64_t F, int n_op, WgShape *s) {
  if (n < 1 || H < 64 || H % 64 != 0 || F < WG_TILE_F || F % WG_TILE_F != 0 || H > 4096 || F > 4096) return false;
  if (n_op < 1 || n_op > 2) return false;
  s->tiles_h = (int)((H + WG_TILE_H - 1) / WG_TILE_H);
  s->tiles_f = (int)(F / WG_TILE_F);
  const int64_t per_slab = (int64_t)s->tiles_h * s->tiles_f * n_op;
  int64_t slabs = (WG_TARGET_BLOCKS + per_slab - 1) / per_slab;
  const int64_t most = (n + WG_MIN_SLAB_ROWS - 1) / WG_MIN_SLAB_ROWS;
  if (slabs > most) slabs = most;
  if (slabs < 1) slabs = 1;
  int64_t rows = (n + slabs - 1) / slabs;
  rows = (rows + 1) / 2 * 2;                         // a k-step is two rows
  s->slab_rows = rows;
  s->slabs = (n + rows - 1) / rows;
  return true;
}

__global__ __launch_bounds__(HC_BLOCK) void wg_partial(const float *__restrict__ g, const float *__restrict__ x0,
                                                        const float *__restrict__ x1, float *__restrict__ part,
                                                        int64_t n, int H, int F, WgShape sh) {
  const float *__restrict__ x = blockIdx.z == 0 ? x0 : x1;
  const int tile = (int)blockIdx.y;
  const int tf = tile % sh.tiles_f, th = tile / sh.tiles_f;
  const int wave = hc_wave_in_block(), lane = hc_lane();
  const int h0 = th * WG_TILE_H + wave * 64;
  if (h0 >= H) return;                                // narrow outputs leave the upper waves idle
  const int f0 = tf * WG_TILE_F;
  const int64_t lo = (int64_t)blockIdx.x * sh.slab_rows;
  const int64_t hi = lo + sh.slab_rows < n ? lo + sh.slab_rows : n;
  const int kk = lane >> 5, c = lane & 31;
  wg_acc acc00 = {0.f}, acc01 = {0.f}, acc10 = {0.f}, acc11 = {0.f};
  const float *gp = g + (lo + kk) * (int64_t)H + h0 + c;
  const float *xp = x + (lo + kk) * (int64_t)F + f0 + c;
  int64_t r = lo;
  // Full stages of WG_STAGE k-steps (2 * WG_STAGE rows).  The loads of the next stage are issued before the
  // matrix instructions of the current one, so that a wave keeps its matrix pipe busy while they are in flight.
  float a0[WG_STAGE], a1[WG_STAGE], b0[WG_STAGE], b1[WG_STAGE];
  bool have = r + 2 * WG_STAGE <= hi;
  if (have) {
#pragma unroll
    for (int s = 0; s < WG_STAGE; ++s) {
      a0[s] = gp[(int64_t)2 * s * H];
      a1[s] = gp[(int64_t)2 * s * H + 32];
      b0[s] = xp[(int64_t)2 * s * F];
      b1[s] = xp[(int64_t)2 * s * F + 32];
    }
  }
  while (have) {
    gp += (int64_t)2 * WG_STAGE * H;
    xp += (int64_t)2 * WG_STAGE * F;
    r += 2 * WG_STAGE;
    const bool more = r + 2 * WG_STAGE <= hi;
    float na0[WG_STAGE], na1[WG_STAGE], nb0[WG_STAGE], nb1[WG_STAGE];
    if (more) {
#pragma unroll
      for (int s = 0; s < WG_STAGE; ++s) {
        na0[s] = gp[(int64_t)2 * s * H];
        na1[s] = gp[(int64_t)2 * s * H + 32];
        nb0[s] = xp[(int64_t)2 * s * F];
        nb1[s] = xp[(int64_t)2 * s * F + 32];
      }
    }
#pragma unroll
    for (int s = 0; s < WG_STAGE; ++s) {
      acc00 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[s], b0[s], acc00, 0, 0, 0);
      acc01 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[s], b1[s], acc01, 0, 0, 0);
      acc10 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[s], b0[s], acc10, 0, 0, 0);
      acc11 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[s], b1[s], acc11, 0, 0, 0);
    }
    if (more) {
#pragma unroll
      for (int s = 0; s < WG_STAGE; ++s) {
        a0[s] = na0[s];
        a1[s] = na1[s];
        b0[s] = nb0[s];
        b1[s] = nb1[s];
      }
    }
    have = more;
  }
  // tail: k-steps whose second row may lie behind the slab
  for (; r < hi; r += 2) {
    const bool ok = r + kk < hi;
    const float a0 = ok ? gp[0] : 0.f, a1 = ok ? gp[32] : 0.f;
    const float b0 = ok ? xp[0] : 0.f, b1 = ok ? xp[32] : 0.f;
    acc00 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc00, 0, 0, 0);
    acc01 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc01, 0, 0, 0);
    acc10 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc10, 0, 0, 0);
    acc11 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc11, 0, 0, 0);
    gp += (int64_t)2 * H;
    xp += (int64_t)2 * F;
  }
  // partial tile of this block: [WG_TILE_H][WG_TILE_F], tiles ordered (operand, tile, slab)
  const int64_t tiles = (int64_t)sh.tiles_h * sh.tiles_f;
  float *o = part + (((int64_t)blockIdx.z * tiles + tile) * sh.slabs + blockIdx.x) * (WG_TILE_H * WG_TILE_F) +
             (int64_t)(wave * 64) * WG_TILE_F;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int i = 8 * (v / 4) + 4 * kk + (v % 4);
    o[(int64_t)i * WG_TILE_F + c] = acc00[v];
    o[(int64_t)i * WG_TILE_F + 32 + c] = acc01[v];
    o[(int64_t)(32 + i) * WG_TILE_F + c] = acc10[v];
    o[(int64_t)(32 + i) * WG_TILE_F + 32 + c] = acc11[v];
  }
}

// dW[op][h][f] = sum over the slabs, in slab order, of the partial tiles; one thread per four columns
__global__ __launch_bounds__(HC_BLOCK) void wg_reduce(const float *__restrict__ part, float *__restrict__ dw0,
                                                       float *__restrict__ dw1, int H, int F, WgShape sh,
                                                       int64_t per_op) {
  const int64_t t = (int64_t)blockIdx.x * HC_BLOCK + threadIdx.x;
  if (t >= per_op) return;
  const int op = (int)blockIdx.y;
  constexpr int Q = WG_TILE_F / 4;                     // float4 groups per tile row
  const int q = (int)(t % Q);
  const int hl = (int)((t / Q) % WG_TILE_H);
  const int tile = (int)(t / ((int64_t)Q * WG_TILE_H));
  const int tf = tile % sh.tiles_f, th = tile / sh.tiles_f;
  const int h = th * WG_TILE_H + hl;
  if (h >= H) return;
  const int64_t tiles = (int64_t)sh.tiles_h * sh.tiles_f;
  const float *p = part + (((int64_t)op * tiles + tile) * sh.slabs) * (WG_TILE_H * WG_TILE_F) +
                   (int64_t)hl * WG_TILE_F + 4 * q;
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  int64_t k = 0;
  for (; k + 8 <= sh.slabs; k += 8) {
    float4 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const float4 *>(p + (k + j) * (WG_TILE_H * WG_TILE_F));
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      s.x += v[j].x; s.y += v[j].y; s.z += v[j].z; s.w += v[j].w;
    }
  }
  for (; k < sh.slabs; ++k) {
    const float4 v = *reinterpret_cast<const float4 *>(p + k * (WG_TILE_H * WG_TILE_F));
    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
  }
  float *dw = op == 0 ? dw0 : dw1;
  *reinterpret_cast<float4 *>(dw + (int64_t)h * F + tf * WG_TILE_F + 4 * q) = s;
}

}  // namespace

extern "C" size_t hc_weight_grad_workspace_bytes(int64_t n, int64_t H, int64_t F, int n_operands) {
  WgShape sh;
  if (!wg_shape(n, H, F, n_operands, &sh)) return 0;
  return hc_align_up((size_t)n_operands * sh.tiles_h * sh.tiles_f * sh.slabs * WG_TILE_H * WG_TILE_F * sizeof(float),
                     256);
}

extern "C" int hc_weight_grad(const float *g, const float *x0, const float *x1, int64_t n, int64_t H, int64_t F,
                              float *dw0, float *dw1, void *workspace, size_t workspace_bytes, void *stream) {
  HC_REQUIRE(g && x0 && dw0 && (x1 == nullptr) == (dw1 == nullptr));
  const int n_op = x1 != nullptr ? 2 : 1;
  WgShape sh;
  if (!wg_shape(n, H, F, n_op, &sh)) return n >= 1 && H >= 1 && F >= 1 ? HC_EUNSUPPORTED : HC_EINVAL;
  const size_t need = (size_t)n_op * sh.tiles_h * sh.tiles_f * sh.slabs * WG_TILE_H * WG_TILE_F * sizeof(float);
  if (!workspace || workspace_bytes < need || reinterpret_cast<uintptr_t>(workspace) % 16 != 0) return HC_EWORKSPACE;
  if (reinterpret_cast<uintptr_t>(dw0) % 16 != 0 || (dw1 && reinterpret_cast<uintptr_t>(dw1) % 16 != 0))
    return HC_EINVAL;
  hipStream_t st = static_cast<hipStream_t>(stream);
  float *part = static_cast<float *>(workspace);
  wg_partial<<<dim3((unsigned)sh.slabs, (unsigned)(sh.tiles_h * sh.tiles_f), (unsigned)n_op), dim3(HC_BLOCK), 0,
               st>>>(g, x0, x1, part, n, (int)H, (int)F, sh);
  const int64_t per_op = (int64_t)sh.tiles_h * sh.tiles_f * WG_TILE_H * (WG_TILE_F / 4);
  wg_reduce<<<dim3((unsigned)((per_op + HC_BLOCK - 1) / HC_BLOCK), (unsigned)n_op), dim3(HC_BLOCK), 0, st>>>(
      part, dw0, dw1, (int)H, (int)F, sh, per_op);
  return hc_launch_status();
}
