// Per-pixel top-k blend weights of the 2D-Gaussian-surfel rasteriser for gfx950.
//
// Reference behaviour reproduced: fast_2d_gs/_C/src/gaussian_splatting/gaussian_topk.cu:95-210 (kernel) and :230-250
// (host entry gs_2d_topk_weights): front-to-back traversal of the tile list, w = alpha * T, insertion of (w, id) into a
// descending list of k slots where `w >= slot` takes the slot (a later surfel wins ties), indices start at -1 and
// weights at 0. The near test uses the surfel's centre depth when the screen-space low-pass filter wins (:180-181),
// unlike the render kernels.
//
// Same tiling, LDS staging and per-quadrant culling as the blend forward; the k slots live in registers instead of the
// reference's read-modify-write of global memory per contributing pair.
#include "blend.hpp"

namespace fsgs {
namespace {

template <int kK>
__global__ void __launch_bounds__(kBlendThreads) blend_topk_kernel(
    int ordered, int W, int H, int topk, float near_n, const int64_t* __restrict__ ranges, const int32_t* __restrict__ point_list,
    const float2* __restrict__ means2D, const float* __restrict__ trans_mat, const float4* __restrict__ normal_opacity,
    int32_t* __restrict__ top_indices, float* __restrict__ top_weights) {
  __shared__ SplatHot s_hot[kBatch];
  __shared__ int s_id[kBatch];
  __shared__ unsigned char s_mask[kBatch];

  const int gx = (W + kTile - 1) / kTile;
  const int tile = scheduled_tile(ordered), tile_x = tile % gx, tile_y = tile / gx;
  int px, py;
  lane_pixel(tile_x, tile_y, px, py);
  const bool inside = px < W && py < H;
  const size_t pix  = (size_t) W * py + px;
  const float pxf = (float) px, pyf = (float) py;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

  const int64_t r0 = ranges[2 * (size_t) tile], r1 = ranges[2 * (size_t) tile + 1];
  const int n_todo = (int) (r1 - r0);
  const int rounds = (n_todo + kBatch - 1) / kBatch;

  bool done = !inside;
  float T = 1.0f;
  float tw[kK];
  int ti[kK];
#pragma unroll
  for (int k = 0; k < kK; ++k) tw[k] = 0.0f, ti[k] = -1;

  for (int b = 0; b < rounds; ++b) {
    if (__syncthreads_count(done) == kBlendThreads) break;
    const int n_here = min(kBatch, n_todo - b * kBatch);
    if ((int) threadIdx.x < n_here) {
      const int id   = point_list[r0 + b * kBatch + threadIdx.x];
      const float* M = trans_mat + 9 * (size_t) id;
      SplatHot h;
#pragma unroll
      for (int k = 0; k < 9; ++k) h.m[k] = M[k];
      const float2 c = means2D[id];
      h.cx = c.x, h.cy = c.y, h.opacity = normal_opacity[id].w;
      s_hot[threadIdx.x]  = h;
      s_id[threadIdx.x]   = id;
      s_mask[threadIdx.x] = (unsigned char) quadrant_mask(h, tile_x * kTile, tile_y * kTile, ordered);
    }
    __syncthreads();
    for (int c = 0; c < kBatch / kWave; ++c) {
      const int jj = c * kWave + lane;
      unsigned long long todo = __ballot(jj < n_here && ((s_mask[jj] >> wave) & 1u));
      while (todo) {
        if (__ballot(!done) == 0ull) break;
        const int j = c * kWave + __builtin_ctzll(todo);
        todo &= todo - 1;
        if (done) continue;
        const SplatHot& h = s_hot[j];
        const float kx = pxf * h.m[6] - h.m[0], ky = pxf * h.m[7] - h.m[1], kz = pxf * h.m[8] - h.m[2];
        const float lx = pyf * h.m[6] - h.m[3], ly = pyf * h.m[7] - h.m[4], lz = pyf * h.m[8] - h.m[5];
        const float qx = ky * lz - kz * ly, qy = kz * lx - kx * lz, qz = kx * ly - ky * lx;
        if (qz == 0.0f) continue;
        const float rz = __builtin_amdgcn_rcpf(qz);
        const float sx = qx * rz, sy = qy * rz;
        const float rho3d = sx * sx + sy * sy;
        const float dx = h.cx - pxf, dy = h.cy - pyf;
        const float rho2d = 2.0f * (dx * dx + dy * dy);
        const float rho   = fminf(rho3d, rho2d);
        const float depth = (rho3d <= rho2d) ? (sx * h.m[6] + sy * h.m[7]) + h.m[8] : h.m[8];
        if (depth < near_n) continue;
        const float power = -0.5f * rho;
        if (power > 0.0f) continue;
        const float alpha = fminf(0.99f, h.opacity * __expf(power));
        if (alpha < (1.0f / 255.0f)) continue;
        const float test_T = T * (1.0f - alpha);
        if (test_T < 0.0001f) {
          done = true;
          continue;
        }
        float w = alpha * T;
        int idx = s_id[j];
#pragma unroll
        for (int k = 0; k < kK; ++k) {
          if (k < topk && w >= tw[k]) {
            const float ow = tw[k];
            const int oi   = ti[k];
            tw[k] = w, ti[k] = idx;
            w = ow, idx = oi;
          }
        }
        T = test_T;
      }
    }
  }
  if (inside) {
#pragma unroll
    for (int k = 0; k < kK; ++k)
      if (k < topk) {
        top_weights[pix * topk + k] = tw[k];
        top_indices[pix * topk + k] = ti[k];
      }
  }
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API int fsgs_gs_2d_topk_weights(int topk, int P, int W, int H, double near_n, double far_n, const float* means2D,
    const float* normal_opacity, const float* trans_mat, const int64_t* ranges, const int32_t* point_list,
    int32_t* top_indices, float* top_weights, void* stream) {
  (void) far_n;
  FSGS_REQUIRE(topk > 0 && W > 0 && H > 0 && P >= 0 && ranges && top_indices && top_weights,
               "gs_2d_topk_weights: bad arguments");
  FSGS_REQUIRE(topk <= 16, "gs_2d_topk_weights: topk=%d exceeds the supported maximum of 16", topk);
  FSGS_REQUIRE(P == 0 || (means2D && normal_opacity && trans_mat && point_list), "gs_2d_topk_weights: null pointer");
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const dim3 grid(gx * gy), block(kBlendThreads);
  hipStream_t s = (hipStream_t) stream;
  const int ordered = launch_tile_order(gx, gy, ranges, s);
#define FSGS_TOPK(KK)                                                                                            \
  hipLaunchKernelGGL((blend_topk_kernel<KK>), grid, block, 0, s, ordered, W, H, topk, (float) near_n, ranges, point_list, \
                     (const float2*) means2D, trans_mat, (const float4*) normal_opacity, top_indices, top_weights)
  if (topk <= 4) FSGS_TOPK(4);
  else if (topk <= 8) FSGS_TOPK(8);
  else FSGS_TOPK(16);
#undef FSGS_TOPK
  return check_launch("gs_2d_topk_weights");
}
