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

// One staged surfel as gathered from the three tensors (the hot record plus its id).
struct TopkEntry {
  SplatHot hot;
  int id;
};

__device__ __forceinline__ TopkEntry gather_topk(int id, const float2* __restrict__ means2D,
    const float* __restrict__ trans_mat, const float4* __restrict__ normal_opacity) {
  TopkEntry e;
  const float* M = trans_mat + 9 * (size_t) id;
#pragma unroll
  for (int k = 0; k < 9; ++k) e.hot.m[k] = M[k];
  const float2 c = means2D[id];
  e.hot.cx = c.x, e.hot.cy = c.y, e.hot.opacity = normal_opacity[id].w;
  e.id = id;
  return e;
}

template <int kK>
__global__ void __launch_bounds__(kBlendThreads) blend_topk_kernel(
    int ordered, const int* __restrict__ tile_order, int W, int H, int topk, float near_n, const int64_t* __restrict__ ranges, const int32_t* __restrict__ point_list,
    const float2* __restrict__ means2D, const float* __restrict__ trans_mat, const float4* __restrict__ normal_opacity,
    int32_t* __restrict__ top_indices, float* __restrict__ top_weights) {
  constexpr int kB = 128;  // surfels staged per round
  __shared__ SplatHot s_hot[kB];
  __shared__ int s_id[kB];
  __shared__ unsigned char s_mask[kB];

  const int gx = (W + kTile - 1) / kTile;
  const int tile = scheduled_tile(ordered, tile_order), tile_x = tile % gx, tile_y = tile / gx;
  int px, py;
  lane_pixel(tile_x, tile_y, px, py);
  const bool inside = px < W && py < H;
  const size_t pix  = (size_t) W * py + px;
  const float pxf = (float) px, pyf = (float) py;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

  const int64_t r0 = ranges[2 * (size_t) tile], r1 = ranges[2 * (size_t) tile + 1];
  const int n_todo = (int) (r1 - r0);
  const int rounds = (n_todo + kB - 1) / kB;

  bool done = !inside;
  float T = 1.0f;
  float tw[kK];  // descending
  int ti[kK];
#pragma unroll
  for (int k = 0; k < kK; ++k) tw[k] = 0.0f, ti[k] = -1;

  // the next batch's gather is in flight while the current one is walked
  TopkEntry next;
  if ((int) threadIdx.x < min(n_todo, kB)) next = gather_topk(point_list[r0 + threadIdx.x], means2D, trans_mat, normal_opacity);
  for (int b = 0; b < rounds; ++b) {
    if (__syncthreads_count(done) == kBlendThreads) break;
    const int n_here = min(kB, n_todo - b * kB);
    if ((int) threadIdx.x < n_here) {
      s_hot[threadIdx.x]  = next.hot;
      s_id[threadIdx.x]   = next.id;
      s_mask[threadIdx.x] = (unsigned char) quadrant_mask(next.hot, tile_x * kTile, tile_y * kTile, ordered);
    }
    __syncthreads();
    const int nxt = (b + 1) * kB + (int) threadIdx.x;
    if ((int) threadIdx.x < kB && nxt < n_todo)
      next = gather_topk(point_list[r0 + nxt], means2D, trans_mat, normal_opacity);
    for (int c = 0; c < kB / kWave; ++c) {
      const int jj = c * kWave + lane;
      unsigned long long todo = __ballot(jj < n_here && ((s_mask[jj] >> wave) & 1u));
      while (todo) {
        if (__ballot(!done) == 0ull) break;
        const int j = c * kWave + __builtin_ctzll(todo);
        todo &= todo - 1;
        // one predicate, no early exits: the wavefront leaves the entry together when nobody blends it
        const SplatHot& h = s_hot[j];
        const float kx = pxf * h.m[6] - h.m[0], ky = pxf * h.m[7] - h.m[1], kz = pxf * h.m[8] - h.m[2];
        const float lx = pyf * h.m[6] - h.m[3], ly = pyf * h.m[7] - h.m[4], lz = pyf * h.m[8] - h.m[5];
        const float qx = ky * lz - kz * ly, qy = kz * lx - kx * lz, qz = kx * ly - ky * lx;
        const float rz = __builtin_amdgcn_rcpf(qz);
        const float sx = qx * rz, sy = qy * rz;
        const float rho3d = sx * sx + sy * sy;
        const float dx = h.cx - pxf, dy = h.cy - pyf;
        const float rho2d = 2.0f * (dx * dx + dy * dy);
        const float rho   = fminf(rho3d, rho2d);
        const float depth = (rho3d <= rho2d) ? (sx * h.m[6] + sy * h.m[7]) + h.m[8] : h.m[8];
        const float power = -0.5f * rho;
        const float alpha = fminf(0.99f, h.opacity * __expf(power));
        const bool hit = !done & (qz != 0.0f) & !(depth < near_n) & !(power > 0.0f) & !(alpha < (1.0f / 255.0f));
        if (__ballot(hit) == 0ull) continue;
        const float test_T = T * (1.0f - alpha);
        const bool sat     = hit && test_T < 0.0001f;
        done               = done || sat;
        if (hit && !sat) {
          // sorted insertion: a slot's new weight is the offered one clamped between the slot and the slot above, its
          // id follows the comparisons against the old list (`w >= slot` takes the slot: a later surfel wins ties)
          const float w = alpha * T;
          const int idx = s_id[j];
          bool ge[kK];
#pragma unroll
          for (int k = 0; k < kK; ++k) ge[k] = k < topk && w >= tw[k];
#pragma unroll
          for (int k = kK - 1; k >= 1; --k) {
            if (k < topk) {
              tw[k] = __builtin_amdgcn_fmed3f(tw[k - 1], w, tw[k]);
              ti[k] = ge[k - 1] ? ti[k - 1] : (ge[k] ? idx : ti[k]);
            }
          }
          tw[0] = fmaxf(tw[0], w);
          ti[0] = ge[0] ? idx : ti[0];
          T = test_T;
        }
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
  const int* tile_order = nullptr;
  const int ordered = launch_tile_order(gx, gy, ranges, s, &tile_order);
#define FSGS_TOPK(KK)                                                                                            \
  hipLaunchKernelGGL((blend_topk_kernel<KK>), grid, block, 0, s, ordered, tile_order, W, H, topk, (float) near_n, ranges, point_list, \
                     (const float2*) means2D, trans_mat, (const float4*) normal_opacity, top_indices, top_weights)
  if (topk <= 4) FSGS_TOPK(4);
  else if (topk <= 8) FSGS_TOPK(8);
  else FSGS_TOPK(16);
#undef FSGS_TOPK
  return check_launch("gs_2d_topk_weights");
}
