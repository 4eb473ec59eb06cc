// Per-pixel epilogue of the 2DGS render, fused, with its backward, for gfx950.
//
// Reference behaviour reproduced: fast_2d_gs/renderer/gs_2d_render.py:608-617 (normals to world space, nan_to_num of the
// two depth maps, surf_depth mix, pseudo surface normal from the depth map, times the detached opacity), its helpers
// depths_to_points / depth_to_normal (:439-470) and the background composite of fast_2d_gs/network.py:725-726. In the
// reference these are ~25 elementwise / matmul / inverse launches over HW per view and as many again in autograd; here
// one kernel each way. The 3x3 pixel -> world ray matrix (inverse intrinsics, then the camera-to-world rotation) and
// the camera centre are derived from Tw2v / Tv2c by the first lane of every block.
//
// intrins = ((c2w^T (Tv2c Tw2v)^T) ndc2pix^T)[:3,:3]^T of the reference equals (ndc2pix Tv2c)[:3,:3] because
// c2w = Tw2v^-1; it is formed in that closed form.
#include "common.hpp"

namespace fsgs {
namespace {

struct PixelRays {
  float m[9];  // ray direction of pixel (x, y) = m . (x, y, 1)
  float o[3];  // camera centre in world space
};

__device__ inline void invert3(const float* a, float* inv) {
  const float c00 = a[4] * a[8] - a[5] * a[7], c01 = a[5] * a[6] - a[3] * a[8], c02 = a[3] * a[7] - a[4] * a[6];
  const float det = a[0] * c00 + a[1] * c01 + a[2] * c02, r = 1.0f / det;
  inv[0] = c00 * r, inv[1] = (a[2] * a[7] - a[1] * a[8]) * r, inv[2] = (a[1] * a[5] - a[2] * a[4]) * r;
  inv[3] = c01 * r, inv[4] = (a[0] * a[8] - a[2] * a[6]) * r, inv[5] = (a[2] * a[3] - a[0] * a[5]) * r;
  inv[6] = c02 * r, inv[7] = (a[1] * a[6] - a[0] * a[7]) * r, inv[8] = (a[0] * a[4] - a[1] * a[3]) * r;
}

// Tw2v is taken as affine (last row 0 0 0 1, which a world-to-view matrix is): c2w = [R^-1 | -R^-1 t] with a general
// 3x3 inverse, so scaled or sheared view matrices work too.
__device__ inline void pixel_rays(int W, int H, const float* __restrict__ Tw2v, const float* __restrict__ Tv2c,
                                  PixelRays& out) {
  float R[9] = {Tw2v[0], Tw2v[1], Tw2v[2], Tw2v[4], Tw2v[5], Tw2v[6], Tw2v[8], Tw2v[9], Tw2v[10]};
  float Ri[9];
  invert3(R, Ri);  // c2w rotation block
  const float t[3] = {Tw2v[3], Tw2v[7], Tw2v[11]};
#pragma unroll
  for (int a = 0; a < 3; ++a) out.o[a] = -(Ri[a * 3] * t[0] + Ri[a * 3 + 1] * t[1] + Ri[a * 3 + 2] * t[2]);
  const float hw = 0.5f * (float) W, hh = 0.5f * (float) H;
  float K[9], Ki[9];
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    K[c]     = hw * Tv2c[c] + hw * Tv2c[12 + c];
    K[3 + c] = hh * Tv2c[4 + c] + hh * Tv2c[12 + c];
    K[6 + c] = Tv2c[12 + c];
  }
  invert3(K, Ki);
#pragma unroll
  for (int a = 0; a < 3; ++a)
#pragma unroll
    for (int b = 0; b < 3; ++b) out.m[a * 3 + b] = Ri[a * 3] * Ki[b] + Ri[a * 3 + 1] * Ki[3 + b] + Ri[a * 3 + 2] * Ki[6 + b];
}

// torch.nan_to_num(x, 0, 0): NaN and +inf become 0, -inf the lowest finite float.
__device__ __forceinline__ float nan0(float v) {
  if (v != v || v == __builtin_inff()) return 0.0f;
  return v == -__builtin_inff() ? -3.4028234663852886e38f : v;
}
__device__ __forceinline__ bool finite_f(float v) { return v == v && fabsf(v) != __builtin_inff(); }

struct Vec3 {
  float x, y, z;
};
__device__ __forceinline__ Vec3 cross3(Vec3 a, Vec3 b) {
  return {a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x};
}

struct DepthMaps {
  const float* depth;   // extras channel 0
  const float* median;  // extras channel 4
  float ratio;
  int W;
  __device__ __forceinline__ float surf(int x, int y) const {
    const size_t p = (size_t) y * W + x;
    return nan0(depth[p]) * (1.0f - ratio) + ratio * nan0(median[p]);
  }
};

__device__ __forceinline__ Vec3 world_point(const PixelRays& r, const DepthMaps& d, int x, int y) {
  const float fx = (float) x, fy = (float) y, s = d.surf(x, y);
  return {s * (r.m[0] * fx + r.m[1] * fy + r.m[2]) + r.o[0], s * (r.m[3] * fx + r.m[4] * fy + r.m[5]) + r.o[1],
          s * (r.m[6] * fx + r.m[7] * fy + r.m[8]) + r.o[2]};
}

// Unnormalised pseudo normal at an interior pixel: (P(y+1) - P(y-1)) x (P(x+1) - P(x-1)).
__device__ __forceinline__ void central_differences(const PixelRays& r, const DepthMaps& d, int x, int y, Vec3& a,
                                                    Vec3& b) {
  const Vec3 up = world_point(r, d, x, y - 1), dn = world_point(r, d, x, y + 1);
  const Vec3 lf = world_point(r, d, x - 1, y), rt = world_point(r, d, x + 1, y);
  a = {dn.x - up.x, dn.y - up.y, dn.z - up.z};
  b = {rt.x - lf.x, rt.y - lf.y, rt.z - lf.z};
}

__global__ void __launch_bounds__(256) epilogue_forward_kernel(int W, int H, float ratio,
    const float* __restrict__ Tw2v, const float* __restrict__ Tv2c, const float* __restrict__ extras,
    const float* __restrict__ opacity, const float* __restrict__ images, const float* __restrict__ background,
    float* __restrict__ normals, float* __restrict__ depths, float* __restrict__ surf_depth,
    float* __restrict__ surf_normal, float* __restrict__ composited) {
  __shared__ PixelRays s_rays;
  if (threadIdx.x == 0 && threadIdx.y == 0) pixel_rays(W, H, Tw2v, Tv2c, s_rays);
  __syncthreads();
  const int x = blockIdx.x * 32 + threadIdx.x, y = blockIdx.y * 8 + threadIdx.y;
  if (x >= W || y >= H) return;
  const size_t HW = (size_t) H * W, p = (size_t) y * W + x;
  const DepthMaps maps = {extras, extras + 4 * HW, ratio, W};
  // normals to world space: row vector times Tw2v[:3,:3]
  const float n0 = extras[HW + p], n1 = extras[2 * HW + p], n2 = extras[3 * HW + p];
#pragma unroll
  for (int j = 0; j < 3; ++j) normals[j * HW + p] = n0 * Tw2v[j] + n1 * Tw2v[4 + j] + n2 * Tw2v[8 + j];
  depths[p]     = nan0(maps.median[p]);
  surf_depth[p] = maps.surf(x, y);
  Vec3 n = {0.0f, 0.0f, 0.0f};
  if (x >= 1 && y >= 1 && x <= W - 2 && y <= H - 2) {
    Vec3 a, b;
    central_differences(s_rays, maps, x, y, a, b);
    const Vec3 c    = cross3(a, b);
    const float inv = opacity[p] / fmaxf(sqrtf(c.x * c.x + c.y * c.y + c.z * c.z), 1e-12f);
    n = {c.x * inv, c.y * inv, c.z * inv};
  }
  surf_normal[p] = n.x, surf_normal[HW + p] = n.y, surf_normal[2 * HW + p] = n.z;
  if (composited) {
    const float t = 1.0f - opacity[p];
#pragma unroll
    for (int c = 0; c < 3; ++c) composited[c * HW + p] = images[c * HW + p] + t * background[c];
  }
}

// dL/d(a), dL/d(b) of the pseudo normal at interior pixel (x, y) given the gradient of its output.
__device__ __forceinline__ void normal_backward(const PixelRays& r, const DepthMaps& d,
    const float* __restrict__ opacity, const float* __restrict__ g_surf_normal, size_t HW, int x, int y, Vec3& ga,
    Vec3& gb) {
  Vec3 a, b;
  central_differences(r, d, x, y, a, b);
  const Vec3 c    = cross3(a, b);
  const float len = sqrtf(c.x * c.x + c.y * c.y + c.z * c.z);
  const size_t q  = (size_t) y * d.W + x;
  const float o   = opacity[q];
  const Vec3 gn   = {g_surf_normal[q] * o, g_surf_normal[HW + q] * o, g_surf_normal[2 * HW + q] * o};
  Vec3 gc;
  if (len > 1e-12f) {
    const float il = 1.0f / len;
    const Vec3 n   = {c.x * il, c.y * il, c.z * il};
    const float t  = n.x * gn.x + n.y * gn.y + n.z * gn.z;
    gc = {(gn.x - n.x * t) * il, (gn.y - n.y * t) * il, (gn.z - n.z * t) * il};
  } else {
    gc = {gn.x * 1e12f, gn.y * 1e12f, gn.z * 1e12f};
  }
  ga = cross3(b, gc);
  gb = cross3(gc, a);
}

__global__ void __launch_bounds__(256) epilogue_backward_kernel(int W, int H, float ratio,
    const float* __restrict__ Tw2v, const float* __restrict__ Tv2c, const float* __restrict__ extras,
    const float* __restrict__ opacity, const float* __restrict__ background, const float* __restrict__ g_normals,
    const float* __restrict__ g_depths, const float* __restrict__ g_surf_depth,
    const float* __restrict__ g_surf_normal, const float* __restrict__ g_distortion,
    const float* __restrict__ g_composited, float* __restrict__ g_extras, float* __restrict__ g_opacity) {
  __shared__ PixelRays s_rays;
  if (threadIdx.x == 0 && threadIdx.y == 0) pixel_rays(W, H, Tw2v, Tv2c, s_rays);
  __syncthreads();
  const int x = blockIdx.x * 32 + threadIdx.x, y = blockIdx.y * 8 + threadIdx.y;
  if (x >= W || y >= H) return;
  const size_t HW = (size_t) H * W, p = (size_t) y * W + x;
  const DepthMaps maps = {extras, extras + 4 * HW, ratio, W};
  float g_sd = g_surf_depth ? g_surf_depth[p] : 0.0f;
  if (g_surf_normal) {
    // this pixel's world point enters the central differences of its four neighbours (where those are interior)
    Vec3 gp = {0.0f, 0.0f, 0.0f}, ga, gb;
    const bool xin = x >= 1 && x <= W - 2, yin = y >= 1 && y <= H - 2;
    if (xin && y - 1 >= 1 && y - 1 <= H - 2) {  // P(p) is the lower point of (x, y - 1)
      normal_backward(s_rays, maps, opacity, g_surf_normal, HW, x, y - 1, ga, gb);
      gp.x += ga.x, gp.y += ga.y, gp.z += ga.z;
    }
    if (xin && y + 1 >= 1 && y + 1 <= H - 2) {  // ... the upper point of (x, y + 1)
      normal_backward(s_rays, maps, opacity, g_surf_normal, HW, x, y + 1, ga, gb);
      gp.x -= ga.x, gp.y -= ga.y, gp.z -= ga.z;
    }
    if (yin && x - 1 >= 1 && x - 1 <= W - 2) {  // ... the right point of (x - 1, y)
      normal_backward(s_rays, maps, opacity, g_surf_normal, HW, x - 1, y, ga, gb);
      gp.x += gb.x, gp.y += gb.y, gp.z += gb.z;
    }
    if (yin && x + 1 >= 1 && x + 1 <= W - 2) {  // ... the left point of (x + 1, y)
      normal_backward(s_rays, maps, opacity, g_surf_normal, HW, x + 1, y, ga, gb);
      gp.x -= gb.x, gp.y -= gb.y, gp.z -= gb.z;
    }
    const float fx = (float) x, fy = (float) y;
    const float* m = s_rays.m;
    g_sd += gp.x * (m[0] * fx + m[1] * fy + m[2]) + gp.y * (m[3] * fx + m[4] * fy + m[5]) +
            gp.z * (m[6] * fx + m[7] * fy + m[8]);
  }
  const float g_med = ratio * g_sd + (g_depths ? g_depths[p] : 0.0f);
  g_extras[p]          = finite_f(maps.depth[p]) ? (1.0f - ratio) * g_sd : 0.0f;
  g_extras[4 * HW + p] = finite_f(maps.median[p]) ? g_med : 0.0f;
  float gn[3] = {0.0f, 0.0f, 0.0f};
  if (g_normals) {
    const float g0 = g_normals[p], g1 = g_normals[HW + p], g2 = g_normals[2 * HW + p];
#pragma unroll
    for (int i = 0; i < 3; ++i) gn[i] = g0 * Tw2v[4 * i] + g1 * Tw2v[4 * i + 1] + g2 * Tw2v[4 * i + 2];
  }
#pragma unroll
  for (int i = 0; i < 3; ++i) g_extras[(1 + i) * HW + p] = gn[i];
  g_extras[5 * HW + p] = g_distortion ? g_distortion[p] : 0.0f;
#pragma unroll
  for (int c = 6; c < 9; ++c) g_extras[c * HW + p] = 0.0f;
  if (g_opacity) {
    float s = 0.0f;
    if (g_composited)
#pragma unroll
      for (int c = 0; c < 3; ++c) s += g_composited[c * HW + p] * background[c];
    g_opacity[p] = -s;
  }
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API int fsgs_gs_2d_epilogue_forward(int W, int H, double depth_ratio, const float* Tw2v, const float* Tv2c,
    const float* extras, const float* opacity, const float* images, const float* background, float* normals,
    float* depths, float* surf_depth, float* surf_normal, float* composited, void* stream) {
  FSGS_REQUIRE(W >= 0 && H >= 0, "gs_2d_epilogue_forward: bad size");
  if ((size_t) W * H == 0) return kOk;
  FSGS_REQUIRE(Tw2v && Tv2c && extras && opacity && normals && depths && surf_depth && surf_normal,
               "gs_2d_epilogue_forward: null pointer");
  FSGS_REQUIRE(!composited || (images && background), "gs_2d_epilogue_forward: composite needs images and background");
  const dim3 grid(div_up(W, 32), div_up(H, 8)), block(32, 8);
  hipLaunchKernelGGL(epilogue_forward_kernel, grid, block, 0, (hipStream_t) stream, W, H, (float) depth_ratio, Tw2v,
                     Tv2c, extras, opacity, images, background, normals, depths, surf_depth, surf_normal, composited);
  return check_launch("gs_2d_epilogue_forward");
}

FSGS_API int fsgs_gs_2d_epilogue_backward(int W, int H, double depth_ratio, const float* Tw2v, const float* Tv2c,
    const float* extras, const float* opacity, const float* background, const float* g_normals, const float* g_depths,
    const float* g_surf_depth, const float* g_surf_normal, const float* g_distortion, const float* g_composited,
    float* g_extras, float* g_opacity, void* stream) {
  FSGS_REQUIRE(W >= 0 && H >= 0, "gs_2d_epilogue_backward: bad size");
  if ((size_t) W * H == 0) return kOk;
  FSGS_REQUIRE(Tw2v && Tv2c && extras && opacity && g_extras, "gs_2d_epilogue_backward: null pointer");
  FSGS_REQUIRE(!g_composited || (background && g_opacity),
               "gs_2d_epilogue_backward: the composite gradient needs the background and g_opacity");
  const dim3 grid(div_up(W, 32), div_up(H, 8)), block(32, 8);
  hipLaunchKernelGGL(epilogue_backward_kernel, grid, block, 0, (hipStream_t) stream, W, H, (float) depth_ratio, Tw2v,
                     Tv2c, extras, opacity, background, g_normals, g_depths, g_surf_depth, g_surf_normal, g_distortion,
                     g_composited, g_extras, g_opacity);
  return check_launch("gs_2d_epilogue_backward");
}
