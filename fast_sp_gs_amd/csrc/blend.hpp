// Shared pieces of the per-tile alpha-blend kernels: the LDS surfel record, the cooperative gather of a batch of
// surfels, the ray-splat intersection, and wave64 cross-lane reductions.
#pragma once
#include "common.hpp"

namespace fsgs {

constexpr int kBlendThreads = 256;  // one 16x16 tile per block = 4 wavefronts, each owning an 8x8 pixel quadrant
constexpr int kBatch        = 256;  // surfels staged in LDS per round

// Hot part of a staged surfel (what every pixel needs to decide whether the surfel touches it), 48 bytes.
struct __attribute__((aligned(16))) SplatHot {
  float m[9];      // ray-splat matrix rows Tu, Tv, Tw
  float cx, cy;    // screen-space centre (low-pass filter)
  float opacity;
};
// Cold part, only read once a pixel in the wavefront actually blends the surfel, 32 bytes.
struct __attribute__((aligned(16))) SplatCold {
  float nx, ny, nz;
  float r, g, b;
  int id;
  int pad;
};

struct Splat {
  SplatHot hot;
  SplatCold cold;
};

__device__ __forceinline__ Splat gather_splat(int id, const float2* __restrict__ means2D,
                                              const float* __restrict__ colors,
                                              const float4* __restrict__ normal_opacity,
                                              const float* __restrict__ trans_mat) {
  Splat s;
  const float* M = trans_mat + 9 * (size_t) id;
#pragma unroll
  for (int k = 0; k < 9; ++k) s.hot.m[k] = M[k];
  const float2 c = means2D[id];
  const float4 no = normal_opacity[id];
  s.hot.cx = c.x, s.hot.cy = c.y, s.hot.opacity = no.w;
  s.cold.nx = no.x, s.cold.ny = no.y, s.cold.nz = no.z;
  s.cold.r = colors[3 * (size_t) id], s.cold.g = colors[3 * (size_t) id + 1], s.cold.b = colors[3 * (size_t) id + 2];
  s.cold.id = id, s.cold.pad = 0;
  return s;
}

// Pixel owned by a lane: wavefront w covers the 8x8 quadrant (w & 1, w >> 1) of the 16x16 tile.
__device__ __forceinline__ void lane_pixel(int tile_x, int tile_y, int& px, int& py) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  px = tile_x * kTile + (wave & 1) * 8 + (lane & 7);
  py = tile_y * kTile + (wave >> 1) * 8 + (lane >> 3);
}

struct Hit {
  float kx, ky, kz, lx, ly, lz;  // the two homogeneous planes through the pixel
  float pz;                      // z of their cross product
  float sx, sy;                  // intersection in the surfel's tangent frame
  float dx, dy;                  // centre - pixel
  float rho3d, rho2d;
  float depth;
  float G;                       // exp(-rho/2)
  float alpha;
};

// Ray-splat intersection and alpha of one surfel at one pixel (gs_2d_redner.cu:122-155). Returns false when the
// reference would `continue`.
__device__ __forceinline__ bool intersect(const SplatHot& h, float pxf, float pyf, float near_n, Hit& o) {
  o.kx = pxf * h.m[6] - h.m[0], o.ky = pxf * h.m[7] - h.m[1], o.kz = pxf * h.m[8] - h.m[2];
  o.lx = pyf * h.m[6] - h.m[3], o.ly = pyf * h.m[7] - h.m[4], o.lz = pyf * h.m[8] - h.m[5];
  const float px_ = o.ky * o.lz - o.kz * o.ly;
  const float py_ = o.kz * o.lx - o.kx * o.lz;
  o.pz            = o.kx * o.ly - o.ky * o.lx;
  if (o.pz == 0.0f) return false;
  const float rz = __builtin_amdgcn_rcpf(o.pz);
  o.sx = px_ * rz, o.sy = py_ * rz;
  o.rho3d = o.sx * o.sx + o.sy * o.sy;
  o.dx = h.cx - pxf, o.dy = h.cy - pyf;
  o.rho2d = 2.0f * (o.dx * o.dx + o.dy * o.dy);
  const float rho = fminf(o.rho3d, o.rho2d);
  o.depth = (o.sx * h.m[6] + o.sy * h.m[7]) + h.m[8];
  if (o.depth < near_n) return false;
  const float power = -0.5f * rho;
  if (power > 0.0f) return false;
  o.G     = __expf(power);
  o.alpha = fminf(0.99f, h.opacity * o.G);
  return !(o.alpha < (1.0f / 255.0f));
}

// ---- wave64 reductions through DPP --------------------------------------------------------------------------------
template <int kCtrl, int kRowMask, int kBankMask>
__device__ __forceinline__ float dpp_shift_zero(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, kRowMask, kBankMask, true));
}

// Sum over the 64 lanes; the total is valid in lane 63 only.
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
  v += dpp_shift_zero<0x111, 0xf, 0xf>(v);  // row_shr:1
  v += dpp_shift_zero<0x112, 0xf, 0xf>(v);  // row_shr:2
  v += dpp_shift_zero<0x114, 0xf, 0xf>(v);  // row_shr:4
  v += dpp_shift_zero<0x118, 0xf, 0xf>(v);  // row_shr:8  -> lane 15 of every row holds the row total
  v += dpp_shift_zero<0x142, 0xa, 0xf>(v);  // row_bcast:15 into rows 1 and 3
  v += dpp_shift_zero<0x143, 0xc, 0xf>(v);  // row_bcast:31 into rows 2 and 3 -> lane 63 holds the wave total
  return v;
}

}  // namespace fsgs
