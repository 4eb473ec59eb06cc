// The blend kernels' bound on where a surfel can reach alpha >= 1/255, in the form the binning uses it: once per surfel,
// then a cheap test per tile of the surfel's rectangle.
#pragma once
#include "common.hpp"

namespace fsgs {

#ifndef FSGS_CULL_PAD
#define FSGS_CULL_PAD 0.125f
#endif
constexpr float kCullPad = FSGS_CULL_PAD;  // pixels added around the footprint box against rounding

// A pixel can only blend a surfel where alpha = min(0.99, o exp(-rho / 2)) >= 1/255, i.e. inside the perspective image of
// the ellipse u^2 + v^2 <= tau = 2 ln(255 o) of the surfel's tangent plane, or inside the screen-space disc of the
// low-pass filter. The blend kernels test the padded bounding box of that region and its extents along the two
// diagonals against each 8x8 quadrant of a tile (quadrant_mask in blend.hpp); a (surfel, tile) instance that fails the
// same test against the whole tile contributes to no pixel of it, so a binning that leaves it out of the tile's list
// changes no image and no gradient (the lists get shorter, and the positions n_contrib counts in change with them).
// The per-surfel part of the bound is formed once per surfel, the per-tile part is eight comparisons; it is evaluated
// once per surfel and view (in the preprocess kernel, or by cull_mask_kernel) and kept as a bit per tile of the
// surfel's rectangle, which the binning and the sum of the gradient records both read, so they cannot disagree.
struct CullBounds {
  float x0, x1, y0, y1, a0, a1, b0, b1;
  int state;  // 0: alpha never reaches 1/255; 1: no finite bound, every tile of the rectangle is kept; 2: test
};

__device__ __forceinline__ CullBounds cull_bounds(const float* M, float ox, float oy, float opacity) {
#pragma clang fp contract(off)
  CullBounds c;
  c.x0 = c.y0 = c.a0 = c.b0 = -1e30f, c.x1 = c.y1 = c.a1 = c.b1 = 1e30f;
  const float oa = 255.0f * opacity;
  if (!(oa >= 1.0f)) {
    c.state = 0;
    return c;
  }
  c.state = 1;
  const float tau = 2.0f * __logf(oa) * 1.0001f + 1e-3f;
  // v_sqrt_f32 / v_rcp_f32 (1 ulp): the bound is padded by 1/8 pixel + 0.5 % of its extent
  const float r2  = __builtin_amdgcn_sqrtf(0.5f * tau);
  const float u0 = M[0] - ox * M[6], u1 = M[1] - ox * M[7], u2 = M[2] - ox * M[8];
  const float v0 = M[3] - oy * M[6], v1 = M[4] - oy * M[7], v2 = M[5] - oy * M[8];
  const float d  = tau * (M[6] * M[6] + M[7] * M[7]) - M[8] * M[8];
  if (!((M[8] > 0.0f) && (d < -1e-6f * M[8] * M[8]))) return c;
  const float inv = __builtin_amdgcn_rcpf(d), f0 = tau * inv, f2 = -inv;
  // centre and half extent of the footprint along direction (p0, p1, p2) = a combination of the two rows
  auto extent = [&](float p0, float p1, float p2, float& centre, float& half) {
    centre        = f0 * (p0 * M[6] + p1 * M[7]) + f2 * (p2 * M[8]);
    const float h = centre * centre - (f0 * (p0 * p0 + p1 * p1) + f2 * (p2 * p2));
    half          = __builtin_amdgcn_sqrtf(fmaxf(h, 0.0f));
  };
  float cx, ex, cy, ey, ca, ea, cb, eb;
  extent(u0, u1, u2, cx, ex);
  extent(v0, v1, v2, cy, ey);
  if (!((ex == ex) && (ey == ey) && (cx == cx) && (cy == cy))) return c;
  float x0 = fminf(-r2, cx - ex), x1 = fmaxf(r2, cx + ex), y0 = fminf(-r2, cy - ey), y1 = fmaxf(r2, cy + ey);
  const float padx = kCullPad + 0.005f * (x1 - x0), pady = kCullPad + 0.005f * (y1 - y0);
  c.x0 = x0 - padx, c.x1 = x1 + padx, c.y0 = y0 - pady, c.y1 = y1 + pady;
  c.state = 2;
  extent(u0 + v0, u1 + v1, u2 + v2, ca, ea);
  extent(u0 - v0, u1 - v1, u2 - v2, cb, eb);
  if ((ea == ea) && (eb == eb) && (ca == ca) && (cb == cb)) {
    const float rd = 1.41421357f * r2;  // the low-pass disc along a diagonal
    const float la = fminf(ca - ea, -rd), ua = fmaxf(ca + ea, rd), lb = fminf(cb - eb, -rd), ub = fmaxf(cb + eb, rd);
    const float pa = 1.5f * kCullPad + 0.005f * (ua - la), pb = 1.5f * kCullPad + 0.005f * (ub - lb);
    c.a0 = la - pa, c.a1 = ua + pa, c.b0 = lb - pb, c.b1 = ub + pb;
  }
  return c;
}

// The same for a 3D Gaussian's screen-space conic Q = [[a, b], [b, c]] (offsets relative to its projected mean): alpha =
// min(0.99, o exp(-d^T Q d / 2)) >= 1/255 inside the ellipse d^T Q d <= tau = 2 ln(255 o), whose half extent along a
// direction n is sqrt(tau n^T Q^-1 n): sqrt(tau c / det), sqrt(tau a / det) along the axes, sqrt(tau (a + c -+ 2 b) /
// det) along x + y and x - y. A conic that is not positive definite has no finite bound (state 1).
__device__ __forceinline__ CullBounds conic_cull_bounds(float a, float b, float c, float opacity) {
#pragma clang fp contract(off)
  CullBounds r;
  r.x0 = r.y0 = r.a0 = r.b0 = -1e30f, r.x1 = r.y1 = r.a1 = r.b1 = 1e30f;
  const float oa = 255.0f * opacity;
  if (!(oa >= 1.0f)) {
    r.state = 0;
    return r;
  }
  r.state = 1;
  const float det = a * c - b * b;
  if (!(det > 0.0f) || !(a > 0.0f)) return r;
  const float tau = 2.0f * (__logf(oa) * 1.0001f + 1e-3f);
  const float s   = tau / det;
  const float ex = sqrtf(s * c), ey = sqrtf(s * a);
  if (!(ex == ex) || !(ey == ey)) return r;
  const float padx = kCullPad + 0.01f * ex, pady = kCullPad + 0.01f * ey;
  r.x0 = -(ex + padx), r.x1 = ex + padx, r.y0 = -(ey + pady), r.y1 = ey + pady;
  r.state = 2;
  const float ea = sqrtf(s * fmaxf(a + c - 2.0f * b, 0.0f)), eb = sqrtf(s * fmaxf(a + c + 2.0f * b, 0.0f));
  if ((ea == ea) && (eb == eb)) {
    const float pa = 1.5f * kCullPad + 0.01f * ea, pb = 1.5f * kCullPad + 0.01f * eb;
    r.a0 = -(ea + pa), r.a1 = ea + pa, r.b0 = -(eb + pb), r.b1 = eb + pb;
  }
  return r;
}

// true: some pixel of tile (tile_x, tile_y) may blend the surfel. The four quadrant tests of quadrant_mask folded into
// one over the tile's 16x16 pixel centres (it only lets through, in addition, footprints that fit between two
// quadrants' pixel centres).
__device__ __forceinline__ bool cull_keeps_tile(const CullBounds& c, float ox, float oy, int tile_x, int tile_y) {
#pragma clang fp contract(off)
  if (c.state != 2) return c.state == 1;
  const float qx0 = (float) (tile_x * kTile) - ox, qy0 = (float) (tile_y * kTile) - oy;
  const float qx1 = qx0 + (float) (kTile - 1), qy1 = qy0 + (float) (kTile - 1);
  const bool box  = c.x1 >= qx0 && c.x0 <= qx1 && c.y1 >= qy0 && c.y0 <= qy1;
  const bool diag = c.a1 >= qx0 + qy0 && c.a0 <= qx1 + qy1 && c.b1 >= qx0 - qy1 && c.b0 <= qx1 - qy0;
  return box && diag;
}

// Which tiles of a surfel's rectangle the binning keeps, as a bit per tile in row-major order (bit (ty - y0) * w +
// (tx - x0)); rectangles of more than 32 tiles are kept whole (all bits set).
constexpr int kCullMaskTiles = 32;

}  // namespace fsgs
