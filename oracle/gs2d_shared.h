// TEST INFRASTRUCTURE ONLY (parity oracle). Helpers shared by the standard and the "fast" surfel paths of the oracle:
// float->int conversion, tile rectangles, 4x4 products, the 3-sigma screen bound and its backward, SH -> RGB.
// Reference lines are cited per function.
#pragma once
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>

#include "sh_basis.h"

namespace oracle {

constexpr int kTile = 16;  // BLOCK_X == BLOCK_Y == 16, gaussian_render.h:28-29

// float -> int conversion with the saturating / NaN->0 behaviour of GPU conversion instructions
// (the reference relies on it for surfels whose bounding radius overflows).
template <typename T>
inline int f2i(T v) {
  if (!(v == v)) return 0;
  if (v >= T(2147483647.0)) return std::numeric_limits<int>::max();
  if (v <= T(-2147483648.0)) return std::numeric_limits<int>::min();
  return (int) v;
}

template <typename T>
struct Rect {
  int x0, y0, x1, y1;
};

// gaussian_render.h:33-39. Note the evaluation order ((p + r) + 16) - 1, all in the scalar type.
template <typename T>
inline Rect<T> get_rect(T px, T py, int r, int gx, int gy) {
  Rect<T> q;
  q.x0 = std::min(gx, std::max(0, f2i((px - T(r)) / T(kTile))));
  q.y0 = std::min(gy, std::max(0, f2i((py - T(r)) / T(kTile))));
  q.x1 = std::min(gx, std::max(0, f2i((((px + T(r)) + T(kTile)) - T(1)) / T(kTile))));
  q.y1 = std::min(gy, std::max(0, f2i((((py + T(r)) + T(kTile)) - T(1)) / T(kTile))));
  return q;
}

template <typename T>
inline void mat4_mul(const T* A, const T* B, T* C) {  // ops_3d_types.h:229-268 (sum order k=0..3)
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 4; ++j)
      C[i * 4 + j] = A[i * 4 + 0] * B[0 * 4 + j] + A[i * 4 + 1] * B[1 * 4 + j] + A[i * 4 + 2] * B[2 * 4 + j] +
                     A[i * 4 + 3] * B[3 * 4 + j];
}

// gs_2d_preprocess.cu:125-156. cutoff = 3.
template <typename T>
inline bool compute_aabb(const T* M, T cutoff, T* centre, T* extent) {
  const T t[3] = {cutoff * cutoff, cutoff * cutoff, T(-1.0)};
  const T d    = t[0] * (M[6] * M[6]) + t[1] * (M[7] * M[7]) + t[2] * (M[8] * M[8]);
  if (d == T(0)) return false;
  const T inv  = 1 / d;
  const T f[3] = {inv * t[0], inv * t[1], inv * t[2]};
  const T px   = f[0] * (M[0] * M[6]) + f[1] * (M[1] * M[7]) + f[2] * (M[2] * M[8]);
  const T py   = f[0] * (M[3] * M[6]) + f[1] * (M[4] * M[7]) + f[2] * (M[5] * M[8]);
  const T hx   = px * px - (f[0] * (M[0] * M[0]) + f[1] * (M[1] * M[1]) + f[2] * (M[2] * M[2]));
  const T hy   = py * py - (f[0] * (M[3] * M[3]) + f[1] * (M[4] * M[4]) + f[2] * (M[5] * M[5]));
  centre[0] = px, centre[1] = py;
  extent[0] = std::sqrt(std::max(T(1e-4), hx));
  extent[1] = std::sqrt(std::max(T(1e-4), hy));
  return true;
}

// gs_2d_preprocess.cu:248-266. Adds into gM.
template <typename T>
inline void compute_aabb_backward(T cutoff, const T* M, const T* g2, T* gM) {
  const T t[3] = {cutoff * cutoff, cutoff * cutoff, T(-1.0)};
  const T d    = t[0] * (M[6] * M[6]) + t[1] * (M[7] * M[7]) + t[2] * (M[8] * M[8]);
  const T inv  = T(1.0) / d;
  T f[3], g0[3], g1[3], gr2[3], df[3];
  for (int a = 0; a < 3; ++a) f[a] = t[a] * inv;
  for (int a = 0; a < 3; ++a) {
    g0[a]  = g2[0] * f[a] * M[6 + a];
    g1[a]  = g2[1] * f[a] * M[6 + a];
    gr2[a] = g2[0] * f[a] * M[a] + g2[1] * f[a] * M[3 + a];
    df[a]  = g2[0] * M[a] * M[6 + a] + g2[1] * M[3 + a] * M[6 + a];
  }
  const T dd = (df[0] * f[0] + df[1] * f[1] + df[2] * f[2]) * -(T(1.0) / d);
  for (int a = 0; a < 3; ++a) {
    const T dd_dT2 = t[a] * M[6 + a] * T(2.0);
    gr2[a] += dd * dd_dT2;
    gM[a] += g0[a];
    gM[3 + a] += g1[a];
    gM[6 + a] += gr2[a];
  }
}

// spherical_harmonic.h:18-202 (degree <= 3). sh / sh_rest follow the split layout of the reference:
// coefficient l is sh[l] when sh_rest == nullptr, else sh[0] for l == 0 and sh_rest[l-1] otherwise.
template <typename T>
inline void sh_to_rgb(int degree, const T* pos, const T* campos, const T* sh, const T* sh_rest, bool clamp,
                             T* rgb) {
  T x = pos[0], y = pos[1], z = pos[2];
  if (campos) {
    x = x - campos[0], y = y - campos[1], z = z - campos[2];
    const T n = T(1) / std::sqrt(x * x + y * y + z * z + T(1e-12));
    x = x * n, y = y * n, z = z * n;
  }
  T Y[kMaxShCoeffs];
  sh_basis(degree, x, y, z, Y);
  const int n = (degree + 1) * (degree + 1);
  for (int c = 0; c < 3; ++c) {
    T r = sh[c] * Y[0];
    for (int l = 1; l < n; ++l) r += (sh_rest ? sh_rest[(l - 1) * 3 + c] : sh[l * 3 + c]) * Y[l];
    r += T(0.5);
    rgb[c] = clamp ? std::max(T(0), r) : r;
  }
}

// spherical_harmonic.h:204-676. Writes (assigns) coefficient gradients, returns d/d(pos).
template <typename T>
inline void sh_to_rgb_backward(int degree, const T* pos, const T* campos, const T* rgb, const T* sh,
                                      const T* sh_rest, const T* grad_rgb_in, T* g_sh, T* g_sh_rest,
                                      bool need_dir, bool clamp, T* g_pos) {
  T x = pos[0], y = pos[1], z = pos[2];
  T n = T(1);
  if (campos) {
    x = x - campos[0], y = y - campos[1], z = z - campos[2];
    n = T(1) / std::sqrt(x * x + y * y + z * z + T(1e-12));
    x = x * n, y = y * n, z = z * n;
  }
  T g[3] = {grad_rgb_in[0], grad_rgb_in[1], grad_rgb_in[2]};
  if (clamp)
    for (int c = 0; c < 3; ++c) g[c] *= T(rgb[c] > 0);
  const int cnt = (degree + 1) * (degree + 1);
  T Y[kMaxShCoeffs], dY[3 * kMaxShCoeffs];
  sh_basis(degree, x, y, z, Y);
  if (g_sh) {
    for (int c = 0; c < 3; ++c) g_sh[c] = g[c] * Y[0];
    for (int l = 1; l < cnt; ++l)
      for (int c = 0; c < 3; ++c) {
        if (g_sh_rest) g_sh_rest[(l - 1) * 3 + c] = g[c] * Y[l];
        else g_sh[l * 3 + c] = g[c] * Y[l];
      }
  }
  g_pos[0] = g_pos[1] = g_pos[2] = T(0);
  if (!need_dir) return;
  sh_basis_grad(degree, x, y, z, dY);
  T dx = 0, dy = 0, dz = 0;
  for (int l = 1; l < cnt; ++l) {
    const T* v = sh_rest ? sh_rest + (l - 1) * 3 : sh + l * 3;
    const T t  = g[0] * v[0] + g[1] * v[1] + g[2] * v[2];
    dx += t * dY[l * 3 + 0], dy += t * dY[l * 3 + 1], dz += t * dY[l * 3 + 2];
  }
  if (campos) {  // through the normalisation, spherical_harmonic.h:665-674
    const T vx = pos[0] - campos[0], vy = pos[1] - campos[1], vz = pos[2] - campos[2];
    const T t  = -(vx * dx + vy * dy + vz * dz) * n * n * n;
    dx = dx * n + t * vx, dy = dy * n + t * vy, dz = dz * n + t * vz;
  }
  g_pos[0] = dx, g_pos[1] = dy, g_pos[2] = dz;
}

inline uint32_t higher_msb(uint32_t n) {  // gaussian_prepare.cu:32-44
  uint32_t msb = sizeof(n) * 4, step = msb;
  while (step > 1) {
    step /= 2;
    if (n >> msb) msb += step;
    else msb -= step;
  }
  if (n >> msb) msb++;
  return msb;
}


}  // namespace oracle
