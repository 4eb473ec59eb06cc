// Screen-space bound of a surfel from its 3x3 ray-splat transform and the matching backward, shared by the standard
// and the "fast" preprocess kernels. Contraction is off inside both functions and the operation order is fixed, so the
// results are reproducible bit for bit against a plain IEEE evaluation
// (fast_2d_gs/_C/src/gaussian_splatting/gs_2d_preprocess.cu:126-141, :248-267; gs_2d_fast_preprocess.cu:143-158, :516-535).
#pragma once
#include <hip/hip_runtime.h>

namespace fsgs {

__device__ __forceinline__ bool bound_3sigma(const float* M, float* c, float* ext) {
#pragma clang fp contract(off)
  const float t0 = 9.0f, t1 = 9.0f, t2 = -1.0f;
  const float d  = t0 * (M[6] * M[6]) + t1 * (M[7] * M[7]) + t2 * (M[8] * M[8]);
  if (d == 0.0f) return false;
  const float inv = 1 / d;
  const float f0 = inv * t0, f1 = inv * t1, f2 = inv * t2;
  const float px = f0 * (M[0] * M[6]) + f1 * (M[1] * M[7]) + f2 * (M[2] * M[8]);
  const float py = f0 * (M[3] * M[6]) + f1 * (M[4] * M[7]) + f2 * (M[5] * M[8]);
  const float hx = px * px - (f0 * (M[0] * M[0]) + f1 * (M[1] * M[1]) + f2 * (M[2] * M[2]));
  const float hy = py * py - (f0 * (M[3] * M[3]) + f1 * (M[4] * M[4]) + f2 * (M[5] * M[5]));
  c[0] = px, c[1] = py;
  ext[0] = sqrtf(fmaxf(1e-4f, hx));
  ext[1] = sqrtf(fmaxf(1e-4f, hy));
  return true;
}

__device__ __forceinline__ void bound_backward(const float* M, float g2x, float g2y, float* gM) {
#pragma clang fp contract(off)
  const float t[3] = {9.0f, 9.0f, -1.0f};
  const float d    = t[0] * (M[6] * M[6]) + t[1] * (M[7] * M[7]) + t[2] * (M[8] * M[8]);
  const float inv  = 1.0f / d;
  float f[3], df[3];
#pragma unroll
  for (int a = 0; a < 3; ++a) f[a] = t[a] * inv;
  float g0[3], g1[3], gr2[3];
#pragma unroll
  for (int a = 0; a < 3; ++a) {
    g0[a]  = g2x * f[a] * M[6 + a];
    g1[a]  = g2y * f[a] * M[6 + a];
    gr2[a] = g2x * f[a] * M[a] + g2y * f[a] * M[3 + a];
    df[a]  = g2x * M[a] * M[6 + a] + g2y * M[3 + a] * M[6 + a];
  }
  const float dd = (df[0] * f[0] + df[1] * f[1] + df[2] * f[2]) * -(1.0f / d);
#pragma unroll
  for (int a = 0; a < 3; ++a) {
    gr2[a] += dd * (t[a] * M[6 + a] * 2.0f);
    gM[a] += g0[a];
    gM[3 + a] += g1[a];
    gM[6 + a] += gr2[a];
  }
}

}  // namespace fsgs
