// Device-side real spherical harmonics (degree 0..7) in the reference's convention
// (fast_2d_gs/_C/include/spherical_harmonic.h:40-193): l=1 is (-y, +z, -x), colours get +0.5 and a clamp at 0.
// Values and Cartesian gradients are produced into register arrays so callers can fuse them with coefficient
// loads of any layout. Degree <= 3 is written out here; degree 4..7 comes from sh_generated.hpp (derived from the
// closed form by gen_sh_tables.py). Kernels are instantiated for 16 coefficients (degree <= 3, the common case, small
// register footprint) and for 64.
#pragma once
#include <hip/hip_runtime.h>

#include "sh_generated.hpp"

namespace fsgs {

constexpr int kMaxShDegree = 7;

__device__ __forceinline__ int sh_count(int degree) { return (degree + 1) * (degree + 1); }

// Entries beyond (degree+1)^2 are left untouched. kN = 16 serves degree <= 3, kN = 64 degree <= 7. T is float or double;
// the coefficients are single-precision literals for either (shencoder.cu:36-176 writes them so for every scalar_t).
template <int kN, typename T>
__device__ __forceinline__ void sh_eval(int degree, T x, T y, T z, T (&Y)[kN]) {
  Y[0] = 0.28209479177387814f;
  if (degree < 1) return;
  Y[1] = -0.48860251190291987f * y;
  Y[2] = 0.48860251190291987f * z;
  Y[3] = -0.48860251190291987f * x;
  if (degree < 2) return;
  const T xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
  Y[4] = 1.0925484305920792f * xy;
  Y[5] = -1.0925484305920792f * yz;
  Y[6] = 0.94617469575755997f * zz - 0.31539156525251999f;
  Y[7] = -1.0925484305920792f * xz;
  Y[8] = 0.54627421529603959f * xx - 0.54627421529603959f * yy;
  if (degree < 3) return;
  Y[9]  = 0.59004358992664352f * y * (-3.0f * xx + yy);
  Y[10] = 2.8906114426405538f * xy * z;
  Y[11] = 0.45704579946446572f * y * (1.0f - 5.0f * zz);
  Y[12] = 0.3731763325901154f * z * (5.0f * zz - 3.0f);
  Y[13] = 0.45704579946446572f * x * (1.0f - 5.0f * zz);
  Y[14] = 1.4453057213202769f * z * (xx - yy);
  Y[15] = 0.59004358992664352f * x * (-xx + 3.0f * yy);
  if constexpr (kN > 16) sh_eval_high(degree, x, y, z, Y);
}

// Accumulates t_l * grad(Y_l) for l >= 1 into (dx, dy, dz); t[l] is the caller's per-basis scalar
// (dot(grad_rgb, coeff_l) for SH->RGB, the upstream gradient for the bare encoder).
template <int kN, typename T>
__device__ __forceinline__ void sh_grad_accumulate(int degree, T x, T y, T z, const T (&t)[kN], T& dx, T& dy, T& dz) {
  if (degree < 1) return;
  dy += t[1] * -0.48860251190291992f;
  dz += t[2] * 0.48860251190291992f;
  dx += t[3] * -0.48860251190291992f;
  if (degree < 2) return;
  const T xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
  dx += t[4] * (1.0925484305920792f * y);
  dy += t[4] * (1.0925484305920792f * x);
  dy += t[5] * (-1.0925484305920792f * z);
  dz += t[5] * (-1.0925484305920792f * y);
  dz += t[6] * (1.8923493915151202f * z);
  dx += t[7] * (-1.0925484305920792f * z);
  dz += t[7] * (-1.0925484305920792f * x);
  dx += t[8] * (1.0925484305920792f * x);
  dy += t[8] * (-1.0925484305920792f * y);
  if (degree < 3) return;
  dx += t[9] * (-3.5402615395598609f * xy);
  dy += t[9] * (-1.7701307697799304f * xx + 1.7701307697799304f * yy);
  dx += t[10] * (2.8906114426405538f * yz);
  dy += t[10] * (2.8906114426405538f * xz);
  dz += t[10] * (2.8906114426405538f * xy);
  dy += t[11] * (0.45704579946446572f - 2.2852289973223288f * zz);
  dz += t[11] * (-4.5704579946446566f * yz);
  dz += t[12] * (5.597644988851731f * zz - 1.1195289977703462f);
  dx += t[13] * (0.45704579946446572f - 2.2852289973223288f * zz);
  dz += t[13] * (-4.5704579946446566f * xz);
  dx += t[14] * (2.8906114426405538f * xz);
  dy += t[14] * (-2.8906114426405538f * yz);
  dz += t[14] * (1.4453057213202769f * xx - 1.4453057213202769f * yy);
  dx += t[15] * (-1.7701307697799304f * xx + 1.7701307697799304f * yy);
  dy += t[15] * (3.5402615395598609f * xy);
  if constexpr (kN > 16) sh_grad_accumulate_high(degree, x, y, z, t, dx, dy, dz);
}

// ---- the bare encoder on half tensors, degree <= 3 -----------------------------------------------------------------------
// With scalar_t = at::Half the reference keeps its monomials (xy, xz, yz, x2, y2, z2) and, in the backward, the three
// running sums in half: a product of two halves is formed in float and rounded to half (shencoder.cu:31-33, 190-193),
// `dx += term` rounds the term to half and then the sum (:204-281; terms whose factor is the literal 0 add nothing). The
// basis values themselves are float expressions of those monomials, rounded once on store. Restated here for degree
// <= 3; degrees 4 - 7 on half tensors use the float routines above (one rounding on store).
__device__ __forceinline__ float round_half(float v) { return (float) (_Float16) v; }

__device__ __forceinline__ void sh_eval_half(int degree, float x, float y, float z, float (&Y)[16]) {
  Y[0] = 0.28209479177387814f;
  if (degree < 1) return;
  Y[1] = -0.48860251190291987f * y;
  Y[2] = 0.48860251190291987f * z;
  Y[3] = -0.48860251190291987f * x;
  if (degree < 2) return;
  const float xy = round_half(x * y), xz = round_half(x * z), yz = round_half(y * z);
  const float xx = round_half(x * x), yy = round_half(y * y), zz = round_half(z * z);
  Y[4] = 1.0925484305920792f * xy;
  Y[5] = -1.0925484305920792f * yz;
  Y[6] = 0.94617469575755997f * zz - 0.31539156525251999f;
  Y[7] = -1.0925484305920792f * xz;
  Y[8] = 0.54627421529603959f * xx - 0.54627421529603959f * yy;
  if (degree < 3) return;
  Y[9]  = 0.59004358992664352f * y * (-3.0f * xx + yy);
  Y[10] = 2.8906114426405538f * xy * z;
  Y[11] = 0.45704579946446572f * y * (1.0f - 5.0f * zz);
  Y[12] = 0.3731763325901154f * z * (5.0f * zz - 3.0f);
  Y[13] = 0.45704579946446572f * x * (1.0f - 5.0f * zz);
  Y[14] = 1.4453057213202769f * z * (xx - yy);
  Y[15] = 0.59004358992664352f * x * (-xx + 3.0f * yy);
}

__device__ __forceinline__ void sh_grad_half(int degree, float x, float y, float z, const float (&t)[16], float& dx,
                                             float& dy, float& dz) {
  auto add = [](float& acc, float term) { acc = round_half(acc + round_half(term)); };
  dx = dy = dz = 0.0f;
  if (degree < 1) return;
  const float xy = round_half(x * y), xz = round_half(x * z), yz = round_half(y * z);
  const float xx = round_half(x * x), yy = round_half(y * y), zz = round_half(z * z);
  // the reference finishes dx over all degrees, then dy, then dz; the sums do not interact, so the order across the
  // three does not matter, the order inside each does
  add(dx, t[3] * -0.48860251190291992f);
  add(dy, t[1] * -0.48860251190291992f);
  add(dz, t[2] * 0.48860251190291992f);
  if (degree < 2) return;
  add(dx, t[4] * (1.0925484305920792f * y)), add(dx, t[7] * (-1.0925484305920792f * z));
  add(dx, t[8] * (1.0925484305920792f * x));
  add(dy, t[4] * (1.0925484305920792f * x)), add(dy, t[5] * (-1.0925484305920792f * z));
  add(dy, t[8] * (-1.0925484305920792f * y));
  add(dz, t[5] * (-1.0925484305920792f * y)), add(dz, t[6] * (1.8923493915151204f * z));
  add(dz, t[7] * (-1.0925484305920792f * x));
  if (degree < 3) return;
  add(dx, t[9] * (-3.5402615395598609f * xy)), add(dx, t[10] * (2.8906114426405538f * yz));
  add(dx, t[13] * (0.45704579946446572f - 2.2852289973223288f * zz)), add(dx, t[14] * (2.8906114426405538f * xz));
  add(dx, t[15] * (-1.7701307697799304f * xx + 1.7701307697799304f * yy));
  add(dy, t[9] * (-1.7701307697799304f * xx + 1.7701307697799304f * yy)), add(dy, t[10] * (2.8906114426405538f * xz));
  add(dy, t[11] * (0.45704579946446572f - 2.2852289973223288f * zz)), add(dy, t[14] * (-2.8906114426405538f * yz));
  add(dy, t[15] * (3.5402615395598609f * xy));
  add(dz, t[10] * (2.8906114426405538f * xy)), add(dz, t[11] * (-4.5704579946446566f * yz));
  add(dz, t[12] * (5.597644988851731f * zz - 1.1195289977703462f)), add(dz, t[13] * (-4.5704579946446566f * xz));
  add(dz, t[14] * (1.4453057213202769f * xx - 1.4453057213202769f * yy));
}

// Unit view direction from the camera to p: (p - cam) * rsqrt(|p - cam|^2 + 1e-12) (spherical_harmonic.h:27-35).
__device__ __forceinline__ float view_dir(const float* __restrict__ p, const float* __restrict__ cam, float& x,
                                          float& y, float& z) {
  x = p[0] - cam[0], y = p[1] - cam[1], z = p[2] - cam[2];
  const float n = 1.0f / sqrtf(x * x + y * y + z * z + 1e-12f);
  x *= n, y *= n, z *= n;
  return n;
}

}  // namespace fsgs
