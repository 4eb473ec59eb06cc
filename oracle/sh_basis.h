// TEST INFRASTRUCTURE ONLY (parity oracle). Never linked, imported or called by the product library.
//
// Real spherical-harmonic basis, degree <= 7 (degree <= 3 written out here, 4..7 generated), in the sign/ordering convention of the reference
// (fast_2d_gs/_C/include/spherical_harmonic.h:40-79 for the basis, :387-460 for the derivative
// polynomials; fast_2d_gs/_C/src/nerf/shencoder.cu:36-73 for the encoder form of the same basis).
//
// The basis is written once as a table of values Y[l] and Cartesian gradients dY[l][3]; every SH
// consumer in the oracle (SH_to_RGB, its backward, sh_encode, its backward) is a dot product with
// this table.
//
// Pinned by tests/test_oracle_sh.py: orthonormality under sphere quadrature, degree-0 closed form,
// the l=1 sign convention (-y, +z, -x), and central finite differences of Y for dY.
#pragma once
#include "sh_basis_generated.h"  // degree 4..7, generated from the closed form by gen_sh.py

namespace oracle {

constexpr int kMaxShDegree = 7;
constexpr int kMaxShCoeffs = 64;

template <typename T>
inline void sh_basis(int degree, T x, T y, T z, T* Y) {
  Y[0] = T(0.28209479177387814);
  if (degree < 1) return;
  Y[1] = T(-0.48860251190291987) * y;
  Y[2] = T(0.48860251190291987) * z;
  Y[3] = T(-0.48860251190291987) * x;
  if (degree < 2) return;
  const T xy = x * y, xz = x * z, yz = y * z, x2 = x * x, y2 = y * y, z2 = z * z;
  Y[4] = T(1.0925484305920792) * xy;
  Y[5] = T(-1.0925484305920792) * yz;
  Y[6] = T(0.94617469575755997) * z2 - T(0.31539156525251999);
  Y[7] = T(-1.0925484305920792) * xz;
  Y[8] = T(0.54627421529603959) * x2 - T(0.54627421529603959) * y2;
  if (degree < 3) return;
  Y[9]  = T(0.59004358992664352) * y * (T(-3.0) * x2 + y2);
  Y[10] = T(2.8906114426405538) * xy * z;
  Y[11] = T(0.45704579946446572) * y * (T(1.0) - T(5.0) * z2);
  Y[12] = T(0.3731763325901154) * z * (T(5.0) * z2 - T(3.0));
  Y[13] = T(0.45704579946446572) * x * (T(1.0) - T(5.0) * z2);
  Y[14] = T(1.4453057213202769) * z * (x2 - y2);
  Y[15] = T(0.59004358992664352) * x * (-x2 + T(3.0) * y2);
  sh_basis_high(degree, x, y, z, Y);
}

// dY[l*3 + a] = d Y_l / d (x,y,z)_a, treating x,y,z as independent variables.
template <typename T>
inline void sh_basis_grad(int degree, T x, T y, T z, T* dY) {
  const int n = (degree + 1) * (degree + 1);
  for (int i = 0; i < 3 * n; ++i) dY[i] = T(0);
  if (degree < 1) return;
  dY[1 * 3 + 1] = T(-0.48860251190291992);
  dY[2 * 3 + 2] = T(0.48860251190291992);
  dY[3 * 3 + 0] = T(-0.48860251190291992);
  if (degree < 2) return;
  const T xy = x * y, xz = x * z, yz = y * z, x2 = x * x, y2 = y * y, z2 = z * z;
  dY[4 * 3 + 0] = T(1.0925484305920792) * y;
  dY[4 * 3 + 1] = T(1.0925484305920792) * x;
  dY[5 * 3 + 1] = T(-1.0925484305920792) * z;
  dY[5 * 3 + 2] = T(-1.0925484305920792) * y;
  dY[6 * 3 + 2] = T(1.8923493915151202) * z;
  dY[7 * 3 + 0] = T(-1.0925484305920792) * z;
  dY[7 * 3 + 2] = T(-1.0925484305920792) * x;
  dY[8 * 3 + 0] = T(1.0925484305920792) * x;
  dY[8 * 3 + 1] = T(-1.0925484305920792) * y;
  if (degree < 3) return;
  dY[9 * 3 + 0]  = T(-3.5402615395598609) * xy;
  dY[9 * 3 + 1]  = T(-1.7701307697799304) * x2 + T(1.7701307697799304) * y2;
  dY[10 * 3 + 0] = T(2.8906114426405538) * yz;
  dY[10 * 3 + 1] = T(2.8906114426405538) * xz;
  dY[10 * 3 + 2] = T(2.8906114426405538) * xy;
  dY[11 * 3 + 1] = T(0.45704579946446572) - T(2.2852289973223288) * z2;
  dY[11 * 3 + 2] = T(-4.5704579946446566) * yz;
  dY[12 * 3 + 2] = T(5.597644988851731) * z2 - T(1.1195289977703462);
  dY[13 * 3 + 0] = T(0.45704579946446572) - T(2.2852289973223288) * z2;
  dY[13 * 3 + 2] = T(-4.5704579946446566) * xz;
  dY[14 * 3 + 0] = T(2.8906114426405538) * xz;
  dY[14 * 3 + 1] = T(-2.8906114426405538) * yz;
  dY[14 * 3 + 2] = T(1.4453057213202769) * x2 - T(1.4453057213202769) * y2;
  dY[15 * 3 + 0] = T(-1.7701307697799304) * x2 + T(1.7701307697799304) * y2;
  dY[15 * 3 + 1] = T(3.5402615395598609) * xy;
  sh_basis_grad_high(degree, x, y, z, dY);
}

}  // namespace oracle
