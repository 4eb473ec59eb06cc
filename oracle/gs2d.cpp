// TEST INFRASTRUCTURE ONLY (parity oracle + CPU baseline). Never linked, imported or called by the
// product library; only tests/, the smoke check and the bench's cpu_baseline leg load it.
//
// Scalar CPU restatement of the 2D-Gaussian-surfel render path of the reference:
//   preprocess forward/backward   fast_2d_gs/_C/src/gaussian_splatting/gs_2d_preprocess.cu:24-329
//   tile binning                  fast_2d_gs/_C/src/gaussian_splatting/gaussian_prepare.cu:32-83,192-308
//                                 fast_2d_gs/_C/include/gaussian_render.h:33-39 (getRect)
//   per-tile alpha blend fwd/bwd  fast_2d_gs/_C/src/gaussian_splatting/gs_2d_redner.cu:28-539
//   per-pixel top-k blend weights fast_2d_gs/_C/src/gaussian_splatting/gaussian_topk.cu:95-210
//
// Arithmetic is templated on the scalar type: the float instantiation is the parity oracle (built
// with -ffp-contract=off so every operation is a single IEEE rounding in source order), the double
// instantiation exists so the tests can pin the backward passes by central finite differences of the
// forward passes.
//
// What pins each function is listed in tests/ (test_oracle_*.py); nothing here is "parity unpinned".
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>

#include "gs2d_shared.h"

#ifdef _OPENMP
#include <omp.h>
#endif

namespace oracle {

template <typename T>
static inline void ndc2pix_mat(int W, int H, T* N) {  // gs_2d_preprocess.cu:48-49
  const T v[16] = {T(0.5 * W), T(0), T(0), T(0.5 * (W - 1)), T(0), T(0.5 * H), T(0), T(0.5 * (H - 1)),
                   T(0), T(0), T(0), T(1), T(0), T(0), T(0), T(1)};
  for (int i = 0; i < 16; ++i) N[i] = v[i];
}

// gs_2d_preprocess.cu:24-53. q = (x, y, z, w), used un-normalised.
template <typename T>
static inline void compute_transmat(int W, int H, const T* p, const T* s, const T* q, const T* Tw2c, const T* Tw2v,
                                    T* M, T* normal) {
  T L[16] = {0};
  const T x = q[0], y = q[1], z = q[2], w = q[3];
  L[0]  = (1 - 2 * (y * y + z * z)) * s[0];
  L[1]  = 2 * (x * y - z * w) * s[1];
  L[2]  = p[0];
  L[4]  = (2 * (x * y + z * w)) * s[0];
  L[5]  = (1 - 2 * (x * x + z * z)) * s[1];
  L[6]  = p[1];
  L[8]  = (2 * (x * z - y * w)) * s[0];
  L[9]  = 2 * (x * w + y * z) * s[1];
  L[10] = p[2];
  L[14] = 1;
  const T t0 = 2 * (y * w + x * z), t1 = 2 * (y * z - x * w), t2 = 1 - 2 * (x * x + y * y);
  T N[16], A[16], B[16];
  ndc2pix_mat(W, H, N);
  mat4_mul(Tw2c, L, A);
  mat4_mul(N, A, B);
  for (int i = 0; i < 3; ++i)
    for (int j = 0; j < 3; ++j) M[i * 3 + j] = B[i * 4 + j];
  normal[0] = Tw2v[0] * t0 + Tw2v[1] * t1 + Tw2v[2] * t2;  // xfm_v_4x3, ops_3d.h:229-236
  normal[1] = Tw2v[4] * t0 + Tw2v[5] * t1 + Tw2v[6] * t2;
  normal[2] = Tw2v[8] * t0 + Tw2v[9] * t1 + Tw2v[10] * t2;
}

// gs_2d_preprocess.cu:81-121. gM is the incoming 3x3 gradient; returns grads of p, s, q.
template <typename T>
static inline void compute_transmat_backward(int W, int H, const T* s, const T* q, const T* Tw2c, const T* Tw2v,
                                             const T* gM, const T* gN, T* gp, T* gs, T* gq) {
  T N[16], G[16] = {0}, GL[16] = {0}, dR[16] = {0};
  ndc2pix_mat(W, H, N);
  for (int i = 0; i < 3; ++i)
    for (int j = 0; j < 3; ++j) G[i * 4 + j] = gM[i * 3 + j];
  for (int i = 0; i < 4; ++i)  // matmul_tn, ops_3d.h:44-57 (accumulates k = 0..3 onto 0)
    for (int j = 0; j < 4; ++j)
      for (int k = 0; k < 4; ++k) GL[i * 4 + j] += N[k * 4 + i] * G[k * 4 + j];
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 4; ++j)
      for (int k = 0; k < 4; ++k) dR[i * 4 + j] += Tw2c[k * 4 + i] * GL[k * 4 + j];
  gp[0] = dR[2], gp[1] = dR[6], gp[2] = dR[10];
  dR[2]  = gN[0] * Tw2v[0] + gN[1] * Tw2v[4] + gN[2] * Tw2v[8];
  dR[6]  = gN[0] * Tw2v[1] + gN[1] * Tw2v[5] + gN[2] * Tw2v[9];
  dR[10] = gN[0] * Tw2v[2] + gN[1] * Tw2v[6] + gN[2] * Tw2v[10];
  const T x = q[0], y = q[1], z = q[2], w = q[3];
  gs[0] = dR[0] * (1 - 2 * (y * y + z * z)) + dR[4] * (2 * (x * y + z * w)) + dR[8] * (2 * (x * z - y * w));
  gs[1] = dR[1] * (2 * (x * y - z * w)) + dR[5] * (1 - 2 * (x * x + z * z)) + dR[9] * (2 * (x * w + y * z));
  dR[0] *= s[0], dR[1] *= s[1], dR[4] *= s[0], dR[5] *= s[1], dR[8] *= s[0], dR[9] *= s[1];
  gq[0] = 2 * (-2 * x * (dR[5] + dR[10]) + y * (dR[1] + dR[4]) + z * (dR[2] + dR[8]) + w * (dR[9] - dR[6]));
  gq[1] = 2 * (x * (dR[1] + dR[4]) - 2 * y * (dR[0] + dR[10]) + z * (dR[6] + dR[9]) + w * (dR[2] - dR[8]));
  gq[2] = 2 * (x * (dR[2] + dR[8]) + y * (dR[6] + dR[9]) - 2 * z * (dR[0] + dR[5]) + w * (dR[4] - dR[1]));
  gq[3] = 2 * (x * (dR[9] - dR[6]) + y * (dR[2] - dR[8]) + z * (dR[4] - dR[1]));
}

// ---------------------------------------------------------------------------------------------
// Preprocess forward: gs_2d_preprocess.cu:158-246 (kernel) and :331-421 (host: outputs start at 0,
// Tw2c = Tv2c @ Tw2v). Every output row is written here (0 for rejected surfels) except rows of a
// caller-supplied means2D buffer that belong to rejected surfels, which keep their content.
template <typename T>
static void preprocess_forward(int P, int W, int H, int sh_degree, int n_sh, const T* means3D, const T* scales,
                               const T* rotations, const T* opacities, const T* shs, const T* sh_rest,
                               const T* Tw2v, const T* Tv2c, const T* campos, const T* trans_precomp,
                               const uint8_t* culling, int means2D_preserve, T* means2D, T* colors, T* trans_mat,
                               T* normal_opacity, T* depths, int32_t* radii, int32_t* tiles_touched) {
  T Tw2c[16];
  mat4_mul(Tv2c, Tw2v, Tw2c);
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
#pragma omp parallel for schedule(static)
  for (int i = 0; i < P; ++i) {
    bool ok = true;
    T M[9] = {0}, nrm[3] = {0}, c2[2] = {0}, rgb[3] = {0}, depth = 0, radius = 0;
    int area = 0;
    do {
      ok = false;
      if (culling && culling[i]) break;
      const T* p = means3D + 3 * i;
      const T pv[3] = {Tw2v[0] * p[0] + Tw2v[1] * p[1] + Tw2v[2] * p[2] + Tw2v[3],
                       Tw2v[4] * p[0] + Tw2v[5] * p[1] + Tw2v[6] * p[2] + Tw2v[7],
                       Tw2v[8] * p[0] + Tw2v[9] * p[1] + Tw2v[10] * p[2] + Tw2v[11]};
      if (pv[2] <= T(0.2)) break;
      if (!trans_precomp) {
        compute_transmat(W, H, p, scales + 2 * i, rotations + 4 * i, Tw2c, Tw2v, M, nrm);
      } else {
        for (int k = 0; k < 9; ++k) M[k] = trans_precomp[9 * i + k];
        nrm[0] = 0, nrm[1] = 0, nrm[2] = 1;
      }
      const T cosv = -(pv[0] * nrm[0] + pv[1] * nrm[1] + pv[2] * nrm[2]);
      if (cosv == 0) break;
      const T mult = cosv > 0 ? T(1) : T(-1);
      for (int a = 0; a < 3; ++a) nrm[a] = mult * nrm[a];
      T ext[2];
      if (!compute_aabb(M, T(3.0), c2, ext)) break;
      radius = std::ceil(std::max(std::max(ext[0], ext[1]), T(3.0) * T(0.707106)));
      const Rect<T> r = get_rect<T>(c2[0], c2[1], f2i(radius), gx, gy);
      area = (r.y1 - r.y0) * (r.x1 - r.x0);
      if ((r.x1 - r.x0) * (r.y1 - r.y0) == 0) break;
      if (sh_degree >= 0)
        sh_to_rgb(sh_degree, p, campos, shs + (size_t) i * (sh_rest ? 1 : n_sh) * 3,
                  sh_rest ? sh_rest + (size_t) i * n_sh * 3 : nullptr, true, rgb);
      depth = pv[2];
      ok    = true;
    } while (false);
    if (ok) {
      if (!trans_precomp)
        for (int k = 0; k < 9; ++k) trans_mat[9 * i + k] = M[k];
      if (sh_degree >= 0)
        for (int c = 0; c < 3; ++c) colors[3 * i + c] = rgb[c];
      depths[i] = depth, radii[i] = f2i(radius), tiles_touched[i] = area;
      means2D[2 * i] = c2[0], means2D[2 * i + 1] = c2[1];
      for (int a = 0; a < 3; ++a) normal_opacity[4 * i + a] = nrm[a];
      normal_opacity[4 * i + 3] = opacities[i];
    } else {
      if (!trans_precomp)
        for (int k = 0; k < 9; ++k) trans_mat[9 * i + k] = 0;
      if (sh_degree >= 0)
        for (int c = 0; c < 3; ++c) colors[3 * i + c] = 0;
      depths[i] = 0, radii[i] = 0, tiles_touched[i] = 0;
      if (!means2D_preserve) means2D[2 * i] = 0, means2D[2 * i + 1] = 0;
      for (int a = 0; a < 4; ++a) normal_opacity[4 * i + a] = 0;
    }
  }
}

// Preprocess backward: gs_2d_preprocess.cu:268-329. Gradients of visible surfels are assigned into
// caller-zeroed buffers; grad_mean2D is overwritten in place with the densification proxy (:325-328).
template <typename T>
static void preprocess_backward(int P, int W, int H, int sh_degree, int n_sh, const T* means3D, const T* scales,
                                const T* rotations, const T* shs, const T* sh_rest, const T* Tw2v, const T* Tv2c,
                                const T* campos, const T* trans_mat, const int32_t* radii, const T* colors,
                                T* grad_mean2D, const T* grad_trans, const T* grad_colors,
                                const T* grad_normal_opacity, T* g_means3D, T* g_scales, T* g_rot, T* g_opac,
                                T* g_shs, T* g_sh_rest) {
  T Tw2c[16];
  mat4_mul(Tv2c, Tw2v, Tw2c);
#pragma omp parallel for schedule(static)
  for (int i = 0; i < P; ++i) {
    if (radii[i] <= 0) continue;
    g_opac[i] = grad_normal_opacity[4 * i + 3];
    T gM[9];
    for (int k = 0; k < 9; ++k) gM[k] = grad_trans[9 * i + k];
    compute_aabb_backward(T(3.0), trans_mat + 9 * i, grad_mean2D + 2 * i, gM);
    T gN[3] = {grad_normal_opacity[4 * i], grad_normal_opacity[4 * i + 1], grad_normal_opacity[4 * i + 2]};
    const T* q = rotations + 4 * i;
    const T* p = means3D + 3 * i;
    const T t0 = 2 * (q[1] * q[3] + q[0] * q[2]), t1 = 2 * (q[1] * q[2] - q[0] * q[3]),
            t2 = 1 - 2 * (q[0] * q[0] + q[1] * q[1]);
    const T nrm[3] = {Tw2v[0] * t0 + Tw2v[1] * t1 + Tw2v[2] * t2, Tw2v[4] * t0 + Tw2v[5] * t1 + Tw2v[6] * t2,
                      Tw2v[8] * t0 + Tw2v[9] * t1 + Tw2v[10] * t2};
    const T pv[3] = {Tw2v[0] * p[0] + Tw2v[1] * p[1] + Tw2v[2] * p[2] + Tw2v[3],
                     Tw2v[4] * p[0] + Tw2v[5] * p[1] + Tw2v[6] * p[2] + Tw2v[7],
                     Tw2v[8] * p[0] + Tw2v[9] * p[1] + Tw2v[10] * p[2] + Tw2v[11]};
    const T cosv = -(pv[0] * nrm[0] + pv[1] * nrm[1] + pv[2] * nrm[2]);
    const T mult = cosv > 0 ? T(1) : T(-1);
    for (int a = 0; a < 3; ++a) gN[a] = mult * gN[a];
    T gp[3], gs[2], gq[4];
    compute_transmat_backward(W, H, scales + 2 * i, q, Tw2c, Tw2v, gM, gN, gp, gs, gq);
    if (sh_degree >= 0) {
      T gdir[3];
      const int m1 = sh_rest ? 1 : n_sh;
      sh_to_rgb_backward(sh_degree, p, campos, colors + 3 * i, shs + (size_t) i * m1 * 3,
                         sh_rest ? sh_rest + (size_t) i * n_sh * 3 : nullptr, grad_colors + 3 * i,
                         g_shs ? g_shs + (size_t) i * m1 * 3 : nullptr,
                         g_sh_rest ? g_sh_rest + (size_t) i * n_sh * 3 : nullptr, true, true, gdir);
      for (int a = 0; a < 3; ++a) gp[a] = gp[a] + gdir[a];
    }
    for (int a = 0; a < 3; ++a) g_means3D[3 * i + a] = gp[a];
    g_scales[2 * i] = gs[0], g_scales[2 * i + 1] = gs[1];
    for (int a = 0; a < 4; ++a) g_rot[4 * i + a] = gq[a];
    const T depth = trans_mat[9 * i + 8];
    grad_mean2D[2 * i]     = grad_trans[9 * i + 2] * depth * T(0.5) * T(W);
    grad_mean2D[2 * i + 1] = grad_trans[9 * i + 5] * depth * T(0.5) * T(H);
  }
}

// ---------------------------------------------------------------------------------------------
// Binning: gaussian_prepare.cu:222-308. Float only (keys carry the float bit pattern of the depth).
static int64_t prepare_count(int P, const int32_t* tiles_touched, int64_t* offsets) {
  int64_t run = 0;
  for (int i = 0; i < P; ++i) run += tiles_touched[i], offsets[i] = run;
  return P > 0 ? offsets[P - 1] : 0;
}

static void prepare_fill(int P, int W, int H, const float* means2D, const float* depths, const int32_t* radii,
                         const int64_t* offsets, int64_t R, int64_t* ranges, int32_t* point_list,
                         int64_t* keys_sorted_out) {
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  std::vector<uint64_t> keys((size_t) R);
  std::vector<int32_t> vals((size_t) R);
  for (int i = 0; i < P; ++i) {  // duplicateWithKeys, gaussian_prepare.cu:47-83
    if (radii[i] <= 0) continue;
    int64_t off = i == 0 ? 0 : offsets[i - 1];
    const Rect<float> r = get_rect<float>(means2D[2 * i], means2D[2 * i + 1], radii[i], gx, gy);
    uint32_t bits;
    std::memcpy(&bits, depths + i, 4);
    for (int y = r.y0; y < r.y1; ++y)
      for (int x = r.x0; x < r.x1; ++x) {
        keys[(size_t) off] = ((uint64_t) (uint32_t) (y * gx + x) << 32) | bits;
        vals[(size_t) off] = i;
        ++off;
      }
  }
  // Stable ascending sort restricted to bits [0, 32 + msb(T)) as cub::DeviceRadixSort::SortPairs does.
  const uint32_t bit  = 32 + higher_msb((uint32_t) (gx * gy));
  const uint64_t mask = bit >= 64 ? ~0ull : ((1ull << bit) - 1);
  std::vector<int64_t> order((size_t) R);
  for (int64_t i = 0; i < R; ++i) order[(size_t) i] = i;
  std::stable_sort(order.begin(), order.end(),
                   [&](int64_t a, int64_t b) { return (keys[(size_t) a] & mask) < (keys[(size_t) b] & mask); });
  for (int64_t i = 0; i < (int64_t) gx * gy * 2; ++i) ranges[i] = 0;
  for (int64_t i = 0; i < R; ++i) {  // identifyTileRanges, gaussian_prepare.cu:192-220
    const uint64_t k = keys[(size_t) order[(size_t) i]];
    point_list[i]    = vals[(size_t) order[(size_t) i]];
    if (keys_sorted_out) keys_sorted_out[i] = (int64_t) k;
    const uint32_t cur = (uint32_t) (k >> 32);
    if (i == 0) ranges[2 * cur] = 0;
    else {
      const uint32_t prev = (uint32_t) (keys[(size_t) order[(size_t) i - 1]] >> 32);
      if (cur != prev) ranges[2 * prev + 1] = i, ranges[2 * cur] = i;
    }
    if (i == R - 1) ranges[2 * cur + 1] = R;
  }
}

// ---------------------------------------------------------------------------------------------
// Blend forward: gs_2d_redner.cu:28-236. One pixel at a time over its tile list in sorted order.
template <typename T>
static void render_forward(int P, int W, int H, T near_n, T far_n, int only_image, const T* means2D,
                           const T* colors, const T* normal_opacity, const T* trans_mat, const int32_t* point_list,
                           const int64_t* ranges, const T* trans_mat_t2, int32_t* accum_max_count,
                           T* accum_weights_p, int32_t* accum_weights_count, T* out_color, T* out_opacity,
                           T* out_extras, T* out_flow, int32_t* n_contrib) {
  (void) P;
  const int gx = (W + kTile - 1) / kTile;
  const size_t HW = (size_t) H * W;
  const bool aux = !only_image;
  // accum_* are racy integer/float atomics in the reference; the oracle serialises pixels when they
  // are requested so that integer results are deterministic.
  const bool serial = accum_max_count || accum_weights_p || accum_weights_count;
#pragma omp parallel for schedule(dynamic, 8) if (!serial)
  for (int py = 0; py < H; ++py)
    for (int px = 0; px < W; ++px) {
      const size_t pix = (size_t) W * py + px;
      const int tile   = (py / kTile) * gx + (px / kTile);
      const int64_t r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
      const T pxf = (T) px, pyf = (T) py;
      T t = 1, C[3] = {0}, N[3] = {0}, D = 0, M1 = 0, M2 = 0, dist = 0, med = 0, wsum = 0, fl[2] = {0};
      uint32_t contributor = 0, last = 0;
      int32_t med_c = -1, wmax_id = -1;
      T wmax = 0;
      bool flag = false;
      for (int64_t e = r0; e < r1; ++e) {
        contributor++;
        const int id = point_list[e];
        const T* Mx  = trans_mat + 9 * (size_t) id;
        const T k[3] = {pxf * Mx[6] - Mx[0], pxf * Mx[7] - Mx[1], pxf * Mx[8] - Mx[2]};
        const T l[3] = {pyf * Mx[6] - Mx[3], pyf * Mx[7] - Mx[4], pyf * Mx[8] - Mx[5]};
        const T p[3] = {k[1] * l[2] - k[2] * l[1], k[2] * l[0] - k[0] * l[2], k[0] * l[1] - k[1] * l[0]};
        if (p[2] == 0.0) continue;
        const T s[2]  = {p[0] / p[2], p[1] / p[2]};
        const T rho3d = s[0] * s[0] + s[1] * s[1];
        const T d[2]  = {means2D[2 * id] - pxf, means2D[2 * id + 1] - pyf};
        const T rho2d = T(2.0) * (d[0] * d[0] + d[1] * d[1]);
        const T rho   = std::min(rho3d, rho2d);
        const T depth = (s[0] * Mx[6] + s[1] * Mx[7]) + Mx[8];
        if (depth < near_n) continue;
        const T* no   = normal_opacity + 4 * (size_t) id;
        const T power = -T(0.5) * rho;
        if (power > T(0.0)) continue;
        const T alpha = std::min(T(0.99), no[3] * std::exp(power));
        if (alpha < T(1.0 / 255.0)) continue;
        const T test_T = t * (1 - alpha);
        if (test_T < T(0.0001)) break;  // done = true
        const T w = alpha * t;
        if (aux) {
          const T A = 1 - t;
          const T m = far_n / (far_n - near_n) * (1 - near_n / depth);
          dist += (m * m * A + M2 - 2 * m * M1) * w;
          D += depth * w;
          M1 += m * w;
          M2 += m * m * w;
          if (t > 0.5) med = depth, med_c = (int32_t) contributor;
          for (int c = 0; c < 3; ++c) N[c] += no[c] * w;
          if (wmax < w) wmax = w, wmax_id = id, flag = true;
          if (accum_weights_p) accum_weights_p[id] += w;
          if (accum_weights_count) accum_weights_count[id] += 1;
          if (trans_mat_t2) {
            const T* Q = trans_mat_t2 + 9 * (size_t) id;
            const T u2 = Q[0] * s[0] + Q[1] * s[1] + Q[2];
            const T v2 = Q[3] * s[0] + Q[4] * s[1] + Q[5];
            T w2       = Q[6] * s[0] + Q[7] * s[1] + Q[8];
            w2         = std::abs(w2) < T(1e-5) ? T(1e-5) : w2;
            fl[0] += (u2 / w2 - pxf) * w;
            fl[1] += (v2 / w2 - pyf) * w;
          }
          wsum += w;
        }
        if (flag && accum_max_count) accum_max_count[wmax_id] += 1;  // flag is never reset, :180-197
        for (int c = 0; c < 3; ++c) C[c] += colors[3 * (size_t) id + c] * w;
        t    = test_T;
        last = contributor;
      }
      out_opacity[pix] = T(1) - t;
      n_contrib[pix]   = (int32_t) last;
      for (int c = 0; c < 3; ++c) out_color[c * HW + pix] = C[c];
      n_contrib[pix + HW] = aux ? med_c : 0;
      if (aux) {
        out_extras[pix + HW * 0] = D;
        for (int c = 0; c < 3; ++c) out_extras[pix + HW * (1 + c)] = N[c];
        out_extras[pix + HW * 4] = med;
        out_extras[pix + HW * 5] = dist;
        out_extras[pix + HW * 6] = M1;
        out_extras[pix + HW * 7] = M2;
        out_extras[pix + HW * 8] = wsum;
        if (out_flow) {
          const T ws        = wsum == 0 ? T(1e-7) : wsum;
          out_flow[2 * pix] = fl[0] / ws, out_flow[2 * pix + 1] = fl[1] / ws;
        }
      }
    }
}

// Blend backward: gs_2d_redner.cu:238-539. Back-to-front per pixel; per-surfel gradients are summed
// into caller-zeroed buffers. Tiles are processed in parallel with per-thread private accumulators
// when OpenMP is on, so summation order differs from both the reference and the GPU (atomics).
template <typename T>
static void render_backward(int P, int W, int H, T near_n, T far_n, const T* means2D, const T* normal_opacity,
                            const T* colors, const T* trans_mat, const T* trans_mat_t2, const T* out_opacity,
                            const T* out_extras, const T* out_flow, const T* dL_dpix, const T* dL_dopacity,
                            const T* dL_dextras, const T* dL_dflow, const int64_t* ranges,
                            const int32_t* point_list, const int32_t* n_contrib, T* g_colors, T* g_means2D,
                            T* g_trans, T* g_normal_opacity) {
  const int gx = (W + kTile - 1) / kTile;
  const size_t HW = (size_t) H * W;
  const bool aux  = out_extras && dL_dextras;
  (void) P;
#pragma omp parallel
  {
    std::vector<T> acc;  // private accumulators: [P][18] = colors 3, means2D 2, trans 9, normal_opacity 4
#ifdef _OPENMP
    const bool priv = omp_get_num_threads() > 1;
#else
    const bool priv = false;
#endif
    if (priv) acc.assign((size_t) P * 18, T(0));
    auto add = [&](int id, int slot, T v) {
      if (priv) acc[(size_t) id * 18 + slot] += v;
      else if (slot < 3) g_colors[3 * (size_t) id + slot] += v;
      else if (slot < 5) g_means2D[2 * (size_t) id + slot - 3] += v;
      else if (slot < 14) g_trans[9 * (size_t) id + slot - 5] += v;
      else g_normal_opacity[4 * (size_t) id + slot - 14] += v;
    };
#pragma omp for schedule(dynamic, 8)
    for (int py = 0; py < H; ++py)
      for (int px = 0; px < W; ++px) {
        const size_t pix = (size_t) W * py + px;
        const int tile   = (py / kTile) * gx + (px / kTile);
        const int64_t r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
        const T pxf = (T) px, pyf = (T) py;
        const T t_final = 1 - out_opacity[pix];
        T t = t_final;
        uint32_t contributor = (uint32_t) (r1 - r0);
        const int last_contributor = n_contrib[pix];
        const int median_contributor = aux ? n_contrib[pix + HW] : 0;
        T accum_rec[3] = {0}, dLp[3], last_color[3] = {0};
        for (int c = 0; c < 3; ++c) dLp[c] = dL_dpix[c * HW + pix];
        T dL_dreg = 0, dL_ddepth = 0, dL_daccum = 0, dL_dn[3] = {0}, dL_dmedian = 0;
        if (aux) {
          dL_daccum = dL_dopacity[pix];
          dL_ddepth = dL_dextras[0 * HW + pix];
          dL_dreg   = dL_dextras[5 * HW + pix];
          for (int c = 0; c < 3; ++c) dL_dn[c] = dL_dextras[(1 + c) * HW + pix];
          dL_dmedian = dL_dextras[4 * HW + pix];
        }
        T last_depth = 0, last_normal[3] = {0}, acc_depth = 0, acc_alpha = 0, acc_normal[3] = {0};
        const T final_D  = aux ? out_extras[pix + 6 * HW] : T(0);
        const T final_D2 = aux ? out_extras[pix + 7 * HW] : T(0);
        const T final_A  = 1 - t_final;
        T last_dL_dT     = 0;
        const T sum_w    = aux ? out_extras[pix + 8 * HW] : T(0);
        T acc_flow[2] = {0}, last_flow[2] = {0}, dLf[2] = {0};
        T dL_dsum_w = 0, acc_w = 0;
        if (dL_dflow) {
          dLf[0] = dL_dflow[2 * pix], dLf[1] = dL_dflow[2 * pix + 1];
          dL_dsum_w = -(dLf[0] * out_flow[2 * pix] + dLf[1] * out_flow[2 * pix + 1]) / (sum_w * sum_w);
          dLf[0] = dLf[0] / sum_w, dLf[1] = dLf[1] / sum_w;
        }
        T last_alpha = 0;
        for (int64_t e = r1 - 1; e >= r0; --e) {
          contributor--;
          if ((int64_t) contributor >= (int64_t) last_contributor) continue;
          const int id = point_list[e];
          const T* Mx  = trans_mat + 9 * (size_t) id;
          const T k[3] = {pxf * Mx[6] - Mx[0], pxf * Mx[7] - Mx[1], pxf * Mx[8] - Mx[2]};
          const T l[3] = {pyf * Mx[6] - Mx[3], pyf * Mx[7] - Mx[4], pyf * Mx[8] - Mx[5]};
          const T p[3] = {k[1] * l[2] - k[2] * l[1], k[2] * l[0] - k[0] * l[2], k[0] * l[1] - k[1] * l[0]};
          if (p[2] == 0.0) continue;
          const T s[2]  = {p[0] / p[2], p[1] / p[2]};
          const T rho3d = s[0] * s[0] + s[1] * s[1];
          const T d[2]  = {means2D[2 * id] - pxf, means2D[2 * id + 1] - pyf};
          const T rho2d = T(2.0) * (d[0] * d[0] + d[1] * d[1]);
          const T rho   = std::min(rho3d, rho2d);
          const T c_d   = (s[0] * Mx[6] + s[1] * Mx[7]) + Mx[8];
          if (c_d < near_n) continue;
          const T* no   = normal_opacity + 4 * (size_t) id;
          const T power = -T(0.5) * rho;
          if (power > T(0.0)) continue;
          const T G     = std::exp(power);
          const T alpha = std::min(T(0.99), no[3] * G);
          if (alpha < T(1.0 / 255.0)) continue;
          t         = t / (T(1.) - alpha);
          const T w = alpha * t;
          T dL_dalpha = 0;
          for (int c = 0; c < 3; ++c) {
            const T col   = colors[3 * (size_t) id + c];
            accum_rec[c]  = last_alpha * last_color[c] + (T(1.) - last_alpha) * accum_rec[c];
            last_color[c] = col;
            dL_dalpha += (col - accum_rec[c]) * dLp[c];
            add(id, c, w * dLp[c]);
          }
          T dL_dz = 0, dL_dweight = 0, dL_ds[2] = {0, 0};
          if (aux) {
            const T m_d    = far_n / (far_n - near_n) * (1 - near_n / c_d);
            const T dmd_dd = (far_n * near_n) / ((far_n - near_n) * c_d * c_d);
            if ((int64_t) contributor == (int64_t) median_contributor - 1) dL_dz += dL_dmedian;
            dL_dweight += (final_D2 + m_d * m_d * final_A - 2 * m_d * final_D) * dL_dreg;
            dL_dalpha += dL_dweight - last_dL_dT;
            last_dL_dT     = dL_dweight * alpha + (1 - alpha) * last_dL_dT;
            const T dL_dmd = T(2.0) * (t * alpha) * (m_d * final_A - final_D) * dL_dreg;
            dL_dz += dL_dmd * dmd_dd;
            acc_depth  = last_alpha * last_depth + (T(1.) - last_alpha) * acc_depth;
            last_depth = c_d;
            dL_dalpha += (c_d - acc_depth) * dL_ddepth;
            acc_alpha = last_alpha * T(1.0) + (T(1.) - last_alpha) * acc_alpha;
            dL_dalpha += (1 - acc_alpha) * dL_daccum;
            for (int c = 0; c < 3; ++c) {
              acc_normal[c]  = last_alpha * last_normal[c] + (T(1.) - last_alpha) * acc_normal[c];
              last_normal[c] = no[c];
              dL_dalpha += (no[c] - acc_normal[c]) * dL_dn[c];
              add(id, 14 + c, alpha * t * dL_dn[c]);
            }
            dL_dz += alpha * t * dL_ddepth;
            dL_ds[0] = dL_dz * Mx[6], dL_ds[1] = dL_dz * Mx[7];
          }
          if (dL_dflow) {
            const T* Q = trans_mat_t2 + 9 * (size_t) id;
            const T u2 = Q[0] * s[0] + Q[1] * s[1] + Q[2];
            const T v2 = Q[3] * s[0] + Q[4] * s[1] + Q[5];
            T w2       = Q[6] * s[0] + Q[7] * s[1] + Q[8];
            w2         = std::abs(w2) < T(1e-5) ? T(1e-5) : w2;
            acc_flow[0] = last_alpha * last_flow[0] + (T(1.) - last_alpha) * acc_flow[0];
            acc_flow[1] = last_alpha * last_flow[1] + (T(1.) - last_alpha) * acc_flow[1];
            last_flow[0] = u2 / w2 - pxf, last_flow[1] = v2 / w2 - pyf;
            dL_dalpha += (last_flow[0] - acc_flow[0]) * dLf[0] + (last_flow[1] - acc_flow[1]) * dLf[1];
            const T gu = w / w2 * dLf[0], gv = w / w2 * dLf[1];
            const T gw = -w / (w2 * w2) * (u2 * dLf[0] + v2 * dLf[1]);
            dL_ds[0] += Q[0] * gu + Q[3] * gv + Q[6] * gw;
            dL_ds[1] += Q[1] * gu + Q[4] * gv + Q[7] * gw;
          }
          acc_w = last_alpha + (T(1.0) - last_alpha) * acc_w;
          dL_dalpha += (T(1) - acc_w) * dL_dsum_w;
          dL_dalpha *= t;
          last_alpha  = alpha;
          const T dL_dG = no[3] * dL_dalpha;
          if (rho3d <= rho2d) {
            dL_ds[0] = dL_ds[0] + dL_dG * -G * s[0];
            dL_ds[1] = dL_ds[1] + dL_dG * -G * s[1];
            const T dsx = dL_ds[0] / p[2], dsy = dL_ds[1] / p[2];
            const T dp[3] = {dsx, dsy, -(dsx * s[0] + dsy * s[1])};
            const T dk[3] = {l[1] * dp[2] - l[2] * dp[1], l[2] * dp[0] - l[0] * dp[2], l[0] * dp[1] - l[1] * dp[0]};
            const T dl[3] = {dp[1] * k[2] - dp[2] * k[1], dp[2] * k[0] - dp[0] * k[2], dp[0] * k[1] - dp[1] * k[0]};
            const T dz_dTw[3] = {s[0], s[1], T(1.0)};
            for (int a = 0; a < 3; ++a) {
              add(id, 5 + a, -dk[a]);
              add(id, 8 + a, -dl[a]);
              add(id, 11 + a, pxf * dk[a] + pyf * dl[a] + dL_dz * dz_dTw[a]);
            }
          } else {
            const T dG_dx = -G * T(2.0) * d[0], dG_dy = -G * T(2.0) * d[1];
            add(id, 3, dL_dG * dG_dx);
            add(id, 4, dL_dG * dG_dy);
            add(id, 11, dL_dz * s[0]);
            add(id, 12, dL_dz * s[1]);
            add(id, 13, dL_dz);
          }
          add(id, 17, G * dL_dalpha);
        }
      }
    if (priv) {
#pragma omp critical
      for (int i = 0; i < P; ++i) {
        const T* a = acc.data() + (size_t) i * 18;
        for (int c = 0; c < 3; ++c) g_colors[3 * (size_t) i + c] += a[c];
        for (int c = 0; c < 2; ++c) g_means2D[2 * (size_t) i + c] += a[3 + c];
        for (int c = 0; c < 9; ++c) g_trans[9 * (size_t) i + c] += a[5 + c];
        for (int c = 0; c < 4; ++c) g_normal_opacity[4 * (size_t) i + c] += a[14 + c];
      }
    }
  }
}

// Per-pixel top-k blend weights: gaussian_topk.cu:95-210. Uses the older depth rule for the near test.
template <typename T>
static void topk_weights(int topk, int W, int H, T near_n, T far_n, const T* means2D, const T* normal_opacity,
                         const T* trans_mat, const int64_t* ranges, const int32_t* point_list, int32_t* top_idx,
                         T* top_w) {
  (void) far_n;
  const int gx = (W + kTile - 1) / kTile;
#pragma omp parallel for schedule(dynamic, 8)
  for (int py = 0; py < H; ++py)
    for (int px = 0; px < W; ++px) {
      const size_t pix = (size_t) W * py + px;
      int32_t* ti = top_idx + pix * topk;
      T* tw       = top_w + pix * topk;
      for (int k = 0; k < topk; ++k) ti[k] = -1, tw[k] = 0;
      const int tile   = (py / kTile) * gx + (px / kTile);
      const int64_t r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
      const T pxf = (T) px, pyf = (T) py;
      T t = 1;
      for (int64_t e = r0; e < r1; ++e) {
        const int id = point_list[e];
        const T* Mx  = trans_mat + 9 * (size_t) id;
        const T k[3] = {pxf * Mx[6] - Mx[0], pxf * Mx[7] - Mx[1], pxf * Mx[8] - Mx[2]};
        const T l[3] = {pyf * Mx[6] - Mx[3], pyf * Mx[7] - Mx[4], pyf * Mx[8] - Mx[5]};
        const T p[3] = {k[1] * l[2] - k[2] * l[1], k[2] * l[0] - k[0] * l[2], k[0] * l[1] - k[1] * l[0]};
        if (p[2] == 0.0) continue;
        const T s[2]  = {p[0] / p[2], p[1] / p[2]};
        const T rho3d = s[0] * s[0] + s[1] * s[1];
        const T d[2]  = {means2D[2 * id] - pxf, means2D[2 * id + 1] - pyf};
        const T rho2d = T(2.0) * (d[0] * d[0] + d[1] * d[1]);
        const T rho   = std::min(rho3d, rho2d);
        const T depth = (rho3d <= rho2d) ? (s[0] * Mx[6] + s[1] * Mx[7]) + Mx[8] : Mx[8];
        if (depth < near_n) continue;
        const T power = -T(0.5) * rho;
        if (power > T(0.0)) continue;
        const T alpha = std::min(T(0.99), normal_opacity[4 * (size_t) id + 3] * std::exp(power));
        if (alpha < T(1.0 / 255.0)) continue;
        const T test_T = t * (1 - alpha);
        if (test_T < T(0.0001)) break;
        const T w = alpha * t;
        // insertion, gaussian_topk.cu (ties: a later splat with w >= slot takes the slot)
        T cw = w;
        int32_t ci = id;
        for (int q = 0; q < topk; ++q) {
          if (cw >= tw[q]) {
            std::swap(cw, tw[q]);
            std::swap(ci, ti[q]);
          }
        }
        t = test_T;
      }
    }
}

}  // namespace oracle

using namespace oracle;

#define ORACLE_API extern "C" __attribute__((visibility("default")))

#define INSTANTIATE(SUF, T)                                                                                       \
  ORACLE_API int oracle_gs_2d_preprocess_forward_##SUF(                                                           \
      int P, int W, int H, int sh_degree, int n_sh, const T* means3D, const T* scales, const T* rotations,        \
      const T* opacities, const T* shs, const T* sh_rest, const T* Tw2v, const T* Tv2c, const T* campos,          \
      const T* trans_precomp, const uint8_t* culling, int means2D_preserve, T* means2D, T* colors, T* trans_mat,  \
      T* normal_opacity, T* depths, int32_t* radii, int32_t* tiles_touched) {                                     \
    if (sh_degree > kMaxShDegree) return 1;                                                                       \
    preprocess_forward<T>(P, W, H, sh_degree, n_sh, means3D, scales, rotations, opacities, shs, sh_rest, Tw2v,    \
                          Tv2c, campos, trans_precomp, culling, means2D_preserve, means2D, colors, trans_mat,     \
                          normal_opacity, depths, radii, tiles_touched);                                          \
    return 0;                                                                                                     \
  }                                                                                                               \
  ORACLE_API int oracle_gs_2d_preprocess_backward_##SUF(                                                          \
      int P, int W, int H, int sh_degree, int n_sh, const T* means3D, const T* scales, const T* rotations,        \
      const T* shs, const T* sh_rest, const T* Tw2v, const T* Tv2c, const T* campos, const T* trans_mat,          \
      const int32_t* radii, const T* colors, T* grad_mean2D, const T* grad_trans, const T* grad_colors,           \
      const T* grad_normal_opacity, T* g_means3D, T* g_scales, T* g_rot, T* g_opac, T* g_shs, T* g_sh_rest) {     \
    if (sh_degree > kMaxShDegree) return 1;                                                                       \
    preprocess_backward<T>(P, W, H, sh_degree, n_sh, means3D, scales, rotations, shs, sh_rest, Tw2v, Tv2c,        \
                           campos, trans_mat, radii, colors, grad_mean2D, grad_trans, grad_colors,                \
                           grad_normal_opacity, g_means3D, g_scales, g_rot, g_opac, g_shs, g_sh_rest);            \
    return 0;                                                                                                     \
  }                                                                                                               \
  ORACLE_API int oracle_gs_2d_compute_transmat_forward_##SUF(int P, int W, int H, const T* means3D,               \
      const T* scales, const T* rotations, const T* Tw2v, const T* Tw2c, T* trans_mat, T* normals) {              \
    for (int i = 0; i < P; ++i)                                                                                   \
      compute_transmat<T>(W, H, means3D + 3 * i, scales + 2 * i, rotations + 4 * i, Tw2c, Tw2v,                   \
                          trans_mat + 9 * i, normals + 3 * i);                                                    \
    return 0;                                                                                                     \
  }                                                                                                               \
  ORACLE_API int oracle_gs_2d_compute_transmat_backward_##SUF(int P, int W, int H, const T* means3D,              \
      const T* scales, const T* rotations, const T* Tw2v, const T* Tw2c, const T* g_mat, const T* g_normals,      \
      T* g_means3D, T* g_scales, T* g_rot) {                                                                      \
    (void) means3D;                                                                                               \
    for (int i = 0; i < P; ++i)                                                                                   \
      compute_transmat_backward<T>(W, H, scales + 2 * i, rotations + 4 * i, Tw2c, Tw2v, g_mat + 9 * i,            \
                                   g_normals + 3 * i, g_means3D + 3 * i, g_scales + 2 * i, g_rot + 4 * i);        \
    return 0;                                                                                                     \
  }                                                                                                               \
  ORACLE_API int oracle_gs_2d_render_forward_##SUF(                                                               \
      int P, int W, int H, double near_n, double far_n, int only_image, const T* means2D, const T* colors,        \
      const T* normal_opacity, const T* trans_mat, const int32_t* point_list, const int64_t* ranges,              \
      const T* trans_mat_t2, int32_t* accum_max_count, T* accum_weights_p, int32_t* accum_weights_count,          \
      T* out_color, T* out_opacity, T* out_extras, T* out_flow, int32_t* n_contrib) {                             \
    render_forward<T>(P, W, H, (T) near_n, (T) far_n, only_image, means2D, colors, normal_opacity, trans_mat,     \
                      point_list, ranges, trans_mat_t2, accum_max_count, accum_weights_p, accum_weights_count,    \
                      out_color, out_opacity, out_extras, out_flow, n_contrib);                                   \
    return 0;                                                                                                     \
  }                                                                                                               \
  ORACLE_API int oracle_gs_2d_render_backward_##SUF(                                                              \
      int P, int W, int H, double near_n, double far_n, const T* means2D, const T* normal_opacity,                \
      const T* colors, const T* trans_mat, const T* trans_mat_t2, const T* out_opacity, const T* out_extras,      \
      const T* out_flow, const T* dL_dpix, const T* dL_dopacity, const T* dL_dextras, const T* dL_dflow,          \
      const int64_t* ranges, const int32_t* point_list, const int32_t* n_contrib, T* g_colors, T* g_means2D,      \
      T* g_trans, T* g_normal_opacity) {                                                                          \
    render_backward<T>(P, W, H, (T) near_n, (T) far_n, means2D, normal_opacity, colors, trans_mat, trans_mat_t2,  \
                       out_opacity, out_extras, out_flow, dL_dpix, dL_dopacity, dL_dextras, dL_dflow, ranges,     \
                       point_list, n_contrib, g_colors, g_means2D, g_trans, g_normal_opacity);                    \
    return 0;                                                                                                     \
  }                                                                                                               \
  ORACLE_API int oracle_gs_2d_topk_weights_##SUF(int topk, int W, int H, double near_n, double far_n,             \
      const T* means2D, const T* normal_opacity, const T* trans_mat, const int64_t* ranges,                       \
      const int32_t* point_list, int32_t* top_idx, T* top_w) {                                                    \
    topk_weights<T>(topk, W, H, (T) near_n, (T) far_n, means2D, normal_opacity, trans_mat, ranges, point_list,    \
                    top_idx, top_w);                                                                              \
    return 0;                                                                                                     \
  }

INSTANTIATE(f32, float)
INSTANTIATE(f64, double)

ORACLE_API int64_t oracle_gs_prepare_count(int P, const int32_t* tiles_touched, int64_t* offsets) {
  return prepare_count(P, tiles_touched, offsets);
}

ORACLE_API int oracle_gs_prepare_fill(int P, int W, int H, const float* means2D, const float* depths,
                                      const int32_t* radii, const int64_t* offsets, int64_t R, int64_t* ranges,
                                      int32_t* point_list, int64_t* keys_sorted_out) {
  prepare_fill(P, W, H, means2D, depths, radii, offsets, R, ranges, point_list, keys_sorted_out);
  return 0;
}

ORACLE_API uint32_t oracle_higher_msb(uint32_t n) { return higher_msb(n); }

ORACLE_API int oracle_num_threads() {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
