// TEST INFRASTRUCTURE ONLY (parity oracle; never linked into or called by the product library).
// CPU restatement of the reference's 3D-Gaussian (EWA) path:
//   preprocess forward / backward   fast_2d_gs/_C/src/gaussian_splatting/gaussian_preprocess.cu:44-128, :246-372
//   3D covariance forward/backward  gaussian_compute_cov3D.cu:18-36, :76-118
//   2D covariance forward/backward  gaussian_compute_cov2D.cu:18-62, :64-186
//   rasterise forward / backward    gaussian_render.cu:20-173, :296-444
//   feature-channel blend fwd/bwd   gaussian_rasterizer_extra.cu:12-101, :103-209
//   bucket snapshots + per-Gaussian backward  gaussian_render.cu:51-63, :100-106, :540-812
// Pre-computed 3D / 2D covariances and the camera gradients (dL/dTw2v rows 0-2, dL/dcampos) included.
//
// Pinned by tests/test_oracle_gs3d.py: cov3D = R S^2 R^T and cov2D = J W cov3D W^T J^T + 0.3 I with numpy, the conic as
// a matrix inverse, a single-Gaussian closed form for the image, an independent numpy compositor, and central finite
// differences (fp64) of the oracle forward for both backward passes.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <limits>
#include <vector>

#include "gs2d_shared.h"

#define ORACLE_API extern "C" __attribute__((visibility("default")))

namespace oracle {
namespace {

// quaternion (x, y, z, w) -> rotation matrix, no normalisation inside: ops_3d.h:101-124
template <typename T>
inline void quat_to_R(const T* q, T* R) {
  R[0] = 1 - 2 * (q[1] * q[1] + q[2] * q[2]);
  R[1] = 2 * (q[0] * q[1] - q[2] * q[3]);
  R[2] = 2 * (q[1] * q[3] + q[0] * q[2]);
  R[3] = 2 * (q[0] * q[1] + q[2] * q[3]);
  R[4] = 1 - 2 * (q[0] * q[0] + q[2] * q[2]);
  R[5] = 2 * (q[1] * q[2] - q[0] * q[3]);
  R[6] = 2 * (q[0] * q[2] - q[1] * q[3]);
  R[7] = 2 * (q[0] * q[3] + q[1] * q[2]);
  R[8] = 1 - 2 * (q[0] * q[0] + q[1] * q[1]);
}

// ops_3d.h:137-142
template <typename T>
inline void dL_quat_to_R(const T* q, const T* dR, T* dq) {
  dq[0] = 2 * (-2 * q[0] * (dR[4] + dR[8]) + q[1] * (dR[1] + dR[3]) + q[2] * (dR[2] + dR[6]) + q[3] * (dR[7] - dR[5]));
  dq[1] = 2 * (q[0] * (dR[1] + dR[3]) - 2 * q[1] * (dR[0] + dR[8]) + q[2] * (dR[5] + dR[7]) + q[3] * (dR[2] - dR[6]));
  dq[2] = 2 * (q[0] * (dR[2] + dR[6]) + q[1] * (dR[5] + dR[7]) - 2 * q[2] * (dR[0] + dR[4]) + q[3] * (dR[3] - dR[1]));
  dq[3] = 2 * (q[0] * (dR[7] - dR[5]) + q[1] * (dR[2] - dR[6]) + q[2] * (dR[3] - dR[1]));
}

// gaussian_compute_cov3D.cu:18-36: upper triangle of R diag(s^2) R^T
template <typename T>
inline void cov3d_forward(const T* s, const T* q, T* c) {
  T R[9];
  quat_to_R(q, R);
  const T sx2 = s[0] * s[0], sy2 = s[1] * s[1], sz2 = s[2] * s[2];
  c[0] = R[0] * R[0] * sx2 + R[1] * R[1] * sy2 + R[2] * R[2] * sz2;
  c[1] = R[0] * R[3] * sx2 + R[1] * R[4] * sy2 + R[2] * R[5] * sz2;
  c[2] = R[0] * R[6] * sx2 + R[1] * R[7] * sy2 + R[2] * R[8] * sz2;
  c[3] = R[3] * R[3] * sx2 + R[4] * R[4] * sy2 + R[5] * R[5] * sz2;
  c[4] = R[3] * R[6] * sx2 + R[4] * R[7] * sy2 + R[5] * R[8] * sz2;
  c[5] = R[6] * R[6] * sx2 + R[7] * R[7] * sy2 + R[8] * R[8] * sz2;
}

// gaussian_compute_cov3D.cu:76-118
template <typename T>
inline void cov3d_backward(const T* s, const T* q, const T* g, T* gs, T* gq) {
  T R[9];
  quat_to_R(q, R);
  for (int a = 0; a < 3; ++a) {
    const T v = R[a] * R[a] * g[0] + R[a] * R[3 + a] * g[1] + R[a] * R[6 + a] * g[2] + R[3 + a] * R[3 + a] * g[3] +
                R[3 + a] * R[6 + a] * g[4] + R[6 + a] * R[6 + a] * g[5];
    gs[a] = v * 2 * s[a];
  }
  const T s2[3] = {s[0] * s[0], s[1] * s[1], s[2] * s[2]};
  T dR[9];
  for (int a = 0; a < 3; ++a) {
    dR[a]     = (2 * R[a] * g[0] + R[3 + a] * g[1] + R[6 + a] * g[2]) * s2[a];
    dR[3 + a] = (2 * R[3 + a] * g[3] + R[a] * g[1] + R[6 + a] * g[4]) * s2[a];
    dR[6 + a] = (2 * R[6 + a] * g[5] + R[a] * g[2] + R[3 + a] * g[4]) * s2[a];
  }
  dL_quat_to_R(q, dR, gq);
}

template <typename T>
struct Cov2DTerms {
  T t[3], J[6], M[6], x_mul, y_mul;
};

// Shared front of computeCov2D / computeCov2DBackward (gaussian_compute_cov2D.cu:22-47, :71-87).
template <typename T>
inline void cov2d_terms(const T* mean, T fx, T fy, T tanx, T tany, const T* V, Cov2DTerms<T>& o) {
  for (int a = 0; a < 3; ++a) o.t[a] = V[4 * a] * mean[0] + V[4 * a + 1] * mean[1] + V[4 * a + 2] * mean[2] + V[4 * a + 3];
  const T limx = T(1.3) * tanx * o.t[2], limy = T(1.3) * tany * o.t[2];
  o.x_mul = (o.t[0] < -limx || o.t[0] > limx) ? T(0) : T(1);
  o.y_mul = (o.t[1] < -limy || o.t[1] > limy) ? T(0) : T(1);
  o.t[0] = std::min(std::max(o.t[0], -limx), limx);
  o.t[1] = std::min(std::max(o.t[1], -limy), limy);
  const T tz = o.t[2];
  o.J[0] = fx / tz, o.J[1] = 0, o.J[2] = -(fx * o.t[0]) / (tz * tz);
  o.J[3] = 0, o.J[4] = fy / tz, o.J[5] = -(fy * o.t[1]) / (tz * tz);
  for (int i = 0; i < 2; ++i)
    for (int j = 0; j < 3; ++j) {
      T s = 0;
      for (int k = 0; k < 3; ++k) s += o.J[i * 3 + k] * V[4 * k + j];
      o.M[i * 3 + j] = s;
    }
}

// M cov3D M^T without the low-pass term: returns (a, b, c) of the symmetric 2x2
template <typename T>
inline void cov2d_product(const T* M, const T* c, T* out) {
  const T Vrk[9] = {c[0], c[1], c[2], c[1], c[3], c[4], c[2], c[4], c[5]};
  T tmp[6];
  for (int i = 0; i < 2; ++i)
    for (int j = 0; j < 3; ++j) {
      T s = 0;
      for (int k = 0; k < 3; ++k) s += M[i * 3 + k] * Vrk[k * 3 + j];
      tmp[i * 3 + j] = s;
    }
  T cov[4];
  for (int i = 0; i < 2; ++i)
    for (int j = 0; j < 2; ++j) {
      T s = 0;
      for (int k = 0; k < 3; ++k) s += tmp[i * 3 + k] * M[j * 3 + k];
      cov[i * 2 + j] = s;
    }
  out[0] = cov[0], out[1] = cov[1], out[2] = cov[3];
}

// gaussian_compute_cov2D.cu:96-186: from dL/dcov2D = (da, db, dc) (b is the one stored off-diagonal entry) to dL/dcov3D,
// dL/dmean and, when g_vm is given, the 12 entries of dL/d(view matrix rows 0-2) ADDED to g_vm (:163-183).
template <typename T>
inline void cov2d_backward_cov(const Cov2DTerms<T>& k, const T* mean, const T* c3, T fx, T fy, const T* V, T da, T db,
                               T dc, T* g_cov3D, T* g_mean, T* g_vm = nullptr) {
  const T* M = k.M;
  if (g_cov3D) {
    g_cov3D[0] = (M[0] * M[0] * da + M[0] * M[3] * db + M[3] * M[3] * dc);
    g_cov3D[3] = (M[1] * M[1] * da + M[1] * M[4] * db + M[4] * M[4] * dc);
    g_cov3D[5] = (M[2] * M[2] * da + M[2] * M[5] * db + M[5] * M[5] * dc);
    g_cov3D[1] = 2 * M[0] * M[1] * da + (M[0] * M[4] + M[1] * M[3]) * db + 2 * M[3] * M[4] * dc;
    g_cov3D[2] = 2 * M[0] * M[2] * da + (M[0] * M[5] + M[2] * M[3]) * db + 2 * M[3] * M[5] * dc;
    g_cov3D[4] = 2 * M[1] * M[2] * da + (M[1] * M[5] + M[2] * M[4]) * db + 2 * M[4] * M[5] * dc;
  }
  T dT[6];
  dT[0] = 2 * (M[0] * c3[0] + M[1] * c3[1] + M[2] * c3[2]) * da + (M[3] * c3[0] + M[4] * c3[1] + M[5] * c3[2]) * db;
  dT[1] = 2 * (M[0] * c3[1] + M[1] * c3[3] + M[2] * c3[4]) * da + (M[3] * c3[1] + M[4] * c3[3] + M[5] * c3[4]) * db;
  dT[2] = 2 * (M[0] * c3[2] + M[1] * c3[4] + M[2] * c3[5]) * da + (M[3] * c3[2] + M[4] * c3[4] + M[5] * c3[5]) * db;
  dT[3] = 2 * (M[3] * c3[0] + M[4] * c3[1] + M[5] * c3[2]) * dc + (M[0] * c3[0] + M[1] * c3[1] + M[2] * c3[2]) * db;
  dT[4] = 2 * (M[3] * c3[1] + M[4] * c3[3] + M[5] * c3[4]) * dc + (M[0] * c3[1] + M[1] * c3[3] + M[2] * c3[4]) * db;
  dT[5] = 2 * (M[3] * c3[2] + M[4] * c3[4] + M[5] * c3[5]) * dc + (M[0] * c3[2] + M[1] * c3[4] + M[2] * c3[5]) * db;
  const T R[9] = {V[0], V[1], V[2], V[4], V[5], V[6], V[8], V[9], V[10]};
  const T dJ00 = dT[0] * R[0] + dT[1] * R[1] + dT[2] * R[2];
  const T dJ02 = dT[0] * R[6] + dT[1] * R[7] + dT[2] * R[8];
  const T dJ11 = dT[3] * R[3] + dT[4] * R[4] + dT[5] * R[5];
  const T dJ12 = dT[3] * R[6] + dT[4] * R[7] + dT[5] * R[8];
  const T tz = T(1) / k.t[2], tz2 = tz * tz, tz3 = tz2 * tz;
  const T dtx = k.x_mul * -fx * tz2 * dJ02;
  const T dty = k.y_mul * -fy * tz2 * dJ12;
  const T dtz = -fx * tz2 * dJ00 - fy * tz2 * dJ11 + (2 * fx * k.t[0]) * tz3 * dJ02 + (2 * fy * k.t[1]) * tz3 * dJ12;
  for (int a2 = 0; a2 < 3; ++a2) g_mean[a2] = V[a2] * dtx + V[4 + a2] * dty + V[8 + a2] * dtz;
  if (g_vm) {
    // M = J W  ->  dL/dW = J^T dL/dM (3x3), plus the view-space mean t = W mean + translation (:163-183)
    const T dt[3] = {dtx, dty, dtz};
    for (int i = 0; i < 3; ++i) {
      for (int j = 0; j < 3; ++j) g_vm[4 * i + j] += k.J[i] * dT[j] + k.J[3 + i] * dT[3 + j] + dt[i] * mean[j];
      g_vm[4 * i + 3] += dt[i];
    }
  }
}

// gaussian_compute_cov2D.cu:64-95 in front of the above: dL_dconic given (dL_dcov2D absent).
// Returns false when the determinant is exactly zero (the reference returns without writing).
template <typename T>
inline bool cov2d_backward(const T* mean, const T* c3, T fx, T fy, T tanx, T tany, const T* V, const T* g_conic,
                           T* g_cov3D, T* g_mean, T* g_vm = nullptr) {
  Cov2DTerms<T> k;
  cov2d_terms(mean, fx, fy, tanx, tany, V, k);
  T cov[3];
  cov2d_product(k.M, c3, cov);
  const T a = cov[0] + T(0.3), b = cov[1], c = cov[2] + T(0.3);
  const T denom = a * c - b * b;
  if (denom == 0) return false;
  const T denom2inv = T(1.) / ((denom * denom) + T(0.0000001));
  const T tt = c * g_conic[0] - b * g_conic[1] + a * g_conic[2];
  const T da = denom2inv * (-c * tt + denom * g_conic[2]);
  const T dc = denom2inv * (-a * tt + denom * g_conic[0]);
  const T db = denom2inv * (T(2) * b * tt - denom * g_conic[1]);
  cov2d_backward_cov(k, mean, c3, fx, fy, V, da, db, dc, g_cov3D, g_mean, g_vm);
  return true;
}

// gaussian_topk_weights -- gaussian_topk.cu:12-93 (kernel) and :212-228: per pixel the k largest blend weights
// w = alpha * T of the front-to-back traversal with their Gaussian ids; `w >= slot` takes a slot, so a later Gaussian
// wins ties; indices start at -1, weights at 0.
template <typename T>
void topk_weights(int topk, int W, int H, const T* means2D, const T* conic_opacity, const int64_t* ranges,
                  const int32_t* point_list, int32_t* top_idx, T* top_w) {
  const int gx = (W + 15) / 16;
#pragma omp parallel for schedule(dynamic, 4)
  for (int py = 0; py < H; ++py)
    for (int px = 0; px < W; ++px) {
      const size_t pix = (size_t) py * W + px;
      int32_t* ti = top_idx + pix * topk;
      T* tw       = top_w + pix * topk;
      for (int k = 0; k < topk; ++k) ti[k] = -1, tw[k] = 0;
      const int tile = (py / 16) * gx + px / 16;
      T t = 1;
      for (int64_t e = ranges[2 * tile]; e < ranges[2 * tile + 1]; ++e) {
        const int id = point_list[e];
        const T dx = means2D[2 * (size_t) id] - (T) px, dy = means2D[2 * (size_t) id + 1] - (T) py;
        const T* co = conic_opacity + 4 * (size_t) id;
        const T power = T(-0.5) * (co[0] * dx * dx + co[2] * dy * dy) - co[1] * dx * dy;
        if (power > 0) continue;
        const T alpha = std::min(T(0.99), co[3] * std::exp(power));
        if (alpha < T(1) / T(255)) continue;
        const T test_T = t * (1 - alpha);
        if (test_T < T(0.0001)) break;
        T w = alpha * t;
        int idx = id;
        for (int k = 0; k < topk; ++k)
          if (w >= tw[k]) std::swap(w, tw[k]), std::swap(idx, ti[k]);
        t = test_T;
      }
    }
}

// gs_compute_cov3D_forward / _backward (gaussian_compute_cov3D.cu:122-161) and gs_compute_cov2D_forward / _backward
// (gaussian_compute_cov2D.cu:186-248, without the view-matrix gradient) as stand-alone operators.
template <typename T>
void compute_cov3D(int N, const T* q, const T* s, T* cov3D) {
#pragma omp parallel for
  for (int i = 0; i < N; ++i) cov3d_forward(s + 3 * (size_t) i, q + 4 * (size_t) i, cov3D + 6 * (size_t) i);
}
template <typename T>
void compute_cov3D_backward(int N, const T* q, const T* s, const T* g, T* gq, T* gs) {
#pragma omp parallel for
  for (int i = 0; i < N; ++i)
    cov3d_backward(s + 3 * (size_t) i, q + 4 * (size_t) i, g + 6 * (size_t) i, gs + 3 * (size_t) i, gq + 4 * (size_t) i);
}
template <typename T>
void compute_cov2D(int N, const T* cov3D, const T* mean, const T* V, T fx, T fy, T tanx, T tany, T* cov2D) {
#pragma omp parallel for
  for (int i = 0; i < N; ++i) {
    Cov2DTerms<T> k;
    cov2d_terms(mean + 3 * (size_t) i, fx, fy, tanx, tany, V, k);
    T* o = cov2D + 3 * (size_t) i;
    cov2d_product(k.M, cov3D + 6 * (size_t) i, o);
    o[0] += T(0.3), o[2] += T(0.3);
  }
}
template <typename T>
void compute_cov2D_backward(int N, const T* cov3D, const T* mean, const T* V, T fx, T fy, T tanx, T tany, const T* g,
                            T* g_cov3D, T* g_mean, T* g_vm) {
  for (int i = 0; i < N; ++i) {  // serial: g_vm (12 sums over all points, added to the caller's buffer) has one order
    Cov2DTerms<T> k;
    cov2d_terms(mean + 3 * (size_t) i, fx, fy, tanx, tany, V, k);
    cov2d_backward_cov(k, mean + 3 * (size_t) i, cov3D + 6 * (size_t) i, fx, fy, V, g[3 * (size_t) i],
                       g[3 * (size_t) i + 1], g[3 * (size_t) i + 2], g_cov3D + 6 * (size_t) i, g_mean + 3 * (size_t) i,
                       g_vm);
  }
}

// gaussian_preprocess.cu:44-128 (preprocess_forward_kernel) + host :372-466. Outputs are expected zero-filled, except
// means2D when the caller passed its own (means2D_preserve).
template <typename T>
void preprocess_forward(int P, int W, int H, int sh_degree, int n_sh, int is_opengl, const T* means3D, const T* scales,
                        const T* rotations, const T* opacities, const T* shs, const T* sh_rest, const T* Tw2v,
                        const T* Tv2c, const T* campos, T tanx, T tany, const uint8_t* culling,
                        const T* cov3D_precomp, const T* cov2D_precomp, T* means2D, T* depths, T* colors,
                        int32_t* radii, int32_t* tiles_touched, T* cov3Ds, T* conic_opacity) {
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const T fx = T(0.5) * W / tanx, fy = T(0.5) * H / tany;
#pragma omp parallel for schedule(static)
  for (int i = 0; i < P; ++i) {
    radii[i] = 0, tiles_touched[i] = 0;
    if (culling && culling[i]) continue;
    const T* p = means3D + 3 * (size_t) i;
    T pv[3], ph[4];
    for (int a = 0; a < 3; ++a) pv[a] = Tw2v[4 * a] * p[0] + Tw2v[4 * a + 1] * p[1] + Tw2v[4 * a + 2] * p[2] + Tw2v[4 * a + 3];
    for (int a = 0; a < 4; ++a) ph[a] = Tv2c[4 * a] * pv[0] + Tv2c[4 * a + 1] * pv[1] + Tv2c[4 * a + 2] * pv[2] + Tv2c[4 * a + 3];
    const T pw = T(1.0) / (ph[3] + T(0.0000001));
    const T proj[3] = {ph[0] * pw, ph[1] * pw, ph[2] * pw};
    if (is_opengl ? (proj[2] < T(-1.0) || proj[2] > T(1.)) : pv[2] <= T(0.2)) continue;
    // a pre-computed 2D covariance is taken as it is (no low-pass term), a pre-computed 3D one replaces R S^2 R^T; the
    // host returns cov3D_precomp itself as `cov3Ds` then (gaussian_preprocess.cu:76-92, :424)
    T cov[3];
    if (cov2D_precomp) {
      for (int a = 0; a < 3; ++a) cov[a] = cov2D_precomp[3 * (size_t) i + a];
    } else {
      const T* c3 = cov3D_precomp ? cov3D_precomp + 6 * (size_t) i : cov3Ds + 6 * (size_t) i;
      if (!cov3D_precomp) cov3d_forward(scales + 3 * (size_t) i, rotations + 4 * (size_t) i, cov3Ds + 6 * (size_t) i);
      Cov2DTerms<T> k;
      cov2d_terms(p, fx, fy, tanx, tany, Tw2v, k);
      cov2d_product(k.M, c3, cov);
      cov[0] += T(0.3), cov[2] += T(0.3);
    }
    const T det = cov[0] * cov[2] - cov[1] * cov[1];
    if (det == T(0.0)) continue;
    const T mid = T(0.5) * (cov[0] + cov[2]);
    const T l1 = mid + std::sqrt(std::max(T(0.1), mid * mid - det));
    const T l2 = mid - std::sqrt(std::max(T(0.1), mid * mid - det));
    const T radius = std::ceil(T(3.) * std::sqrt(std::max(l1, l2)));
    T px, py;
    if (is_opengl) px = (T(1.0) + proj[0]) * T(0.5) * W, py = (T(1.0) + -proj[1]) * T(0.5) * H;
    else px = (T(1.0) + proj[0]) * T(0.5) * W - T(0.5), py = (T(1.0) + proj[1]) * T(0.5) * H - T(0.5);
    const Rect<T> r = get_rect<T>(px, py, f2i(radius), gx, gy);
    if ((r.x1 - r.x0) * (r.y1 - r.y0) == 0) continue;
    if (sh_degree >= 0)
      sh_to_rgb(sh_degree, p, campos, shs + (size_t) i * (sh_rest ? 1 : n_sh) * 3,
                sh_rest ? sh_rest + (size_t) i * n_sh * 3 : nullptr, true, colors + 3 * (size_t) i);
    depths[i] = is_opengl ? proj[2] : pv[2];
    radii[i]  = f2i(radius);
    means2D[2 * (size_t) i] = px, means2D[2 * (size_t) i + 1] = py;
    const T det_inv = T(1.) / det;
    T* co = conic_opacity + 4 * (size_t) i;
    co[0] = cov[2] * det_inv, co[1] = -cov[1] * det_inv, co[2] = cov[0] * det_inv, co[3] = opacities[i];
    tiles_touched[i] = (r.y1 - r.y0) * (r.x1 - r.x0);
  }
}

// gaussian_preprocess.cu:246-372 (preprocess_backward_kernel).
// grad_mean2D is overwritten with (0.5 W g.x, +-0.5 H g.y) as the reference does; rows with radii <= 0 are untouched.
// cov2Ds (pre-computed 2D covariances): g_cov is [P,3] and gets the conic's gradient (:293-301), nothing flows to the
// mean or to scales / rotations through the covariance. Otherwise cov3Ds (computed or pre-computed) is differentiated
// and g_cov is [P,6]. g_Tw2v (16 values, rows 0-2 written) and g_campos (3) are ADDED to, as the reference's atomics do.
template <typename T>
void preprocess_backward(int P, int W, int H, int sh_degree, int n_sh, int is_opengl, const T* means3D, const T* scales,
                         const T* rotations, const T* shs, const T* sh_rest, const T* Tw2v, const T* Tv2c,
                         const T* campos, T tanx, T tany, const int32_t* radii, const T* colors, const T* cov3Ds,
                         const T* cov2Ds, T* grad_mean2D, const T* grad_colors, const T* grad_conic, T* g_means3D,
                         T* g_scales, T* g_rot, T* g_opac, T* g_shs, T* g_sh_rest, T* g_cov3D, T* g_Tw2v,
                         T* g_campos) {
  const T fx = T(0.5) * W / tanx, fy = T(0.5) * H / tany;
#pragma omp parallel for schedule(static) if (!g_Tw2v && !g_campos)
  for (int i = 0; i < P; ++i) {
    if (radii[i] <= 0) continue;
    const T* p = means3D + 3 * (size_t) i;
    T pv[3], pc[4];
    for (int a = 0; a < 3; ++a) pv[a] = Tw2v[4 * a] * p[0] + Tw2v[4 * a + 1] * p[1] + Tw2v[4 * a + 2] * p[2] + Tw2v[4 * a + 3];
    for (int a = 0; a < 4; ++a) pc[a] = Tv2c[4 * a] * pv[0] + Tv2c[4 * a + 1] * pv[1] + Tv2c[4 * a + 2] * pv[2] + Tv2c[4 * a + 3];
    const T mw = T(1.0) / (pc[3] + T(0.0000001));
    const T du = T(0.5 * W) * grad_mean2D[2 * (size_t) i];
    const T dv = T((is_opengl ? -0.5 : 0.5) * H) * grad_mean2D[2 * (size_t) i + 1];
    grad_mean2D[2 * (size_t) i] = du, grad_mean2D[2 * (size_t) i + 1] = dv;
    const T tmp1 = (pc[0] * du + pc[1] * dv) * mw * mw;
    T dpv[3];
    for (int a = 0; a < 3; ++a) dpv[a] = (Tv2c[a] * du + Tv2c[4 + a] * dv) * mw - Tv2c[12 + a] * tmp1;
    T gm[3];
    for (int a = 0; a < 3; ++a) gm[a] = Tw2v[a] * dpv[0] + Tw2v[4 + a] * dpv[1] + Tw2v[8 + a] * dpv[2];
    if (g_opac) g_opac[i] = grad_conic[4 * (size_t) i + 3];
    T gcov[6] = {0, 0, 0, 0, 0, 0}, gmean_cov[3];
    if (cov2Ds) {
      if (g_cov3D) {
        const T a = cov2Ds[3 * (size_t) i], b = cov2Ds[3 * (size_t) i + 1], c = cov2Ds[3 * (size_t) i + 2];
        const T* gc = grad_conic + 4 * (size_t) i;
        const T denom = a * c - b * b;
        const T denom2inv = T(1.) / ((denom * denom) + T(0.0000001));
        const T tt = c * gc[0] - b * gc[1] + a * gc[2];
        g_cov3D[3 * (size_t) i + 0] = denom2inv * (-c * tt + denom * gc[2]);
        g_cov3D[3 * (size_t) i + 2] = denom2inv * (-a * tt + denom * gc[0]);
        g_cov3D[3 * (size_t) i + 1] = denom2inv * (T(2) * b * tt - denom * gc[1]);
      }
    } else {
      if (cov2d_backward(p, cov3Ds + 6 * (size_t) i, fx, fy, tanx, tany, Tw2v, grad_conic + 4 * (size_t) i, gcov,
                         gmean_cov, g_Tw2v))
        for (int a = 0; a < 3; ++a) gm[a] += gmean_cov[a];
      if (g_cov3D)
        for (int a = 0; a < 6; ++a) g_cov3D[6 * (size_t) i + a] = gcov[a];
    }
    if (g_Tw2v)
      for (int a = 0; a < 3; ++a) {
        for (int b = 0; b < 3; ++b) g_Tw2v[4 * a + b] += p[b] * dpv[a];
        g_Tw2v[4 * a + 3] += dpv[a];
      }
    if (sh_degree >= 0 && grad_colors) {
      T gdir[3];
      const int m1 = sh_rest ? 1 : n_sh;
      sh_to_rgb_backward(sh_degree, p, campos, colors + 3 * (size_t) i, shs + (size_t) i * m1 * 3,
                         sh_rest ? sh_rest + (size_t) i * n_sh * 3 : nullptr, grad_colors + 3 * (size_t) i,
                         g_shs ? g_shs + (size_t) i * m1 * 3 : nullptr,
                         g_sh_rest ? g_sh_rest + (size_t) i * n_sh * 3 : nullptr, true, true, gdir);
      for (int a = 0; a < 3; ++a) gm[a] += gdir[a];
      if (g_campos)  // the direction is normalize(p - campos): the camera position gets minus the point's share
        for (int a = 0; a < 3; ++a) g_campos[a] -= gdir[a];
    }
    for (int a = 0; a < 3; ++a) g_means3D[3 * (size_t) i + a] = gm[a];
    if (!g_scales && !g_rot) continue;
    T gs[3], gq[4];
    cov3d_backward(scales + 3 * (size_t) i, rotations + 4 * (size_t) i, gcov, gs, gq);
    if (g_scales)
      for (int a = 0; a < 3; ++a) g_scales[3 * (size_t) i + a] = gs[a];
    if (g_rot)
      for (int a = 0; a < 4; ++a) g_rot[4 * (size_t) i + a] = gq[a];
  }
}

// gaussian_render.cu:20-173. Planar outputs; accum_* are optional accumulators (not reset here).
// With bucket_offset (inclusive cumsum of ceil(len / 32) per tile): bucket_to_tile[B], max_contrib[T] (deepest
// contributor of the tile) and, for pixels still blending, the state before every 32nd list entry: sampled_T[B,256],
// sampled_ar[B,3+E,256] (position inside the tile row-major). The reference indexes its colour accumulator past its
// end for the extra channels (:103, `C[ch]` with ch >= 3); the running sums of the extras are what is stored here.
template <typename T>
void render_forward(int W, int H, int E, const T* means2D, const T* conic_opacity, const T* colors, const T* extras,
                    const int32_t* point_list, const int64_t* ranges, T* out_color, T* out_opacity, T* out_extras,
                    int32_t* n_contrib, int32_t* accum_max_count, T* accum_weights_p, int32_t* accum_weights_count,
                    const int64_t* bucket_offset = nullptr, int32_t* max_contrib = nullptr,
                    int32_t* bucket_to_tile = nullptr, T* sampled_T = nullptr, T* sampled_ar = nullptr) {
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const size_t HW = (size_t) H * W;
  if (bucket_offset)
    for (int t = 0; t < gx * gy; ++t) {
      const int64_t b0 = t == 0 ? 0 : bucket_offset[t - 1];
      for (int64_t b = 0; b < (ranges[2 * t + 1] - ranges[2 * t] + 31) / 32; ++b) bucket_to_tile[b0 + b] = t;
      max_contrib[t] = 0;
    }
  for (int py = 0; py < H; ++py)
    for (int px = 0; px < W; ++px) {
      const int tile = (py / kTile) * gx + px / kTile;
      const int64_t r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
      const int rank = (py % kTile) * kTile + (px % kTile);
      int64_t bbm = bucket_offset ? (tile == 0 ? 0 : bucket_offset[tile - 1]) : 0;
      T t = 1, C[3] = {0, 0, 0}, wmax = 0;
      std::vector<T> Ex(E, T(0));
      int contributor = 0, last = 0, wmax_id = -1;
      bool flag = false;
      for (int64_t e = r0; e < r1; ++e) {
        if (bucket_offset && (e - r0) % 32 == 0) {
          sampled_T[bbm * 256 + rank] = t;
          for (int c = 0; c < 3; ++c) sampled_ar[(bbm * (3 + E) + c) * 256 + rank] = C[c];
          for (int c = 0; c < E; ++c) sampled_ar[(bbm * (3 + E) + 3 + c) * 256 + rank] = Ex[c];
          ++bbm;
        }
        const int id = point_list[e];
        ++contributor;
        const T dx = means2D[2 * (size_t) id] - T(px), dy = means2D[2 * (size_t) id + 1] - T(py);
        const T* co = conic_opacity + 4 * (size_t) id;
        const T power = T(-0.5) * (co[0] * dx * dx + co[2] * dy * dy) - co[1] * dx * dy;
        if (power > T(0.0)) continue;
        const T alpha = std::min(T(0.99), co[3] * std::exp(power));
        if (alpha < T(1.0 / 255.0)) continue;
        const T test_T = t * (1 - alpha);
        if (test_T < T(0.0001)) break;
        const T w = alpha * t;
        for (int c = 0; c < 3; ++c) C[c] += colors[3 * (size_t) id + c] * w;
        for (int c = 0; c < E; ++c) Ex[c] += extras[(size_t) E * id + c] * w;
        if (wmax < w) wmax = w, wmax_id = id, flag = true;
        if (accum_weights_p) accum_weights_p[id] += w;
        if (accum_weights_count) accum_weights_count[id] += 1;
        t = test_T;
        last = contributor;
      }
      if (flag && accum_max_count) accum_max_count[wmax_id] += 1;
      const size_t pix = (size_t) py * W + px;
      out_opacity[pix] = T(1) - t;
      n_contrib[pix]   = last;
      for (int c = 0; c < 3; ++c) out_color[c * HW + pix] = C[c];
      for (int c = 0; c < E; ++c) out_extras[c * HW + pix] = Ex[c];
      if (bucket_offset) max_contrib[tile] = std::max(max_contrib[tile], (int32_t) last);
    }
}

// gaussian_rasterize_fast_backward -- gaussian_render.cu:540-694 (kernel), :760-812 (host): one warp per bucket of 32 list
// entries, lane = entry, every pixel of the tile passing through the lanes in turn with its state (transmittance, the
// running sums minus the final image) taken from the forward's snapshots. Restated per (bucket, pixel): the state
// enters at the bucket's first entry and is updated entry by entry, exactly the sequence a pixel sees on its way
// through the warp. The reference reads the gradient of the extra channels into the wrong registers (:636, `e + E`
// where `e + C` is meant) and leaves the right ones uninitialised; the intended assignment is what is restated.
template <typename T>
void render_fast_backward(int W, int H, int E, const T* means2D, const T* conic_opacity, const T* colors,
                          const T* extras, const T* images, const T* out_extras, const T* out_opacity,
                          const int32_t* n_contrib, const int32_t* max_contrib, const int64_t* bucket_offset,
                          const int32_t* bucket_to_tile, const T* sampled_T, const T* sampled_ar, const T* dL_dpix,
                          const T* dL_dout_extras, const T* dL_dout_opacity, const int32_t* point_list,
                          const int64_t* ranges, int64_t B, T* g_means2D, T* g_conic_opacity, T* g_colors,
                          T* g_extras) {
  const int gx = (W + kTile - 1) / kTile;
  const size_t HW = (size_t) H * W;
  const int CE = 3 + E;
  std::vector<T> ar(CE), g(CE), c(CE);
  for (int64_t bucket = 0; bucket < B; ++bucket) {
    const int tile = bucket_to_tile[bucket];
    const int64_t r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
    const int64_t bbm = tile == 0 ? 0 : bucket_offset[tile - 1];
    const int64_t in_tile = bucket - bbm;
    if (in_tile * 32 >= max_contrib[tile]) continue;
    const int tx = tile % gx, ty = tile / gx;
    for (int idx = 0; idx < 256; ++idx) {
      const int px = tx * kTile + idx % kTile, py = ty * kTile + idx / kTile;
      if (px >= W || py >= H) continue;
      const size_t pix = (size_t) W * py + px;
      T t = sampled_T[bucket * 256 + idx];
      for (int ch = 0; ch < 3; ++ch)
        ar[ch] = -images[ch * HW + pix] + sampled_ar[(bucket * CE + ch) * 256 + idx], g[ch] = dL_dpix[ch * HW + pix];
      for (int e = 0; e < E; ++e)
        ar[3 + e] = -out_extras[e * HW + pix] + sampled_ar[(bucket * CE + 3 + e) * 256 + idx],
               g[3 + e] = dL_dout_extras[e * HW + pix];
      const T t_final = 1 - out_opacity[pix];
      const int last = n_contrib[pix];
      const T dL_dt_final = -dL_dout_opacity[pix];
      for (int lane = 0; lane < 32; ++lane) {
        const int64_t s = in_tile * 32 + lane;
        if (s >= r1 - r0) break;
        if (s >= last) continue;
        const int id = point_list[r0 + s];
        const T dx = means2D[2 * (size_t) id] - T(px), dy = means2D[2 * (size_t) id + 1] - T(py);
        const T* co = conic_opacity + 4 * (size_t) id;
        const T power = -T(0.5) * (co[0] * dx * dx + co[2] * dy * dy) - co[1] * dx * dy;
        if (power > 0) continue;
        const T G = std::exp(power);
        const T alpha = std::min(T(0.99), co[3] * G);
        if (alpha < T(1.0 / 255.)) continue;
        const T dch = alpha * t;
        for (int ch = 0; ch < 3; ++ch) c[ch] = colors[3 * (size_t) id + ch];
        for (int e = 0; e < E; ++e) c[3 + e] = extras[(size_t) E * id + e];
        T dL_dalpha = 0;
        for (int ch = 0; ch < CE; ++ch) {
          ar[ch] += t * alpha * c[ch];
          if (ch < 3) g_colors[3 * (size_t) id + ch] += dch * g[ch];
          else g_extras[(size_t) E * id + (ch - 3)] += dch * g[ch];
          dL_dalpha += ((c[ch] * t) + (T(1.0) / (T(1.0) - alpha)) * ar[ch]) * g[ch];
        }
        dL_dalpha += (-t_final / (T(1.0) - alpha)) * dL_dt_final;
        t *= (1 - alpha);
        const T dL_dG = -co[3] * G * dL_dalpha;
        g_means2D[2 * (size_t) id] += dL_dG * (dx * co[0] + dy * co[1]);
        g_means2D[2 * (size_t) id + 1] += dL_dG * (dy * co[2] + dx * co[1]);
        T* gc = g_conic_opacity + 4 * (size_t) id;
        gc[0] += T(0.5) * dx * dx * dL_dG;
        gc[1] += T(1.0) * dx * dy * dL_dG;
        gc[2] += T(0.5) * dy * dy * dL_dG;
        gc[3] += G * dL_dalpha;
      }
    }
  }
}

// gaussian_render.cu:296-444. Gradients are accumulated into zero-filled outputs, pixel by pixel in raster order.
template <typename T>
void render_backward(int W, int H, int E, const T* means2D, const T* conic_opacity, const T* colors, const T* extras,
                     const T* out_opacity, const int32_t* n_contrib, const T* dL_dpix, const T* dL_dout_extras,
                     const T* dL_dout_opacity, const int32_t* point_list, const int64_t* ranges, T* g_means2D,
                     T* g_conic_opacity, T* g_colors, T* g_extras) {
  const int gx = (W + kTile - 1) / kTile;
  const size_t HW = (size_t) H * W;
  for (int py = 0; py < H; ++py)
    for (int px = 0; px < W; ++px) {
      const int tile = (py / kTile) * gx + px / kTile;
      const int64_t r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
      const size_t pix = (size_t) py * W + px;
      const T T_final = T(1.0) - out_opacity[pix];
      T t = T_final;
      const T dL_dT = -dL_dout_opacity[pix];
      const int last = n_contrib[pix];
      std::vector<T> accum(3 + E, T(0)), g(3 + E);
      for (int c = 0; c < 3; ++c) g[c] = dL_dpix[c * HW + pix];
      for (int c = 0; c < E; ++c) g[3 + c] = dL_dout_extras[c * HW + pix];
      int contributor = (int) (r1 - r0);
      for (int64_t e = r1 - 1; e >= r0; --e) {
        --contributor;
        if (contributor >= last) continue;
        const int id = point_list[e];
        const T dx = means2D[2 * (size_t) id] - T(px), dy = means2D[2 * (size_t) id + 1] - T(py);
        const T* co = conic_opacity + 4 * (size_t) id;
        const T power = T(-0.5) * (co[0] * dx * dx + co[2] * dy * dy) - co[1] * dx * dy;
        if (power > T(0.0)) continue;
        const T G = std::exp(power);
        const T alpha = std::min(T(0.99), co[3] * G);
        if (alpha < T(1.0 / 255.0)) continue;
        t = t / (T(1.0) - alpha);
        const T dch = alpha * t;
        T dL_dalpha = 0;
        for (int c = 0; c < 3 + E; ++c) {
          const T v = c < 3 ? colors[3 * (size_t) id + c] : extras[(size_t) E * id + (c - 3)];
          dL_dalpha += (v * t * (T(1.0) - alpha) - accum[c]) * g[c];
          accum[c] += v * dch;
          if (c < 3) g_colors[3 * (size_t) id + c] += dch * g[c];
          else g_extras[(size_t) E * id + (c - 3)] += dch * g[c];
        }
        dL_dalpha = (dL_dalpha - T_final * dL_dT) / (T(1.0) - alpha);
        const T dL_dG = -co[3] * G * dL_dalpha;
        g_means2D[2 * (size_t) id] += dL_dG * (co[0] * dx + co[1] * dy);
        g_means2D[2 * (size_t) id + 1] += dL_dG * (co[2] * dy + co[1] * dx);
        T* gc = g_conic_opacity + 4 * (size_t) id;
        gc[0] += T(0.5) * dx * dx * dL_dG;
        gc[1] += T(1.0) * dx * dy * dL_dG;
        gc[2] += T(0.5) * dy * dy * dL_dG;
        gc[3] += G * dL_dalpha;
      }
    }
}

// gaussian_rasterize_extra_forward -- gaussian_rasterizer_extra.cu:12-101 (kernel), :317-339 (host): any number of
// per-Gaussian feature channels blended with the weights of the main forward pass, whose n_contrib bounds the
// traversal; output pixel-major [H, W, E]. The reference walks the list once per group of 16 channels; the weights do not
// depend on the group, so one walk is the same computation.
template <typename T>
void extra_forward(int W, int H, int E, const T* extras, const T* means2D, const T* conic_opacity,
                   const int64_t* ranges, const int32_t* point_list, const int32_t* n_contrib, T* out) {
  const int gx = (W + kTile - 1) / kTile;
  for (int py = 0; py < H; ++py)
    for (int px = 0; px < W; ++px) {
      const int tile = (py / kTile) * gx + px / kTile;
      const size_t pix = (size_t) py * W + px;
      const int last = n_contrib[pix];
      std::vector<T> acc(E, T(0));
      T t = 1;
      int contributor = 0;
      for (int64_t e = ranges[2 * tile]; e < ranges[2 * tile + 1]; ++e) {
        if (++contributor > last) break;
        const int id = point_list[e];
        const T dx = means2D[2 * (size_t) id] - T(px), dy = means2D[2 * (size_t) id + 1] - T(py);
        const T* co = conic_opacity + 4 * (size_t) id;
        const T power = T(-0.5) * (co[0] * dx * dx + co[2] * dy * dy) - co[1] * dx * dy;
        if (power > T(0.0)) continue;
        const T alpha = std::min(T(0.99), co[3] * std::exp(power));
        if (alpha < T(1.0 / 255.0)) continue;
        const T test_T = t * (1 - alpha);
        if (test_T < T(0.0001)) break;
        for (int c = 0; c < E; ++c) acc[c] += extras[(size_t) E * id + c] * alpha * t;
        t = test_T;
      }
      for (int c = 0; c < E; ++c) out[pix * E + c] = acc[c];
    }
}

// gaussian_rasterize_extra_backward -- gaussian_rasterizer_extra.cu:103-209 (kernel), :341-365 (host): back to front
// from T_final = 1 - out_opacity, entries behind n_contrib skipped, no background and no opacity term. Each of the three
// gradients is optional and accumulated into. The reference adds the mean / conic / opacity gradient once per group of
// 16 channels; the sum over groups is the single sum over all channels taken here.
template <typename T>
void extra_backward(int W, int H, int E, const T* extras, const T* out_opacity, const T* grad_out, const T* means2D,
                    const T* conic_opacity, const int64_t* ranges, const int32_t* point_list,
                    const int32_t* n_contrib, T* g_extras, T* g_means2D, T* g_conic_opacity) {
  const int gx = (W + kTile - 1) / kTile;
  for (int py = 0; py < H; ++py)
    for (int px = 0; px < W; ++px) {
      const int tile = (py / kTile) * gx + px / kTile;
      const int64_t r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
      const size_t pix = (size_t) py * W + px;
      T t = T(1.0) - out_opacity[pix];
      const int last = n_contrib[pix];
      std::vector<T> accum(E, T(0));
      const T* g = grad_out + pix * E;
      int contributor = (int) (r1 - r0);
      for (int64_t e = r1 - 1; e >= r0; --e) {
        --contributor;
        if (contributor >= last) continue;
        const int id = point_list[e];
        const T dx = means2D[2 * (size_t) id] - T(px), dy = means2D[2 * (size_t) id + 1] - T(py);
        const T* co = conic_opacity + 4 * (size_t) id;
        const T power = T(-0.5) * (co[0] * dx * dx + co[2] * dy * dy) - co[1] * dx * dy;
        if (power > T(0.0)) continue;
        const T G = std::exp(power);
        const T alpha = std::min(T(0.99), co[3] * G);
        if (alpha < T(1.0 / 255.0)) continue;
        t = t / (T(1.0) - alpha);
        const T dch = alpha * t;
        T dL_dalpha = 0;
        for (int c = 0; c < E; ++c) {
          const T v = extras[(size_t) E * id + c];
          dL_dalpha += (v * t * (T(1.0) - alpha) - accum[c]) * g[c];
          accum[c] += v * dch;
          if (g_extras) g_extras[(size_t) E * id + c] += dch * g[c];
        }
        dL_dalpha = dL_dalpha / (T(1.0) - alpha);
        const T dL_dG = -co[3] * G * dL_dalpha;
        if (g_means2D) {
          g_means2D[2 * (size_t) id] += dL_dG * (co[0] * dx + co[1] * dy);
          g_means2D[2 * (size_t) id + 1] += dL_dG * (co[2] * dy + co[1] * dx);
        }
        if (g_conic_opacity) {
          T* gc = g_conic_opacity + 4 * (size_t) id;
          gc[0] += T(0.5) * dx * dx * dL_dG;
          gc[1] += T(1.0) * dx * dy * dL_dG;
          gc[2] += T(0.5) * dy * dy * dL_dG;
          gc[3] += G * dL_dalpha;
        }
      }
    }
}

}  // namespace
}  // namespace oracle

using namespace oracle;

#define INSTANTIATE_GS3D(SUF, T)                                                                                     \
  ORACLE_API int oracle_gs3d_preprocess_forward_##SUF(int P, int W, int H, int sh_degree, int n_sh, int is_opengl,   \
      const T* means3D, const T* scales, const T* rotations, const T* opacities, const T* shs, const T* sh_rest,     \
      const T* Tw2v, const T* Tv2c, const T* campos, double tanx, double tany, const uint8_t* culling,               \
      const T* cov3D_precomp, const T* cov2D_precomp, T* means2D, T* depths, T* colors, int32_t* radii,              \
      int32_t* tiles_touched, T* cov3Ds, T* conic_opacity) {                                                         \
    preprocess_forward<T>(P, W, H, sh_degree, n_sh, is_opengl, means3D, scales, rotations, opacities, shs, sh_rest,  \
                          Tw2v, Tv2c, campos, (T) tanx, (T) tany, culling, cov3D_precomp, cov2D_precomp, means2D,    \
                          depths, colors, radii, tiles_touched, cov3Ds, conic_opacity);                              \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs3d_preprocess_backward_##SUF(int P, int W, int H, int sh_degree, int n_sh, int is_opengl,  \
      const T* means3D, const T* scales, const T* rotations, const T* shs, const T* sh_rest, const T* Tw2v,          \
      const T* Tv2c, const T* campos, double tanx, double tany, const int32_t* radii, const T* colors,               \
      const T* cov3Ds, const T* cov2Ds, T* grad_mean2D, const T* grad_colors, const T* grad_conic, T* g_means3D,     \
      T* g_scales, T* g_rot, T* g_opac, T* g_shs, T* g_sh_rest, T* g_cov3D, T* g_Tw2v, T* g_campos) {                \
    preprocess_backward<T>(P, W, H, sh_degree, n_sh, is_opengl, means3D, scales, rotations, shs, sh_rest, Tw2v,      \
                           Tv2c, campos, (T) tanx, (T) tany, radii, colors, cov3Ds, cov2Ds, grad_mean2D,             \
                           grad_colors, grad_conic, g_means3D, g_scales, g_rot, g_opac, g_shs, g_sh_rest, g_cov3D,   \
                           g_Tw2v, g_campos);                                                                        \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs3d_render_forward_##SUF(int W, int H, int E, const T* means2D, const T* conic_opacity,     \
      const T* colors, const T* extras, const int32_t* point_list, const int64_t* ranges, T* out_color,              \
      T* out_opacity, T* out_extras, int32_t* n_contrib, int32_t* accum_max_count, T* accum_weights_p,               \
      int32_t* accum_weights_count, const int64_t* bucket_offset, int32_t* max_contrib, int32_t* bucket_to_tile,     \
      T* sampled_T, T* sampled_ar) {                                                                                 \
    render_forward<T>(W, H, E, means2D, conic_opacity, colors, extras, point_list, ranges, out_color, out_opacity,   \
                      out_extras, n_contrib, accum_max_count, accum_weights_p, accum_weights_count, bucket_offset,   \
                      max_contrib, bucket_to_tile, sampled_T, sampled_ar);                                           \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs3d_render_fast_backward_##SUF(int W, int H, int E, const T* means2D,                       \
      const T* conic_opacity, const T* colors, const T* extras, const T* images, const T* out_extras,                \
      const T* out_opacity, const int32_t* n_contrib, const int32_t* max_contrib, const int64_t* bucket_offset,      \
      const int32_t* bucket_to_tile, const T* sampled_T, const T* sampled_ar, const T* dL_dpix,                      \
      const T* dL_dout_extras, const T* dL_dout_opacity, const int32_t* point_list, const int64_t* ranges,           \
      int64_t B, T* g_means2D, T* g_conic_opacity, T* g_colors, T* g_extras) {                                       \
    render_fast_backward<T>(W, H, E, means2D, conic_opacity, colors, extras, images, out_extras, out_opacity,        \
                            n_contrib, max_contrib, bucket_offset, bucket_to_tile, sampled_T, sampled_ar, dL_dpix,   \
                            dL_dout_extras, dL_dout_opacity, point_list, ranges, B, g_means2D, g_conic_opacity,      \
                            g_colors, g_extras);                                                                     \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs3d_render_backward_##SUF(int W, int H, int E, const T* means2D, const T* conic_opacity,    \
      const T* colors, const T* extras, const T* out_opacity, const int32_t* n_contrib, const T* dL_dpix,            \
      const T* dL_dout_extras, const T* dL_dout_opacity, const int32_t* point_list, const int64_t* ranges,           \
      T* g_means2D, T* g_conic_opacity, T* g_colors, T* g_extras) {                                                  \
    render_backward<T>(W, H, E, means2D, conic_opacity, colors, extras, out_opacity, n_contrib, dL_dpix,             \
                       dL_dout_extras, dL_dout_opacity, point_list, ranges, g_means2D, g_conic_opacity, g_colors,    \
                       g_extras);                                                                                    \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs3d_extra_forward_##SUF(int W, int H, int E, const T* extras, const T* means2D,             \
      const T* conic_opacity, const int64_t* ranges, const int32_t* point_list, const int32_t* n_contrib, T* out) {  \
    extra_forward<T>(W, H, E, extras, means2D, conic_opacity, ranges, point_list, n_contrib, out);                   \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs3d_extra_backward_##SUF(int W, int H, int E, const T* extras, const T* out_opacity,        \
      const T* grad_out, const T* means2D, const T* conic_opacity, const int64_t* ranges, const int32_t* point_list, \
      const int32_t* n_contrib, T* g_extras, T* g_means2D, T* g_conic_opacity) {                                     \
    extra_backward<T>(W, H, E, extras, out_opacity, grad_out, means2D, conic_opacity, ranges, point_list, n_contrib, \
                      g_extras, g_means2D, g_conic_opacity);                                                         \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs3d_topk_weights_##SUF(int topk, int W, int H, const T* means2D, const T* conic_opacity,    \
      const int64_t* ranges, const int32_t* point_list, int32_t* top_idx, T* top_w) {                                \
    topk_weights<T>(topk, W, H, means2D, conic_opacity, ranges, point_list, top_idx, top_w);                         \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs3d_compute_cov3D_##SUF(int N, const T* q, const T* s, T* cov3D) {                          \
    compute_cov3D<T>(N, q, s, cov3D);                                                                                \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs3d_compute_cov3D_backward_##SUF(int N, const T* q, const T* s, const T* g, T* gq, T* gs) { \
    compute_cov3D_backward<T>(N, q, s, g, gq, gs);                                                                   \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs3d_compute_cov2D_##SUF(int N, const T* cov3D, const T* mean, const T* Tw2v, double fx,     \
      double fy, double tanx, double tany, T* cov2D) {                                                               \
    compute_cov2D<T>(N, cov3D, mean, Tw2v, (T) fx, (T) fy, (T) tanx, (T) tany, cov2D);                               \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs3d_compute_cov2D_backward_##SUF(int N, const T* cov3D, const T* mean, const T* Tw2v,       \
      double fx, double fy, double tanx, double tany, const T* g, T* g_cov3D, T* g_mean, T* g_vm) {                  \
    compute_cov2D_backward<T>(N, cov3D, mean, Tw2v, (T) fx, (T) fy, (T) tanx, (T) tany, g, g_cov3D, g_mean, g_vm);   \
    return 0;                                                                                                        \
  }

INSTANTIATE_GS3D(f32, float)
INSTANTIATE_GS3D(f64, double)
