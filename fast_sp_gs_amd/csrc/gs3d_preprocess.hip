// Per-Gaussian preprocessing of the 3D-Gaussian (EWA splatting) path and its backward, for gfx950.
//
// Reference behaviour reproduced: fast_2d_gs/_C/src/gaussian_splatting/gaussian_preprocess.cu:44-128 (forward kernel),
// :246-372 (backward kernel), hosts :372-466 and :567-636; 3D covariance gaussian_compute_cov3D.cu:18-36 / :76-118;
// 2D covariance (EWA, 1.3 x FoV clamp, +0.3 low-pass) gaussian_compute_cov2D.cu:18-62 / :64-186; SH colour
// spherical_harmonic.h:18-202 / :204-676. Covariances come from scales + rotations; pre-computed cov3D / cov2D inputs and
// camera gradients are not implemented.
//
// One lane per Gaussian. The geometry is evaluated with contraction off in the reference's operation order, so radii,
// tile counts, screen positions and conics are bit-identical to a plain IEEE evaluation; SH rows (degree <= 3) are
// moved between HBM and LDS by the whole block on consecutive addresses as in the surfel preprocess. Every output row
// is written (zeros for Gaussians that are not rendered), so callers allocate uninitialised memory.
#include "common.hpp"
#include "sh.hpp"
#include "sh_stage.hpp"

namespace fsgs {
namespace {

__device__ __forceinline__ void quat_to_R(const float4 q, float* R) {
#pragma clang fp contract(off)
  R[0] = 1 - 2 * (q.y * q.y + q.z * q.z);
  R[1] = 2 * (q.x * q.y - q.z * q.w);
  R[2] = 2 * (q.y * q.w + q.x * q.z);
  R[3] = 2 * (q.x * q.y + q.z * q.w);
  R[4] = 1 - 2 * (q.x * q.x + q.z * q.z);
  R[5] = 2 * (q.y * q.z - q.x * q.w);
  R[6] = 2 * (q.x * q.z - q.y * q.w);
  R[7] = 2 * (q.x * q.w + q.y * q.z);
  R[8] = 1 - 2 * (q.x * q.x + q.y * q.y);
}

// upper triangle of R diag(s^2) R^T
__device__ __forceinline__ void cov3d_forward(const float* s, const float4 q, float* c) {
#pragma clang fp contract(off)
  float R[9];
  quat_to_R(q, R);
  const float sx2 = s[0] * s[0], sy2 = s[1] * s[1], sz2 = s[2] * s[2];
  c[0] = R[0] * R[0] * sx2 + R[1] * R[1] * sy2 + R[2] * R[2] * sz2;
  c[1] = R[0] * R[3] * sx2 + R[1] * R[4] * sy2 + R[2] * R[5] * sz2;
  c[2] = R[0] * R[6] * sx2 + R[1] * R[7] * sy2 + R[2] * R[8] * sz2;
  c[3] = R[3] * R[3] * sx2 + R[4] * R[4] * sy2 + R[5] * R[5] * sz2;
  c[4] = R[3] * R[6] * sx2 + R[4] * R[7] * sy2 + R[5] * R[8] * sz2;
  c[5] = R[6] * R[6] * sx2 + R[7] * R[7] * sy2 + R[8] * R[8] * sz2;
}

__device__ __forceinline__ void cov3d_backward(const float* s, const float4 q, const float* g, float* gs, float* gq) {
#pragma clang fp contract(off)
  float R[9];
  quat_to_R(q, R);
#pragma unroll
  for (int a = 0; a < 3; ++a) {
    const float v = R[a] * R[a] * g[0] + R[a] * R[3 + a] * g[1] + R[a] * R[6 + a] * g[2] +
                    R[3 + a] * R[3 + a] * g[3] + R[3 + a] * R[6 + a] * g[4] + R[6 + a] * R[6 + a] * g[5];
    gs[a] = v * 2 * s[a];
  }
  const float s2[3] = {s[0] * s[0], s[1] * s[1], s[2] * s[2]};
  float dR[9];
#pragma unroll
  for (int a = 0; a < 3; ++a) {
    dR[a]     = (2 * R[a] * g[0] + R[3 + a] * g[1] + R[6 + a] * g[2]) * s2[a];
    dR[3 + a] = (2 * R[3 + a] * g[3] + R[a] * g[1] + R[6 + a] * g[4]) * s2[a];
    dR[6 + a] = (2 * R[6 + a] * g[5] + R[a] * g[2] + R[3 + a] * g[4]) * s2[a];
  }
  const float x = q.x, y = q.y, z = q.z, w = q.w;
  gq[0] = 2 * (-2 * x * (dR[4] + dR[8]) + y * (dR[1] + dR[3]) + z * (dR[2] + dR[6]) + w * (dR[7] - dR[5]));
  gq[1] = 2 * (x * (dR[1] + dR[3]) - 2 * y * (dR[0] + dR[8]) + z * (dR[5] + dR[7]) + w * (dR[2] - dR[6]));
  gq[2] = 2 * (x * (dR[2] + dR[6]) + y * (dR[5] + dR[7]) - 2 * z * (dR[0] + dR[4]) + w * (dR[3] - dR[1]));
  gq[3] = 2 * (x * (dR[7] - dR[5]) + y * (dR[2] - dR[6]) + z * (dR[3] - dR[1]));
}

struct Cov2DTerms {
  float t[3], M[6], J[6], x_mul, y_mul;
};

// View-space mean with the 1.3 x FoV clamp, the projection Jacobian J and M = J W (W = rotation block of Tw2v).
__device__ __forceinline__ void cov2d_terms(const float* mean, float fx, float fy, float tanx, float tany,
                                            const float* V, Cov2DTerms& o) {
#pragma clang fp contract(off)
#pragma unroll
  for (int a = 0; a < 3; ++a)
    o.t[a] = V[4 * a] * mean[0] + V[4 * a + 1] * mean[1] + V[4 * a + 2] * mean[2] + V[4 * a + 3];
  const float limx = 1.3f * tanx * o.t[2], limy = 1.3f * tany * o.t[2];
  o.x_mul = (o.t[0] < -limx || o.t[0] > limx) ? 0.0f : 1.0f;
  o.y_mul = (o.t[1] < -limy || o.t[1] > limy) ? 0.0f : 1.0f;
  o.t[0]  = fminf(fmaxf(o.t[0], -limx), limx);
  o.t[1]  = fminf(fmaxf(o.t[1], -limy), limy);
  const float tz = o.t[2];
  const float J[6] = {fx / tz, 0.0f, -(fx * o.t[0]) / (tz * tz), 0.0f, fy / tz, -(fy * o.t[1]) / (tz * tz)};
#pragma unroll
  for (int k = 0; k < 6; ++k) o.J[k] = J[k];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      float s = 0.0f;
#pragma unroll
      for (int k = 0; k < 3; ++k) s += J[i * 3 + k] * V[4 * k + j];
      o.M[i * 3 + j] = s;
    }
}

// M cov3D M^T without the low-pass term -> (a, b, c) of the symmetric 2x2
__device__ __forceinline__ void cov2d_product(const float* M, const float* c, float* out) {
#pragma clang fp contract(off)
  const float Vrk[9] = {c[0], c[1], c[2], c[1], c[3], c[4], c[2], c[4], c[5]};
  float tmp[6];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      float s = 0.0f;
#pragma unroll
      for (int k = 0; k < 3; ++k) s += M[i * 3 + k] * Vrk[k * 3 + j];
      tmp[i * 3 + j] = s;
    }
  float cov[4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      float s = 0.0f;
#pragma unroll
      for (int k = 0; k < 3; ++k) s += tmp[i * 3 + k] * M[j * 3 + k];
      cov[i * 2 + j] = s;
    }
  out[0] = cov[0], out[1] = cov[1], out[2] = cov[3];
}

// dL/dcov2D = (da, db, dc) (b is the one stored off-diagonal entry) -> dL/dcov3D (6), dL/dmean (3) and, when g_vm is
// given, this point's share of dL/d(view matrix rows 0-2) (12 values, row-major with the translation in column 3;
// gaussian_compute_cov2D.cu:163-183), ADDED to g_vm.
__device__ __forceinline__ void cov2d_backward_cov(const Cov2DTerms& k, const float* mean, const float* c3, float fx,
                                                   float fy, const float* V, float da, float db, float dc,
                                                   float* g_cov3D, float* g_mean, float* g_vm = nullptr) {
#pragma clang fp contract(off)
  const float* M = k.M;
  g_cov3D[0] = (M[0] * M[0] * da + M[0] * M[3] * db + M[3] * M[3] * dc);
  g_cov3D[3] = (M[1] * M[1] * da + M[1] * M[4] * db + M[4] * M[4] * dc);
  g_cov3D[5] = (M[2] * M[2] * da + M[2] * M[5] * db + M[5] * M[5] * dc);
  g_cov3D[1] = 2 * M[0] * M[1] * da + (M[0] * M[4] + M[1] * M[3]) * db + 2 * M[3] * M[4] * dc;
  g_cov3D[2] = 2 * M[0] * M[2] * da + (M[0] * M[5] + M[2] * M[3]) * db + 2 * M[3] * M[5] * dc;
  g_cov3D[4] = 2 * M[1] * M[2] * da + (M[1] * M[5] + M[2] * M[4]) * db + 2 * M[4] * M[5] * dc;
  float dT[6];
  dT[0] = 2 * (M[0] * c3[0] + M[1] * c3[1] + M[2] * c3[2]) * da + (M[3] * c3[0] + M[4] * c3[1] + M[5] * c3[2]) * db;
  dT[1] = 2 * (M[0] * c3[1] + M[1] * c3[3] + M[2] * c3[4]) * da + (M[3] * c3[1] + M[4] * c3[3] + M[5] * c3[4]) * db;
  dT[2] = 2 * (M[0] * c3[2] + M[1] * c3[4] + M[2] * c3[5]) * da + (M[3] * c3[2] + M[4] * c3[4] + M[5] * c3[5]) * db;
  dT[3] = 2 * (M[3] * c3[0] + M[4] * c3[1] + M[5] * c3[2]) * dc + (M[0] * c3[0] + M[1] * c3[1] + M[2] * c3[2]) * db;
  dT[4] = 2 * (M[3] * c3[1] + M[4] * c3[3] + M[5] * c3[4]) * dc + (M[0] * c3[1] + M[1] * c3[3] + M[2] * c3[4]) * db;
  dT[5] = 2 * (M[3] * c3[2] + M[4] * c3[4] + M[5] * c3[5]) * dc + (M[0] * c3[2] + M[1] * c3[4] + M[2] * c3[5]) * db;
  const float R[9] = {V[0], V[1], V[2], V[4], V[5], V[6], V[8], V[9], V[10]};
  const float dJ00 = dT[0] * R[0] + dT[1] * R[1] + dT[2] * R[2];
  const float dJ02 = dT[0] * R[6] + dT[1] * R[7] + dT[2] * R[8];
  const float dJ11 = dT[3] * R[3] + dT[4] * R[4] + dT[5] * R[5];
  const float dJ12 = dT[3] * R[6] + dT[4] * R[7] + dT[5] * R[8];
  const float tz = 1.0f / k.t[2], tz2 = tz * tz, tz3 = tz2 * tz;
  const float dtx = k.x_mul * -fx * tz2 * dJ02;
  const float dty = k.y_mul * -fy * tz2 * dJ12;
  const float dtz =
      -fx * tz2 * dJ00 - fy * tz2 * dJ11 + (2 * fx * k.t[0]) * tz3 * dJ02 + (2 * fy * k.t[1]) * tz3 * dJ12;
#pragma unroll
  for (int a2 = 0; a2 < 3; ++a2) g_mean[a2] = V[a2] * dtx + V[4 + a2] * dty + V[8 + a2] * dtz;
  if (g_vm) {
    const float dt[3] = {dtx, dty, dtz};
#pragma unroll
    for (int i = 0; i < 3; ++i) {
#pragma unroll
      for (int j = 0; j < 3; ++j) g_vm[4 * i + j] += k.J[i] * dT[j] + k.J[3 + i] * dT[3 + j] + dt[i] * mean[j];
      g_vm[4 * i + 3] += dt[i];
    }
  }
}

// dL/dconic -> dL/dcov3D (6) and dL/dmean (3); false when the covariance determinant is exactly zero.
__device__ __forceinline__ bool cov2d_backward(const float* mean, const float* c3, float fx, float fy, float tanx,
                                               float tany, const float* V, const float* g_conic, float* g_cov3D,
                                               float* g_mean, float* g_vm = nullptr) {
#pragma clang fp contract(off)
  Cov2DTerms k;
  cov2d_terms(mean, fx, fy, tanx, tany, V, k);
  float cov[3];
  cov2d_product(k.M, c3, cov);
  const float a = cov[0] + 0.3f, b = cov[1], c = cov[2] + 0.3f;
  const float denom = a * c - b * b;
  if (denom == 0.0f) return false;
  const float denom2inv = 1.0f / ((denom * denom) + 0.0000001f);
  const float tt = c * g_conic[0] - b * g_conic[1] + a * g_conic[2];
  const float da = denom2inv * (-c * tt + denom * g_conic[2]);
  const float dc = denom2inv * (-a * tt + denom * g_conic[0]);
  const float db = denom2inv * (2.0f * b * tt - denom * g_conic[1]);
  cov2d_backward_cov(k, mean, c3, fx, fy, V, da, db, dc, g_cov3D, g_mean, g_vm);
  return true;
}

struct Projected {
  float pv[3], proj[3], pw, ph[4];
};

__device__ __forceinline__ void project(const float* p, const float* Tw2v, const float* Tv2c, Projected& o) {
#pragma clang fp contract(off)
#pragma unroll
  for (int a = 0; a < 3; ++a)
    o.pv[a] = Tw2v[4 * a] * p[0] + Tw2v[4 * a + 1] * p[1] + Tw2v[4 * a + 2] * p[2] + Tw2v[4 * a + 3];
#pragma unroll
  for (int a = 0; a < 4; ++a)
    o.ph[a] = Tv2c[4 * a] * o.pv[0] + Tv2c[4 * a + 1] * o.pv[1] + Tv2c[4 * a + 2] * o.pv[2] + Tv2c[4 * a + 3];
  o.pw = 1.0f / (o.ph[3] + 0.0000001f);
  o.proj[0] = o.ph[0] * o.pw, o.proj[1] = o.ph[1] * o.pw, o.proj[2] = o.ph[2] * o.pw;
}

struct Screen {
  float px, py, radius, conic[3], depth;
  int area;
};

// Everything between the frustum test and the SH colour; false = rejected.
// cov2D_given: a pre-computed 2D covariance, taken as it is (gaussian_preprocess.cu:76-78).
__device__ __forceinline__ bool screen_geometry(int W, int H, int gx, int gy, bool is_opengl, const float* p,
                                                const Projected& pr, const float* c3, const float* cov2D_given,
                                                float fx, float fy, float tanx, float tany, const float* Tw2v,
                                                Screen& o) {
#pragma clang fp contract(off)
  float cov[3];
  if (cov2D_given) {
    cov[0] = cov2D_given[0], cov[1] = cov2D_given[1], cov[2] = cov2D_given[2];
  } else {
    Cov2DTerms k;
    cov2d_terms(p, fx, fy, tanx, tany, Tw2v, k);
    cov2d_product(k.M, c3, cov);
    cov[0] += 0.3f, cov[2] += 0.3f;
  }
  const float det = cov[0] * cov[2] - cov[1] * cov[1];
  if (det == 0.0f) return false;
  const float mid = 0.5f * (cov[0] + cov[2]);
  const float l1  = mid + sqrtf(fmaxf(0.1f, mid * mid - det));
  const float l2  = mid - sqrtf(fmaxf(0.1f, mid * mid - det));
  o.radius = ceilf(3.0f * sqrtf(fmaxf(l1, l2)));
  if (is_opengl) o.px = (1.0f + pr.proj[0]) * 0.5f * (float) W, o.py = (1.0f + -pr.proj[1]) * 0.5f * (float) H;
  else o.px = (1.0f + pr.proj[0]) * 0.5f * (float) W - 0.5f, o.py = (1.0f + pr.proj[1]) * 0.5f * (float) H - 0.5f;
  const TileRect r = tile_rect(o.px, o.py, f2i_sat(o.radius), gx, gy);
  o.area = (r.y1 - r.y0) * (r.x1 - r.x0);
  if (o.area == 0) return false;
  const float det_inv = 1.0f / det;
  o.conic[0] = cov[2] * det_inv, o.conic[1] = -cov[1] * det_inv, o.conic[2] = cov[0] * det_inv;
  o.depth = is_opengl ? pr.proj[2] : pr.pv[2];
  return true;
}

// kWave: complete degree-3 rows in one 16-byte aligned [P,16,3] tensor, moved by each wavefront on its own.
template <int kSh, bool kWave>
__global__ void __launch_bounds__(256) gs3d_preprocess_forward_kernel(int P, int W, int H, int sh_degree, int n_sh,
    int is_opengl, const float* __restrict__ means3D, const float* __restrict__ scales,
    const float4* __restrict__ rotations, const float* __restrict__ opacities, const float* __restrict__ shs,
    const float* __restrict__ sh_rest, const float* __restrict__ Tw2v_g, const float* __restrict__ Tv2c_g,
    const float* __restrict__ campos, float tanx, float tany, const uint8_t* __restrict__ culling,
    const float* __restrict__ cov3D_precomp, const float* __restrict__ cov2D_precomp,
    int means2D_preserve, float2* __restrict__ means2D, float* __restrict__ depths, float* __restrict__ colors,
    int32_t* __restrict__ radii, int32_t* __restrict__ tiles_touched, float* __restrict__ cov3Ds,
    float4* __restrict__ conic_opacity) {
  constexpr bool kStage = kSh == 16;
  __shared__ float s_Tw2v[16], s_Tv2c[16];
  __shared__ float s_rows[kStage ? kShStageRows * kShStageStride : 1];
  __shared__ unsigned char s_flag[kShStageRows];
  if (threadIdx.x < 16) s_Tw2v[threadIdx.x] = Tw2v_g[threadIdx.x], s_Tv2c[threadIdx.x] = Tv2c_g[threadIdx.x];
  __syncthreads();
  const int i      = blockIdx.x * blockDim.x + threadIdx.x;
  const bool valid = i < P;
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const float fx = 0.5f * (float) W / tanx, fy = 0.5f * (float) H / tany;

  bool ok = false;
  float p[3] = {0, 0, 0}, c3[6] = {0, 0, 0, 0, 0, 0}, rgb[3] = {0, 0, 0};
  Screen sc = {};
  if (valid) p[0] = means3D[3 * (size_t) i], p[1] = means3D[3 * (size_t) i + 1], p[2] = means3D[3 * (size_t) i + 2];
  const int wave_base = blockIdx.x * blockDim.x + (threadIdx.x & ~63);
  float* s_wave_rows  = &s_rows[kWave ? (threadIdx.x & ~63) * kShStageStride : 0];
  ShWaveRows sh_regs;
  unsigned long long wanted = 0;
  if (kWave) {  // the fetch of the rows is in flight during the geometry
    wanted = __ballot(valid && !(culling && culling[i]));
    if (wanted) wave_fetch_sh_rows(sh_regs, wanted, wave_base, (const float4*) shs);
  }
  do {
    if (!valid || (culling && culling[i])) break;
    float Tw2v[16], Tv2c[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) Tw2v[k] = s_Tw2v[k], Tv2c[k] = s_Tv2c[k];
    Projected pr;
    project(p, Tw2v, Tv2c, pr);
    if (is_opengl ? (pr.proj[2] < -1.0f || pr.proj[2] > 1.0f) : pr.pv[2] <= 0.2f) break;
    float cov2[3] = {0, 0, 0};
    if (cov2D_precomp) {
#pragma unroll
      for (int k = 0; k < 3; ++k) cov2[k] = cov2D_precomp[3 * (size_t) i + k];
    } else if (cov3D_precomp) {
#pragma unroll
      for (int k = 0; k < 6; ++k) c3[k] = cov3D_precomp[6 * (size_t) i + k];
    } else {
      const float s[3] = {scales[3 * (size_t) i], scales[3 * (size_t) i + 1], scales[3 * (size_t) i + 2]};
      cov3d_forward(s, rotations[i], c3);  // kept even when a later test rejects the Gaussian, as in the reference
    }
    ok = screen_geometry(W, H, gx, gy, is_opengl != 0, p, pr, c3, cov2D_precomp ? cov2 : nullptr, fx, fy, tanx, tany,
                         Tw2v, sc);
  } while (false);

  if (sh_degree >= 0) {
    const int n = sh_count(sh_degree);
    if (kWave) {
      if (wanted) wave_rows_to_lds(sh_regs, s_wave_rows);
      wave_lds_sync();
    } else if (kStage) {
      s_flag[threadIdx.x] = ok;
      __syncthreads();
      stage_sh_rows(s_rows, s_flag, blockIdx.x * blockDim.x, P, n, n_sh, shs, sh_rest);
      __syncthreads();
    }
    if (ok) {
      float x, y, z, Y[kSh];
      view_dir(p, campos, x, y, z);
      sh_eval(sh_degree, x, y, z, Y);
      const float* c0 = kStage ? &s_rows[threadIdx.x * kShStageStride] : shs + (size_t) i * (sh_rest ? 1 : n_sh) * 3;
      const float* cr = kStage ? c0 : (sh_rest ? sh_rest + (size_t) i * n_sh * 3 - 3 : c0);
      float r = c0[0] * Y[0], g = c0[1] * Y[0], b = c0[2] * Y[0];
      for (int l = 1; l < n; ++l) r += cr[3 * l] * Y[l], g += cr[3 * l + 1] * Y[l], b += cr[3 * l + 2] * Y[l];
      rgb[0] = fmaxf(0.0f, r + 0.5f), rgb[1] = fmaxf(0.0f, g + 0.5f), rgb[2] = fmaxf(0.0f, b + 0.5f);
    }
  }
  if (!valid) return;
  if (cov3Ds)  // absent with a pre-computed 3D covariance: the caller hands that tensor on as the operator's output
#pragma unroll
    for (int k = 0; k < 6; ++k) cov3Ds[6 * (size_t) i + k] = c3[k];
  if (sh_degree >= 0) {
    colors[3 * (size_t) i] = rgb[0], colors[3 * (size_t) i + 1] = rgb[1], colors[3 * (size_t) i + 2] = rgb[2];
  }
  depths[i]        = ok ? sc.depth : 0.0f;
  radii[i]         = ok ? f2i_sat(sc.radius) : 0;
  tiles_touched[i] = ok ? sc.area : 0;
  if (ok || !means2D_preserve) means2D[i] = ok ? make_float2(sc.px, sc.py) : make_float2(0.0f, 0.0f);
  conic_opacity[i] = ok ? make_float4(sc.conic[0], sc.conic[1], sc.conic[2], opacities[i]) : make_float4(0, 0, 0, 0);
}

template <int kSh, bool kWave>
__global__ void __launch_bounds__(256) gs3d_preprocess_backward_kernel(int P, int W, int H, int sh_degree, int n_sh,
    int is_opengl, const float* __restrict__ means3D, const float* __restrict__ scales,
    const float4* __restrict__ rotations, const float* __restrict__ shs, const float* __restrict__ sh_rest,
    const float* __restrict__ Tw2v_g, const float* __restrict__ Tv2c_g, const float* __restrict__ campos, float tanx,
    float tany, const int32_t* __restrict__ radii, const float* __restrict__ colors,
    const float* __restrict__ cov3Ds, const float* __restrict__ cov2Ds, float2* __restrict__ grad_mean2D,
    const float* __restrict__ grad_colors,
    const float4* __restrict__ grad_conic, float* __restrict__ g_means3D, float* __restrict__ g_scales,
    float4* __restrict__ g_rot, float* __restrict__ g_opac, float* __restrict__ g_shs, float* __restrict__ g_sh_rest,
    float* __restrict__ g_cov3D, float* __restrict__ g_Tw2v, float* __restrict__ g_campos) {
  constexpr bool kStage = kSh == 16;
  __shared__ float s_Tw2v[16], s_Tv2c[16];
  __shared__ float s_rows[kStage ? kShStageRows * kShStageStride : 1];
  __shared__ unsigned char s_flag[kShStageRows];
  if (threadIdx.x < 16) s_Tw2v[threadIdx.x] = Tw2v_g[threadIdx.x], s_Tv2c[threadIdx.x] = Tv2c_g[threadIdx.x];
  __syncthreads();
  const int i      = blockIdx.x * blockDim.x + threadIdx.x;
  const bool valid = i < P;
  const bool vis   = valid && radii[i] > 0;
  const int n      = sh_degree >= 0 ? sh_count(sh_degree) : 0;
  const int m1     = sh_rest ? 1 : n_sh;
  float* my_row    = &s_rows[kStage ? threadIdx.x * kShStageStride : 0];
  const float fx = 0.5f * (float) W / tanx, fy = 0.5f * (float) H / tany;
  const int wave_base = blockIdx.x * blockDim.x + (threadIdx.x & ~63);
  float* s_wave_rows  = &s_rows[kWave ? (threadIdx.x & ~63) * kShStageStride : 0];
  if (kWave) {
    const unsigned long long wanted = __ballot(vis);
    if (wanted) {
      ShWaveRows sh_regs;
      wave_fetch_sh_rows(sh_regs, wanted, wave_base, (const float4*) shs);
      wave_rows_to_lds(sh_regs, s_wave_rows);
    }
    wave_lds_sync();
  } else if (kStage && sh_degree >= 0) {
    s_flag[threadIdx.x] = vis;
    __syncthreads();
    stage_sh_rows(s_rows, s_flag, blockIdx.x * blockDim.x, P, n, n_sh, shs, sh_rest);
    __syncthreads();
  }
  // this lane's share of the camera gradients: dL/dTw2v rows 0-2 (12 values) and dL/dcampos (3)
  float cam[15];
#pragma unroll
  for (int k = 0; k < 15; ++k) cam[k] = 0.0f;
  const int cov_w = cov2Ds ? 3 : 6;  // columns of g_cov3D
  if (vis) {
    float Tw2v[16], Tv2c[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) Tw2v[k] = s_Tw2v[k], Tv2c[k] = s_Tv2c[k];
    const float p[3] = {means3D[3 * (size_t) i], means3D[3 * (size_t) i + 1], means3D[3 * (size_t) i + 2]};
    float gm[3], gcov[6] = {0, 0, 0, 0, 0, 0};
    {
#pragma clang fp contract(off)
      Projected pr;
      project(p, Tw2v, Tv2c, pr);
      const float2 g2 = grad_mean2D[i];
      const float du = (0.5f * (float) W) * g2.x, dv = ((is_opengl ? -0.5f : 0.5f) * (float) H) * g2.y;
      grad_mean2D[i] = make_float2(du, dv);
      const float tmp1 = (pr.ph[0] * du + pr.ph[1] * dv) * pr.pw * pr.pw;
      float dpv[3];
#pragma unroll
      for (int a = 0; a < 3; ++a) dpv[a] = (Tv2c[a] * du + Tv2c[4 + a] * dv) * pr.pw - Tv2c[12 + a] * tmp1;
#pragma unroll
      for (int a = 0; a < 3; ++a) gm[a] = Tw2v[a] * dpv[0] + Tw2v[4 + a] * dpv[1] + Tw2v[8 + a] * dpv[2];
      const float4 gc = grad_conic[i];
      g_opac[i] = gc.w;
      const float gcv[3] = {gc.x, gc.y, gc.z};
      if (cov2Ds) {
        // a pre-computed 2D covariance: the conic's derivative, nothing reaches the mean (gaussian_preprocess.cu:293-301)
        if (g_cov3D) {
          const float a = cov2Ds[3 * (size_t) i], b = cov2Ds[3 * (size_t) i + 1], c = cov2Ds[3 * (size_t) i + 2];
          const float denom = a * c - b * b;
          const float denom2inv = 1.0f / ((denom * denom) + 0.0000001f);
          const float tt = c * gcv[0] - b * gcv[1] + a * gcv[2];
          g_cov3D[3 * (size_t) i + 0] = denom2inv * (-c * tt + denom * gcv[2]);
          g_cov3D[3 * (size_t) i + 2] = denom2inv * (-a * tt + denom * gcv[0]);
          g_cov3D[3 * (size_t) i + 1] = denom2inv * (2.0f * b * tt - denom * gcv[1]);
        }
      } else {
        float c3[6], gmc[3];
#pragma unroll
        for (int k = 0; k < 6; ++k) c3[k] = cov3Ds[6 * (size_t) i + k];
        if (cov2d_backward(p, c3, fx, fy, tanx, tany, Tw2v, gcv, gcov, gmc, g_Tw2v ? cam : nullptr)) {
#pragma unroll
          for (int a = 0; a < 3; ++a) gm[a] += gmc[a];
        }
      }
      if (g_Tw2v) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
#pragma unroll
          for (int b = 0; b < 3; ++b) cam[4 * a + b] += p[b] * dpv[a];
          cam[4 * a + 3] += dpv[a];
        }
      }
    }
    if (g_cov3D && !cov2Ds)
#pragma unroll
      for (int k = 0; k < 6; ++k) g_cov3D[6 * (size_t) i + k] = gcov[k];
    if (sh_degree >= 0) {
      float x, y, z, Y[kSh], tl[kSh];
      const float nn = view_dir(p, campos, x, y, z);
      sh_eval(sh_degree, x, y, z, Y);
      float g[3];
#pragma unroll
      for (int c = 0; c < 3; ++c) g[c] = grad_colors[3 * (size_t) i + c] * (float) (colors[3 * (size_t) i + c] > 0);
      const float* c0 = kStage ? my_row : shs + (size_t) i * m1 * 3;
      const float* cr = kStage ? my_row : (sh_rest ? sh_rest + (size_t) i * n_sh * 3 - 3 : c0);
      float* o0  = kStage ? my_row : (g_shs ? g_shs + (size_t) i * m1 * 3 : nullptr);
      float* orr = kStage ? my_row
                          : (sh_rest ? (g_sh_rest ? g_sh_rest + (size_t) i * n_sh * 3 - 3 : nullptr) : o0);
      if (o0) o0[0] = g[0] * Y[0], o0[1] = g[1] * Y[0], o0[2] = g[2] * Y[0];
      tl[0] = 0.0f;
      for (int l = 1; l < n; ++l) {
        tl[l] = g[0] * cr[3 * l] + g[1] * cr[3 * l + 1] + g[2] * cr[3 * l + 2];
        if (orr) orr[3 * l] = g[0] * Y[l], orr[3 * l + 1] = g[1] * Y[l], orr[3 * l + 2] = g[2] * Y[l];
      }
      if (!kStage && orr) {
        for (int l = n; l < (sh_rest ? n_sh + 1 : n_sh); ++l)
          orr[3 * l] = 0.0f, orr[3 * l + 1] = 0.0f, orr[3 * l + 2] = 0.0f;
      }
      float dx = 0, dy = 0, dz = 0;
      sh_grad_accumulate(sh_degree, x, y, z, tl, dx, dy, dz);
      const float vx = p[0] - campos[0], vy = p[1] - campos[1], vz = p[2] - campos[2];
      const float tt = -(vx * dx + vy * dy + vz * dz) * nn * nn * nn;
      const float gd[3] = {dx * nn + tt * vx, dy * nn + tt * vy, dz * nn + tt * vz};
      gm[0] = gm[0] + gd[0];
      gm[1] = gm[1] + gd[1];
      gm[2] = gm[2] + gd[2];
      cam[12] = -gd[0], cam[13] = -gd[1], cam[14] = -gd[2];  // the view direction is normalize(p - campos)
    }
    g_means3D[3 * (size_t) i] = gm[0], g_means3D[3 * (size_t) i + 1] = gm[1], g_means3D[3 * (size_t) i + 2] = gm[2];
    if (g_scales || g_rot) {
      const float s[3] = {scales[3 * (size_t) i], scales[3 * (size_t) i + 1], scales[3 * (size_t) i + 2]};
      float gs[3], gq[4];
      cov3d_backward(s, rotations[i], gcov, gs, gq);
      if (g_scales)
        g_scales[3 * (size_t) i] = gs[0], g_scales[3 * (size_t) i + 1] = gs[1], g_scales[3 * (size_t) i + 2] = gs[2];
      if (g_rot) g_rot[i] = make_float4(gq[0], gq[1], gq[2], gq[3]);
    }
  } else if (valid) {
    g_opac[i] = 0.0f;
    g_means3D[3 * (size_t) i] = 0.0f, g_means3D[3 * (size_t) i + 1] = 0.0f, g_means3D[3 * (size_t) i + 2] = 0.0f;
    if (g_scales) g_scales[3 * (size_t) i] = 0.0f, g_scales[3 * (size_t) i + 1] = 0.0f, g_scales[3 * (size_t) i + 2] = 0.0f;
    if (g_rot) g_rot[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (g_cov3D)
      for (int k = 0; k < cov_w; ++k) g_cov3D[(size_t) cov_w * i + k] = 0.0f;
    if (sh_degree >= 0) {
      if (kStage) {
        for (int c = 0; c < n * 3; ++c) my_row[c] = 0.0f;
      } else {
        if (g_shs)
          for (int c = 0; c < m1 * 3; ++c) g_shs[(size_t) i * m1 * 3 + c] = 0.0f;
        if (g_sh_rest)
          for (int c = 0; c < n_sh * 3; ++c) g_sh_rest[(size_t) i * n_sh * 3 + c] = 0.0f;
      }
    }
  }
  if (g_Tw2v || g_campos) {
    // sums over the wavefront, then one atomic per value and wavefront (the reference: one per value and block,
    // gaussian_preprocess.cu:340-355); rows of invisible points contribute zeros
#pragma unroll
    for (int k = 0; k < 15; ++k) {
      float v = cam[k];
#pragma unroll
      for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
      cam[k] = v;
    }
    if ((threadIdx.x & 63) == 0) {
      if (g_Tw2v)
#pragma unroll
        for (int k = 0; k < 12; ++k)
          if (cam[k] != 0.0f) atomicAdd(&g_Tw2v[k], cam[k]);
      if (g_campos)
#pragma unroll
        for (int k = 0; k < 3; ++k)
          if (cam[12 + k] != 0.0f) atomicAdd(&g_campos[k], cam[12 + k]);
    }
  }
  if (kWave) {
    wave_lds_sync();
    wave_rows_to_global(s_wave_rows, wave_base, P, (float4*) g_shs);
  } else if (kStage && sh_degree >= 0 && (g_shs || g_sh_rest)) {
    __syncthreads();
    unstage_sh_grads(s_rows, blockIdx.x * blockDim.x, P, n, n_sh, sh_rest != nullptr, g_shs, g_sh_rest);
  }
}

// ---- the covariance steps as operators of their own --------------------------------------------------------------
__global__ void __launch_bounds__(256) cov3d_forward_kernel(int N, const float4* __restrict__ q,
                                                            const float* __restrict__ s, float* __restrict__ cov3D) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= N) return;
  const float sc[3] = {s[3 * (size_t) i], s[3 * (size_t) i + 1], s[3 * (size_t) i + 2]};
  float c[6];
  cov3d_forward(sc, q[i], c);
#pragma unroll
  for (int k = 0; k < 6; ++k) cov3D[6 * (size_t) i + k] = c[k];
}

__global__ void __launch_bounds__(256) cov3d_backward_kernel(int N, const float4* __restrict__ q,
    const float* __restrict__ s, const float* __restrict__ g, float4* __restrict__ gq, float* __restrict__ gs) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= N) return;
  const float sc[3] = {s[3 * (size_t) i], s[3 * (size_t) i + 1], s[3 * (size_t) i + 2]};
  float gc[6], os[3], oq[4];
#pragma unroll
  for (int k = 0; k < 6; ++k) gc[k] = g[6 * (size_t) i + k];
  cov3d_backward(sc, q[i], gc, os, oq);
  gq[i] = make_float4(oq[0], oq[1], oq[2], oq[3]);
#pragma unroll
  for (int k = 0; k < 3; ++k) gs[3 * (size_t) i + k] = os[k];
}

__global__ void __launch_bounds__(256) cov2d_forward_kernel(int N, const float* __restrict__ cov3D,
    const float* __restrict__ mean, const float* __restrict__ Tw2v, float fx, float fy, float tanx, float tany,
    float* __restrict__ cov2D) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= N) return;
  float V[16], c3[6], o[3];
#pragma unroll
  for (int k = 0; k < 16; ++k) V[k] = Tw2v[k];
#pragma unroll
  for (int k = 0; k < 6; ++k) c3[k] = cov3D[6 * (size_t) i + k];
  const float p[3] = {mean[3 * (size_t) i], mean[3 * (size_t) i + 1], mean[3 * (size_t) i + 2]};
  Cov2DTerms t;
  cov2d_terms(p, fx, fy, tanx, tany, V, t);
  cov2d_product(t.M, c3, o);
  cov2D[3 * (size_t) i] = o[0] + 0.3f, cov2D[3 * (size_t) i + 1] = o[1], cov2D[3 * (size_t) i + 2] = o[2] + 0.3f;
}

__global__ void __launch_bounds__(256) cov2d_backward_kernel(int N, const float* __restrict__ cov3D,
    const float* __restrict__ mean, const float* __restrict__ Tw2v, float fx, float fy, float tanx, float tany,
    const float* __restrict__ g, float* __restrict__ g_cov3D, float* __restrict__ g_mean, float* __restrict__ g_vm) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  float vm[12];
#pragma unroll
  for (int k = 0; k < 12; ++k) vm[k] = 0.0f;
  if (i < N) {
    float V[16], c3[6], gc[6], gm[3];
#pragma unroll
    for (int k = 0; k < 16; ++k) V[k] = Tw2v[k];
#pragma unroll
    for (int k = 0; k < 6; ++k) c3[k] = cov3D[6 * (size_t) i + k];
    const float p[3] = {mean[3 * (size_t) i], mean[3 * (size_t) i + 1], mean[3 * (size_t) i + 2]};
    Cov2DTerms t;
    cov2d_terms(p, fx, fy, tanx, tany, V, t);
    cov2d_backward_cov(t, p, c3, fx, fy, V, g[3 * (size_t) i], g[3 * (size_t) i + 1], g[3 * (size_t) i + 2], gc, gm,
                       g_vm ? vm : nullptr);
#pragma unroll
    for (int k = 0; k < 6; ++k) g_cov3D[6 * (size_t) i + k] = gc[k];
#pragma unroll
    for (int k = 0; k < 3; ++k) g_mean[3 * (size_t) i + k] = gm[k];
  }
  if (g_vm) {  // gaussian_compute_cov2D.cu:223-227: added to the caller's buffer
#pragma unroll
    for (int k = 0; k < 12; ++k) {
      float v = vm[k];
#pragma unroll
      for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
      if ((threadIdx.x & 63) == 0 && v != 0.0f) atomicAdd(&g_vm[k], v);
    }
  }
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API int fsgs_gs_compute_cov3D_forward(int N, const float* q, const float* s, float* cov3D, void* stream) {
  FSGS_REQUIRE(N >= 0, "gs_compute_cov3D_forward: bad size");
  if (N == 0) return kOk;
  FSGS_REQUIRE(q && s && cov3D, "gs_compute_cov3D_forward: null pointer");
  hipLaunchKernelGGL(cov3d_forward_kernel, dim3(div_up(N, 256)), dim3(256), 0, (hipStream_t) stream, N,
                     (const float4*) q, s, cov3D);
  return check_launch("gs_compute_cov3D_forward");
}

FSGS_API int fsgs_gs_compute_cov3D_backward(int N, const float* q, const float* s, const float* g_cov3D, float* g_q,
                                            float* g_s, void* stream) {
  FSGS_REQUIRE(N >= 0, "gs_compute_cov3D_backward: bad size");
  if (N == 0) return kOk;
  FSGS_REQUIRE(q && s && g_cov3D && g_q && g_s, "gs_compute_cov3D_backward: null pointer");
  hipLaunchKernelGGL(cov3d_backward_kernel, dim3(div_up(N, 256)), dim3(256), 0, (hipStream_t) stream, N,
                     (const float4*) q, s, g_cov3D, (float4*) g_q, g_s);
  return check_launch("gs_compute_cov3D_backward");
}

FSGS_API int fsgs_gs_compute_cov2D_forward(int N, const float* cov3D, const float* mean, const float* Tw2v,
    double focal_x, double focal_y, double tan_fovx, double tan_fovy, float* cov2D, void* stream) {
  FSGS_REQUIRE(N >= 0, "gs_compute_cov2D_forward: bad size");
  if (N == 0) return kOk;
  FSGS_REQUIRE(cov3D && mean && Tw2v && cov2D, "gs_compute_cov2D_forward: null pointer");
  hipLaunchKernelGGL(cov2d_forward_kernel, dim3(div_up(N, 256)), dim3(256), 0, (hipStream_t) stream, N, cov3D, mean,
                     Tw2v, (float) focal_x, (float) focal_y, (float) tan_fovx, (float) tan_fovy, cov2D);
  return check_launch("gs_compute_cov2D_forward");
}

FSGS_API int fsgs_gs_compute_cov2D_backward(int N, const float* cov3D, const float* mean, const float* Tw2v,
    double focal_x, double focal_y, double tan_fovx, double tan_fovy, const float* g_cov2D, float* g_cov3D,
    float* g_mean, float* g_vm, void* stream) {
  FSGS_REQUIRE(N >= 0, "gs_compute_cov2D_backward: bad size");
  if (N == 0) return kOk;
  FSGS_REQUIRE(cov3D && mean && Tw2v && g_cov2D && g_cov3D && g_mean, "gs_compute_cov2D_backward: null pointer");
  hipLaunchKernelGGL(cov2d_backward_kernel, dim3(div_up(N, 256)), dim3(256), 0, (hipStream_t) stream, N, cov3D, mean,
                     Tw2v, (float) focal_x, (float) focal_y, (float) tan_fovx, (float) tan_fovy, g_cov2D, g_cov3D,
                     g_mean, g_vm);
  return check_launch("gs_compute_cov2D_backward");
}

FSGS_API int fsgs_gs_preprocess_forward(int P, int W, int H, int sh_degree, int n_sh, int is_opengl,
    const float* means3D, const float* scales, const float* rotations, const float* opacities, const float* shs,
    const float* sh_rest, const float* Tw2v, const float* Tv2c, const float* campos, double tan_fovx, double tan_fovy,
    const uint8_t* culling, const float* cov3D_precomp, const float* cov2D_precomp, int means2D_preserve,
    float* means2D, float* depths, float* colors, int32_t* radii, int32_t* tiles_touched, float* cov3Ds,
    float* conic_opacity, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0 && tan_fovx > 0 && tan_fovy > 0, "gs_preprocess_forward: bad sizes");
  FSGS_REQUIRE(sh_degree <= kMaxShDegree, "gs_preprocess_forward: sh_degree %d > %d not supported", sh_degree,
               kMaxShDegree);
  if (sh_degree >= 0)
    FSGS_REQUIRE(n_sh + (sh_rest ? 1 : 0) >= (sh_degree + 1) * (sh_degree + 1),
                 "gs_preprocess_forward: %d SH coefficients are too few for degree %d", n_sh, sh_degree);
  if (P == 0) return kOk;
  FSGS_REQUIRE(means3D && scales && rotations && opacities && shs && Tw2v && Tv2c && campos && means2D && depths &&
                   radii && tiles_touched && (cov3Ds || cov3D_precomp) && conic_opacity && (colors || sh_degree < 0),
               "gs_preprocess_forward: null pointer");
  const bool wave_rows = sh_degree == 3 && n_sh == 16 && !sh_rest && (uintptr_t) shs % 16 == 0;
  auto kernel = sh_degree > 3 ? gs3d_preprocess_forward_kernel<64, false>
                              : (wave_rows ? gs3d_preprocess_forward_kernel<16, true>
                                           : gs3d_preprocess_forward_kernel<16, false>);
  hipLaunchKernelGGL(kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P, W, H, sh_degree, n_sh,
                     is_opengl, means3D, scales, (const float4*) rotations, opacities, shs, sh_rest, Tw2v, Tv2c,
                     campos, (float) tan_fovx, (float) tan_fovy, culling, cov3D_precomp, cov2D_precomp, means2D_preserve,
                     (float2*) means2D, depths, colors, radii, tiles_touched, cov3D_precomp ? nullptr : cov3Ds,
                     (float4*) conic_opacity);
  return check_launch("gs_preprocess_forward");
}

FSGS_API int fsgs_gs_preprocess_backward(int P, int W, int H, int sh_degree, int n_sh, int is_opengl,
    const float* means3D, const float* scales, const float* rotations, const float* shs, const float* sh_rest,
    const float* Tw2v, const float* Tv2c, const float* campos, double tan_fovx, double tan_fovy, const int32_t* radii,
    const float* colors, const float* cov3Ds, const float* cov2Ds, float* grad_mean2D, const float* grad_colors,
    const float* grad_conic, float* g_means3D, float* g_scales, float* g_rot, float* g_opac, float* g_shs,
    float* g_sh_rest, float* g_cov, float* g_Tw2v, float* g_campos, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0 && tan_fovx > 0 && tan_fovy > 0, "gs_preprocess_backward: bad sizes");
  FSGS_REQUIRE(sh_degree <= kMaxShDegree, "gs_preprocess_backward: sh_degree %d > %d not supported", sh_degree,
               kMaxShDegree);
  if (P == 0) return kOk;
  FSGS_REQUIRE(means3D && scales && rotations && Tw2v && Tv2c && campos && radii && (cov3Ds || cov2Ds) &&
                   grad_mean2D && grad_conic && g_means3D && g_opac,
               "gs_preprocess_backward: null pointer");
  FSGS_REQUIRE(!cov2Ds || (!g_scales && !g_rot),
               "gs_preprocess_backward: no scale / rotation gradients with pre-computed 2D covariances");
  if (sh_degree >= 0)
    FSGS_REQUIRE(shs && colors && grad_colors, "gs_preprocess_backward: SH path needs shs, colors and grad_colors");
  const bool wave_rows = sh_degree == 3 && n_sh == 16 && !sh_rest && g_shs && (uintptr_t) shs % 16 == 0 &&
                         (uintptr_t) g_shs % 16 == 0;
  auto kernel = sh_degree > 3 ? gs3d_preprocess_backward_kernel<64, false>
                              : (wave_rows ? gs3d_preprocess_backward_kernel<16, true>
                                           : gs3d_preprocess_backward_kernel<16, false>);
  hipLaunchKernelGGL(kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P, W, H, sh_degree, n_sh,
                     is_opengl, means3D, scales, (const float4*) rotations, shs, sh_rest, Tw2v, Tv2c, campos,
                     (float) tan_fovx, (float) tan_fovy, radii, colors, cov3Ds, cov2Ds, (float2*) grad_mean2D,
                     grad_colors, (const float4*) grad_conic, g_means3D, g_scales, (float4*) g_rot, g_opac, g_shs,
                     g_sh_rest, g_cov, g_Tw2v, g_campos);
  return check_launch("gs_preprocess_backward");
}
