// TEST INFRASTRUCTURE ONLY (parity oracle). Never linked, imported or called by the product library.
//
// Scalar CPU restatement of the reference's "fast" 2DGS surfel path:
//   transform with intrinsics + adjugate   fast_2d_gs/_C/src/gaussian_splatting/gs_2d_fast_preprocess.cu:60-158
//   preprocess forward                     gs_2d_fast_preprocess.cu:160-262
//   fused binning with the corner test     gs_2d_fast_preprocess.cu:264-327 (duplicateWithKeys), :484-514 (ranges),
//                                          :711-778 (host: scan, sort on 32 + msb(T + 1) bits)
//   preprocess backward                    gs_2d_fast_preprocess.cu:536-609
//   blend forward (8 aux maps, snapshots)  fast_2d_gs/_C/src/gaussian_splatting/gs_2d_fast_redner.cu:22-271
//   blend backward, per-pixel form         gs_2d_fast_redner.cu:273-561
//   blend backward, per-splat form         gs_2d_fast_redner.cu:563-837 (same gradient with a different channel set:
//                                          no distortion gradient, M1/M2 maps as plain weighted sums, the M1 depth
//                                          term overwritten by the M2 one, :748-757)
//
// One documented deviation: the reference evaluates log2(opacity) in the corner test with PTX `lg2.approx.f32`
// (gs_2d_fast_preprocess.cu:48-52, :282); the oracle and the GPU kernel both evaluate log2 in double precision and
// round the result to the working type.
//
// Pinned by tests/test_oracle_fast.py: equivalence with the (independently pinned) standard path when the intrinsics
// equal (ndc2pix * Tv2c)[:3,:3] and the camera has no x/y translation, brute-force corner tests in double precision,
// and central finite differences.
#include "gs2d_shared.h"

#ifdef _OPENMP
#include <omp.h>
#endif

namespace oracle {

// gs_2d_fast_preprocess.cu:60-98
template <typename T>
static inline void fast_transmat(const T* p, const T* s, const T* q, const T* Tw2v, const T* Tv2s, T* M, T* normal) {
  const T x = q[0], y = q[1], z = q[2], w = q[3];
  T L[9];
  L[0] = (1 - 2 * (y * y + z * z)) * s[0];
  L[1] = 2 * (x * y - z * w) * s[1];
  L[2] = p[0];
  L[3] = (2 * (x * y + z * w)) * s[0];
  L[4] = (1 - 2 * (x * x + z * z)) * s[1];
  L[5] = p[1];
  L[6] = (2 * (x * z - y * w)) * s[0];
  L[7] = 2 * (x * w + y * z) * s[1];
  L[8] = p[2];
  const T t0 = 2 * (y * w + x * z), t1 = 2 * (y * z - x * w), t2 = 1 - 2 * (x * x + y * y);
  T t[9];
  for (int i = 0; i < 3; ++i)
    for (int j = 0; j < 3; ++j) {
      T res = 0;
      for (int k = 0; k < 3; ++k) res += Tw2v[i * 4 + k] * L[k * 3 + j];
      t[i * 3 + j] = res;
    }
  t[8] += Tw2v[11];  // only the z translation of the view matrix enters (:95)
  for (int i = 0; i < 9; ++i) M[i] = 0;
  for (int i = 0; i < 3; ++i)
    for (int j = 0; j < 3; ++j)
      for (int k = 0; k < 3; ++k) M[i * 3 + j] += Tv2s[i * 3 + k] * t[k * 3 + j];
  normal[0] = Tw2v[0] * t0 + Tw2v[1] * t1 + Tw2v[2] * t2;
  normal[1] = Tw2v[4] * t0 + Tw2v[5] * t1 + Tw2v[6] * t2;
  normal[2] = Tw2v[8] * t0 + Tw2v[9] * t1 + Tw2v[10] * t2;
}

// gs_2d_fast_preprocess.cu:100-140
template <typename T>
static inline void fast_transmat_backward(const T* s, const T* q, const T* Tw2v, const T* Tv2s, const T* gM,
                                          const T* gN, T* gp, T* gs, T* gq) {
  T gL[9] = {0}, dR[9];
  for (int i = 0; i < 3; ++i)
    for (int j = 0; j < 3; ++j)
      for (int k = 0; k < 3; ++k) gL[i * 3 + j] += Tv2s[k * 3 + i] * gM[k * 3 + j];
  for (int i = 0; i < 3; ++i)
    for (int j = 0; j < 3; ++j) {
      T res = 0;
      for (int k = 0; k < 3; ++k) res += Tw2v[k * 4 + i] * gL[k * 3 + j];
      dR[i * 3 + j] = res;
    }
  gp[0] = dR[2], gp[1] = dR[5], gp[2] = dR[8];
  dR[2] = gN[0] * Tw2v[0] + gN[1] * Tw2v[4] + gN[2] * Tw2v[8];
  dR[5] = gN[0] * Tw2v[1] + gN[1] * Tw2v[5] + gN[2] * Tw2v[9];
  dR[8] = gN[0] * Tw2v[2] + gN[1] * Tw2v[6] + gN[2] * Tw2v[10];
  const T x = q[0], y = q[1], z = q[2], w = q[3];
  gs[0] = dR[0] * (1 - 2 * (y * y + z * z)) + dR[3] * (2 * (x * y + z * w)) + dR[6] * (2 * (x * z - y * w));
  gs[1] = dR[1] * (2 * (x * y - z * w)) + dR[4] * (1 - 2 * (x * x + z * z)) + dR[7] * (2 * (x * w + y * z));
  dR[0] *= s[0], dR[1] *= s[1], dR[3] *= s[0], dR[4] *= s[1], dR[6] *= s[0], dR[7] *= s[1];
  // dL_quaternion_to_R, ops_3d.h:127-134
  gq[0] = 2 * (-2 * x * (dR[4] + dR[8]) + y * (dR[1] + dR[3]) + z * (dR[2] + dR[6]) + w * (dR[7] - dR[5]));
  gq[1] = 2 * (x * (dR[1] + dR[3]) - 2 * y * (dR[0] + dR[8]) + z * (dR[5] + dR[7]) + w * (dR[2] - dR[6]));
  gq[2] = 2 * (x * (dR[2] + dR[6]) + y * (dR[5] + dR[7]) - 2 * z * (dR[0] + dR[4]) + w * (dR[3] - dR[1]));
  gq[3] = 2 * (x * (dR[7] - dR[5]) + y * (dR[2] - dR[6]) + z * (dR[3] - dR[1]));
}

// gs_2d_fast_preprocess.cu:247-255: columns are the cross products M1xM2, M2xM0, M0xM1 (so p = IM (x, y, 1))
template <typename T>
static inline void adjugate(const T* m, T* a) {
  a[0] = m[4] * m[8] - m[7] * m[5];
  a[1] = m[7] * m[2] - m[1] * m[8];
  a[2] = m[1] * m[5] - m[4] * m[2];
  a[3] = m[6] * m[5] - m[3] * m[8];
  a[4] = m[0] * m[8] - m[6] * m[2];
  a[5] = m[3] * m[2] - m[0] * m[5];
  a[6] = m[3] * m[7] - m[6] * m[4];
  a[7] = m[6] * m[1] - m[0] * m[7];
  a[8] = m[0] * m[4] - m[3] * m[1];
}

template <typename T>
static void fast_preprocess_forward(int P, int W, int H, int sh_degree, int n_sh, const T* means3D, const T* scales,
                                    const T* rotations, const T* opacities, const T* shs, const T* sh_rest,
                                    const T* Tw2v, const T* Tv2s, const T* campos, const T* trans_precomp,
                                    const uint8_t* culling, int means2D_preserve, T* means2D, T* colors, T* trans_mat,
                                    T* inverse_m, T* normal_opacity, T* depths, int32_t* radii,
                                    int32_t* tiles_touched) {
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
#pragma omp parallel for schedule(static)
  for (int i = 0; i < P; ++i) {
    bool ok = false;
    T M[9] = {0}, nrm[3] = {0}, c2[2] = {0}, rgb[3] = {0}, depth = 0, radius = 0;
    int area = 0;
    do {
      if (culling && culling[i]) break;
      const T* p = means3D + 3 * i;
      const T pv[3] = {Tw2v[0] * p[0] + Tw2v[1] * p[1] + Tw2v[2] * p[2] + Tw2v[3],
                       Tw2v[4] * p[0] + Tw2v[5] * p[1] + Tw2v[6] * p[2] + Tw2v[7],
                       Tw2v[8] * p[0] + Tw2v[9] * p[1] + Tw2v[10] * p[2] + Tw2v[11]};
      if (pv[2] <= T(0.2)) break;
      if (!trans_precomp) fast_transmat(p, scales + 2 * i, rotations + 4 * i, Tw2v, Tv2s, M, nrm);
      else {
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
      if (area == 0) break;
      if (sh_degree >= 0)
        sh_to_rgb(sh_degree, p, campos, shs + (size_t) i * (sh_rest ? 1 : n_sh) * 3,
                  sh_rest ? sh_rest + (size_t) i * n_sh * 3 : nullptr, true, rgb);
      depth = pv[2];
      ok    = true;
    } while (false);
    T adj[9] = {0};
    if (ok) adjugate(M, adj);
    for (int k = 0; k < 9; ++k) {
      if (!trans_precomp || ok) trans_mat[9 * i + k] = ok ? M[k] : (trans_precomp ? trans_mat[9 * i + k] : T(0));
      inverse_m[9 * i + k] = adj[k];
    }
    if (sh_degree >= 0)
      for (int c = 0; c < 3; ++c) colors[3 * i + c] = ok ? rgb[c] : T(0);
    depths[i] = depth, radii[i] = ok ? f2i(radius) : 0, tiles_touched[i] = ok ? area : 0;
    if (ok || !means2D_preserve) means2D[2 * i] = ok ? c2[0] : T(0), means2D[2 * i + 1] = ok ? c2[1] : T(0);
    for (int a = 0; a < 3; ++a) normal_opacity[4 * i + a] = ok ? nrm[a] : T(0);
    normal_opacity[4 * i + 3] = ok ? opacities[i] : T(0);
  }
}

// Corner test of gs_2d_fast_preprocess.cu:277-304: the tile is kept iff the implicit conic
// W(u, v) = |IM (u,v,1)|_xy^2 + d (IM_2 . (u,v,1))^2 is <= 0 at one of its four corners, d = -2 ln2 (log2(254)+log2 o).
template <typename T>
struct CornerTest {
  T Wxx, Wyy, Wxy, Wx_, Wy_, W__;
  CornerTest(const T* IM, T opacity) {
    const T d = -T(2) * T(0.69314718055f) * (T(7.9886846867721655) + T(std::log2((double) opacity)));
    Wxx = IM[0] * IM[0] + IM[3] * IM[3] + d * IM[6] * IM[6];
    Wyy = IM[1] * IM[1] + IM[4] * IM[4] + d * IM[7] * IM[7];
    W__ = IM[2] * IM[2] + IM[5] * IM[5] + d * IM[8] * IM[8];
    Wxy = 2 * (IM[0] * IM[1] + IM[3] * IM[4] + d * IM[6] * IM[7]);
    Wx_ = 2 * (IM[0] * IM[2] + IM[3] * IM[5] + d * IM[6] * IM[8]);
    Wy_ = 2 * (IM[1] * IM[2] + IM[4] * IM[5] + d * IM[7] * IM[8]);
    Wxx = Wxx * kTile * kTile, Wyy = Wyy * kTile * kTile, Wxy = Wxy * kTile * kTile;
    Wx_ = Wx_ * kTile, Wy_ = Wy_ * kTile;
  }
  bool at(T u, T v) const { return Wxx * u * u + Wyy * v * v + Wxy * u * v + Wx_ * u + Wy_ * v + W__ <= 0; }
  bool tile(int x, int y) const {
    return at((T) x, (T) y) || at((T) (x + 1), (T) y) || at((T) x, (T) (y + 1)) || at((T) (x + 1), (T) (y + 1));
  }
};

static void fast_prepare_fill(int P, int W, int H, const float* means2D, const float* inverse_m, const float* depths,
                              const float* opacities, const int32_t* radii, const int64_t* offsets, int64_t R,
                              int64_t* ranges, int32_t* point_list, int64_t* keys_sorted_out) {
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const uint32_t T_ = (uint32_t) (gx * gy);
  std::vector<uint64_t> keys((size_t) R);
  std::vector<int32_t> vals((size_t) R);
  for (int i = 0; i < P; ++i) {
    if (radii[i] <= 0) continue;
    int64_t off          = i == 0 ? 0 : offsets[i - 1];
    const int64_t off_to = offsets[i];
    const Rect<float> r  = get_rect<float>(means2D[2 * i], means2D[2 * i + 1], radii[i], gx, gy);
    uint32_t bits;
    std::memcpy(&bits, depths + i, 4);
    const CornerTest<float> ct(inverse_m + 9 * (size_t) i, opacities[i]);
    for (int x = r.x0; x < r.x1; ++x)  // x-major here, unlike the standard path
      for (int y = r.y0; y < r.y1; ++y)
        if (ct.tile(x, y)) {
          keys[(size_t) off] = ((uint64_t) (uint32_t) (y * gx + x) << 32) | bits;
          vals[(size_t) off] = i;
          ++off;
        }
    for (; off < off_to; ++off) keys[(size_t) off] = (uint64_t) T_ << 32, vals[(size_t) off] = -1;  // padding
  }
  const uint32_t bit  = 32 + higher_msb(T_ + 1);
  const uint64_t mask = bit >= 64 ? ~0ull : ((1ull << bit) - 1);
  std::vector<int64_t> order((size_t) R);
  for (int64_t i = 0; i < R; ++i) order[(size_t) i] = i;
  std::stable_sort(order.begin(), order.end(),
                   [&](int64_t a, int64_t b) { return (keys[(size_t) a] & mask) < (keys[(size_t) b] & mask); });
  for (int64_t i = 0; i < (int64_t) T_ * 2; ++i) ranges[i] = 0;
  for (int64_t i = 0; i < R; ++i) {
    const uint64_t k = keys[(size_t) order[(size_t) i]];
    point_list[i]    = vals[(size_t) order[(size_t) i]];
    if (keys_sorted_out) keys_sorted_out[i] = (int64_t) k;
    const uint32_t cur = (uint32_t) (k >> 32);
    const bool valid   = cur < T_;
    if (i == 0) {
      if (valid) ranges[2 * cur] = 0;
    } else {
      const uint32_t prev = (uint32_t) (keys[(size_t) order[(size_t) i - 1]] >> 32);
      if (cur != prev) {
        ranges[2 * prev + 1] = i;
        if (valid) ranges[2 * cur] = i;
      }
    }
    if (i == R - 1 && valid) ranges[2 * cur + 1] = R;
  }
}

// gs_2d_fast_preprocess.cu:536-609
template <typename T>
static void fast_preprocess_backward(int P, int W, int H, int sh_degree, int n_sh, const T* means3D, const T* scales,
                                     const T* rotations, const T* shs, const T* sh_rest, const T* Tw2v, const T* Tv2s,
                                     const T* campos, const T* trans_mat, const int32_t* radii, const T* colors,
                                     T* grad_mean2D, const T* grad_trans, const T* grad_inv_m, const T* grad_colors,
                                     const T* grad_normal_opacity, T* g_means3D, T* g_scales, T* g_rot, T* g_opac,
                                     T* g_shs, T* g_sh_rest) {
#pragma omp parallel for schedule(static)
  for (int i = 0; i < P; ++i) {
    if (radii[i] <= 0) continue;
    g_opac[i] = grad_normal_opacity[4 * i + 3];
    const T* m = trans_mat + 9 * i;
    const T* gM = grad_inv_m + 9 * i;
    T gT[9];
    for (int k = 0; k < 9; ++k) gT[k] = grad_trans[9 * i + k];
#define MM(r, c) m[(r) * 3 + (c)]
#define GM(r, c) gM[(r) * 3 + (c)]
    gT[0] += GM(1, 1) * MM(2, 2) + GM(2, 2) * MM(1, 1) - GM(1, 2) * MM(1, 2) - GM(2, 1) * MM(2, 1);
    gT[1] += GM(0, 2) * MM(1, 2) + GM(2, 1) * MM(2, 0) - GM(0, 1) * MM(2, 2) - GM(2, 2) * MM(1, 0);
    gT[2] += GM(0, 1) * MM(2, 1) + GM(1, 2) * MM(1, 0) - GM(0, 2) * MM(1, 1) - GM(1, 1) * MM(2, 0);
    gT[3] += GM(1, 2) * MM(0, 2) + GM(2, 0) * MM(2, 1) - GM(1, 0) * MM(2, 2) - GM(2, 2) * MM(0, 1);
    gT[4] += GM(0, 0) * MM(2, 2) + GM(2, 2) * MM(0, 0) - GM(0, 2) * MM(0, 2) - GM(2, 0) * MM(2, 0);
    gT[5] += GM(0, 2) * MM(0, 1) + GM(1, 0) * MM(2, 0) - GM(0, 0) * MM(2, 1) - GM(1, 2) * MM(0, 0);
    gT[6] += GM(1, 0) * MM(1, 2) + GM(2, 1) * MM(0, 1) - GM(1, 1) * MM(0, 2) - GM(2, 0) * MM(1, 1);
    gT[7] += GM(0, 1) * MM(0, 2) + GM(2, 0) * MM(1, 0) - GM(0, 0) * MM(1, 2) - GM(2, 1) * MM(0, 0);
    gT[8] += GM(0, 0) * MM(1, 1) + GM(1, 1) * MM(0, 0) - GM(0, 1) * MM(0, 1) - GM(1, 0) * MM(1, 0);
#undef MM
#undef GM
    compute_aabb_backward(T(3.0), m, grad_mean2D + 2 * i, gT);
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
    fast_transmat_backward(scales + 2 * i, q, Tw2v, Tv2s, gT, gN, gp, gs, gq);
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
    const T depth = m[8];
    grad_mean2D[2 * i]     = gT[2] * depth * T(0.5) * T(W);  // the ACCUMULATED gradient here (:606-608)
    grad_mean2D[2 * i + 1] = gT[5] * depth * T(0.5) * T(H);
  }
}

// gs_2d_fast_redner.cu:22-271. extras has 8 channels: depth, normal xyz, median depth, distortion, M1, M2.
// Snapshot outputs (when bucket_offset != nullptr): state before every 32nd list entry, per pixel of the tile in
// row-major (16 x 16) order, for pixels that are still blending; sampled_aux has 8 channels, or 10 with optical flow
// (channels 8, 9 = the unnormalised flow sums, :141-144). Optical flow (trans_mat_t2 given, :247-255) is normalised by
// the final opacity, 0 where that is 0 (:259-263) -- the standard path divides by the sum of weights instead. The
// accum_* side outputs are those of the standard path (:236-246, the arg-max flag is never reset).
template <typename T>
static void fast_render_forward(int W, int H, T near_n, T far_n, int only_image, const T* means2D, const T* colors,
                                const T* normal_opacity, const T* trans_mat, const T* inverse_m,
                                const int32_t* point_list, const int64_t* ranges, const int64_t* bucket_offset,
                                const T* trans_mat_t2, int32_t* accum_max_count, T* accum_weights_p,
                                int32_t* accum_weights_count, T* out_color, T* out_opacity, T* out_extras,
                                T* out_flow, int32_t* n_contrib, int32_t* max_contrib, int32_t* bucket_to_tile,
                                T* sampled_T, T* sampled_acc, T* sampled_aux) {
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const size_t HW = (size_t) H * W;
  const bool aux  = !only_image;
  const bool snap = aux && bucket_offset != nullptr;
  const bool flow = aux && trans_mat_t2 != nullptr && out_flow != nullptr;
  const int NUM   = flow ? 10 : 8;
  const bool accum = accum_max_count || accum_weights_p || accum_weights_count;
  if (snap) {
    for (int t = 0; t < gx * gy; ++t) {
      const int64_t b0 = t == 0 ? 0 : bucket_offset[t - 1];
      const int64_t nb = (ranges[2 * t + 1] - ranges[2 * t] + 31) / 32;
      for (int64_t b = 0; b < nb; ++b) bucket_to_tile[b0 + b] = t;
      max_contrib[t] = 0;
    }
  }
  // the side outputs are sums over pixels of different tiles: serial when they are asked for
#pragma omp parallel for schedule(dynamic, 1) if (!accum)
  for (int tile = 0; tile < gx * gy; ++tile) {
    const int tx = tile % gx, ty = tile / gx;
    const int64_t r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
    int tile_max = 0;
    for (int ly = 0; ly < kTile; ++ly)
      for (int lx = 0; lx < kTile; ++lx) {
        const int px = tx * kTile + lx, py = ty * kTile + ly;
        if (px >= W || py >= H) continue;
        const int rank   = ly * kTile + lx;
        const size_t pix = (size_t) W * py + px;
        const T pxf = (T) px, pyf = (T) py;
        T t = 1, C[3] = {0}, N[3] = {0}, D = 0, M1 = 0, M2 = 0, dist = 0, med = 0, fl[2] = {0, 0};
        T wmax = 0;
        int32_t wmax_id = -1;
        bool flag = false;
        int32_t contributor = 0, last = 0, med_c = -1;
        int64_t bbm = snap ? (tile == 0 ? 0 : bucket_offset[tile - 1]) : 0;
        for (int64_t e = r0; e < r1; ++e) {
          if (snap && (e - r0) % 32 == 0) {
            sampled_T[bbm * 256 + rank] = t;
            for (int c = 0; c < 3; ++c) sampled_acc[(bbm * 3 + c) * 256 + rank] = C[c];
            sampled_aux[(bbm * NUM + 0) * 256 + rank] = D;
            for (int c = 0; c < 3; ++c) sampled_aux[(bbm * NUM + 1 + c) * 256 + rank] = N[c];
            sampled_aux[(bbm * NUM + 5) * 256 + rank] = dist;
            sampled_aux[(bbm * NUM + 6) * 256 + rank] = M1;
            sampled_aux[(bbm * NUM + 7) * 256 + rank] = M2;
            if (flow) sampled_aux[(bbm * NUM + 8) * 256 + rank] = fl[0], sampled_aux[(bbm * NUM + 9) * 256 + rank] = fl[1];
            ++bbm;
          }
          contributor++;
          const int id = point_list[e];
          const T* A   = inverse_m + 9 * (size_t) id;
          const T* Mx  = trans_mat + 9 * (size_t) id;
          const T p[3] = {A[0] * pxf + A[1] * pyf + A[2], A[3] * pxf + A[4] * pyf + A[5], A[6] * pxf + A[7] * pyf + A[8]};
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
          if (test_T < T(0.0001)) break;
          const T w = alpha * t;
          if (aux) {
            const T Aacc = 1 - t;
            const T m    = far_n / (far_n - near_n) * (1 - near_n / depth);
            dist += (m * m * Aacc + M2 - 2 * m * M1) * w;
            D += depth * w;
            M1 += m * w;
            M2 += m * m * w;
            if (t > 0.5) med = depth, med_c = contributor;
            for (int c = 0; c < 3; ++c) N[c] += no[c] * w;
            if (wmax < w) wmax = w, wmax_id = id, flag = true;
            if (accum_weights_p) accum_weights_p[id] += w;
            if (accum_weights_count) accum_weights_count[id] += 1;
            if (flow) {
              const T* Q = trans_mat_t2 + 9 * (size_t) id;
              const T u2 = Q[0] * s[0] + Q[1] * s[1] + Q[2];
              const T v2 = Q[3] * s[0] + Q[4] * s[1] + Q[5];
              T w2       = Q[6] * s[0] + Q[7] * s[1] + Q[8];
              w2         = std::abs(w2) < 1e-5 ? T(1e-5) : w2;
              fl[0] += (u2 / w2 - pxf) * w;
              fl[1] += (v2 / w2 - pyf) * w;
            }
          }
          if (flag && accum_max_count) accum_max_count[wmax_id] += 1;
          for (int c = 0; c < 3; ++c) C[c] += colors[3 * (size_t) id + c] * w;
          t    = test_T;
          last = contributor;
        }
        out_opacity[pix] = T(1) - t;
        n_contrib[pix]   = last;
        for (int c = 0; c < 3; ++c) out_color[c * HW + pix] = C[c];
        n_contrib[pix + HW] = aux ? med_c : 0;
        if (aux) {
          out_extras[pix + HW * 0] = D;
          for (int c = 0; c < 3; ++c) out_extras[pix + HW * (1 + c)] = N[c];
          out_extras[pix + HW * 4] = med;
          out_extras[pix + HW * 5] = dist;
          out_extras[pix + HW * 6] = M1;
          out_extras[pix + HW * 7] = M2;
          if (flow) {
            const T op = T(1) - t;
            out_flow[2 * pix]     = op > 0 ? fl[0] / op : T(0);
            out_flow[2 * pix + 1] = op > 0 ? fl[1] / op : T(0);
          }
        }
        tile_max = std::max(tile_max, (int) last);
      }
    if (snap) max_contrib[tile] = tile_max;
  }
}

// gs_2d_fast_redner.cu:273-561 (per_splat_form == 0) and :563-837 (per_splat_form == 1, same derivative written as a
// back-to-front recursion here; only the set of channels that carry gradient differs).
// Optical flow (dL_dflow given): both kernels take dL_dflow as the gradient of the UNNORMALISED flow sum (no division by
// the opacity the forward divided by, :366, :704) and send it to alpha and, through the second transform, to the
// intersection (s.x, s.y) (:494-510, :765-782); no gradient goes to trans_mat_t2. The per-splat kernel forms "partial
// sum up to and including this entry minus the total" with the NORMALISED out_flow as the total (:706); that is
// restated literally here from a front-to-back pass over the pixel's contributors.
template <typename T>
static void fast_render_backward(int P, int W, int H, T near_n, T far_n, int per_splat_form, const T* means2D,
                                 const T* normal_opacity, const T* colors, const T* trans_mat, const T* inverse_m,
                                 const T* trans_mat_t2, const T* out_opacity, const T* out_extras, const T* out_flow,
                                 const T* dL_dpix, const T* dL_dopacity, const T* dL_dextras, const T* dL_dflow,
                                 const int64_t* ranges, const int32_t* point_list, const int32_t* n_contrib,
                                 T* g_colors, T* g_means2D, T* g_trans, T* g_inv, T* g_normal_opacity) {
  const int gx = (W + kTile - 1) / kTile;
  const size_t HW = (size_t) H * W;
  const bool aux  = out_extras && dL_dextras;
  const bool flow = dL_dflow != nullptr && trans_mat_t2 != nullptr;
  (void) P;
  std::vector<T> pre_T, pre_P0, pre_P1;  // per list position of the current pixel (per-splat form with flow)
  for (int py = 0; py < H; ++py)
    for (int px = 0; px < W; ++px) {
      const size_t pix = (size_t) W * py + px;
      const int tile   = (py / kTile) * gx + (px / kTile);
      const int64_t r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
      const T pxf = (T) px, pyf = (T) py;
      const T t_final = 1 - out_opacity[pix];
      T t = t_final;
      int64_t contributor = r1 - r0;
      const int last_contributor   = n_contrib[pix];
      const int median_contributor = aux ? n_contrib[pix + HW] : 0;
      T acc_c[3] = {0}, last_c[3] = {0}, dLp[3];
      for (int c = 0; c < 3; ++c) dLp[c] = dL_dpix[c * HW + pix];
      T g_reg = 0, g_depth = 0, g_acc = 0, g_n[3] = {0}, g_med = 0, g_M1 = 0, g_M2 = 0;
      if (aux) {
        g_acc   = dL_dopacity[pix];
        g_depth = dL_dextras[0 * HW + pix];
        for (int c = 0; c < 3; ++c) g_n[c] = dL_dextras[(1 + c) * HW + pix];
        g_med = dL_dextras[4 * HW + pix];
        if (per_splat_form) g_M1 = dL_dextras[6 * HW + pix], g_M2 = dL_dextras[7 * HW + pix];
        else g_reg = dL_dextras[5 * HW + pix];
      } else if (per_splat_form) {
        g_acc = dL_dopacity[pix];
      }
      T last_depth = 0, acc_depth = 0, acc_alpha = 0, last_n[3] = {0}, acc_n[3] = {0};
      T last_m = 0, acc_m = 0, last_m2 = 0, acc_m2 = 0;
      const T final_D  = aux ? out_extras[pix + 6 * HW] : T(0);
      const T final_D2 = aux ? out_extras[pix + 7 * HW] : T(0);
      const T final_A  = 1 - t_final;
      T last_dL_dT = 0, last_alpha = 0;
      T acc_f[2] = {0, 0}, last_f[2] = {0, 0}, gF[2] = {0, 0};
      if (flow) gF[0] = dL_dflow[2 * pix], gF[1] = dL_dflow[2 * pix + 1];
      if (flow && per_splat_form) {
        // front-to-back: transmittance before each contributing entry and the flow sum up to and including it
        pre_T.assign((size_t) (r1 - r0), T(0)), pre_P0.assign((size_t) (r1 - r0), T(0)),
            pre_P1.assign((size_t) (r1 - r0), T(0));
        T tt = 1, f0 = 0, f1 = 0;
        for (int64_t e = r0; e < r0 + last_contributor; ++e) {
          const int id = point_list[e];
          const T* A   = inverse_m + 9 * (size_t) id;
          const T* Mx  = trans_mat + 9 * (size_t) id;
          const T p[3] = {A[0] * pxf + A[1] * pyf + A[2], A[3] * pxf + A[4] * pyf + A[5], A[6] * pxf + A[7] * pyf + A[8]};
          if (p[2] == 0.0) continue;
          const T s[2]  = {p[0] / p[2], p[1] / p[2]};
          const T d[2]  = {means2D[2 * id] - pxf, means2D[2 * id + 1] - pyf};
          const T rho   = std::min(s[0] * s[0] + s[1] * s[1], T(2.0) * (d[0] * d[0] + d[1] * d[1]));
          if (s[0] * Mx[6] + s[1] * Mx[7] + Mx[8] < near_n) continue;
          const T power = -T(0.5) * rho;
          if (power > T(0.0)) continue;
          const T alpha = std::min(T(0.99), normal_opacity[4 * (size_t) id + 3] * std::exp(power));
          if (alpha < T(1.0 / 255.0)) continue;
          const T* Q = trans_mat_t2 + 9 * (size_t) id;
          T w2       = Q[6] * s[0] + Q[7] * s[1] + Q[8];
          w2         = std::abs(w2) < 1e-5 ? T(1e-5) : w2;
          pre_T[(size_t) (e - r0)] = tt;
          f0 += alpha * tt * ((Q[0] * s[0] + Q[1] * s[1] + Q[2]) / w2 - pxf);
          f1 += alpha * tt * ((Q[3] * s[0] + Q[4] * s[1] + Q[5]) / w2 - pyf);
          pre_P0[(size_t) (e - r0)] = f0, pre_P1[(size_t) (e - r0)] = f1;
          tt *= 1 - alpha;
        }
      }
      for (int64_t e = r1 - 1; e >= r0; --e) {
        contributor--;
        if (contributor >= (int64_t) last_contributor) continue;
        const int id = point_list[e];
        const T* A   = inverse_m + 9 * (size_t) id;
        const T* Mx  = trans_mat + 9 * (size_t) id;
        const T p[3] = {A[0] * pxf + A[1] * pyf + A[2], A[3] * pxf + A[4] * pyf + A[5], A[6] * pxf + A[7] * pyf + A[8]};
        if (p[2] == 0.0) continue;
        const T s[2]  = {p[0] / p[2], p[1] / p[2]};
        const T rho3d = s[0] * s[0] + s[1] * s[1];
        const T d[2]  = {means2D[2 * id] - pxf, means2D[2 * id + 1] - pyf};
        const T rho2d = T(2.0) * (d[0] * d[0] + d[1] * d[1]);
        const T rho   = std::min(rho3d, rho2d);
        const T c_d   = s[0] * Mx[6] + s[1] * Mx[7] + Mx[8];
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
          const T col = colors[3 * (size_t) id + c];
          acc_c[c]    = last_alpha * last_c[c] + (T(1.) - last_alpha) * acc_c[c];
          last_c[c]   = col;
          dL_dalpha += (col - acc_c[c]) * dLp[c];
          g_colors[3 * (size_t) id + c] += w * dLp[c];
        }
        T dL_dz = 0, dL_dsx = 0, dL_dsy = 0;
        if (aux) {
          const T m_d    = far_n / (far_n - near_n) * (1 - near_n / c_d);
          const T dmd_dd = (far_n * near_n) / ((far_n - near_n) * c_d * c_d);
          if (contributor == (int64_t) median_contributor - 1) dL_dz += g_med;
          if (!per_splat_form) {
            const T dL_dweight = (final_D2 + m_d * m_d * final_A - 2 * m_d * final_D) * g_reg;
            dL_dalpha += dL_dweight - last_dL_dT;
            last_dL_dT = dL_dweight * alpha + (1 - alpha) * last_dL_dT;
            dL_dz += T(2.0) * (t * alpha) * (m_d * final_A - final_D) * g_reg * dmd_dd;
          } else {
            acc_m  = last_alpha * last_m + (T(1.) - last_alpha) * acc_m, last_m = m_d;
            acc_m2 = last_alpha * last_m2 + (T(1.) - last_alpha) * acc_m2, last_m2 = m_d * m_d;
            dL_dalpha += (m_d - acc_m) * g_M1 + (m_d * m_d - acc_m2) * g_M2;
            dL_dz += dmd_dd * (T(2) * m_d * w * g_M2);  // the M1 term is overwritten in the reference (:751, :755)
          }
          acc_depth  = last_alpha * last_depth + (T(1.) - last_alpha) * acc_depth;
          last_depth = c_d;
          dL_dalpha += (c_d - acc_depth) * g_depth;
          for (int c = 0; c < 3; ++c) {
            acc_n[c]  = last_alpha * last_n[c] + (T(1.) - last_alpha) * acc_n[c];
            last_n[c] = no[c];
            dL_dalpha += (no[c] - acc_n[c]) * g_n[c];
            g_normal_opacity[4 * (size_t) id + c] += w * g_n[c];
          }
          dL_dz += w * g_depth;
        }
        if (aux || per_splat_form) {
          acc_alpha = last_alpha * T(1.0) + (T(1.) - last_alpha) * acc_alpha;
          dL_dalpha += (1 - acc_alpha) * g_acc;
        }
        T flow_alpha = 0;  // the per-splat form's alpha term, already carrying its transmittance factors
        if (flow) {
          const T* Q = trans_mat_t2 + 9 * (size_t) id;
          const T u2 = Q[0] * s[0] + Q[1] * s[1] + Q[2];
          const T v2 = Q[3] * s[0] + Q[4] * s[1] + Q[5];
          T w2       = Q[6] * s[0] + Q[7] * s[1] + Q[8];
          w2         = std::abs(w2) < 1e-5 ? T(1e-5) : w2;
          const T f[2] = {u2 / w2 - pxf, v2 / w2 - pyf};
          if (!per_splat_form) {
            for (int c = 0; c < 2; ++c) {
              acc_f[c]  = last_alpha * last_f[c] + (T(1.) - last_alpha) * acc_f[c];
              last_f[c] = f[c];
              dL_dalpha += (f[c] - acc_f[c]) * gF[c];
            }
          } else {
            const size_t k = (size_t) (e - r0);
            flow_alpha = (f[0] * pre_T[k] + (pre_P0[k] - out_flow[2 * pix]) / (T(1.0) - alpha)) * gF[0] +
                         (f[1] * pre_T[k] + (pre_P1[k] - out_flow[2 * pix + 1]) / (T(1.0) - alpha)) * gF[1];
          }
          const T gu = w / w2 * gF[0], gv = w / w2 * gF[1], gw = -w / (w2 * w2) * (u2 * gF[0] + v2 * gF[1]);
          dL_dsx += Q[0] * gu + Q[3] * gv + Q[6] * gw;
          dL_dsy += Q[1] * gu + Q[4] * gv + Q[7] * gw;
        }
        dL_dalpha *= t;
        dL_dalpha += flow_alpha;
        last_alpha    = alpha;
        const T dL_dG = no[3] * dL_dalpha;
        if (rho3d <= rho2d) {
          dL_dsx += dL_dG * -G * s[0] + dL_dz * Mx[6];
          dL_dsy += dL_dG * -G * s[1] + dL_dz * Mx[7];
          const T a = dL_dsx / p[2], b = dL_dsy / p[2];
          const T dp[3] = {a, b, -(a * s[0] + b * s[1])};
          for (int r = 0; r < 3; ++r) {
            g_inv[9 * (size_t) id + 3 * r + 0] += dp[r] * pxf;
            g_inv[9 * (size_t) id + 3 * r + 1] += dp[r] * pyf;
            g_inv[9 * (size_t) id + 3 * r + 2] += dp[r];
          }
        } else {
          g_means2D[2 * (size_t) id] += dL_dG * (-G * T(2.0) * d[0]);
          g_means2D[2 * (size_t) id + 1] += dL_dG * (-G * T(2.0) * d[1]);
        }
        g_trans[9 * (size_t) id + 6] += dL_dz * s[0];
        g_trans[9 * (size_t) id + 7] += dL_dz * s[1];
        g_trans[9 * (size_t) id + 8] += dL_dz;
        g_normal_opacity[4 * (size_t) id + 3] += G * dL_dalpha;
      }
    }
}

}  // namespace oracle

using namespace oracle;
#define ORACLE_API extern "C" __attribute__((visibility("default")))

#define INSTANTIATE(SUF, T)                                                                                          \
  ORACLE_API int oracle_gs_2d_fast_compute_transmat_forward_##SUF(int P, const T* means3D, const T* scales,          \
      const T* rotations, const T* Tw2v, const T* Tv2s, T* trans_mat, T* normals) {                                  \
    for (int i = 0; i < P; ++i)                                                                                      \
      fast_transmat<T>(means3D + 3 * i, scales + 2 * i, rotations + 4 * i, Tw2v, Tv2s, trans_mat + 9 * i,            \
                       normals + 3 * i);                                                                             \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs_2d_fast_compute_transmat_backward_##SUF(int P, const T* means3D, const T* scales,         \
      const T* rotations, const T* Tw2v, const T* Tv2s, const T* g_mat, const T* g_normals, T* g_means3D,            \
      T* g_scales, T* g_rot) {                                                                                       \
    (void) means3D;                                                                                                  \
    for (int i = 0; i < P; ++i)                                                                                      \
      fast_transmat_backward<T>(scales + 2 * i, rotations + 4 * i, Tw2v, Tv2s, g_mat + 9 * i, g_normals + 3 * i,     \
                                g_means3D + 3 * i, g_scales + 2 * i, g_rot + 4 * i);                                 \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs_2d_fast_preprocess_forward_##SUF(int P, int W, int H, int sh_degree, int n_sh,            \
      const T* means3D, const T* scales, const T* rotations, const T* opacities, const T* shs, const T* sh_rest,     \
      const T* Tw2v, const T* Tv2s, const T* campos, const T* trans_precomp, const uint8_t* culling,                 \
      int means2D_preserve, T* means2D, T* colors, T* trans_mat, T* inverse_m, T* normal_opacity, T* depths,         \
      int32_t* radii, int32_t* tiles_touched) {                                                                      \
    if (sh_degree > kMaxShDegree) return 1;                                                                          \
    fast_preprocess_forward<T>(P, W, H, sh_degree, n_sh, means3D, scales, rotations, opacities, shs, sh_rest, Tw2v,  \
                               Tv2s, campos, trans_precomp, culling, means2D_preserve, means2D, colors, trans_mat,   \
                               inverse_m, normal_opacity, depths, radii, tiles_touched);                             \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs_2d_fast_preprocess_backward_##SUF(int P, int W, int H, int sh_degree, int n_sh,           \
      const T* means3D, const T* scales, const T* rotations, const T* shs, const T* sh_rest, const T* Tw2v,          \
      const T* Tv2s, const T* campos, const T* trans_mat, const int32_t* radii, const T* colors, T* grad_mean2D,     \
      const T* grad_trans, const T* grad_inv_m, const T* grad_colors, const T* grad_normal_opacity, T* g_means3D,    \
      T* g_scales, T* g_rot, T* g_opac, T* g_shs, T* g_sh_rest) {                                                    \
    if (sh_degree > kMaxShDegree) return 1;                                                                          \
    fast_preprocess_backward<T>(P, W, H, sh_degree, n_sh, means3D, scales, rotations, shs, sh_rest, Tw2v, Tv2s,      \
                                campos, trans_mat, radii, colors, grad_mean2D, grad_trans, grad_inv_m, grad_colors,  \
                                grad_normal_opacity, g_means3D, g_scales, g_rot, g_opac, g_shs, g_sh_rest);          \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs_2d_fast_render_forward_##SUF(int W, int H, double near_n, double far_n, int only_image,   \
      const T* means2D, const T* colors, const T* normal_opacity, const T* trans_mat, const T* inverse_m,            \
      const int32_t* point_list, const int64_t* ranges, const int64_t* bucket_offset, const T* trans_mat_t2,         \
      int32_t* accum_max_count, T* accum_weights_p, int32_t* accum_weights_count, T* out_color, T* out_opacity,      \
      T* out_extras, T* out_flow, int32_t* n_contrib, int32_t* max_contrib, int32_t* bucket_to_tile, T* sampled_T,   \
      T* sampled_acc, T* sampled_aux) {                                                                              \
    fast_render_forward<T>(W, H, (T) near_n, (T) far_n, only_image, means2D, colors, normal_opacity, trans_mat,      \
                           inverse_m, point_list, ranges, bucket_offset, trans_mat_t2, accum_max_count,              \
                           accum_weights_p, accum_weights_count, out_color, out_opacity, out_extras, out_flow,       \
                           n_contrib, max_contrib, bucket_to_tile, sampled_T, sampled_acc, sampled_aux);             \
    return 0;                                                                                                        \
  }                                                                                                                  \
  ORACLE_API int oracle_gs_2d_fast_render_backward_##SUF(int P, int W, int H, double near_n, double far_n,           \
      int per_splat_form, const T* means2D, const T* normal_opacity, const T* colors, const T* trans_mat,            \
      const T* inverse_m, const T* trans_mat_t2, const T* out_opacity, const T* out_extras, const T* out_flow,       \
      const T* dL_dpix, const T* dL_dopacity, const T* dL_dextras, const T* dL_dflow, const int64_t* ranges,         \
      const int32_t* point_list, const int32_t* n_contrib, T* g_colors, T* g_means2D, T* g_trans, T* g_inv,          \
      T* g_normal_opacity) {                                                                                         \
    fast_render_backward<T>(P, W, H, (T) near_n, (T) far_n, per_splat_form, means2D, normal_opacity, colors,         \
                            trans_mat, inverse_m, trans_mat_t2, out_opacity, out_extras, out_flow, dL_dpix,          \
                            dL_dopacity, dL_dextras, dL_dflow, ranges, point_list, n_contrib, g_colors, g_means2D,   \
                            g_trans, g_inv, g_normal_opacity);                                                       \
    return 0;                                                                                                        \
  }

INSTANTIATE(f32, float)
INSTANTIATE(f64, double)

ORACLE_API int oracle_gs_fast_prepare_fill(int P, int W, int H, const float* means2D, const float* inverse_m,
                                           const float* depths, const float* opacities, const int32_t* radii,
                                           const int64_t* offsets, int64_t R, int64_t* ranges, int32_t* point_list,
                                           int64_t* keys_sorted_out) {
  fast_prepare_fill(P, W, H, means2D, inverse_m, depths, opacities, radii, offsets, R, ranges, point_list,
                    keys_sorted_out);
  return 0;
}

// Corner test of one tile in double precision, for the brute-force pin of the single-precision test.
ORACLE_API int oracle_fast_corner_test_f64(const double* inverse_m, double opacity, int x, int y) {
  return CornerTest<double>(inverse_m, opacity).tile(x, y) ? 1 : 0;
}
