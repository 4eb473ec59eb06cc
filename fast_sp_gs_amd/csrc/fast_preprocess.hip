// "Fast" 2D-Gaussian-surfel preprocess for gfx950: ray-splat transform through camera intrinsics, its adjugate (so the
// blend evaluates the plane-plane intersection with three dot products), the 3-sigma screen bound, SH -> RGB, and the
// fused binning that only emits the tiles of a surfel's rectangle whose corners reach inside its alpha >= 1/255 conic.
//
// Reference behaviour reproduced: fast_2d_gs/_C/src/gaussian_splatting/gs_2d_fast_preprocess.cu:60-158 (transform,
// its backward, bound), :160-262 (forward kernel), :264-327 (duplicateWithKeys with the corner test, x-major emission,
// padding of unused slots with key = T << 32 / value = -1), :484-514 (ranges), :536-609 (backward), :611-782 (host).
// One documented deviation: log2(opacity) in the corner test is log2 evaluated in double precision and rounded to
// float, not PTX lg2.approx.
//
// Geometry and the corner test are compiled with contraction off in the reference's operation order, so radii, tile
// counts, keys, ranges and point lists are reproducible bit for bit against a plain IEEE evaluation.
#include "binning.hpp"
#include "sh.hpp"
#include "sh_stage.hpp"
#include "surfel_geom.hpp"

FSGS_API int fsgs_gs_prepare_scan(int P, const int32_t* tiles_touched, int64_t* point_offsets, void* workspace,
                                  size_t workspace_bytes, int64_t* num_rendered_host, void* stream);

namespace fsgs {
namespace {

#pragma clang fp contract(off)

__device__ __forceinline__ void fast_transmat(const float* p, float sx, float sy, const float4 q, const float* Tw2v,
                                              const float* Tv2s, float* M, float* nrm) {
  const float x = q.x, y = q.y, z = q.z, w = q.w;
  float L[9];
  L[0] = (1 - 2 * (y * y + z * z)) * sx;
  L[1] = 2 * (x * y - z * w) * sy;
  L[2] = p[0];
  L[3] = (2 * (x * y + z * w)) * sx;
  L[4] = (1 - 2 * (x * x + z * z)) * sy;
  L[5] = p[1];
  L[6] = (2 * (x * z - y * w)) * sx;
  L[7] = 2 * (x * w + y * z) * sy;
  L[8] = p[2];
  const float t0 = 2 * (y * w + x * z), t1 = 2 * (y * z - x * w), t2 = 1 - 2 * (x * x + y * y);
  float t[9];
#pragma unroll
  for (int i = 0; i < 3; ++i)
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      float res = 0.0f;
#pragma unroll
      for (int k = 0; k < 3; ++k) res += Tw2v[i * 4 + k] * L[k * 3 + j];
      t[i * 3 + j] = res;
    }
  t[8] += Tw2v[11];
#pragma unroll
  for (int i = 0; i < 9; ++i) M[i] = 0.0f;
#pragma unroll
  for (int i = 0; i < 3; ++i)
#pragma unroll
    for (int j = 0; j < 3; ++j)
#pragma unroll
      for (int k = 0; k < 3; ++k) M[i * 3 + j] += Tv2s[i * 3 + k] * t[k * 3 + j];
  nrm[0] = Tw2v[0] * t0 + Tw2v[1] * t1 + Tw2v[2] * t2;
  nrm[1] = Tw2v[4] * t0 + Tw2v[5] * t1 + Tw2v[6] * t2;
  nrm[2] = Tw2v[8] * t0 + Tw2v[9] * t1 + Tw2v[10] * t2;
}

__device__ __forceinline__ void fast_transmat_backward(float sx, float sy, const float4 q, const float* Tw2v,
                                                       const float* Tv2s, const float* gM, const float* gN, float* gp,
                                                       float* gs, float* gq) {
  float gL[9], dR[9];
#pragma unroll
  for (int i = 0; i < 9; ++i) gL[i] = 0.0f;
#pragma unroll
  for (int i = 0; i < 3; ++i)
#pragma unroll
    for (int j = 0; j < 3; ++j)
#pragma unroll
      for (int k = 0; k < 3; ++k) gL[i * 3 + j] += Tv2s[k * 3 + i] * gM[k * 3 + j];
#pragma unroll
  for (int i = 0; i < 3; ++i)
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      float res = 0.0f;
#pragma unroll
      for (int k = 0; k < 3; ++k) res += Tw2v[k * 4 + i] * gL[k * 3 + j];
      dR[i * 3 + j] = res;
    }
  gp[0] = dR[2], gp[1] = dR[5], gp[2] = dR[8];
  dR[2] = gN[0] * Tw2v[0] + gN[1] * Tw2v[4] + gN[2] * Tw2v[8];
  dR[5] = gN[0] * Tw2v[1] + gN[1] * Tw2v[5] + gN[2] * Tw2v[9];
  dR[8] = gN[0] * Tw2v[2] + gN[1] * Tw2v[6] + gN[2] * Tw2v[10];
  const float x = q.x, y = q.y, z = q.z, w = q.w;
  gs[0] = dR[0] * (1 - 2 * (y * y + z * z)) + dR[3] * (2 * (x * y + z * w)) + dR[6] * (2 * (x * z - y * w));
  gs[1] = dR[1] * (2 * (x * y - z * w)) + dR[4] * (1 - 2 * (x * x + z * z)) + dR[7] * (2 * (x * w + y * z));
  dR[0] *= sx, dR[1] *= sy, dR[3] *= sx, dR[4] *= sy, dR[6] *= sx, dR[7] *= sy;
  gq[0] = 2 * (-2 * x * (dR[4] + dR[8]) + y * (dR[1] + dR[3]) + z * (dR[2] + dR[6]) + w * (dR[7] - dR[5]));
  gq[1] = 2 * (x * (dR[1] + dR[3]) - 2 * y * (dR[0] + dR[8]) + z * (dR[5] + dR[7]) + w * (dR[2] - dR[6]));
  gq[2] = 2 * (x * (dR[2] + dR[6]) + y * (dR[5] + dR[7]) - 2 * z * (dR[0] + dR[4]) + w * (dR[3] - dR[1]));
  gq[3] = 2 * (x * (dR[7] - dR[5]) + y * (dR[2] - dR[6]) + z * (dR[3] - dR[1]));
}

// kWave: complete degree-3 rows in one 16-byte aligned [P,16,3] tensor, moved by each wavefront on its own (sh_stage.hpp).
constexpr int kCoopThreshold = 32;  // rectangles with more tiles are walked (and corner-tested) by a whole wavefront

template <int kSh, bool kWave>
__global__ void __launch_bounds__(256) fast_preprocess_forward_kernel(
    int P, int W, int H, int sh_degree, int n_sh, const float* __restrict__ means3D, const float2* __restrict__ scales,
    const float4* __restrict__ rotations, const float* __restrict__ opacities, const float* __restrict__ shs,
    const float* __restrict__ sh_rest, const float* __restrict__ Tw2v_g, const float* __restrict__ Tv2s_g,
    const float* __restrict__ campos, const float* __restrict__ trans_precomp, const uint8_t* __restrict__ culling,
    int means2D_preserve, float2* __restrict__ means2D, float* __restrict__ colors, float* __restrict__ trans_mat,
    float* __restrict__ inverse_m, float4* __restrict__ normal_opacity, float* __restrict__ depths,
    int32_t* __restrict__ radii, int32_t* __restrict__ tiles_touched, uint32_t* __restrict__ keep_masks) {
  __shared__ float s_rows[kWave ? kShStageRows * kShStageStride : 1];
  const int i0     = blockIdx.x * blockDim.x + threadIdx.x;
  const bool valid = i0 < P;
  if (!kWave && !valid) return;
  const int i = valid ? i0 : P - 1;  // lanes past the end stay for the wavefront's row movement and write nothing
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  float Tw2v[16], Tv2s[9];
#pragma unroll
  for (int k = 0; k < 16; ++k) Tw2v[k] = Tw2v_g[k];
#pragma unroll
  for (int k = 0; k < 9; ++k) Tv2s[k] = Tv2s_g[k];

  bool ok = false;
  float M[9], nrm[3] = {0, 0, 0}, c2[2] = {0, 0}, rgb[3] = {0, 0, 0}, depth = 0, radius = 0;
  int area = 0;
#pragma unroll
  for (int k = 0; k < 9; ++k) M[k] = 0.0f;
  const float p[3] = {means3D[3 * (size_t) i], means3D[3 * (size_t) i + 1], means3D[3 * (size_t) i + 2]};
  const int wave_base = blockIdx.x * blockDim.x + (threadIdx.x & ~63);
  float* s_wave_rows  = &s_rows[kWave ? (threadIdx.x & ~63) * kShStageStride : 0];
  ShWaveRows sh_regs;
  unsigned long long wanted = 0;
  if (kWave) {
    // the two cheapest rejections decide which rows are fetched; the fetch is then in flight during the geometry
    bool maybe = valid && !(culling && culling[i]);
    maybe = maybe && !((Tw2v[8] * p[0] + Tw2v[9] * p[1] + Tw2v[10] * p[2] + Tw2v[11]) <= 0.2f);
    wanted = __ballot(maybe);
    if (wanted) wave_fetch_sh_rows(sh_regs, wanted, wave_base, (const float4*) shs);
  }
  do {
    if (!valid || (culling && culling[i])) break;
    const float pv[3] = {Tw2v[0] * p[0] + Tw2v[1] * p[1] + Tw2v[2] * p[2] + Tw2v[3],
                         Tw2v[4] * p[0] + Tw2v[5] * p[1] + Tw2v[6] * p[2] + Tw2v[7],
                         Tw2v[8] * p[0] + Tw2v[9] * p[1] + Tw2v[10] * p[2] + Tw2v[11]};
    if (pv[2] <= 0.2f) break;
    if (trans_precomp == nullptr) {
      const float2 s = scales[i];
      fast_transmat(p, s.x, s.y, rotations[i], Tw2v, Tv2s, M, nrm);
    } else {
#pragma unroll
      for (int k = 0; k < 9; ++k) M[k] = trans_precomp[9 * (size_t) i + k];
      nrm[0] = 0.0f, nrm[1] = 0.0f, nrm[2] = 1.0f;
    }
    const float cosv = -(pv[0] * nrm[0] + pv[1] * nrm[1] + pv[2] * nrm[2]);
    if (cosv == 0.0f) break;
    const float mult = cosv > 0 ? 1.0f : -1.0f;
    nrm[0] = mult * nrm[0], nrm[1] = mult * nrm[1], nrm[2] = mult * nrm[2];
    float ext[2];
    if (!bound_3sigma(M, c2, ext)) break;
    radius = ceilf(fmaxf(fmaxf(ext[0], ext[1]), 3.0f * 0.707106f));
    const TileRect r = tile_rect(c2[0], c2[1], f2i_sat(radius), gx, gy);
    area = (r.y1 - r.y0) * (r.x1 - r.x0);
    if (area == 0) break;
    depth = pv[2];
    ok    = true;
  } while (false);

  if (kWave) {
    if (wanted) wave_rows_to_lds(sh_regs, s_wave_rows);
    wave_lds_sync();
  }
  if (ok && sh_degree >= 0) {
    float x, y, z, Y[kSh];
    view_dir(p, campos, x, y, z);
    sh_eval(sh_degree, x, y, z, Y);
    const int n = sh_count(sh_degree);
    const float* c0 = kWave ? &s_rows[threadIdx.x * kShStageStride] : shs + (size_t) i * (sh_rest ? 1 : n_sh) * 3;
    float r = c0[0] * Y[0], g = c0[1] * Y[0], b = c0[2] * Y[0];
    const float* cr = kWave ? c0 : (sh_rest ? sh_rest + (size_t) i * n_sh * 3 - 3 : c0);
    for (int l = 1; l < n; ++l) r += cr[3 * l] * Y[l], g += cr[3 * l + 1] * Y[l], b += cr[3 * l + 2] * Y[l];
    rgb[0] = fmaxf(0.0f, r + 0.5f), rgb[1] = fmaxf(0.0f, g + 0.5f), rgb[2] = fmaxf(0.0f, b + 0.5f);
  }
  if (!valid) return;
  float adj[9];
#pragma unroll
  for (int k = 0; k < 9; ++k) adj[k] = 0.0f;
  if (ok) {
    adj[0] = M[4] * M[8] - M[7] * M[5];
    adj[1] = M[7] * M[2] - M[1] * M[8];
    adj[2] = M[1] * M[5] - M[4] * M[2];
    adj[3] = M[6] * M[5] - M[3] * M[8];
    adj[4] = M[0] * M[8] - M[6] * M[2];
    adj[5] = M[3] * M[2] - M[0] * M[5];
    adj[6] = M[3] * M[7] - M[6] * M[4];
    adj[7] = M[6] * M[1] - M[0] * M[7];
    adj[8] = M[0] * M[4] - M[3] * M[1];
  }
#pragma unroll
  for (int k = 0; k < 9; ++k) {
    if (trans_precomp == nullptr) trans_mat[9 * (size_t) i + k] = ok ? M[k] : 0.0f;
    inverse_m[9 * (size_t) i + k] = adj[k];
  }
  if (sh_degree >= 0) {
    colors[3 * (size_t) i] = rgb[0], colors[3 * (size_t) i + 1] = rgb[1], colors[3 * (size_t) i + 2] = rgb[2];
  }
  depths[i]        = depth;
  radii[i]         = ok ? f2i_sat(radius) : 0;
  tiles_touched[i] = ok ? area : 0;
  if (ok || !means2D_preserve) means2D[i] = ok ? make_float2(c2[0], c2[1]) : make_float2(0.0f, 0.0f);
  normal_opacity[i] = ok ? make_float4(nrm[0], nrm[1], nrm[2], opacities[i]) : make_float4(0, 0, 0, 0);
  if (keep_masks) {
    // The binning's corner test for every tile of a rectangle of at most 32 tiles, here where adjugate, opacity and
    // rectangle are in registers: bit x * h + y (x-major, the order of the surfel's key span). The two walks of the
    // binning and the backward's record sum read the word instead of repeating the test and its set-up; larger
    // rectangles (all bits set here) are tested where they are walked.
    uint32_t m = 0xffffffffu;
    if (ok && area <= kCoopThreshold) {
      const TileRect r = tile_rect(c2[0], c2[1], f2i_sat(radius), gx, gy);
      const int w = r.x1 - r.x0, h = r.y1 - r.y0;
      const CornerTest ct(adj, opacities[i]);
      // a tile passes if one of its four corners does: every corner of the rectangle is evaluated once, a column of
      // corners at a time (h + 1 <= 33 bits), and a column of tiles is the OR of its two corner columns and their
      // shifts
      auto corner_column = [&](int X) {
        unsigned long long c = 0ull;
        for (int y = 0; y <= h; ++y)
          if (ct.at((float) X, (float) (r.y0 + y))) c |= 1ull << y;
        return c;
      };
      m = 0u;
      unsigned long long left = corner_column(r.x0);
      for (int x = 0; x < w; ++x) {
        const unsigned long long right = corner_column(r.x0 + x + 1), any = left | right;
        m |= (uint32_t) ((any | (any >> 1)) & ((1ull << h) - 1ull)) << (x * h);
        left = right;
      }
    }
    keep_masks[i] = m;
  }
}

__global__ void __launch_bounds__(256) fast_duplicate_keys_kernel(int P, int gx, int gy, int64_t R,
    const float2* __restrict__ means2D, const float* __restrict__ inverse_m, const float* __restrict__ depths,
    const float* __restrict__ opacities, const int32_t* __restrict__ radii, const int64_t* __restrict__ offsets,
    uint64_t* __restrict__ keys, int32_t* __restrict__ vals) {
  const int i    = blockIdx.x * blockDim.x + threadIdx.x;
  const int lane = __lane_id();
  const uint64_t pad_key = (uint64_t) (uint32_t) (gx * gy) << 32;
  int x0 = 0, y0 = 0, w = 0, h = 0;
  int64_t off = 0, off_to = 0;
  uint32_t dbits = 0;
  float IM[9], opacity = 1.0f;
#pragma unroll
  for (int k = 0; k < 9; ++k) IM[k] = 0.0f;
  if (i < P && radii[i] > 0) {
    const float2 c   = means2D[i];
    const TileRect r = tile_rect(c.x, c.y, radii[i], gx, gy);
    x0 = r.x0, y0 = r.y0, w = max(r.x1 - r.x0, 0), h = max(r.y1 - r.y0, 0);
    off    = i == 0 ? 0 : offsets[i - 1];
    off_to = offsets[i];
    dbits  = __float_as_uint(depths[i]);
    opacity = opacities[i];
#pragma unroll
    for (int k = 0; k < 9; ++k) IM[k] = inverse_m[9 * (size_t) i + k];
  }
  const int count = w * h;
  if (count > 0 && count <= kCoopThreshold) {
    const CornerTest ct(IM, opacity);
    for (int x = 0; x < w; ++x)
      for (int y = 0; y < h; ++y)
        if (ct.tile(x0 + x, y0 + y)) {
          if (off < R) {
            keys[off] = ((uint64_t) (uint32_t) ((y0 + y) * gx + (x0 + x)) << 32) | dbits;
            vals[off] = i;
          }
          ++off;
        }
    for (; off < off_to; ++off)
      if (off < R) keys[off] = pad_key, vals[off] = -1;
  }
  // Large rectangles: 64 tiles are tested per step by the whole wavefront and compacted in x-major order.
  unsigned long long big = __ballot(count > kCoopThreshold);
  while (big) {
    const int src = __ffsll((long long) big) - 1;
    big &= big - 1;
    float sIM[9];
#pragma unroll
    for (int k = 0; k < 9; ++k) sIM[k] = __shfl(IM[k], src, kWave);
    const CornerTest ct(sIM, __shfl(opacity, src, kWave));
    const int sx0 = __shfl(x0, src, kWave), sy0 = __shfl(y0, src, kWave), sh = __shfl(h, src, kWave);
    const int scount = __shfl(count, src, kWave), sid = __shfl(i, src, kWave);
    const uint32_t sbits = __shfl(dbits, src, kWave);
    int64_t soff         = __shfl((long long) off, src, kWave);
    const int64_t soff_to = __shfl((long long) off_to, src, kWave);
    for (int e0 = 0; e0 < scount; e0 += kWave) {
      const int e = e0 + lane;
      const int x = e / sh, y = e - x * sh;
      const bool keep = e < scount && ct.tile(sx0 + x, sy0 + y);
      const unsigned long long m = __ballot(keep);
      const int rank = __popcll(m & (lane == 0 ? 0ull : (~0ull >> (64 - lane))));
      if (keep && soff + rank < R) {
        keys[soff + rank] = ((uint64_t) (uint32_t) ((sy0 + y) * gx + (sx0 + x)) << 32) | sbits;
        vals[soff + rank] = sid;
      }
      soff += __popcll(m);
    }
    for (int64_t o = soff + lane; o < soff_to; o += kWave)
      if (o < R) keys[o] = pad_key, vals[o] = -1;
  }
}

template <int kSh, bool kWave>
__global__ void __launch_bounds__(256) fast_preprocess_backward_kernel(
    int P, int W, int H, int sh_degree, int n_sh, const float* __restrict__ means3D, const float2* __restrict__ scales,
    const float4* __restrict__ rotations, const float* __restrict__ shs, const float* __restrict__ sh_rest,
    const float* __restrict__ Tw2v_g, const float* __restrict__ Tv2s_g, const float* __restrict__ campos,
    const float* __restrict__ trans_mat, const int32_t* __restrict__ radii, const float* __restrict__ colors,
    float2* __restrict__ grad_mean2D, const float* __restrict__ grad_trans, const float* __restrict__ grad_inv_m,
    const float* __restrict__ grad_colors, const float4* __restrict__ grad_normal_opacity,
    float* __restrict__ g_means3D, float2* __restrict__ g_scales, float4* __restrict__ g_rot,
    float* __restrict__ g_opac, float* __restrict__ g_shs, float* __restrict__ g_sh_rest) {
  __shared__ float s_rows[kWave ? kShStageRows * kShStageStride : 1];
  const int i      = blockIdx.x * blockDim.x + threadIdx.x;
  const bool valid = i < P;
  const bool vis   = valid && radii[i] > 0;
  const int wave_base = blockIdx.x * blockDim.x + (threadIdx.x & ~63);
  float* s_wave_rows  = &s_rows[kWave ? (threadIdx.x & ~63) * kShStageStride : 0];
  float* my_row       = &s_rows[kWave ? threadIdx.x * kShStageStride : 0];
  // Rows of surfels that were not rendered get explicit zeros, so the outputs need no initialisation (the reference
  // leaves them to the caller's zero fill; a caller that zero-fills gets the same result).
  auto zero_geometry = [&]() {
    g_opac[i] = 0.0f;
    g_means3D[3 * (size_t) i] = 0.0f, g_means3D[3 * (size_t) i + 1] = 0.0f, g_means3D[3 * (size_t) i + 2] = 0.0f;
    g_scales[i] = make_float2(0.0f, 0.0f);
    g_rot[i]    = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  };
  if (kWave) {
    const unsigned long long wanted = __ballot(vis);
    if (wanted == 0ull) {  // nothing of this wavefront was rendered: its gradient rows are zeros
      if (wave_base < P) {
#pragma unroll
        for (int k = 0; k < kShWavePieces; ++k) {
          int r, c4;
          wave_piece(k, r, c4);
          if (wave_base + r < P)
            ((float4*) g_shs)[(size_t) (wave_base + r) * kShWavePieces + c4] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
      }
      if (valid) zero_geometry();
      return;
    }
    ShWaveRows sh_regs;
    wave_fetch_sh_rows(sh_regs, wanted, wave_base, (const float4*) shs);
    wave_rows_to_lds(sh_regs, s_wave_rows);
    wave_lds_sync();
    if (!vis) {
#pragma unroll
      for (int c = 0; c < kShStageFloats; ++c) my_row[c] = 0.0f;
      if (valid) zero_geometry();
    }
  } else if (!vis) {
    if (valid) {
      zero_geometry();
      if (sh_degree >= 0) {
        const int m1 = sh_rest ? 1 : n_sh;
        if (g_shs)
          for (int c = 0; c < m1 * 3; ++c) g_shs[(size_t) i * m1 * 3 + c] = 0.0f;
        if (g_sh_rest)
          for (int c = 0; c < n_sh * 3; ++c) g_sh_rest[(size_t) i * n_sh * 3 + c] = 0.0f;
      }
    }
    return;
  }
  if (vis) {
  float Tw2v[16], Tv2s[9];
#pragma unroll
  for (int k = 0; k < 16; ++k) Tw2v[k] = Tw2v_g[k];
#pragma unroll
  for (int k = 0; k < 9; ++k) Tv2s[k] = Tv2s_g[k];
  const float4 gno = grad_normal_opacity[i];
  g_opac[i]        = gno.w;
  float m[9], gT[9], gA[9];
#pragma unroll
  for (int k = 0; k < 9; ++k)
    m[k] = trans_mat[9 * (size_t) i + k], gT[k] = grad_trans[9 * (size_t) i + k], gA[k] = grad_inv_m[9 * (size_t) i + k];
#define MM(r, c) m[(r) * 3 + (c)]
#define GA(r, c) gA[(r) * 3 + (c)]
  gT[0] += GA(1, 1) * MM(2, 2) + GA(2, 2) * MM(1, 1) - GA(1, 2) * MM(1, 2) - GA(2, 1) * MM(2, 1);
  gT[1] += GA(0, 2) * MM(1, 2) + GA(2, 1) * MM(2, 0) - GA(0, 1) * MM(2, 2) - GA(2, 2) * MM(1, 0);
  gT[2] += GA(0, 1) * MM(2, 1) + GA(1, 2) * MM(1, 0) - GA(0, 2) * MM(1, 1) - GA(1, 1) * MM(2, 0);
  gT[3] += GA(1, 2) * MM(0, 2) + GA(2, 0) * MM(2, 1) - GA(1, 0) * MM(2, 2) - GA(2, 2) * MM(0, 1);
  gT[4] += GA(0, 0) * MM(2, 2) + GA(2, 2) * MM(0, 0) - GA(0, 2) * MM(0, 2) - GA(2, 0) * MM(2, 0);
  gT[5] += GA(0, 2) * MM(0, 1) + GA(1, 0) * MM(2, 0) - GA(0, 0) * MM(2, 1) - GA(1, 2) * MM(0, 0);
  gT[6] += GA(1, 0) * MM(1, 2) + GA(2, 1) * MM(0, 1) - GA(1, 1) * MM(0, 2) - GA(2, 0) * MM(1, 1);
  gT[7] += GA(0, 1) * MM(0, 2) + GA(2, 0) * MM(1, 0) - GA(0, 0) * MM(1, 2) - GA(2, 1) * MM(0, 0);
  gT[8] += GA(0, 0) * MM(1, 1) + GA(1, 1) * MM(0, 0) - GA(0, 1) * MM(0, 1) - GA(1, 0) * MM(1, 0);
#undef MM
#undef GA
  const float2 g2 = grad_mean2D[i];
  bound_backward(m, g2.x, g2.y, gT);

  const float4 q   = rotations[i];
  const float p[3] = {means3D[3 * (size_t) i], means3D[3 * (size_t) i + 1], means3D[3 * (size_t) i + 2]};
  const float t0 = 2 * (q.y * q.w + q.x * q.z), t1 = 2 * (q.y * q.z - q.x * q.w), t2 = 1 - 2 * (q.x * q.x + q.y * q.y);
  const float nrm[3] = {Tw2v[0] * t0 + Tw2v[1] * t1 + Tw2v[2] * t2, Tw2v[4] * t0 + Tw2v[5] * t1 + Tw2v[6] * t2,
                        Tw2v[8] * t0 + Tw2v[9] * t1 + Tw2v[10] * t2};
  const float pv[3] = {Tw2v[0] * p[0] + Tw2v[1] * p[1] + Tw2v[2] * p[2] + Tw2v[3],
                       Tw2v[4] * p[0] + Tw2v[5] * p[1] + Tw2v[6] * p[2] + Tw2v[7],
                       Tw2v[8] * p[0] + Tw2v[9] * p[1] + Tw2v[10] * p[2] + Tw2v[11]};
  const float cosv = -(pv[0] * nrm[0] + pv[1] * nrm[1] + pv[2] * nrm[2]);
  const float mult = cosv > 0 ? 1.0f : -1.0f;
  const float gN[3] = {mult * gno.x, mult * gno.y, mult * gno.z};
  const float2 s = scales[i];
  float gp[3], gs[2], gq[4];
  fast_transmat_backward(s.x, s.y, q, Tw2v, Tv2s, gT, gN, gp, gs, gq);

  if (sh_degree >= 0) {
    float x, y, z, Y[kSh], tl[kSh];
    const float nn = view_dir(p, campos, x, y, z);
    sh_eval(sh_degree, x, y, z, Y);
    float g[3];
#pragma unroll
    for (int c = 0; c < 3; ++c) g[c] = grad_colors[3 * (size_t) i + c] * (float) (colors[3 * (size_t) i + c] > 0);
    const int n  = sh_count(sh_degree);
    const int m1 = sh_rest ? 1 : n_sh;
    // with kWave the coefficients are read from the lane's staged row and the gradient row is written over them
    const float* c0 = kWave ? my_row : shs + (size_t) i * m1 * 3;
    const float* cr = kWave ? my_row : (sh_rest ? sh_rest + (size_t) i * n_sh * 3 - 3 : c0);
    float* o0  = kWave ? my_row : (g_shs ? g_shs + (size_t) i * m1 * 3 : nullptr);
    float* orr = kWave ? my_row : (g_sh_rest ? g_sh_rest + (size_t) i * n_sh * 3 - 3 : o0);
    if (o0) o0[0] = g[0] * Y[0], o0[1] = g[1] * Y[0], o0[2] = g[2] * Y[0];
    tl[0] = 0.0f;
    for (int l = 1; l < n; ++l) {
      tl[l] = g[0] * cr[3 * l] + g[1] * cr[3 * l + 1] + g[2] * cr[3 * l + 2];
      if (o0) orr[3 * l] = g[0] * Y[l], orr[3 * l + 1] = g[1] * Y[l], orr[3 * l + 2] = g[2] * Y[l];
    }
    float dx = 0, dy = 0, dz = 0;
    sh_grad_accumulate(sh_degree, x, y, z, tl, dx, dy, dz);
    const float vx = p[0] - campos[0], vy = p[1] - campos[1], vz = p[2] - campos[2];
    const float tt = -(vx * dx + vy * dy + vz * dz) * nn * nn * nn;
    gp[0] = gp[0] + (dx * nn + tt * vx);
    gp[1] = gp[1] + (dy * nn + tt * vy);
    gp[2] = gp[2] + (dz * nn + tt * vz);
  }
  g_means3D[3 * (size_t) i] = gp[0], g_means3D[3 * (size_t) i + 1] = gp[1], g_means3D[3 * (size_t) i + 2] = gp[2];
  g_scales[i] = make_float2(gs[0], gs[1]);
  g_rot[i]    = make_float4(gq[0], gq[1], gq[2], gq[3]);
  // densification proxy from the ACCUMULATED transform gradient (gs_2d_fast_preprocess.cu:606-608)
  const float depth = m[8];
  grad_mean2D[i] = make_float2(gT[2] * depth * 0.5f * (float) W, gT[5] * depth * 0.5f * (float) H);
  }
  if (kWave) {
    wave_lds_sync();
    wave_rows_to_global(s_wave_rows, wave_base, P, (float4*) g_shs);
  }
}

__global__ void __launch_bounds__(256) fast_transmat_forward_kernel(int P, const float* __restrict__ means3D,
    const float2* __restrict__ scales, const float4* __restrict__ rotations, const float* __restrict__ Tw2v_g,
    const float* __restrict__ Tv2s_g, float* __restrict__ trans_mat, float* __restrict__ normals) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= P) return;
  float Tw2v[16], Tv2s[9], M[9], nrm[3];
#pragma unroll
  for (int k = 0; k < 16; ++k) Tw2v[k] = Tw2v_g[k];
#pragma unroll
  for (int k = 0; k < 9; ++k) Tv2s[k] = Tv2s_g[k];
  const float p[3] = {means3D[3 * (size_t) i], means3D[3 * (size_t) i + 1], means3D[3 * (size_t) i + 2]};
  const float2 s = scales[i];
  fast_transmat(p, s.x, s.y, rotations[i], Tw2v, Tv2s, M, nrm);
#pragma unroll
  for (int k = 0; k < 9; ++k) trans_mat[9 * (size_t) i + k] = M[k];
#pragma unroll
  for (int k = 0; k < 3; ++k) normals[3 * (size_t) i + k] = nrm[k];
}

__global__ void __launch_bounds__(256) fast_transmat_backward_kernel(int P, const float2* __restrict__ scales,
    const float4* __restrict__ rotations, const float* __restrict__ Tw2v_g, const float* __restrict__ Tv2s_g,
    const float* __restrict__ g_mat, const float* __restrict__ g_normals, float* __restrict__ g_means3D,
    float2* __restrict__ g_scales, float4* __restrict__ g_rot) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= P) return;
  float Tw2v[16], Tv2s[9], gM[9], gN[3], gp[3], gs[2], gq[4];
#pragma unroll
  for (int k = 0; k < 16; ++k) Tw2v[k] = Tw2v_g[k];
#pragma unroll
  for (int k = 0; k < 9; ++k) Tv2s[k] = Tv2s_g[k], gM[k] = g_mat[9 * (size_t) i + k];
#pragma unroll
  for (int k = 0; k < 3; ++k) gN[k] = g_normals[3 * (size_t) i + k];
  const float2 s = scales[i];
  fast_transmat_backward(s.x, s.y, rotations[i], Tw2v, Tv2s, gM, gN, gp, gs, gq);
#pragma unroll
  for (int k = 0; k < 3; ++k) g_means3D[3 * (size_t) i + k] = gp[k];
  g_scales[i] = make_float2(gs[0], gs[1]);
  g_rot[i]    = make_float4(gq[0], gq[1], gq[2], gq[3]);
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API int fsgs_gs_2d_fast_preprocess_forward(int P, int W, int H, int sh_degree, int n_sh, const float* means3D,
    const float* scales, const float* rotations, const float* opacities, const float* shs, const float* sh_rest,
    const float* Tw2v, const float* Tv2s, const float* campos, const float* trans_precomp, const uint8_t* culling,
    int means2D_preserve, float* means2D, float* colors, float* trans_mat, float* inverse_m, float* normal_opacity,
    float* depths, int32_t* radii, int32_t* tiles_touched, uint32_t* keep_masks, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0, "gs_2d_fast_preprocess_forward: bad sizes");
  FSGS_REQUIRE(sh_degree <= kMaxShDegree, "gs_2d_fast_preprocess_forward: sh_degree %d not supported", sh_degree);
  if (sh_degree >= 0)
    FSGS_REQUIRE(n_sh + (sh_rest ? 1 : 0) >= (sh_degree + 1) * (sh_degree + 1),
                 "gs_2d_fast_preprocess_forward: %d SH coefficients are too few for degree %d", n_sh, sh_degree);
  FSGS_REQUIRE(means3D && scales && rotations && opacities && shs && Tw2v && Tv2s && campos && means2D && inverse_m &&
                   normal_opacity && depths && radii && tiles_touched && (trans_mat || trans_precomp) &&
                   (colors || sh_degree < 0),
               "gs_2d_fast_preprocess_forward: null pointer");
  if (P == 0) return kOk;
  const bool wave_rows = sh_degree == 3 && n_sh == 16 && !sh_rest && (uintptr_t) shs % 16 == 0;
  auto kernel = sh_degree > 3 ? fast_preprocess_forward_kernel<64, false>
                              : (wave_rows ? fast_preprocess_forward_kernel<16, true>
                                           : fast_preprocess_forward_kernel<16, false>);
  hipLaunchKernelGGL(kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P, W, H, sh_degree, n_sh,
                     means3D, (const float2*) scales, (const float4*) rotations, opacities, shs, sh_rest, Tw2v, Tv2s,
                     campos, trans_precomp, culling, means2D_preserve, (float2*) means2D, colors, trans_mat, inverse_m,
                     (float4*) normal_opacity, depths, radii, tiles_touched, keep_masks);
  return check_launch("gs_2d_fast_preprocess_forward");
}

FSGS_API int fsgs_gs_2d_fast_prepare_sort_bits(int W, int H) {
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  return 32 + (int) higher_msb((uint32_t) (gx * gy) + 1u);
}

FSGS_API size_t fsgs_gs_2d_fast_prepare_fill_workspace_bytes(int P, int W, int H, int64_t R) {
  return align_up(sort_workspace_bytes(R), 256) + fast_bucket_bins_bytes(P, W, H);
}

FSGS_API int fsgs_gs_2d_fast_prepare_fill(int P, int W, int H, const float* means2D, const float* inverse_m,
    const float* depths, const float* opacities, const int32_t* radii, const int64_t* point_offsets, int64_t R,
    int64_t* ranges, int32_t* point_list, int64_t* sorted_keys_out, void* workspace, size_t workspace_bytes,
    const uint32_t* keep_masks, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0 && R >= 0 && ranges, "gs_2d_fast_prepare_fill: bad arguments");
  FSGS_REQUIRE(R < (int64_t) 0x7fffffff, "gs_2d_fast_prepare_fill: %lld instances exceed the 2^31-1 limit",
               (long long) R);
  hipStream_t s = (hipStream_t) stream;
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const int T  = gx * gy;
  tile_order_invalidate(s);  // the ranges are rewritten: the blend schedule of this stream is stale
  if (R == 0 || P == 0) {
    launch_zero_ranges(T, ranges, s);
    return check_launch("gs_2d_fast_prepare_fill(zero)");
  }
  FSGS_REQUIRE(means2D && inverse_m && depths && opacities && radii && point_offsets && point_list && workspace,
               "gs_2d_fast_prepare_fill: null pointer");
  if (workspace_bytes < sort_workspace_bytes(R))
    return fail(kWorkspaceSmall, "gs_2d_fast_prepare_fill: workspace %zu < %zu bytes", workspace_bytes,
                sort_workspace_bytes(R));
  // With room for the per-tile counters behind the sort buffers (fsgs_gs_2d_fast_prepare_fill_workspace_bytes) the kept
  // instances are counted, scattered and sorted per tile, as on the standard path; the same lists, keys and ranges come
  // out of the device-wide sort of the padded key array below, which serves tile grids too large for that scheme and
  // callers that size the workspace for the sort alone.
  const size_t bins_at = align_up(sort_workspace_bytes(R), 256), bins_bytes = fast_bucket_bins_bytes(P, W, H);
  if (bins_bytes > 0 && workspace_bytes >= bins_at + bins_bytes)
    return fast_bucket_fill(P, W, H, means2D, inverse_m, depths, opacities, radii, keep_masks, R, ranges, point_list,
                            sorted_keys_out, workspace, (char*) workspace + bins_at, s);
  // the range kernel below writes the tiles that have entries (the per-tile scheme above writes every range itself)
  launch_zero_ranges(T, ranges, s);
  const int bits = fsgs_gs_2d_fast_prepare_sort_bits(W, H);
  hipLaunchKernelGGL(fast_duplicate_keys_kernel, dim3(div_up(P, 256)), dim3(256), 0, s, P, gx, gy, R,
                     (const float2*) means2D, inverse_m, depths, opacities, radii, point_offsets,
                     sort_keys_in(R, workspace), sort_vals_in(R, bits, workspace, point_list));
  const uint64_t* sorted = nullptr;
  radix_sort_pairs(R, bits, workspace, point_list, &sorted, s);
  launch_tile_ranges(R, T, sorted, ranges, s);
  if (sorted_keys_out)
    FSGS_HIP(hipMemcpyAsync(sorted_keys_out, sorted, (size_t) R * 8, hipMemcpyDeviceToDevice, s));
  return check_launch("gs_2d_fast_prepare_fill");
}

FSGS_API int fsgs_gs_2d_fast_preprocess_backward(int P, int W, int H, int sh_degree, int n_sh, const float* means3D,
    const float* scales, const float* rotations, const float* shs, const float* sh_rest, const float* Tw2v,
    const float* Tv2s, const float* campos, const float* trans_mat, const int32_t* radii, const float* colors,
    float* grad_mean2D, const float* grad_trans, const float* grad_inv_m, const float* grad_colors,
    const float* grad_normal_opacity, float* g_means3D, float* g_scales, float* g_rot, float* g_opac, float* g_shs,
    float* g_sh_rest, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0, "gs_2d_fast_preprocess_backward: bad sizes");
  FSGS_REQUIRE(sh_degree <= kMaxShDegree, "gs_2d_fast_preprocess_backward: sh_degree %d not supported", sh_degree);
  FSGS_REQUIRE(means3D && scales && rotations && Tw2v && Tv2s && campos && trans_mat && radii && grad_mean2D &&
                   grad_trans && grad_inv_m && grad_normal_opacity && g_means3D && g_scales && g_rot && g_opac,
               "gs_2d_fast_preprocess_backward: null pointer");
  if (sh_degree >= 0)
    FSGS_REQUIRE(shs && colors && grad_colors, "gs_2d_fast_preprocess_backward: SH path needs shs, colors, grad_colors");
  if (P == 0) return kOk;
  const bool wave_rows = sh_degree == 3 && n_sh == 16 && !sh_rest && g_shs && (uintptr_t) shs % 16 == 0 &&
                         (uintptr_t) g_shs % 16 == 0;
  auto kernel = sh_degree > 3 ? fast_preprocess_backward_kernel<64, false>
                              : (wave_rows ? fast_preprocess_backward_kernel<16, true>
                                           : fast_preprocess_backward_kernel<16, false>);
  hipLaunchKernelGGL(kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P, W, H, sh_degree, n_sh,
                     means3D, (const float2*) scales, (const float4*) rotations, shs, sh_rest, Tw2v, Tv2s, campos,
                     trans_mat, radii, colors, (float2*) grad_mean2D, grad_trans, grad_inv_m, grad_colors,
                     (const float4*) grad_normal_opacity, g_means3D, (float2*) g_scales, (float4*) g_rot, g_opac, g_shs,
                     g_sh_rest);
  return check_launch("gs_2d_fast_preprocess_backward");
}

FSGS_API int fsgs_gs_2d_fast_compute_transmat_forward(int P, const float* means3D, const float* scales,
    const float* rotations, const float* Tw2v, const float* Tv2s, float* trans_mat, float* normals, void* stream) {
  FSGS_REQUIRE(P >= 0 && means3D && scales && rotations && Tw2v && Tv2s && trans_mat && normals,
               "gs_2d_fast_compute_transmat_forward: bad arguments");
  if (P == 0) return kOk;
  hipLaunchKernelGGL(fast_transmat_forward_kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P,
                     means3D, (const float2*) scales, (const float4*) rotations, Tw2v, Tv2s, trans_mat, normals);
  return check_launch("gs_2d_fast_compute_transmat_forward");
}

FSGS_API int fsgs_gs_2d_fast_compute_transmat_backward(int P, const float* means3D, const float* scales,
    const float* rotations, const float* Tw2v, const float* Tv2s, const float* g_mat, const float* g_normals,
    float* g_means3D, float* g_scales, float* g_rot, void* stream) {
  (void) means3D;
  FSGS_REQUIRE(P >= 0 && scales && rotations && Tw2v && Tv2s && g_mat && g_normals && g_means3D && g_scales && g_rot,
               "gs_2d_fast_compute_transmat_backward: bad arguments");
  if (P == 0) return kOk;
  hipLaunchKernelGGL(fast_transmat_backward_kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P,
                     (const float2*) scales, (const float4*) rotations, Tw2v, Tv2s, g_mat, g_normals, g_means3D,
                     (float2*) g_scales, (float4*) g_rot);
  return check_launch("gs_2d_fast_compute_transmat_backward");
}
