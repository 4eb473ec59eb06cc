// 2D-Gaussian-surfel preprocess for gfx950: ray-splat transform, screen-space bound, tile rectangle, SH -> RGB,
// and the matching backward. One lane per surfel; pure HBM streaming.
//
// Reference behaviour reproduced: fast_2d_gs/_C/src/gaussian_splatting/gs_2d_preprocess.cu:24-329.
// The geometric part (transform, bound, radius, rectangle) is compiled with floating-point contraction off and in the
// reference's operation order, so radii / tiles_touched / means2D / trans_mat / depths are reproducible bit for bit
// against a plain IEEE evaluation of the same expressions.
#include "common.hpp"
#include "cull_bound.hpp"
#include "sh.hpp"
#include "sh_stage.hpp"
#include "surfel_geom.hpp"

namespace fsgs {
namespace {

#pragma clang fp contract(off)

struct Mat4 {
  float m[16];
};

__device__ __forceinline__ void mat4_mul(const float* A, const float* B, float* C) {
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      C[i * 4 + j] = A[i * 4 + 0] * B[0 * 4 + j] + A[i * 4 + 1] * B[1 * 4 + j] + A[i * 4 + 2] * B[2 * 4 + j] +
                     A[i * 4 + 3] * B[3 * 4 + j];
}

__device__ __forceinline__ void ndc2pix(int W, int H, float* N) {
#pragma unroll
  for (int i = 0; i < 16; ++i) N[i] = 0.0f;
  N[0] = (float) (0.5 * W), N[3] = (float) (0.5 * (W - 1));
  N[5] = (float) (0.5 * H), N[7] = (float) (0.5 * (H - 1));
  N[11] = 1.0f, N[15] = 1.0f;
}

// Block-wide: Tw2c = Tv2c * Tw2v into shared memory (the reference does this product with a device matmul on the
// host side, gs_2d_preprocess.cu:381).
__device__ __forceinline__ void load_camera(const float* __restrict__ Tw2v, const float* __restrict__ Tv2c,
                                            float* s_Tw2v, float* s_Tw2c) {
  const int t = threadIdx.x;
  if (t < 16) {
    const int i = t >> 2, j = t & 3;
    s_Tw2v[t] = Tw2v[t];
    s_Tw2c[t] = Tv2c[i * 4 + 0] * Tw2v[0 * 4 + j] + Tv2c[i * 4 + 1] * Tw2v[1 * 4 + j] +
                Tv2c[i * 4 + 2] * Tw2v[2 * 4 + j] + Tv2c[i * 4 + 3] * Tw2v[3 * 4 + j];
  }
  __syncthreads();
}

__device__ __forceinline__ void transmat(int W, int H, const float* p, float sx, float sy, const float4 q,
                                         const float* Tw2c, const float* Tw2v, float* M, float* nrm) {
  float L[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) L[i] = 0.0f;
  const float x = q.x, y = q.y, z = q.z, w = q.w;
  L[0]  = (1 - 2 * (y * y + z * z)) * sx;
  L[1]  = 2 * (x * y - z * w) * sy;
  L[2]  = p[0];
  L[4]  = (2 * (x * y + z * w)) * sx;
  L[5]  = (1 - 2 * (x * x + z * z)) * sy;
  L[6]  = p[1];
  L[8]  = (2 * (x * z - y * w)) * sx;
  L[9]  = 2 * (x * w + y * z) * sy;
  L[10] = p[2];
  L[14] = 1.0f;
  const float t0 = 2 * (y * w + x * z), t1 = 2 * (y * z - x * w), t2 = 1 - 2 * (x * x + y * y);
  float N[16], A[16], B[16];
  ndc2pix(W, H, N);
  mat4_mul(Tw2c, L, A);
  mat4_mul(N, A, B);
#pragma unroll
  for (int i = 0; i < 3; ++i)
#pragma unroll
    for (int j = 0; j < 3; ++j) M[i * 3 + j] = B[i * 4 + j];
  nrm[0] = Tw2v[0] * t0 + Tw2v[1] * t1 + Tw2v[2] * t2;
  nrm[1] = Tw2v[4] * t0 + Tw2v[5] * t1 + Tw2v[6] * t2;
  nrm[2] = Tw2v[8] * t0 + Tw2v[9] * t1 + Tw2v[10] * t2;
}

// kWave: complete degree-3 rows in one 16-byte aligned [P,16,3] tensor, moved by each wavefront on its own.
template <int kSh, bool kWave>
__global__ void __launch_bounds__(256) preprocess_forward_kernel(
    int P, int W, int H, int sh_degree, int n_sh, const float* __restrict__ means3D, const float2* __restrict__ scales,
    const float4* __restrict__ rotations, const float* __restrict__ opacities, const float* __restrict__ shs,
    const float* __restrict__ sh_rest, const float* __restrict__ Tw2v_g, const float* __restrict__ Tv2c_g,
    const float* __restrict__ campos, const float* __restrict__ trans_precomp, const uint8_t* __restrict__ culling,
    int means2D_preserve, float2* __restrict__ means2D, float* __restrict__ colors, float* __restrict__ trans_mat,
    float4* __restrict__ normal_opacity, float* __restrict__ depths, int32_t* __restrict__ radii,
    int32_t* __restrict__ tiles_touched, float4* __restrict__ records, uint32_t* __restrict__ keep_masks) {
  constexpr bool kStage = kSh == 16;  // degree <= 3: SH rows travel through LDS, read from HBM line by line
  __shared__ float s_Tw2v[16], s_Tw2c[16];
  __shared__ float s_rows[kStage ? kShStageRows * kShStageStride : 1];
  __shared__ unsigned char s_flag[kShStageRows];
  load_camera(Tw2v_g, Tv2c_g, s_Tw2v, s_Tw2c);
  const int i      = blockIdx.x * blockDim.x + threadIdx.x;
  const bool valid = i < P;
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;

  bool ok = false;
  float M[9], nrm[3] = {0, 0, 0}, c2[2] = {0, 0}, rgb[3] = {0, 0, 0}, depth = 0, radius = 0;
  int area = 0;
#pragma unroll
  for (int k = 0; k < 9; ++k) M[k] = 0.0f;
  float p[3] = {0, 0, 0};
  if (valid) p[0] = means3D[3 * (size_t) i], p[1] = means3D[3 * (size_t) i + 1], p[2] = means3D[3 * (size_t) i + 2];
  const int wave_base = blockIdx.x * blockDim.x + (threadIdx.x & ~63);
  float* s_wave_rows  = &s_rows[kWave ? (threadIdx.x & ~63) * kShStageStride : 0];
  ShWaveRows sh_regs;
  unsigned long long wanted = 0;
  if (kWave) {
    // the two cheapest rejections decide which rows are fetched; the fetch is then in flight during the geometry
    bool maybe = valid && !(culling && culling[i]);
    maybe = maybe && !((s_Tw2v[8] * p[0] + s_Tw2v[9] * p[1] + s_Tw2v[10] * p[2] + s_Tw2v[11]) <= 0.2f);
    wanted = __ballot(maybe);
    if (wanted) wave_fetch_sh_rows(sh_regs, wanted, wave_base, (const float4*) shs);
  }
  do {
    if (!valid || (culling && culling[i])) break;
    float Tw2v[16], Tw2c[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) Tw2v[k] = s_Tw2v[k], Tw2c[k] = s_Tw2c[k];
    const float pv[3] = {Tw2v[0] * p[0] + Tw2v[1] * p[1] + Tw2v[2] * p[2] + Tw2v[3],
                         Tw2v[4] * p[0] + Tw2v[5] * p[1] + Tw2v[6] * p[2] + Tw2v[7],
                         Tw2v[8] * p[0] + Tw2v[9] * p[1] + Tw2v[10] * p[2] + Tw2v[11]};
    if (pv[2] <= 0.2f) break;
    if (trans_precomp == nullptr) {
      const float2 s = scales[i];
      transmat(W, H, p, s.x, s.y, rotations[i], Tw2c, Tw2v, M, nrm);
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

  if (trans_precomp == nullptr) {
#pragma unroll
    for (int k = 0; k < 9; ++k) trans_mat[9 * (size_t) i + k] = ok ? M[k] : 0.0f;
  }
  if (sh_degree >= 0) {
    colors[3 * (size_t) i] = rgb[0], colors[3 * (size_t) i + 1] = rgb[1], colors[3 * (size_t) i + 2] = rgb[2];
  }
  depths[i]        = depth;
  radii[i]         = ok ? f2i_sat(radius) : 0;
  tiles_touched[i] = ok ? area : 0;
  if (ok || !means2D_preserve) means2D[i] = ok ? make_float2(c2[0], c2[1]) : make_float2(0.0f, 0.0f);
  normal_opacity[i] = ok ? make_float4(nrm[0], nrm[1], nrm[2], opacities[i]) : make_float4(0, 0, 0, 0);
  if (records) {
    // The blend kernels' 80-byte record (layout of pack_records_kernel), written here while every field is in
    // registers. Surfels that are not rendered never enter a tile list; their records are zeros.
    const float* col = sh_degree >= 0 ? rgb : shs + 3 * (size_t) i;
    const float op   = opacities[i];
    float4* r        = records + 5 * (size_t) i;
    if (ok) {
      r[0] = make_float4(M[0], M[1], M[2], M[3]);
      r[1] = make_float4(M[4], M[5], M[6], M[7]);
      r[2] = make_float4(M[8], c2[0], c2[1], op);
      r[3] = make_float4(nrm[0], nrm[1], nrm[2], col[0]);
      r[4] = make_float4(col[1], col[2], __int_as_float(f2i_sat(radius)), __int_as_float(-1));  // offset: not known yet
    } else {
#pragma unroll
      for (int k = 0; k < 5; ++k) r[k] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
  }
  if (keep_masks) {
    // Which tiles of the surfel's rectangle some pixel of which can blend it (the culled binning's input): a bit per
    // tile, row-major; rectangles above kCullMaskTiles tiles keep every bit. Evaluated here, where transform, centre
    // and radius are in registers and the vector units wait for memory anyway.
    uint32_t m = 0xffffffffu;
    if (ok) {
      const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
      const TileRect r = tile_rect(c2[0], c2[1], f2i_sat(radius), gx, gy);
      const int w = max(r.x1 - r.x0, 0), h = max(r.y1 - r.y0, 0);
      if (w * h <= kCullMaskTiles) {
        const CullBounds cb = cull_bounds(M, c2[0], c2[1], opacities[i]);
        m = 0u;
        int e = 0;
        for (int y = 0; y < h; ++y)
          for (int x = 0; x < w; ++x, ++e)
            if (cull_keeps_tile(cb, c2[0], c2[1], r.x0 + x, r.y0 + y)) m |= 1u << e;
      }
    }
    keep_masks[i] = m;
  }
}

__device__ __forceinline__ void transmat_backward(int W, int H, float sx, float sy, const float4 q, const float* Tw2c,
                                                  const float* Tw2v, const float* gM, const float* gN, float* gp,
                                                  float* gs, float* gq) {
  float N[16], G[16], GL[16], dR[16];
  ndc2pix(W, H, N);
#pragma unroll
  for (int i = 0; i < 16; ++i) G[i] = 0.0f, GL[i] = 0.0f, dR[i] = 0.0f;
#pragma unroll
  for (int i = 0; i < 3; ++i)
#pragma unroll
    for (int j = 0; j < 3; ++j) G[i * 4 + j] = gM[i * 3 + j];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int k = 0; k < 4; ++k) GL[i * 4 + j] += N[k * 4 + i] * G[k * 4 + j];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int k = 0; k < 4; ++k) dR[i * 4 + j] += Tw2c[k * 4 + i] * GL[k * 4 + j];
  gp[0] = dR[2], gp[1] = dR[6], gp[2] = dR[10];
  dR[2]  = gN[0] * Tw2v[0] + gN[1] * Tw2v[4] + gN[2] * Tw2v[8];
  dR[6]  = gN[0] * Tw2v[1] + gN[1] * Tw2v[5] + gN[2] * Tw2v[9];
  dR[10] = gN[0] * Tw2v[2] + gN[1] * Tw2v[6] + gN[2] * Tw2v[10];
  const float x = q.x, y = q.y, z = q.z, w = q.w;
  gs[0] = dR[0] * (1 - 2 * (y * y + z * z)) + dR[4] * (2 * (x * y + z * w)) + dR[8] * (2 * (x * z - y * w));
  gs[1] = dR[1] * (2 * (x * y - z * w)) + dR[5] * (1 - 2 * (x * x + z * z)) + dR[9] * (2 * (x * w + y * z));
  dR[0] *= sx, dR[1] *= sy, dR[4] *= sx, dR[5] *= sy, dR[8] *= sx, dR[9] *= sy;
  gq[0] = 2 * (-2 * x * (dR[5] + dR[10]) + y * (dR[1] + dR[4]) + z * (dR[2] + dR[8]) + w * (dR[9] - dR[6]));
  gq[1] = 2 * (x * (dR[1] + dR[4]) - 2 * y * (dR[0] + dR[10]) + z * (dR[6] + dR[9]) + w * (dR[2] - dR[8]));
  gq[2] = 2 * (x * (dR[2] + dR[8]) + y * (dR[6] + dR[9]) - 2 * z * (dR[0] + dR[5]) + w * (dR[4] - dR[1]));
  gq[3] = 2 * (x * (dR[9] - dR[6]) + y * (dR[2] - dR[8]) + z * (dR[4] - dR[1]));
}

template <int kSh, bool kWave>
__global__ void __launch_bounds__(256) preprocess_backward_kernel(
    int P, int W, int H, int sh_degree, int n_sh, const float* __restrict__ means3D, const float2* __restrict__ scales,
    const float4* __restrict__ rotations, const float* __restrict__ shs, const float* __restrict__ sh_rest,
    const float* __restrict__ Tw2v_g, const float* __restrict__ Tv2c_g, const float* __restrict__ campos,
    const float* __restrict__ trans_mat, const int32_t* __restrict__ radii, const float* __restrict__ colors,
    float2* __restrict__ grad_mean2D, const float* __restrict__ grad_trans, const float* __restrict__ grad_colors,
    const float4* __restrict__ grad_normal_opacity, float* __restrict__ g_means3D, float2* __restrict__ g_scales,
    float4* __restrict__ g_rot, float* __restrict__ g_opac, float* __restrict__ g_shs,
    float* __restrict__ g_sh_rest) {
  constexpr bool kStage = kSh == 16;
  __shared__ float s_Tw2v[16], s_Tw2c[16];
  __shared__ float s_rows[kStage ? kShStageRows * kShStageStride : 1];
  __shared__ unsigned char s_flag[kShStageRows];
  load_camera(Tw2v_g, Tv2c_g, s_Tw2v, s_Tw2c);
  const int i      = blockIdx.x * blockDim.x + threadIdx.x;
  const bool valid = i < P;
  const bool vis   = valid && radii[i] > 0;
  const int n      = sh_degree >= 0 ? sh_count(sh_degree) : 0;
  const int m1     = sh_rest ? 1 : n_sh;
  float* my_row    = &s_rows[kStage ? threadIdx.x * kShStageStride : 0];
  const int wave_base = blockIdx.x * blockDim.x + (threadIdx.x & ~63);
  float* s_wave_rows  = &s_rows[kWave ? (threadIdx.x & ~63) * kShStageStride : 0];
  const unsigned long long wanted = kWave ? __ballot(vis) : 0ull;
  if (kWave) {
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
      if (valid) {
        g_opac[i] = 0.0f;
        g_means3D[3 * (size_t) i] = 0.0f, g_means3D[3 * (size_t) i + 1] = 0.0f, g_means3D[3 * (size_t) i + 2] = 0.0f;
        g_scales[i] = make_float2(0.0f, 0.0f);
        g_rot[i]    = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      }
      return;
    }
    ShWaveRows sh_regs;
    wave_fetch_sh_rows(sh_regs, wanted, wave_base, (const float4*) shs);
    wave_rows_to_lds(sh_regs, s_wave_rows);
    wave_lds_sync();
  } else if (kStage && sh_degree >= 0) {
    s_flag[threadIdx.x] = vis;
    __syncthreads();
    stage_sh_rows(s_rows, s_flag, blockIdx.x * blockDim.x, P, n, n_sh, shs, sh_rest);
    __syncthreads();
  }

  if (vis) {
    float Tw2v[16], Tw2c[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) Tw2v[k] = s_Tw2v[k], Tw2c[k] = s_Tw2c[k];

    const float4 gno = grad_normal_opacity[i];
    g_opac[i]        = gno.w;
    float gM[9], M[9], gM_in2, gM_in5;
#pragma unroll
    for (int k = 0; k < 9; ++k) gM[k] = grad_trans[9 * (size_t) i + k], M[k] = trans_mat[9 * (size_t) i + k];
    gM_in2 = gM[2], gM_in5 = gM[5];
    const float2 g2 = grad_mean2D[i];
    bound_backward(M, g2.x, g2.y, gM);

    const float4 q   = rotations[i];
    const float p[3] = {means3D[3 * (size_t) i], means3D[3 * (size_t) i + 1], means3D[3 * (size_t) i + 2]};
    const float t0 = 2 * (q.y * q.w + q.x * q.z), t1 = 2 * (q.y * q.z - q.x * q.w),
                t2 = 1 - 2 * (q.x * q.x + q.y * q.y);
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
    transmat_backward(W, H, s.x, s.y, q, Tw2c, Tw2v, gM, gN, gp, gs, gq);

    if (sh_degree >= 0) {
      float x, y, z, Y[kSh], tl[kSh];
      const float nn = view_dir(p, campos, x, y, z);
      sh_eval(sh_degree, x, y, z, Y);
      float g[3];
#pragma unroll
      for (int c = 0; c < 3; ++c) g[c] = grad_colors[3 * (size_t) i + c] * (float) (colors[3 * (size_t) i + c] > 0);
      // coefficient rows are read from LDS when staged, and each gradient row is written over the coefficients it
      // was computed from (a lane only ever touches its own row)
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
      if (!kStage && orr) {  // coefficients above the active degree
        for (int l = n; l < (sh_rest ? n_sh + 1 : n_sh); ++l)
          orr[3 * l] = 0.0f, orr[3 * l + 1] = 0.0f, orr[3 * l + 2] = 0.0f;
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
    // densification proxy written over the incoming screen-space gradient (gs_2d_preprocess.cu:325-328)
    const float depth = M[8];
    grad_mean2D[i] = make_float2(gM_in2 * depth * 0.5f * (float) W, gM_in5 * depth * 0.5f * (float) H);
  } else if (valid) {
    // rows of surfels that were not rendered get explicit zeros, so the outputs need no initialisation
    g_opac[i] = 0.0f;
    g_means3D[3 * (size_t) i] = 0.0f, g_means3D[3 * (size_t) i + 1] = 0.0f, g_means3D[3 * (size_t) i + 2] = 0.0f;
    g_scales[i] = make_float2(0.0f, 0.0f);
    g_rot[i]    = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
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
  if (kWave) {
    wave_lds_sync();
    wave_rows_to_global(s_wave_rows, wave_base, P, (float4*) g_shs);
  } else if (kStage && sh_degree >= 0 && (g_shs || g_sh_rest)) {
    __syncthreads();
    unstage_sh_grads(s_rows, blockIdx.x * blockDim.x, P, n, n_sh, sh_rest != nullptr, g_shs, g_sh_rest);
  }
}

__global__ void __launch_bounds__(256) transmat_forward_kernel(int P, int W, int H, const float* __restrict__ means3D,
    const float2* __restrict__ scales, const float4* __restrict__ rotations, const float* __restrict__ Tw2v_g,
    const float* __restrict__ Tw2c_g, float* __restrict__ trans_mat, float* __restrict__ normals) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= P) return;
  float Tw2v[16], Tw2c[16], M[9], nrm[3];
#pragma unroll
  for (int k = 0; k < 16; ++k) Tw2v[k] = Tw2v_g[k], Tw2c[k] = Tw2c_g[k];
  const float p[3] = {means3D[3 * (size_t) i], means3D[3 * (size_t) i + 1], means3D[3 * (size_t) i + 2]};
  const float2 s = scales[i];
  transmat(W, H, p, s.x, s.y, rotations[i], Tw2c, Tw2v, M, nrm);
#pragma unroll
  for (int k = 0; k < 9; ++k) trans_mat[9 * (size_t) i + k] = M[k];
#pragma unroll
  for (int k = 0; k < 3; ++k) normals[3 * (size_t) i + k] = nrm[k];
}

__global__ void __launch_bounds__(256) transmat_backward_kernel(int P, int W, int H, const float2* __restrict__ scales,
    const float4* __restrict__ rotations, const float* __restrict__ Tw2v_g, const float* __restrict__ Tw2c_g,
    const float* __restrict__ g_mat, const float* __restrict__ g_normals, float* __restrict__ g_means3D,
    float2* __restrict__ g_scales, float4* __restrict__ g_rot) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= P) return;
  float Tw2v[16], Tw2c[16], gM[9], gN[3], gp[3], gs[2], gq[4];
#pragma unroll
  for (int k = 0; k < 16; ++k) Tw2v[k] = Tw2v_g[k], Tw2c[k] = Tw2c_g[k];
#pragma unroll
  for (int k = 0; k < 9; ++k) gM[k] = g_mat[9 * (size_t) i + k];
#pragma unroll
  for (int k = 0; k < 3; ++k) gN[k] = g_normals[3 * (size_t) i + k];
  const float2 s = scales[i];
  transmat_backward(W, H, s.x, s.y, rotations[i], Tw2c, Tw2v, gM, gN, gp, gs, gq);
#pragma unroll
  for (int k = 0; k < 3; ++k) g_means3D[3 * (size_t) i + k] = gp[k];
  g_scales[i] = make_float2(gs[0], gs[1]);
  g_rot[i]    = make_float4(gq[0], gq[1], gq[2], gq[3]);
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API int fsgs_gs_2d_preprocess_forward(int P, int W, int H, int sh_degree, int n_sh, const float* means3D,
    const float* scales, const float* rotations, const float* opacities, const float* shs, const float* sh_rest,
    const float* Tw2v, const float* Tv2c, const float* campos, const float* trans_precomp, const uint8_t* culling,
    int means2D_preserve, float* means2D, float* colors, float* trans_mat, float* normal_opacity, float* depths,
    int32_t* radii, int32_t* tiles_touched, float* records, uint32_t* keep_masks, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0, "gs_2d_preprocess_forward: bad sizes P=%d W=%d H=%d", P, W, H);
  FSGS_REQUIRE(((uintptr_t) records & 15) == 0, "gs_2d_preprocess_forward: records must be 16-byte aligned");
  FSGS_REQUIRE(sh_degree <= kMaxShDegree, "gs_2d_preprocess_forward: sh_degree %d > %d not supported", sh_degree,
               kMaxShDegree);
  if (sh_degree >= 0)
    FSGS_REQUIRE(n_sh + (sh_rest ? 1 : 0) >= (sh_degree + 1) * (sh_degree + 1),
                 "gs_2d_preprocess_forward: %d SH coefficients are too few for degree %d", n_sh, sh_degree);
  FSGS_REQUIRE(means3D && scales && rotations && opacities && shs && Tw2v && Tv2c && campos && means2D &&
                   normal_opacity && depths && radii && tiles_touched && (trans_mat || trans_precomp) &&
                   (colors || sh_degree < 0),
               "gs_2d_preprocess_forward: null pointer");
  if (P == 0) return kOk;
  const bool wave_rows = sh_degree == 3 && n_sh == 16 && !sh_rest && (uintptr_t) shs % 16 == 0;
  auto kernel = sh_degree > 3 ? preprocess_forward_kernel<64, false>
                              : (wave_rows ? preprocess_forward_kernel<16, true> : preprocess_forward_kernel<16, false>);
  hipLaunchKernelGGL(kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P, W, H, sh_degree, n_sh, means3D, (const float2*) scales, (const float4*) rotations, opacities, shs,
                     sh_rest, Tw2v, Tv2c, campos, trans_precomp, culling, means2D_preserve, (float2*) means2D, colors,
                     trans_mat, (float4*) normal_opacity, depths, radii, tiles_touched, (float4*) records, keep_masks);
  return check_launch("gs_2d_preprocess_forward");
}

FSGS_API int fsgs_gs_2d_preprocess_backward(int P, int W, int H, int sh_degree, int n_sh, const float* means3D,
    const float* scales, const float* rotations, const float* shs, const float* sh_rest, const float* Tw2v,
    const float* Tv2c, const float* campos, const float* trans_mat, const int32_t* radii, const float* colors,
    float* grad_mean2D, const float* grad_trans, const float* grad_colors, const float* grad_normal_opacity,
    float* g_means3D, float* g_scales, float* g_rot, float* g_opac, float* g_shs, float* g_sh_rest, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0, "gs_2d_preprocess_backward: bad sizes");
  FSGS_REQUIRE(sh_degree <= kMaxShDegree, "gs_2d_preprocess_backward: sh_degree %d > %d not supported", sh_degree,
               kMaxShDegree);
  FSGS_REQUIRE(means3D && scales && rotations && Tw2v && Tv2c && campos && trans_mat && radii && grad_mean2D &&
                   grad_trans && grad_normal_opacity && g_means3D && g_scales && g_rot && g_opac,
               "gs_2d_preprocess_backward: null pointer");
  if (sh_degree >= 0)
    FSGS_REQUIRE(shs && colors && grad_colors, "gs_2d_preprocess_backward: SH path needs shs, colors and grad_colors");
  if (P == 0) return kOk;
  const bool wave_rows = sh_degree == 3 && n_sh == 16 && !sh_rest && g_shs && (uintptr_t) shs % 16 == 0 &&
                         (uintptr_t) g_shs % 16 == 0;
  auto kernel = sh_degree > 3 ? preprocess_backward_kernel<64, false>
                              : (wave_rows ? preprocess_backward_kernel<16, true> : preprocess_backward_kernel<16, false>);
  hipLaunchKernelGGL(kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P, W, H, sh_degree, n_sh, means3D, (const float2*) scales, (const float4*) rotations, shs, sh_rest, Tw2v,
                     Tv2c, campos, trans_mat, radii, colors, (float2*) grad_mean2D, grad_trans, grad_colors,
                     (const float4*) grad_normal_opacity, g_means3D, (float2*) g_scales, (float4*) g_rot, g_opac,
                     g_shs, g_sh_rest);
  return check_launch("gs_2d_preprocess_backward");
}

FSGS_API int fsgs_gs_2d_compute_transmat_forward(int P, int W, int H, const float* means3D, const float* scales,
    const float* rotations, const float* Tw2v, const float* Tw2c, float* trans_mat, float* normals, void* stream) {
  FSGS_REQUIRE(P >= 0 && means3D && scales && rotations && Tw2v && Tw2c && trans_mat && normals,
               "gs_2d_compute_transmat_forward: bad arguments");
  if (P == 0) return kOk;
  hipLaunchKernelGGL(transmat_forward_kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P, W, H,
                     means3D, (const float2*) scales, (const float4*) rotations, Tw2v, Tw2c, trans_mat, normals);
  return check_launch("gs_2d_compute_transmat_forward");
}

FSGS_API int fsgs_gs_2d_compute_transmat_backward(int P, int W, int H, const float* means3D, const float* scales,
    const float* rotations, const float* Tw2v, const float* Tw2c, const float* g_mat, const float* g_normals,
    float* g_means3D, float* g_scales, float* g_rot, void* stream) {
  (void) means3D;
  FSGS_REQUIRE(P >= 0 && scales && rotations && Tw2v && Tw2c && g_mat && g_normals && g_means3D && g_scales && g_rot,
               "gs_2d_compute_transmat_backward: bad arguments");
  if (P == 0) return kOk;
  hipLaunchKernelGGL(transmat_backward_kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P, W, H,
                     (const float2*) scales, (const float4*) rotations, Tw2v, Tw2c, g_mat, g_normals, g_means3D,
                     (float2*) g_scales, (float4*) g_rot);
  return check_launch("gs_2d_compute_transmat_backward");
}
