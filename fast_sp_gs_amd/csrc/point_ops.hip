// Stand-alone per-point operators for gfx950: SH -> RGB and its backward, the bare SH and frequency encoders,
// nearest / farthest point (cdist top-1) with backward, K-nearest control points, LBS skinning, masked Adam.
//
// Reference behaviour reproduced:
//   SH_to_RGB_forward / _backward   fast_2d_gs/_C/src/ops_3d/spherical_harmonics.cu:6-66
//   sh_encode_forward / _backward   fast_2d_gs/_C/src/nerf/shencoder.cu:18-176, 178-655
//   freq_encode_forward / _backward fast_2d_gs/_C/src/nerf/freqencoder.cu:7-60
//   cdist_top / cdist_top_backward  fast_2d_gs/_C/src/other/cdist_top.cu:3-32, 86-105
//   AdamMasksedUpdated              fast_2d_gs/_C/src/other/adam_masked_update.cu:9-28
//   K-NN + LBS blend                fast_2d_gs/network.py:498-573 (pytorch3d.ops.knn_points + lietorch.SE3 there)
//
// All of these are HBM-streaming or small brute-force searches: one lane per point, control points staged in LDS and
// read as wave-wide broadcasts, distances accumulated in the reference's order with contraction off so that indices
// are reproducible bit for bit.
#include <algorithm>
#include <type_traits>

#include "../../include/fsgs.h"
#include "common.hpp"
#include "lbs.hpp"
#include "sh.hpp"
#include "sh_stage.hpp"

namespace fsgs {
namespace {

// ---- SH -> RGB ----------------------------------------------------------------------------------------------------
// kRows: all 16 coefficients of a point sit in one 16-byte-aligned 192-byte row (F == 16, degree 3). A lane that walks its
// own row touches one 128-byte line per load instruction (920 GB/s measured at 1M points); each wavefront therefore moves
// its 64 rows as twelve 16-byte pieces per lane, 1 KB of consecutive addresses per instruction, through its own slice of
// LDS, and every lane then reads its row there (the scheme of the preprocess kernels, sh_stage.hpp).
template <int kSh, bool kRows>
__global__ void __launch_bounds__(256) sh_to_rgb_forward_kernel(int P, int F, int degree, int clamp,
    const float* __restrict__ pos, const float* __restrict__ campos, const float* __restrict__ sh,
    float* __restrict__ rgb) {
  __shared__ float s_rows[kRows ? 4 * kWave * kShStageStride : 1];
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  float* my_rows = s_rows + (kRows ? (threadIdx.x >> 6) * kWave * kShStageStride : 0);
  if (kRows) {
    const unsigned long long live = __ballot(i < P);
    if (live != 0ull) {
      ShWaveRows regs;
      wave_fetch_sh_rows(regs, live, (int) (blockIdx.x * blockDim.x + (threadIdx.x & ~63)), (const float4*) sh);
      wave_rows_to_lds(regs, my_rows);
      wave_lds_sync();
    }
  }
  if (i >= P) return;
  float x = pos[3 * (size_t) i], y = pos[3 * (size_t) i + 1], z = pos[3 * (size_t) i + 2];
  if (campos) {
    const float p[3] = {x, y, z};
    view_dir(p, campos, x, y, z);
  }
  float Y[kSh];
  sh_eval(degree, x, y, z, Y);
  const int n    = sh_count(degree);
  const float* c = kRows ? my_rows + (threadIdx.x & 63) * kShStageStride : sh + (size_t) i * F * 3;
  float r = c[0] * Y[0], g = c[1] * Y[0], b = c[2] * Y[0];
  for (int l = 1; l < n; ++l) r += c[3 * l] * Y[l], g += c[3 * l + 1] * Y[l], b += c[3 * l + 2] * Y[l];
  r += 0.5f, g += 0.5f, b += 0.5f;
  if (clamp) r = fmaxf(0.0f, r), g = fmaxf(0.0f, g), b = fmaxf(0.0f, b);
  rgb[3 * (size_t) i] = r, rgb[3 * (size_t) i + 1] = g, rgb[3 * (size_t) i + 2] = b;
}

__device__ __forceinline__ float wave_sum_xor(float v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, kWave);
  return v;
}

template <int kSh, bool kRows>
__global__ void __launch_bounds__(256) sh_to_rgb_backward_kernel(int P, int F, int degree, int clamp,
    const float* __restrict__ pos, const float* __restrict__ campos, const float* __restrict__ sh,
    const float* __restrict__ rgb, const float* __restrict__ grad_rgb, float* __restrict__ grad_dir,
    float* __restrict__ grad_campos, float* __restrict__ grad_sh) {
  __shared__ float s_cam[4][3];
  __shared__ float s_rows[kRows ? 4 * kWave * kShStageStride : 1];
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const int wave_base = (int) (blockIdx.x * blockDim.x + (threadIdx.x & ~63));
  float* my_rows = s_rows + (kRows ? (threadIdx.x >> 6) * kWave * kShStageStride : 0);
  if (kRows) {  // coefficient rows in through LDS; the gradient rows leave the same way (a lane overwrites its own row)
    const unsigned long long live = __ballot(i < P);
    if (live != 0ull) {
      ShWaveRows regs;
      wave_fetch_sh_rows(regs, live, wave_base, (const float4*) sh);
      wave_rows_to_lds(regs, my_rows);
      wave_lds_sync();
    }
  }
  float dx = 0, dy = 0, dz = 0;
  if (i < P) {
    const float p[3] = {pos[3 * (size_t) i], pos[3 * (size_t) i + 1], pos[3 * (size_t) i + 2]};
    float x = p[0], y = p[1], z = p[2], nn = 1.0f;
    if (campos) nn = view_dir(p, campos, x, y, z);
    float g[3];
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      g[c] = grad_rgb[3 * (size_t) i + c];
      if (clamp) g[c] *= (float) (rgb[3 * (size_t) i + c] > 0);
    }
    float Y[kSh], tl[kSh];
    sh_eval(degree, x, y, z, Y);
    const int n    = sh_count(degree);
    float* row     = my_rows + (threadIdx.x & 63) * kShStageStride;
    const float* c = kRows ? row : sh + (size_t) i * F * 3;
    float* o       = kRows ? (grad_sh ? row : nullptr) : (grad_sh ? grad_sh + (size_t) i * F * 3 : nullptr);
    tl[0] = 0.0f;
    for (int l = 0; l < n; ++l) {  // a coefficient is read before its slot takes the gradient
      const float c0 = c[3 * l], c1 = c[3 * l + 1], c2 = c[3 * l + 2];
      tl[l] = g[0] * c0 + g[1] * c1 + g[2] * c2;
      if (o) o[3 * l] = g[0] * Y[l], o[3 * l + 1] = g[1] * Y[l], o[3 * l + 2] = g[2] * Y[l];
    }
    if (grad_dir || grad_campos) {
      sh_grad_accumulate(degree, x, y, z, tl, dx, dy, dz);
      if (campos) {
        const float vx = p[0] - campos[0], vy = p[1] - campos[1], vz = p[2] - campos[2];
        const float t  = -(vx * dx + vy * dy + vz * dz) * nn * nn * nn;
        dx = dx * nn + t * vx, dy = dy * nn + t * vy, dz = dz * nn + t * vz;
      }
      if (grad_dir) grad_dir[3 * (size_t) i] = dx, grad_dir[3 * (size_t) i + 1] = dy, grad_dir[3 * (size_t) i + 2] = dz;
    }
  }
  if (kRows && grad_sh) {
    wave_lds_sync();
    wave_rows_to_global(my_rows, wave_base, P, (float4*) grad_sh);
  }
  if (grad_campos) {  // block reduction, then 3 atomics per block (spherical_harmonics.cu:56-65)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float sx = wave_sum_xor(dx), sy = wave_sum_xor(dy), sz = wave_sum_xor(dz);
    if (lane == 0) s_cam[wave][0] = sx, s_cam[wave][1] = sy, s_cam[wave][2] = sz;
    __syncthreads();
    if (threadIdx.x < 3) {
      const float t = s_cam[0][threadIdx.x] + s_cam[1][threadIdx.x] + s_cam[2][threadIdx.x] + s_cam[3][threadIdx.x];
      atomicAdd(grad_campos + threadIdx.x, -t);
    }
  }
}

// ---- element types of the small operators -------------------------------------------------------------------------------
// The encoders and the nearest / farthest search accept the floating types the reference dispatches on. Half precision
// is a storage format: values are widened on load, the arithmetic is single precision, the result is rounded once on
// store -- except where the reference itself keeps intermediates in half (the SH encoder's monomials and backward sums,
// restated for degree <= 3 in sh_eval_half / sh_grad_half).
template <typename T> struct Arith { using type = T; };
template <> struct Arith<_Float16> { using type = float; };

// ---- bare SH encoder ------------------------------------------------------------------------------------------------
template <int kSh, typename T>
__global__ void __launch_bounds__(256) sh_encode_forward_kernel(int B, int D, int C, const T* __restrict__ in,
                                                                T* __restrict__ out) {
  using A = typename Arith<T>::type;
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  A Y[kSh];
  if constexpr (std::is_same<T, _Float16>::value && kSh == 16)
    sh_eval_half(C, (A) in[(size_t) b * D], (A) in[(size_t) b * D + 1], (A) in[(size_t) b * D + 2], Y);
  else
    sh_eval(C, (A) in[(size_t) b * D], (A) in[(size_t) b * D + 1], (A) in[(size_t) b * D + 2], Y);
  const int n = sh_count(C);
  T* o        = out + (size_t) b * n;
  if constexpr (std::is_same<T, float>::value) {
    if ((n & 3) == 0) {
      for (int l = 0; l < n; l += 4) *(float4*) (o + l) = make_float4(Y[l], Y[l + 1], Y[l + 2], Y[l + 3]);
      return;
    }
  }
  for (int l = 0; l < n; ++l) o[l] = (T) Y[l];
}

template <int kSh, typename T>
__global__ void __launch_bounds__(256) sh_encode_backward_kernel(int B, int D, int C, const T* __restrict__ grad,
    const T* __restrict__ in, T* __restrict__ grad_in) {
  using A = typename Arith<T>::type;
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  const int n = sh_count(C);
  A t[kSh];
  const T* g = grad + (size_t) b * n;
  bool loaded = false;
  if constexpr (std::is_same<T, float>::value) {
    if ((n & 3) == 0) {
      for (int l = 0; l < n; l += 4) {
        const float4 v = *(const float4*) (g + l);
        t[l] = v.x, t[l + 1] = v.y, t[l + 2] = v.z, t[l + 3] = v.w;
      }
      loaded = true;
    }
  }
  if (!loaded)
    for (int l = 0; l < n; ++l) t[l] = (A) g[l];
  A dx = 0, dy = 0, dz = 0;
  if constexpr (std::is_same<T, _Float16>::value && kSh == 16)
    sh_grad_half(C, (A) in[(size_t) b * D], (A) in[(size_t) b * D + 1], (A) in[(size_t) b * D + 2], t, dx, dy, dz);
  else
    sh_grad_accumulate(C, (A) in[(size_t) b * D], (A) in[(size_t) b * D + 1], (A) in[(size_t) b * D + 2], t, dx, dy, dz);
  grad_in[(size_t) b * D] = (T) dx, grad_in[(size_t) b * D + 1] = (T) dy, grad_in[(size_t) b * D + 2] = (T) dz;
}

// ---- frequency encoder ------------------------------------------------------------------------------------------------
// The angle is scaled and its sine / cosine taken in single precision for double tensors too: the reference goes through
// scalbnf, whose argument and result are float (freqencoder.cu:27-28). The backward is in T throughout (:54).
template <typename T>
__global__ void __launch_bounds__(128) freq_encode_forward_kernel(int B, int Din, int degree, int include_input,
    T scale, const T* __restrict__ in, T* __restrict__ out) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= B * Din) return;
  const int b = t / Din, c = t - b * Din;
  const int Dout = Din * (2 * degree + (include_input ? 1 : 0));
  T* o = out + (size_t) b * Dout + c;
  T x  = in[t];
  if (include_input) o[0] = x, o += Din;
  x = x * scale;
  const float xf = (float) x;
  for (int d = 0; d < degree; ++d) {
    const float v = ldexpf(xf, d);
    o[(2 * d + 0) * Din] = (T) sinf(v);
    o[(2 * d + 1) * Din] = (T) cosf(v);
  }
}

template <typename T>
__global__ void __launch_bounds__(128) freq_encode_backward_kernel(int B, int Din, int degree, int include_input,
    T scale, const T* __restrict__ grad, const T* __restrict__ outv, T* __restrict__ gin) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= B * Din) return;
  const int b = t / Din, c = t - b * Din;
  const int Dout = Din * (2 * degree + (include_input ? 1 : 0));
  const T* g = grad + (size_t) b * Dout + c;
  const T* o = outv + (size_t) b * Dout + c;
  T gx = 0;
  if (include_input) gx = g[0], g += Din, o += Din;
  for (int f = 0; f < degree; ++f) {
    gx += ldexpf(1.0f, f) * scale * (g[0] * o[Din] - g[Din] * o[0]);
    g += 2 * Din, o += 2 * Din;
  }
  gin[t] = gx;
}

// ---- nearest / farthest point -------------------------------------------------------------------------------------------
constexpr int kCtrlChunk = 1024;  // control points staged per LDS round (x 3 values for the D == 3 fast path)

template <int kD, typename T>
__global__ void __launch_bounds__(128) cdist_top_kernel(int N, int M, int D, int largest, const T* __restrict__ x,
    const T* __restrict__ y, T* __restrict__ dist, int64_t* __restrict__ index) {
#pragma clang fp contract(off)
  __shared__ T s_y[kD > 0 ? kCtrlChunk * kD : 1];
  const int b = blockIdx.y;
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  const T* yb = y + (size_t) b * M * D;
  const T* xp = x + ((size_t) b * N + (n < N ? n : 0)) * D;
  T xr[kD > 0 ? kD : 1];
  if (kD > 0)
#pragma unroll
    for (int d = 0; d < kD; ++d) xr[d] = xp[d];
  T top    = 0;
  int topi = 0;
  if (kD > 0) {
    for (int m0 = 0; m0 < M; m0 += kCtrlChunk) {
      const int mc = min(kCtrlChunk, M - m0);
      __syncthreads();
      for (int k = threadIdx.x; k < mc * kD; k += blockDim.x) s_y[k] = yb[(size_t) m0 * kD + k];
      __syncthreads();
      for (int m = 0; m < mc; ++m) {
        T sum = 0;
#pragma unroll
        for (int d = 0; d < kD; ++d) {
          const T t = xr[d] - s_y[m * kD + d];
          sum += t * t;
        }
        if ((m0 + m) == 0 || (sum > top) == (bool) largest) top = sum, topi = m0 + m;
      }
    }
  } else {
    for (int m = 0; m < M; ++m) {
      T sum = 0;
      for (int d = 0; d < D; ++d) {
        const T t = xp[d] - yb[(size_t) m * D + d];
        sum += t * t;
      }
      if (m == 0 || (sum > top) == (bool) largest) top = sum, topi = m;
    }
  }
  if (n < N) {
    dist[(size_t) b * N + n]  = sqrt(top);
    index[(size_t) b * N + n] = topi;
  }
}

template <typename T>
__global__ void __launch_bounds__(256) cdist_top_backward_kernel(int B, int N, int M, int D, const T* __restrict__ p1,
    const T* __restrict__ p2, const T* __restrict__ gdist, const T* __restrict__ dist,
    const int64_t* __restrict__ index, T* __restrict__ g1, T* __restrict__ g2) {
  const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t) B * N) return;
  const int b  = (int) (i / N);
  const int j2 = (int) index[i];
  const T g    = gdist[i] / dist[i];
  for (int d = 0; d < D; ++d) {
    const T t = g * (p1[(size_t) i * D + d] - p2[((size_t) b * M + j2) * D + d]);
    g1[(size_t) i * D + d] = t;
    atomicAdd(&g2[((size_t) b * M + j2) * D + d], -t);
  }
}

// ---- K nearest control points ---------------------------------------------------------------------------------------------
// Squared distances ascending, ties -> lower index first. One lane per query, candidates broadcast from LDS eight at a
// time: the eight distances are formed first (their LDS reads are issued together instead of one exposed round trip per
// candidate), then each is offered to the sorted list. The list update is a clamp per slot for the distances
// (new[k] = med3(old[k-1], d, old[k]), the list being sorted) and two selects per slot for the indices, decided by the
// strict comparisons against the old list, so an equal distance never displaces an earlier (lower) index.
constexpr int kKnnUnroll = 8;
template <int kD, int kK>
__global__ void __launch_bounds__(256) knn_topk_kernel(int N, int M, int D, int K, const float* __restrict__ x,
    const float* __restrict__ y, float* __restrict__ dist2, int64_t* __restrict__ index) {
#pragma clang fp contract(off)
  __shared__ __attribute__((aligned(16))) float s_y[kD > 0 ? (kCtrlChunk + kKnnUnroll) * kD : 1];
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  const float* xp = x + (size_t) (n < N ? n : 0) * D;
  float xr[kD > 0 ? kD : 1];
  if (kD > 0)
#pragma unroll
    for (int d = 0; d < kD; ++d) xr[d] = xp[d];
  float bd[kK];
  int bi[kK];
#pragma unroll
  for (int k = 0; k < kK; ++k) bd[k] = __builtin_inff(), bi[k] = -1;
  auto offer = [&](float cd, int ci) {
    if (cd < bd[kK - 1]) {
      bool lt[kK];
#pragma unroll
      for (int k = 0; k < kK; ++k) lt[k] = cd < bd[k];
#pragma unroll
      for (int k = kK - 1; k >= 1; --k) {
        bd[k] = __builtin_amdgcn_fmed3f(bd[k - 1], cd, bd[k]);
        bi[k] = lt[k - 1] ? bi[k - 1] : (lt[k] ? ci : bi[k]);
      }
      bd[0] = lt[0] ? cd : bd[0];  // a select on the comparison already made (fminf adds two canonicalising moves)
      bi[0] = lt[0] ? ci : bi[0];
    }
  };
  for (int m0 = 0; m0 < M; m0 += kCtrlChunk) {
    const int mc = min(kCtrlChunk, M - m0);
    if (kD > 0) {
      __syncthreads();
      const int padded = (mc + kKnnUnroll - 1) / kKnnUnroll * kKnnUnroll;  // candidates past the end sit at infinity
      for (int k = threadIdx.x; k < padded * kD; k += blockDim.x)
        s_y[k] = k < mc * kD ? y[(size_t) m0 * kD + k] : __builtin_inff();
      __syncthreads();
      for (int m = 0; m < mc; m += kKnnUnroll) {
        float cand[kKnnUnroll];
#pragma unroll
        for (int u = 0; u < kKnnUnroll; ++u) {
          float sum = 0.0f;
#pragma unroll
          for (int d = 0; d < kD; ++d) {
            const float t = xr[d] - s_y[(m + u) * kD + d];
            sum += t * t;
          }
          cand[u] = sum;
        }
#pragma unroll
        for (int u = 0; u < kKnnUnroll; ++u) offer(cand[u], m0 + m + u);
      }
    } else {
      for (int m = 0; m < mc; ++m) {
        float sum = 0.0f;
        for (int d = 0; d < D; ++d) {
          const float t = xp[d] - y[(size_t) (m0 + m) * D + d];
          sum += t * t;
        }
        offer(sum, m0 + m);
      }
    }
  }
  if (n < N) {
#pragma unroll
    for (int k = 0; k < kK; ++k)
      if (k < K) {
        dist2[(size_t) n * K + k] = bi[k] >= 0 ? bd[k] : -1.0f;
        index[(size_t) n * K + k] = bi[k];
      }
  }
}

// ---- LBS skinning (per-control-point table and weights: lbs.hpp) -----------------------------------------------------
template <int kMaxK>
__global__ void __launch_bounds__(256) lbs_blend_kernel(int N, int M, int K, int S, int warp_mode, int weight_mode,
    float temperature, const float* __restrict__ points, const float* __restrict__ xf, const float* __restrict__ sp_r,
    const float* __restrict__ sp_s, const float* __restrict__ pair_in, const int64_t* __restrict__ index,
    float* __restrict__ weights_out, float* __restrict__ d_xyz, float* __restrict__ d_rot,
    float* __restrict__ d_scale) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N) return;
  const int64_t* id = index + (size_t) n * K;
  float u[kMaxK], inv_den;
  lbs_weights<kMaxK>(weight_mode, K, M, 1.0f / temperature, pair_in + (size_t) n * K, id, xf, u, inv_den);
  const float p[3] = {points[3 * (size_t) n], points[3 * (size_t) n + 1], points[3 * (size_t) n + 2]};
  float acc[3] = {0, 0, 0}, ar[4] = {0, 0, 0, 0}, as[4] = {0, 0, 0, 0};
#pragma unroll
  for (int k = 0; k < kMaxK; ++k) {
    if (k >= K) break;
    const int64_t j = id[k];
    if (j < 0 || j >= M) {
      if (weights_out) weights_out[(size_t) n * K + k] = 0.0f;
      continue;
    }
    const float w  = u[k] * inv_den;
    const float* X = xf + (size_t) kXf * j;
    if (warp_mode != 0) {
#pragma unroll
      for (int a = 0; a < 3; ++a) acc[a] += w * (X[a * 3] * p[0] + X[a * 3 + 1] * p[1] + X[a * 3 + 2] * p[2] + X[9 + a]);
    } else {
#pragma unroll
      for (int a = 0; a < 3; ++a) acc[a] += w * X[9 + a];
    }
#pragma unroll
    for (int a = 0; a < 4; ++a) ar[a] += w * sp_r[4 * j + a];
    for (int a = 0; a < S; ++a) as[a] += w * sp_s[(size_t) S * j + a];
    if (weights_out) weights_out[(size_t) n * K + k] = w;
  }
#pragma unroll
  for (int a = 0; a < 3; ++a) d_xyz[3 * (size_t) n + a] = warp_mode != 0 ? acc[a] - p[a] : acc[a];
#pragma unroll
  for (int a = 0; a < 4; ++a) d_rot[4 * (size_t) n + a] = ar[a];
  for (int a = 0; a < S; ++a) d_scale[(size_t) S * n + a] = as[a];
}

// ---- masked Adam ------------------------------------------------------------------------------------------------------------
// One lane per 4 consecutive elements when rows are a multiple of 4 floats, else one lane per element.
template <int kVec>
__global__ void __launch_bounds__(256) adam_masked_kernel(int64_t total, int64_t M, const uint8_t* __restrict__ mask,
    float lr, float b1, float b2, float eps, float* __restrict__ param, const float* __restrict__ grad,
    float* __restrict__ m, float* __restrict__ v) {
#pragma clang fp contract(off)
  const int64_t e = ((int64_t) blockIdx.x * blockDim.x + threadIdx.x) * kVec;
  if (e >= total) return;
  if (!mask[e / M]) return;
  float g[kVec], mm[kVec], vv[kVec], pp[kVec];
  if (kVec == 4) {
    *(float4*) g  = *(const float4*) (grad + e);
    *(float4*) mm = *(const float4*) (m + e);
    *(float4*) vv = *(const float4*) (v + e);
    *(float4*) pp = *(const float4*) (param + e);
  } else {
    g[0] = grad[e], mm[0] = m[e], vv[0] = v[e], pp[0] = param[e];
  }
#pragma unroll
  for (int k = 0; k < kVec; ++k) {
    mm[k] = b1 * mm[k] + (1.0f - b1) * g[k];
    vv[k] = b2 * vv[k] + (1.0f - b2) * g[k] * g[k];
    pp[k] += -lr * mm[k] / (sqrtf(vv[k]) + eps);
  }
  if (kVec == 4) {
    *(float4*) (param + e) = *(float4*) pp;
    *(float4*) (m + e)     = *(float4*) mm;
    *(float4*) (v + e)     = *(float4*) vv;
  } else {
    param[e] = pp[0], m[e] = mm[0], v[e] = vv[0];
  }
}

// ---- deformed parameters --------------------------------------------------------------------------------------------
// network.py:630, :643, :645: points + d_xyz, scaling_activation(scales) + d_scale (exp when the scales are stored as
// logarithms), normalize(rotations + d_rotation) with torch.nn.functional.normalize's 1e-12 floor on the norm. One lane
// per point; the reference runs these as separate torch operators with their autograd nodes.
template <int S>
__global__ void __launch_bounds__(256) deform_apply_forward_kernel(int N, int log_scales,
    const float* __restrict__ points, const float* __restrict__ d_xyz, const float* __restrict__ scales,
    const float* __restrict__ d_scale, const float* __restrict__ rot, const float* __restrict__ d_rot,
    float* __restrict__ out_points, float* __restrict__ out_scales, float* __restrict__ out_rot) {
#pragma clang fp contract(off)
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N) return;
#pragma unroll
  for (int c = 0; c < 3; ++c) out_points[3 * (size_t) i + c] = points[3 * (size_t) i + c] + d_xyz[3 * (size_t) i + c];
#pragma unroll
  for (int c = 0; c < S; ++c) {
    const float v = scales[S * (size_t) i + c];
    out_scales[S * (size_t) i + c] = (log_scales ? expf(v) : v) + d_scale[S * (size_t) i + c];
  }
  const float4 a = ((const float4*) rot)[i], b = ((const float4*) d_rot)[i];
  const float x = a.x + b.x, y = a.y + b.y, z = a.z + b.z, w = a.w + b.w;
  const float inv = 1.0f / fmaxf(sqrtf(x * x + y * y + z * z + w * w), 1e-12f);
  ((float4*) out_rot)[i] = make_float4(x * inv, y * inv, z * inv, w * inv);
}

// Gradients that are not the upstream gradient itself: through the normalisation to rotations / d_rotation (the same
// tensor for both) and, for logarithmic scales, g * exp(scale). points, d_xyz and d_scale receive their output's
// gradient unchanged, so nothing is computed for them.
template <int S>
__global__ void __launch_bounds__(256) deform_apply_backward_kernel(int N, int log_scales,
    const float* __restrict__ scales, const float* __restrict__ rot, const float* __restrict__ d_rot,
    const float* __restrict__ g_out_scales, const float* __restrict__ g_out_rot, float* __restrict__ g_scales,
    float* __restrict__ g_rot) {
#pragma clang fp contract(off)
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N) return;
  if (log_scales)
#pragma unroll
    for (int c = 0; c < S; ++c)
      g_scales[S * (size_t) i + c] = g_out_scales[S * (size_t) i + c] * expf(scales[S * (size_t) i + c]);
  const float4 a = ((const float4*) rot)[i], b = ((const float4*) d_rot)[i], g = ((const float4*) g_out_rot)[i];
  const float x = a.x + b.x, y = a.y + b.y, z = a.z + b.z, w = a.w + b.w;
  const float n = sqrtf(x * x + y * y + z * z + w * w);
  float4 o;
  if (n > 1e-12f) {
    const float inv = 1.0f / n;
    const float qx = x * inv, qy = y * inv, qz = z * inv, qw = w * inv;
    const float dot = qx * g.x + qy * g.y + qz * g.z + qw * g.w;
    o = make_float4((g.x - qx * dot) * inv, (g.y - qy * dot) * inv, (g.z - qz * dot) * inv, (g.w - qw * dot) * inv);
  } else {
    o = make_float4(g.x * 1e12f, g.y * 1e12f, g.z * 1e12f, g.w * 1e12f);
  }
  ((float4*) g_rot)[i] = o;
}

// The same update for every parameter tensor of a point set in one launch: the reference steps its parameter groups one
// kernel at a time (sparse_gaussian_adam.py:20-45), each a few microseconds of work behind a launch. Table passed by
// value; the blocks of all tensors form one grid (a block finds its tensor in the table's block prefix), so no block
// is launched for nothing, and every tensor whose element count and addresses allow it moves as 16-byte pieces whatever
// its row length: the four elements of a piece look up their own rows in the mask. Same arithmetic as
// adam_masked_kernel, element for element.
constexpr int kMaxAdamTensors = 12;
struct AdamTable {
  float* param[kMaxAdamTensors];
  const float* grad[kMaxAdamTensors];
  float* m[kMaxAdamTensors];
  float* v[kMaxAdamTensors];
  int64_t M[kMaxAdamTensors];
  float lr[kMaxAdamTensors], eps[kMaxAdamTensors];
  int vec4[kMaxAdamTensors];
  unsigned first_block[kMaxAdamTensors + 1];
  int n;
};

__global__ void __launch_bounds__(256) adam_masked_multi_kernel(AdamTable t, int64_t N, float b1, float b2,
                                                                const uint8_t* __restrict__ mask) {
#pragma clang fp contract(off)
  int q = 0;
  while (q + 1 < t.n && blockIdx.x >= t.first_block[q + 1]) ++q;
  const int64_t M = t.M[q], total = N * M;
  const int vec   = t.vec4[q] ? 4 : 1;
  const int64_t e = ((int64_t) (blockIdx.x - t.first_block[q]) * blockDim.x + threadIdx.x) * vec;
  if (e >= total) return;
  const float lr = t.lr[q], eps = t.eps[q];
  float* __restrict__ param = t.param[q];
  const float* __restrict__ grad = t.grad[q];
  float* __restrict__ m = t.m[q];
  float* __restrict__ v = t.v[q];
  if (vec == 1) {
    if (!mask[e / M]) return;
    const float g = grad[e];
    const float mm = b1 * m[e] + (1.0f - b1) * g;
    const float vv = b2 * v[e] + (1.0f - b2) * g * g;
    param[e] += -lr * mm / (sqrtf(vv) + eps);
    m[e] = mm, v[e] = vv;
    return;
  }
  // rows of the piece's four elements (a piece may straddle rows, several of them when rows are shorter than four)
  int64_t row = e / M, rem = e - row * M;
  bool on[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    on[k] = mask[row] != 0;
    if (++rem == M) rem = 0, ++row;
    if (row >= N) row = N - 1;  // only past the last element of the tensor, which e + k < total excludes
  }
  if (!(on[0] | on[1] | on[2] | on[3])) return;
  float g[4], mm[4], vv[4], pp[4];
  *(float4*) g  = *(const float4*) (grad + e);
  *(float4*) mm = *(const float4*) (m + e);
  *(float4*) vv = *(const float4*) (v + e);
  *(float4*) pp = *(const float4*) (param + e);
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float m1 = b1 * mm[k] + (1.0f - b1) * g[k];
    const float v1 = b2 * vv[k] + (1.0f - b2) * g[k] * g[k];
    const float p1 = pp[k] + -lr * m1 / (sqrtf(v1) + eps);
    mm[k] = on[k] ? m1 : mm[k], vv[k] = on[k] ? v1 : vv[k], pp[k] = on[k] ? p1 : pp[k];
  }
  *(float4*) (param + e) = *(float4*) pp;  // elements of masked rows are written back as they were
  *(float4*) (m + e)     = *(float4*) mm;
  *(float4*) (v + e)     = *(float4*) vv;
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API int fsgs_deform_apply_forward(int N, int S, int log_scales, const float* points, const float* d_xyz,
    const float* scales, const float* d_scale, const float* rot, const float* d_rot, float* out_points,
    float* out_scales, float* out_rot, void* stream) {
  FSGS_REQUIRE(N >= 0 && (S == 2 || S == 3), "deform_apply: N >= 0 and 2 or 3 scales per point");
  if (N == 0) return kOk;
  FSGS_REQUIRE(points && d_xyz && scales && d_scale && rot && d_rot && out_points && out_scales && out_rot,
               "deform_apply: null pointer");
  FSGS_REQUIRE((((uintptr_t) rot | (uintptr_t) d_rot | (uintptr_t) out_rot) & 15) == 0,
               "deform_apply: rotations must be 16-byte aligned");
  auto kernel = S == 2 ? deform_apply_forward_kernel<2> : deform_apply_forward_kernel<3>;
  hipLaunchKernelGGL(kernel, dim3(div_up(N, 256)), dim3(256), 0, (hipStream_t) stream, N, log_scales, points, d_xyz,
                     scales, d_scale, rot, d_rot, out_points, out_scales, out_rot);
  return check_launch("deform_apply");
}

FSGS_API int fsgs_deform_apply_backward(int N, int S, int log_scales, const float* scales, const float* rot,
    const float* d_rot, const float* g_out_scales, const float* g_out_rot, float* g_scales, float* g_rot,
    void* stream) {
  FSGS_REQUIRE(N >= 0 && (S == 2 || S == 3), "deform_apply_backward: N >= 0 and 2 or 3 scales per point");
  if (N == 0) return kOk;
  FSGS_REQUIRE(rot && d_rot && g_out_rot && g_rot && (!log_scales || (scales && g_out_scales && g_scales)),
               "deform_apply_backward: null pointer");
  FSGS_REQUIRE((((uintptr_t) rot | (uintptr_t) d_rot | (uintptr_t) g_out_rot | (uintptr_t) g_rot) & 15) == 0,
               "deform_apply_backward: rotations must be 16-byte aligned");
  auto kernel = S == 2 ? deform_apply_backward_kernel<2> : deform_apply_backward_kernel<3>;
  hipLaunchKernelGGL(kernel, dim3(div_up(N, 256)), dim3(256), 0, (hipStream_t) stream, N, log_scales, scales, rot,
                     d_rot, g_out_scales, g_out_rot, g_scales, g_rot);
  return check_launch("deform_apply_backward");
}

FSGS_API int fsgs_adam_masked_update_max_tensors(void) { return kMaxAdamTensors; }

FSGS_API int fsgs_adam_masked_update_multi(int n_tensors, int64_t N, const int64_t* M, const uint8_t* mask,
    const double* lr, double b1, double b2, const double* eps, float* const* param, const float* const* grad,
    float* const* m, float* const* v, void* stream) {
  FSGS_REQUIRE(n_tensors >= 0 && n_tensors <= kMaxAdamTensors && N >= 0,
               "AdamMasksedUpdated (multi): bad arguments (at most %d tensors)", kMaxAdamTensors);
  if (n_tensors == 0 || N == 0) return kOk;
  FSGS_REQUIRE(M && mask && lr && eps && param && grad && m && v, "AdamMasksedUpdated (multi): null pointer");
  AdamTable t{};
  t.n = n_tensors;
  unsigned blocks = 0;
  for (int q = 0; q < n_tensors; ++q) {
    FSGS_REQUIRE(M[q] > 0 && param[q] && grad[q] && m[q] && v[q], "AdamMasksedUpdated (multi): bad tensor %d", q);
    t.param[q] = param[q], t.grad[q] = grad[q], t.m[q] = m[q], t.v[q] = v[q], t.M[q] = M[q];
    t.lr[q] = (float) lr[q], t.eps[q] = (float) eps[q];
    const int64_t total = N * M[q];
    t.vec4[q] = (total % 4 == 0) &&
                (((uintptr_t) param[q] | (uintptr_t) grad[q] | (uintptr_t) m[q] | (uintptr_t) v[q]) % 16 == 0);
    t.first_block[q] = blocks;
    const int64_t nb = div_up(t.vec4[q] ? total / 4 : total, (int64_t) 256);
    FSGS_REQUIRE((int64_t) blocks + nb < (int64_t) 0x7fffffff, "AdamMasksedUpdated (multi): too many elements");
    blocks += (unsigned) nb;
  }
  t.first_block[n_tensors] = blocks;
  hipLaunchKernelGGL(adam_masked_multi_kernel, dim3(blocks), dim3(256), 0, (hipStream_t) stream, t, N, (float) b1,
                     (float) b2, mask);
  return check_launch("AdamMasksedUpdated");
}

FSGS_API int fsgs_sh_to_rgb_forward(int P, int F, int degree, int clamp, const float* pos, const float* campos,
                                    const float* sh, float* rgb, void* stream) {
  FSGS_REQUIRE(P >= 0 && pos && sh && rgb, "SH_to_RGB_forward: bad arguments");
  FSGS_REQUIRE(0 <= degree && degree <= kMaxShDegree && (degree + 1) * (degree + 1) <= F,
               "SH_to_RGB_forward: degree %d unsupported or > features %d", degree, F);
  if (P == 0) return kOk;
  const bool rows = degree == 3 && F == 16 && ((uintptr_t) sh & 15) == 0;
  auto kernel = degree > 3 ? sh_to_rgb_forward_kernel<64, false>
                           : (rows ? sh_to_rgb_forward_kernel<16, true> : sh_to_rgb_forward_kernel<16, false>);
  hipLaunchKernelGGL(kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P, F, degree,
                     clamp, pos, campos, sh, rgb);
  return check_launch("SH_to_RGB_forward");
}

FSGS_API int fsgs_sh_to_rgb_backward(int P, int F, int degree, int clamp, const float* pos, const float* campos,
    const float* sh, const float* rgb, const float* grad_rgb, float* grad_dir, float* grad_campos, float* grad_sh,
    void* stream) {
  FSGS_REQUIRE(P >= 0 && pos && sh && rgb && grad_rgb, "SH_to_RGB_backward: bad arguments");
  FSGS_REQUIRE(0 <= degree && degree <= kMaxShDegree && (degree + 1) * (degree + 1) <= F,
               "SH_to_RGB_backward: degree %d unsupported or > features %d", degree, F);
  FSGS_REQUIRE(!grad_campos || campos, "SH_to_RGB_backward: grad_campos without campos");
  if (P == 0) return kOk;
  const bool rows = degree == 3 && F == 16 && (((uintptr_t) sh | (uintptr_t) grad_sh) & 15) == 0;
  auto kernel = degree > 3 ? sh_to_rgb_backward_kernel<64, false>
                           : (rows ? sh_to_rgb_backward_kernel<16, true> : sh_to_rgb_backward_kernel<16, false>);
  hipLaunchKernelGGL(kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P, F, degree,
                     clamp, pos, campos, sh, rgb, grad_rgb, grad_dir, grad_campos, grad_sh);
  return check_launch("SH_to_RGB_backward");
}

// ---- encoders and nearest / farthest search: one typed entry each plus the single-precision shorthand -----------------
namespace {
template <typename T>
int sh_encode_forward_t(int B, int D, int C, const void* in, void* out, hipStream_t s) {
  auto kernel = C > 3 ? sh_encode_forward_kernel<64, T> : sh_encode_forward_kernel<16, T>;
  hipLaunchKernelGGL(kernel, dim3(div_up(B, 256)), dim3(256), 0, s, B, D, C, (const T*) in, (T*) out);
  return check_launch("sh_encode_forward");
}
template <typename T>
int sh_encode_backward_t(int B, int D, int C, const void* grad, const void* in, void* grad_in, hipStream_t s) {
  auto kernel = C > 3 ? sh_encode_backward_kernel<64, T> : sh_encode_backward_kernel<16, T>;
  hipLaunchKernelGGL(kernel, dim3(div_up(B, 256)), dim3(256), 0, s, B, D, C, (const T*) grad, (const T*) in,
                     (T*) grad_in);
  return check_launch("sh_encode_backward");
}
template <typename T>
int freq_encode_forward_t(int B, int Din, int degree, int include_input, double scale, const void* in, void* out,
                          hipStream_t s) {
  hipLaunchKernelGGL(freq_encode_forward_kernel<T>, dim3(div_up((int64_t) B * Din, 128)), dim3(128), 0, s, B, Din,
                     degree, include_input, (T) scale, (const T*) in, (T*) out);
  return check_launch("freq_encode_forward");
}
template <typename T>
int freq_encode_backward_t(int B, int Din, int degree, int include_input, double scale, const void* grad,
                           const void* outv, void* gin, hipStream_t s) {
  hipLaunchKernelGGL(freq_encode_backward_kernel<T>, dim3(div_up((int64_t) B * Din, 128)), dim3(128), 0, s, B, Din,
                     degree, include_input, (T) scale, (const T*) grad, (const T*) outv, (T*) gin);
  return check_launch("freq_encode_backward");
}
template <typename T>
int cdist_top_forward_t(int B, int N, int M, int D, int largest, const void* x, const void* y, void* dist,
                        int64_t* index, hipStream_t s) {
  const dim3 grid(div_up(N, 128), B), block(128);
  if (D == 3)
    hipLaunchKernelGGL((cdist_top_kernel<3, T>), grid, block, 0, s, N, M, D, largest, (const T*) x, (const T*) y,
                       (T*) dist, index);
  else
    hipLaunchKernelGGL((cdist_top_kernel<0, T>), grid, block, 0, s, N, M, D, largest, (const T*) x, (const T*) y,
                       (T*) dist, index);
  return check_launch("cdist_top");
}
template <typename T>
int cdist_top_backward_t(int B, int N, int M, int D, const void* p1, const void* p2, const void* dist,
                         const int64_t* index, const void* gdist, void* g1, void* g2, hipStream_t s) {
  hipLaunchKernelGGL(cdist_top_backward_kernel<T>, dim3(div_up((int64_t) B * N, 256)), dim3(256), 0, s, B, N, M, D,
                     (const T*) p1, (const T*) p2, (const T*) gdist, (const T*) dist, index, (T*) g1, (T*) g2);
  return check_launch("cdist_top_backward");
}
}  // namespace

FSGS_API int fsgs_sh_encode_forward_typed(int dtype, int B, int D, int C, const void* in, void* out, void* stream) {
  FSGS_REQUIRE(B >= 0 && D >= 3 && in && out, "sh_encode_forward: bad arguments");
  FSGS_REQUIRE(0 <= C && C <= kMaxShDegree, "sh_encode_forward: degree %d not supported (max %d)", C, kMaxShDegree);
  FSGS_REQUIRE(dtype == FSGS_DTYPE_F32 || dtype == FSGS_DTYPE_F64 || dtype == FSGS_DTYPE_F16,
               "sh_encode_forward: element type %d not supported", dtype);
  if (B == 0) return kOk;
  if (dtype == FSGS_DTYPE_F64) return sh_encode_forward_t<double>(B, D, C, in, out, (hipStream_t) stream);
  if (dtype == FSGS_DTYPE_F16) return sh_encode_forward_t<_Float16>(B, D, C, in, out, (hipStream_t) stream);
  return sh_encode_forward_t<float>(B, D, C, in, out, (hipStream_t) stream);
}

FSGS_API int fsgs_sh_encode_forward(int B, int D, int C, const float* in, float* out, void* stream) {
  return fsgs_sh_encode_forward_typed(FSGS_DTYPE_F32, B, D, C, in, out, stream);
}

FSGS_API int fsgs_sh_encode_backward_typed(int dtype, int B, int D, int C, const void* grad, const void* in,
                                           void* grad_in, void* stream) {
  FSGS_REQUIRE(B >= 0 && D >= 3 && grad && in && grad_in, "sh_encode_backward: bad arguments");
  FSGS_REQUIRE(0 <= C && C <= kMaxShDegree, "sh_encode_backward: degree %d not supported (max %d)", C, kMaxShDegree);
  FSGS_REQUIRE(dtype == FSGS_DTYPE_F32 || dtype == FSGS_DTYPE_F64 || dtype == FSGS_DTYPE_F16,
               "sh_encode_backward: element type %d not supported", dtype);
  if (B == 0) return kOk;
  if (dtype == FSGS_DTYPE_F64) return sh_encode_backward_t<double>(B, D, C, grad, in, grad_in, (hipStream_t) stream);
  if (dtype == FSGS_DTYPE_F16) return sh_encode_backward_t<_Float16>(B, D, C, grad, in, grad_in, (hipStream_t) stream);
  return sh_encode_backward_t<float>(B, D, C, grad, in, grad_in, (hipStream_t) stream);
}

FSGS_API int fsgs_sh_encode_backward(int B, int D, int C, const float* grad, const float* in, float* grad_in,
                                     void* stream) {
  return fsgs_sh_encode_backward_typed(FSGS_DTYPE_F32, B, D, C, grad, in, grad_in, stream);
}

FSGS_API int fsgs_freq_encode_forward_typed(int dtype, int B, int Din, int degree, int include_input, double scale,
                                            const void* in, void* out, void* stream) {
  FSGS_REQUIRE(B >= 0 && Din > 0 && degree >= 0 && in && out, "freq_encode_forward: bad arguments");
  FSGS_REQUIRE(dtype == FSGS_DTYPE_F32 || dtype == FSGS_DTYPE_F64, "freq_encode_forward: element type %d not supported",
               dtype);
  if (B == 0) return kOk;
  if (dtype == FSGS_DTYPE_F64)
    return freq_encode_forward_t<double>(B, Din, degree, include_input, scale, in, out, (hipStream_t) stream);
  return freq_encode_forward_t<float>(B, Din, degree, include_input, scale, in, out, (hipStream_t) stream);
}

FSGS_API int fsgs_freq_encode_forward(int B, int Din, int degree, int include_input, double scale, const float* in,
                                      float* out, void* stream) {
  return fsgs_freq_encode_forward_typed(FSGS_DTYPE_F32, B, Din, degree, include_input, scale, in, out, stream);
}

FSGS_API int fsgs_freq_encode_backward_typed(int dtype, int B, int Din, int degree, int include_input, double scale,
                                             const void* grad, const void* outv, void* gin, void* stream) {
  FSGS_REQUIRE(B >= 0 && Din > 0 && degree >= 0 && grad && outv && gin, "freq_encode_backward: bad arguments");
  FSGS_REQUIRE(dtype == FSGS_DTYPE_F32 || dtype == FSGS_DTYPE_F64,
               "freq_encode_backward: element type %d not supported", dtype);
  if (B == 0) return kOk;
  if (dtype == FSGS_DTYPE_F64)
    return freq_encode_backward_t<double>(B, Din, degree, include_input, scale, grad, outv, gin, (hipStream_t) stream);
  return freq_encode_backward_t<float>(B, Din, degree, include_input, scale, grad, outv, gin, (hipStream_t) stream);
}

FSGS_API int fsgs_freq_encode_backward(int B, int Din, int degree, int include_input, double scale, const float* grad,
                                       const float* outv, float* gin, void* stream) {
  return fsgs_freq_encode_backward_typed(FSGS_DTYPE_F32, B, Din, degree, include_input, scale, grad, outv, gin, stream);
}

FSGS_API int fsgs_cdist_top_forward_typed(int dtype, int B, int N, int M, int D, int largest, const void* x,
                                          const void* y, void* dist, int64_t* index, void* stream) {
  FSGS_REQUIRE(B >= 0 && N >= 0 && M > 0 && D > 0 && x && y && dist && index, "cdist_top: bad arguments");
  FSGS_REQUIRE(dtype == FSGS_DTYPE_F32 || dtype == FSGS_DTYPE_F64, "cdist_top: element type %d not supported", dtype);
  if (B == 0 || N == 0) return kOk;
  if (dtype == FSGS_DTYPE_F64)
    return cdist_top_forward_t<double>(B, N, M, D, largest, x, y, dist, index, (hipStream_t) stream);
  return cdist_top_forward_t<float>(B, N, M, D, largest, x, y, dist, index, (hipStream_t) stream);
}

FSGS_API int fsgs_cdist_top_forward(int B, int N, int M, int D, int largest, const float* x, const float* y,
                                    float* dist, int64_t* index, void* stream) {
  return fsgs_cdist_top_forward_typed(FSGS_DTYPE_F32, B, N, M, D, largest, x, y, dist, index, stream);
}

FSGS_API int fsgs_cdist_top_backward_typed(int dtype, int B, int N, int M, int D, const void* p1, const void* p2,
                                           const void* dist, const int64_t* index, const void* gdist, void* g1,
                                           void* g2, void* stream) {
  FSGS_REQUIRE(B >= 0 && N >= 0 && M > 0 && D > 0 && p1 && p2 && dist && index && gdist && g1 && g2,
               "cdist_top_backward: bad arguments");
  FSGS_REQUIRE(dtype == FSGS_DTYPE_F32 || dtype == FSGS_DTYPE_F64, "cdist_top_backward: element type %d not supported",
               dtype);
  if (B == 0 || N == 0) return kOk;
  if (dtype == FSGS_DTYPE_F64)
    return cdist_top_backward_t<double>(B, N, M, D, p1, p2, dist, index, gdist, g1, g2, (hipStream_t) stream);
  return cdist_top_backward_t<float>(B, N, M, D, p1, p2, dist, index, gdist, g1, g2, (hipStream_t) stream);
}

FSGS_API int fsgs_cdist_top_backward(int B, int N, int M, int D, const float* p1, const float* p2, const float* dist,
                                     const int64_t* index, const float* gdist, float* g1, float* g2, void* stream) {
  return fsgs_cdist_top_backward_typed(FSGS_DTYPE_F32, B, N, M, D, p1, p2, dist, index, gdist, g1, g2, stream);
}

FSGS_API int fsgs_knn_topk(int N, int M, int D, int K, const float* x, const float* y, float* dist2, int64_t* index,
                           void* stream) {
  FSGS_REQUIRE(N >= 0 && M > 0 && D > 0 && K > 0 && x && y && dist2 && index, "knn_topk: bad arguments");
  FSGS_REQUIRE(K <= 16, "knn_topk: K=%d exceeds the supported maximum of 16", K);
  if (N == 0) return kOk;
  const dim3 grid(div_up(N, 256)), block(256);
  hipStream_t s = (hipStream_t) stream;
#define FSGS_KNN(DD, KK) \
  hipLaunchKernelGGL((knn_topk_kernel<DD, KK>), grid, block, 0, s, N, M, D, K, x, y, dist2, index)
  if (D == 3) {
    if (K <= 4) FSGS_KNN(3, 4);
    else if (K <= 8) FSGS_KNN(3, 8);
    else FSGS_KNN(3, 16);
  } else {
    if (K <= 4) FSGS_KNN(0, 4);
    else if (K <= 8) FSGS_KNN(0, 8);
    else FSGS_KNN(0, 16);
  }
#undef FSGS_KNN
  return check_launch("knn_topk");
}

FSGS_API size_t fsgs_lbs_blend_workspace_bytes(int M) { return align_up((size_t) (M > 0 ? M : 1) * kXf * 4, 256); }

FSGS_API int fsgs_lbs_blend(int N, int M, int K, int warp_mode, int weight_mode, double temperature,
    const float* points, const float* sp_points, const float* sp_t, const float* sp_rot, const float* sp_r,
    const float* sp_s, int S, const float* pair_in, const int64_t* index, const float* sp_log_radius,
    const float* sp_weight_logit, float* weights_out, float* d_xyz, float* d_rot, float* d_scale, void* workspace,
    size_t workspace_bytes, void* stream) {
  FSGS_REQUIRE(N >= 0 && M > 0 && K > 0 && K <= 16 && S >= 0 && S <= 4, "lbs_blend: bad sizes (K <= 16, S <= 4)");
  FSGS_REQUIRE(warp_mode >= 0 && warp_mode <= 2 && weight_mode >= 0 && weight_mode <= 3, "lbs_blend: unknown mode");
  FSGS_REQUIRE(points && sp_points && sp_t && sp_r && pair_in && index && d_xyz && d_rot &&
                   (S == 0 || (sp_s && d_scale)) && workspace, "lbs_blend: null pointer");
  FSGS_REQUIRE((warp_mode == 0) == (sp_rot == nullptr),
               "lbs_blend: sp_rot goes with warp modes 1 and 2 and is absent in mode 0 (translation only)");
  FSGS_REQUIRE(weight_mode != 1 || sp_log_radius, "lbs_blend: the kernel weights need sp_log_radius");
  FSGS_REQUIRE(weight_mode != 0 || temperature > 0, "lbs_blend: temperature must be positive");
  if (workspace_bytes < fsgs_lbs_blend_workspace_bytes(M))
    return fail(kWorkspaceSmall, "lbs_blend: workspace %zu < %zu bytes", workspace_bytes,
                fsgs_lbs_blend_workspace_bytes(M));
  if (N == 0) return kOk;
  hipStream_t s = (hipStream_t) stream;
  float* xf     = (float*) workspace;
  hipLaunchKernelGGL(lbs_prepare_kernel, dim3(div_up(M, 256)), dim3(256), 0, s, M, warp_mode, sp_points, sp_t, sp_rot,
                     weight_mode == 1 ? sp_log_radius : nullptr, weight_mode == 1 ? sp_weight_logit : nullptr, xf);
  auto kernel = K <= 4 ? lbs_blend_kernel<4> : lbs_blend_kernel<16>;
  hipLaunchKernelGGL(kernel, dim3(div_up(N, 256)), dim3(256), 0, s, N, M, K, S, warp_mode, weight_mode,
                     (float) temperature, points, xf, sp_r, sp_s, pair_in, index, weights_out, d_xyz, d_rot, d_scale);
  return check_launch("lbs_blend");
}

FSGS_API int fsgs_adam_masked_update(int64_t N, int64_t M, const uint8_t* mask, double lr, double b1, double b2,
                                     double eps, float* param, const float* grad, float* m, float* v, void* stream) {
  FSGS_REQUIRE(N >= 0 && M > 0 && mask && param && grad && m && v, "AdamMasksedUpdated: bad arguments");
  if (N == 0) return kOk;
  const int64_t total = N * M;
  hipStream_t s = (hipStream_t) stream;
  const bool vec4 = (M % 4 == 0) && (((uintptr_t) param | (uintptr_t) grad | (uintptr_t) m | (uintptr_t) v) % 16 == 0);
  if (vec4)
    hipLaunchKernelGGL((adam_masked_kernel<4>), dim3(div_up(total / 4, 256)), dim3(256), 0, s, total, M, mask,
                       (float) lr, (float) b1, (float) b2, (float) eps, param, grad, m, v);
  else
    hipLaunchKernelGGL((adam_masked_kernel<1>), dim3(div_up(total, 256)), dim3(256), 0, s, total, M, mask, (float) lr,
                       (float) b1, (float) b2, (float) eps, param, grad, m, v);
  return check_launch("AdamMasksedUpdated");
}
