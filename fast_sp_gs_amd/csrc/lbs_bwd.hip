// Backward of the LBS blend and of the K-NN squared distances for gfx950.
//
// The reference differentiates fast_2d_gs/network.py:504 (pytorch3d.ops.knn_points), :507-517 (neighbour weights) and
// :545-573 (warp: translations alone, or lietorch.SE3 when a local rotation is given) with torch autograd: ~30 elementwise / gather / scatter launches over [N,K,...] tensors and
// index_add-style atomics into the M control-point rows. Here one kernel walks the Gaussians once:
//   * per-Gaussian outputs (g_points, g_dist2 / g_x) are written directly;
//   * per-control-point sums are accumulated in a block-private LDS table [M][F] with LDS atomics (a few hundred
//     thousand Gaussians share a few hundred control points, so device-scope atomics would serialise on M rows),
//     each block stores its table as one partial, and a second kernel adds the partials in a fixed order;
//   * a last one-lane-per-control-point kernel applies the chain rule through the centring, the rotation matrix and the
//     quaternion normalisation.
// Tables that do not fit in LDS fall back to device-scope atomics on a zeroed accumulator.
#include <algorithm>

#include "common.hpp"
#include "lbs.hpp"

namespace fsgs {
namespace {

constexpr int kTableFloats  = 36864;  // 144 KB of LDS for the per-block table
constexpr int kMaxAccBlocks = 256;    // partial tables per launch
constexpr int kAccThreads   = 1024;  // 16 wavefronts share one LDS table: the loop is bound by gather latency, not by the atomics

__global__ void __launch_bounds__(256) zero_floats_kernel(size_t n, float* __restrict__ p) {
  for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t) gridDim.x * blockDim.x)
    p[i] = 0.0f;
}

// Row of control point j in the table of per-control-point sums (F columns):
//   [G: 9, warp modes 1 and 2 only] sum w g[a] p[b]   [t: 3] sum w g[a]   [r: 4] sum w g_rot[a]   [s: S] sum w g_scale[a]
//   [rho, omega: 2, weight mode 1 only] sum X d2, sum X   with X = (v - <w, v>) / U * exp(-d2 / (2 r^2)), U the sum of the
//   unnormalised weights: the radius and weight-logit gradients follow from them per control point.
struct LbsCols {
  int nG, oT, oR, oS, oK, F;
};
__host__ __device__ inline LbsCols lbs_cols(int warp_mode, int weight_mode, int S) {
  LbsCols c;
  c.nG = warp_mode != 0 ? 9 : 0;
  c.oT = c.nG, c.oR = c.oT + 3, c.oS = c.oR + 4, c.oK = c.oS + S;
  c.F  = c.oK + (weight_mode == 1 ? 2 : 0);
  return c;
}

// What one point contributes: its own outputs (g_points, g_pair) and, per neighbour, the weight w and the kernel-mode
// factor X. v[k] = dL/dw_k = <g_xyz, x_k> + <g_rot, r_j> + <g_scale, s_j> with x_k = R_j p + t_j (or t_j alone).
template <int kMaxK>
struct LbsPoint {
  float p[3], g[3], gr[4], gs[4];
  float w[kMaxK], X[kMaxK];
};
template <int kMaxK>
__device__ __forceinline__ void lbs_point_backward(int n, int M, int K, int S, int warp_mode, int weight_mode,
    float inv_t, const float* __restrict__ points, const float* __restrict__ xf, const float* __restrict__ sp_r,
    const float* __restrict__ sp_s, const float* __restrict__ pair_in, const int64_t* __restrict__ index,
    const float* __restrict__ g_xyz, const float* __restrict__ g_rot, const float* __restrict__ g_scale,
    float* __restrict__ g_points, float* __restrict__ g_pair, LbsPoint<kMaxK>& P) {
  const float* in   = pair_in + (size_t) n * K;
  const int64_t* id = index + (size_t) n * K;
  float u[kMaxK], inv_den;
  lbs_weights<kMaxK>(weight_mode, K, M, inv_t, in, id, xf, u, inv_den);
#pragma unroll
  for (int a = 0; a < 3; ++a) P.p[a] = points[3 * (size_t) n + a], P.g[a] = g_xyz[3 * (size_t) n + a];
#pragma unroll
  for (int a = 0; a < 4; ++a) P.gr[a] = g_rot[4 * (size_t) n + a], P.gs[a] = 0.0f;
#pragma unroll
  for (int a = 0; a < 4; ++a)
    if (a < S) P.gs[a] = g_scale[(size_t) S * n + a];
  float gp[3] = {0, 0, 0}, dot = 0.0f, v[kMaxK];
#pragma unroll
  for (int k = 0; k < kMaxK; ++k) {
    const int64_t j = k < K ? id[k] : -1;
    P.w[k] = 0.0f, P.X[k] = 0.0f, v[k] = 0.0f;
    if (j < 0 || j >= M) continue;
    const float w  = u[k] * inv_den;
    const float* X = xf + (size_t) kXf * j;
    float vk = 0.0f;
    if (warp_mode != 0) {
#pragma unroll
      for (int a = 0; a < 3; ++a) {
        vk += P.g[a] * (X[a * 3] * P.p[0] + X[a * 3 + 1] * P.p[1] + X[a * 3 + 2] * P.p[2] + X[9 + a]);
        gp[a] += w * (X[a] * P.g[0] + X[3 + a] * P.g[1] + X[6 + a] * P.g[2]);
      }
    } else {
#pragma unroll
      for (int a = 0; a < 3; ++a) vk += P.g[a] * X[9 + a];
    }
#pragma unroll
    for (int a = 0; a < 4; ++a) vk += P.gr[a] * sp_r[4 * j + a];
#pragma unroll
    for (int a = 0; a < 4; ++a)
      if (a < S) vk += P.gs[a] * sp_s[(size_t) S * j + a];
    v[k] = vk, P.w[k] = w;
    dot += w * vk;
  }
#pragma unroll
  for (int k = 0; k < kMaxK; ++k) {
    if (k >= K) break;
    const int64_t j = id[k];
    float out = 0.0f;
    if (j >= 0 && j < M) {
      if (weight_mode == 0) out = -(P.w[k] * (v[k] - dot)) * inv_t;
      else if (weight_mode == 2) out = P.w[k] * (v[k] - dot);
      else if (weight_mode == 3) out = v[k];
      else {
        const float* X = xf + (size_t) kXf * j;
        const float e  = expf(-in[k] * X[12]);
        P.X[k]         = (v[k] - dot) * inv_den * e;
        out            = -P.X[k] * X[13] * X[12];
      }
    }
    g_pair[(size_t) n * K + k] = out;
  }
  if (g_points) {
#pragma unroll
    for (int a = 0; a < 3; ++a) g_points[3 * (size_t) n + a] = warp_mode != 0 ? gp[a] - P.g[a] : 0.0f;
  }
}

// kMode 0: atomics into a zeroed accumulator in global memory. 1: block-private table in LDS, stored as one partial.
constexpr int kStageTable = 11264;  // table floats of the binned variant below (44 KB: 512 control points x 22 columns)
template <int kMode>
__global__ void __launch_bounds__(kAccThreads) lbs_backward_accumulate_kernel(int N, int M, int K, int S,
    int warp_mode, int weight_mode, float temperature, const float* __restrict__ points, const float* __restrict__ xf,
    const float* __restrict__ sp_r, const float* __restrict__ sp_s, const float* __restrict__ pair_in,
    const int64_t* __restrict__ index, const float* __restrict__ g_xyz, const float* __restrict__ g_rot,
    const float* __restrict__ g_scale, float* __restrict__ g_points, float* __restrict__ g_pair,
    float* __restrict__ out /* kMode > 0: partial[gridDim.x][M*F]; else accumulator[M*F], zeroed */) {
  constexpr bool kLds = kMode > 0;
  __shared__ float s_tab[kLds ? kTableFloats : 1];
  const LbsCols C = lbs_cols(warp_mode, weight_mode, S);
  const int F = C.F, cells = M * F;
  float* tab = kLds ? s_tab : out;
  if (kLds) {
    for (int e = threadIdx.x; e < cells; e += kAccThreads) s_tab[e] = 0.0f;
    __syncthreads();
  }
  const float inv_t = 1.0f / temperature;
  for (int n = blockIdx.x * kAccThreads + threadIdx.x; n < N; n += gridDim.x * kAccThreads) {
    LbsPoint<16> P;
    lbs_point_backward<16>(n, M, K, S, warp_mode, weight_mode, inv_t, points, xf, sp_r, sp_s, pair_in, index, g_xyz,
                           g_rot, g_scale, g_points, g_pair, P);
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      if (k >= K) break;
      const int64_t j = index[(size_t) n * K + k];
      if (j < 0 || j >= M) continue;
      float* row    = tab + (size_t) j * F;
      const float w = P.w[k];
#pragma unroll
      for (int a = 0; a < 3; ++a) {
        const float wg = w * P.g[a];
        if (C.nG) atomicAdd(&row[a * 3], wg * P.p[0]), atomicAdd(&row[a * 3 + 1], wg * P.p[1]), atomicAdd(&row[a * 3 + 2], wg * P.p[2]);
        atomicAdd(&row[C.oT + a], wg);
      }
#pragma unroll
      for (int a = 0; a < 4; ++a) atomicAdd(&row[C.oR + a], w * P.gr[a]);
#pragma unroll
      for (int a = 0; a < 4; ++a)
        if (a < S) atomicAdd(&row[C.oS + a], w * P.gs[a]);
      if (weight_mode == 1)
        atomicAdd(&row[C.oK], P.X[k] * pair_in[(size_t) n * K + k]), atomicAdd(&row[C.oK + 1], P.X[k]);
    }
  }
  if (kLds) {
    __syncthreads();
    float* mine = out + (size_t) blockIdx.x * cells;
    for (int e = threadIdx.x; e < cells; e += kAccThreads) mine[e] = s_tab[e];
  }
}

// The same sums without float atomics, for tables of up to kStageTable cells and K <= kBinK neighbours: LDS float
// atomics retire about one lane every three cycles on this chip, and the 18 per neighbour above are what that kernel's
// time is made of. A block takes 1024 points at a time. Every lane does its point's own outputs and counts its
// neighbours per control point (integer LDS atomics), the counts are scanned, every (point, neighbour) pair is placed
// in its control point's bin (weight, kernel-mode factor, owning lane and slot), and then each table cell is summed by
// one lane over its control point's bin from the points' gradients parked in LDS. Partial tables go out as in mode 1.
constexpr int kBinK = 4;
constexpr int kBinFeat = 14;  // g[3] p[3] g_rot[4] g_scale[<= 4] per point
__global__ void __launch_bounds__(kAccThreads) lbs_backward_binned_kernel(int N, int M, int K, int S, int warp_mode,
    int weight_mode, float temperature, const float* __restrict__ points, const float* __restrict__ xf,
    const float* __restrict__ sp_r, const float* __restrict__ sp_s, const float* __restrict__ pair_in,
    const int64_t* __restrict__ index, const float* __restrict__ g_xyz, const float* __restrict__ g_rot,
    const float* __restrict__ g_scale, float* __restrict__ g_points, float* __restrict__ g_pair,
    float* __restrict__ out /* partial[gridDim.x][M*F] */) {
  __shared__ float s_tab[kStageTable];
  __shared__ float s_feat[kAccThreads][kBinFeat + 1];
  __shared__ float s_pw[kAccThreads * kBinK];
  __shared__ float s_px[kAccThreads * kBinK];          // kernel-mode factor X of the pair
  __shared__ unsigned short s_pp[kAccThreads * kBinK];  // owning lane (10 bits) | neighbour slot << 10
  __shared__ int s_count[kAccThreads], s_off[kAccThreads + 1], s_cursor[kAccThreads], s_wsum[kAccThreads / kWave];
  const LbsCols C = lbs_cols(warp_mode, weight_mode, S);
  const int F = C.F, cells = M * F;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int e = tid; e < cells; e += kAccThreads) s_tab[e] = 0.0f;
  const float inv_t = 1.0f / temperature;
  for (int n0 = blockIdx.x * kAccThreads; n0 < N; n0 += gridDim.x * kAccThreads) {
    const int n = n0 + tid;
    const bool live = n < N;
    s_count[tid] = 0;
    __syncthreads();
    LbsPoint<kBinK> P;
    if (live) {
      lbs_point_backward<kBinK>(n, M, K, S, warp_mode, weight_mode, inv_t, points, xf, sp_r, sp_s, pair_in, index,
                                g_xyz, g_rot, g_scale, g_points, g_pair, P);
      float* ft = s_feat[tid];
#pragma unroll
      for (int a = 0; a < 3; ++a) ft[a] = P.g[a], ft[3 + a] = P.p[a];
#pragma unroll
      for (int a = 0; a < 4; ++a) ft[6 + a] = P.gr[a], ft[10 + a] = P.gs[a];
      for (int k = 0; k < K; ++k) {
        const int64_t j = index[(size_t) n * K + k];
        if (j >= 0 && j < M) atomicAdd(&s_count[j], 1);
      }
    }
    __syncthreads();
    // exclusive scan of the counts (M <= 1024: one control point per lane)
    const int cnt = tid < M ? s_count[tid] : 0;
    int incl = cnt;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int t = __shfl_up(incl, d, kWave);
      if (lane >= d) incl += t;
    }
    if (lane == kWave - 1) s_wsum[wave] = incl;
    __syncthreads();
    int base = 0;
    for (int w = 0; w < wave; ++w) base += s_wsum[w];
    s_off[tid] = s_cursor[tid] = base + incl - cnt;
    if (tid == kAccThreads - 1) s_off[kAccThreads] = base + incl;
    __syncthreads();
    if (live) {
#pragma unroll
      for (int k = 0; k < kBinK; ++k) {
        if (k >= K) break;
        const int64_t j = index[(size_t) n * K + k];
        if (j < 0 || j >= M) continue;
        const int pos = atomicAdd(&s_cursor[j], 1);
        s_pw[pos] = P.w[k];
        s_px[pos] = P.X[k];
        s_pp[pos] = (unsigned short) (tid | (k << 10));
      }
    }
    __syncthreads();
    for (int cell = tid; cell < cells; cell += kAccThreads) {
      const int j = cell / F, c = cell - j * F;
      float sum = 0.0f;
      if (c < C.oK) {
        // a weighted sum of one per-point feature, or of a product of two (the dL/dR block)
        int fa, fb = -1;
        if (c < C.nG) fa = c / 3, fb = 3 + (c - 3 * (c / 3));
        else if (c < C.oR) fa = c - C.oT;
        else fa = 6 + (c - C.oR);  // g_rot 6..9, g_scale 10..13
        for (int q = s_off[j]; q < s_off[j + 1]; ++q) {
          const float* ft = s_feat[s_pp[q] & 1023];
          const float f   = fb >= 0 ? ft[fa] * ft[fb] : ft[fa];
          sum += s_pw[q] * f;
        }
      } else if (c == C.oK) {
        for (int q = s_off[j]; q < s_off[j + 1]; ++q) {
          const int owner = s_pp[q] & 1023, k = s_pp[q] >> 10;
          sum += s_px[q] * pair_in[(size_t) (n0 + owner) * K + k];
        }
      } else {
        for (int q = s_off[j]; q < s_off[j + 1]; ++q) sum += s_px[q];
      }
      s_tab[cell] += sum;
    }
    __syncthreads();
  }
  float* mine = out + (size_t) blockIdx.x * cells;
  for (int e = tid; e < cells; e += kAccThreads) mine[e] = s_tab[e];
}

// g_x[n] = sum_k 2 g_k (x_n - y_idx) written directly; -that accumulated into row idx of the table [M][D].
template <bool kLds>
__global__ void __launch_bounds__(kAccThreads) knn_backward_accumulate_kernel(int N, int M, int D, int K,
    const float* __restrict__ x, const float* __restrict__ y, const int64_t* __restrict__ index,
    const float* __restrict__ g_dist2, float* __restrict__ g_x, float* __restrict__ out) {
  __shared__ float s_tab[kLds ? kTableFloats : 1];
  const int cells = M * D;
  float* tab = kLds ? s_tab : out;
  if (kLds) {
    for (int e = threadIdx.x; e < cells; e += kAccThreads) s_tab[e] = 0.0f;
    __syncthreads();
  }
  for (int n = blockIdx.x * kAccThreads + threadIdx.x; n < N; n += gridDim.x * kAccThreads) {
    for (int d = 0; d < D; ++d) {
      const float xv = x[(size_t) n * D + d];
      float sum = 0.0f;
      for (int k = 0; k < K; ++k) {
        const int64_t j = index[(size_t) n * K + k];
        if (j < 0 || j >= M) continue;
        const float t = 2.0f * g_dist2[(size_t) n * K + k] * (xv - y[(size_t) j * D + d]);
        sum += t;
        atomicAdd(&tab[(size_t) j * D + d], -t);
      }
      if (g_x) g_x[(size_t) n * D + d] = sum;
    }
  }
  if (kLds) {
    __syncthreads();
    float* mine = out + (size_t) blockIdx.x * cells;
    for (int e = threadIdx.x; e < cells; e += kAccThreads) mine[e] = s_tab[e];
  }
}

// acc[e] = partial[0][e] + partial[1][e] + ... in a fixed association: wavefront w of the block adds its contiguous
// share of the G partials, then the 8 wavefront sums are added in order.
__global__ void __launch_bounds__(512) partial_sum_kernel(int cells, int G, const float* __restrict__ partial,
                                                          float* __restrict__ acc) {
  __shared__ float s_part[8][kWave];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int e    = blockIdx.x * kWave + lane;
  const int per  = (G + 7) / 8;
  float sum = 0.0f;
  if (e < cells)
    for (int g = wv * per; g < min(G, (wv + 1) * per); ++g) sum += partial[(size_t) g * cells + e];
  s_part[wv][lane] = sum;
  __syncthreads();
  if (wv == 0 && e < cells) {
    float tot = s_part[0][lane];
#pragma unroll
    for (int k = 1; k < 8; ++k) tot += s_part[k][lane];
    acc[e] = tot;
  }
}

__global__ void __launch_bounds__(256) lbs_backward_finish_kernel(int M, int S, int warp_mode, int weight_mode,
    const float* __restrict__ sp_points, const float* __restrict__ xf, const float* __restrict__ acc,
    float* __restrict__ g_sp_points, float* __restrict__ g_sp_t, float* __restrict__ g_sp_rot,
    float* __restrict__ g_sp_r, float* __restrict__ g_sp_s, float* __restrict__ g_log_radius,
    float* __restrict__ g_weight_logit) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= M) return;
  const LbsCols C = lbs_cols(warp_mode, weight_mode, S);
  const float* a  = acc + (size_t) j * C.F;
  const float* X  = xf + (size_t) kXf * j;
  const float t[3] = {a[C.oT], a[C.oT + 1], a[C.oT + 2]};
  float gc[3] = {0, 0, 0};
  if (warp_mode != 0) {
    float G[9];
#pragma unroll
    for (int k = 0; k < 9; ++k) G[k] = a[k];
    if (warp_mode == 2) {
      const float* c = sp_points + 3 * j;
#pragma unroll
      for (int r = 0; r < 3; ++r) {
        gc[r] = t[r] - (X[r] * t[0] + X[3 + r] * t[1] + X[6 + r] * t[2]);
#pragma unroll
        for (int b = 0; b < 3; ++b) G[r * 3 + b] -= t[r] * c[b];
      }
    }
    const float x = X[14], y = X[15], z = X[16], w = X[17], nq = X[18];
    float dq[4];
    dq[0] = 2 * (-2 * x * (G[4] + G[8]) + y * (G[1] + G[3]) + z * (G[2] + G[6]) + w * (G[7] - G[5]));
    dq[1] = 2 * (x * (G[1] + G[3]) - 2 * y * (G[0] + G[8]) + z * (G[5] + G[7]) + w * (G[2] - G[6]));
    dq[2] = 2 * (x * (G[2] + G[6]) + y * (G[5] + G[7]) - 2 * z * (G[0] + G[4]) + w * (G[3] - G[1]));
    dq[3] = 2 * (x * (G[7] - G[5]) + y * (G[2] - G[6]) + z * (G[3] - G[1]));
    const float along = X[19] != 0.0f ? 0.0f : x * dq[0] + y * dq[1] + z * dq[2] + w * dq[3];
    const float qh[4] = {x, y, z, w};
#pragma unroll
    for (int k = 0; k < 4; ++k) g_sp_rot[4 * j + k] = nq * (dq[k] - qh[k] * along);
  }
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    g_sp_t[3 * j + k] = t[k];
    if (g_sp_points) g_sp_points[3 * j + k] = gc[k];
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) g_sp_r[4 * j + k] = a[C.oR + k];
  for (int k = 0; k < S; ++k) g_sp_s[(size_t) S * j + k] = a[C.oS + k];
  if (weight_mode == 1) {
    // u = e * sig + 1e-7 with e = exp(-d2 * i2), i2 = 1 / (2 r^2), r = exp(rho): du/drho = e sig d2 2 i2, du/domega =
    // e sig (1 - sig)
    const float i2 = X[12], sig = X[13];
    g_log_radius[j] = a[C.oK] * sig * 2.0f * i2;
    if (g_weight_logit) g_weight_logit[j] = a[C.oK + 1] * sig * (1.0f - sig);
  }
}

struct TablePlan {
  int blocks;   // accumulate blocks (== number of partial tables when lds)
  bool lds;
};

TablePlan plan_table(int N, int cells) {
  TablePlan p;
  p.lds    = cells <= kTableFloats;
  p.blocks = std::max(1, std::min(div_up(N, kAccThreads), p.lds ? kMaxAccBlocks : 1024));
  return p;
}

size_t partial_bytes(int N, int cells) {
  const TablePlan p = plan_table(N, cells);
  return p.lds ? align_up((size_t) p.blocks * cells * 4, 256) : 256;
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API size_t fsgs_lbs_blend_backward_workspace_bytes(int N, int M, int S) {
  if (N < 0 || M <= 0 || S < 0 || S > 4) return 0;
  const int F = 18 + S;  // the widest row: rotation block + kernel-weight columns
  return align_up((size_t) M * kXf * 4, 256) + align_up((size_t) M * F * 4, 256) + partial_bytes(N, M * F);
}

FSGS_API int fsgs_lbs_blend_backward(int N, int M, int K, int warp_mode, int weight_mode, double temperature,
    const float* points, const float* sp_points, const float* sp_t, const float* sp_rot, const float* sp_r,
    const float* sp_s, int S, const float* pair_in, const int64_t* index, const float* sp_log_radius,
    const float* sp_weight_logit, const float* g_xyz, const float* g_rot, const float* g_scale, float* g_points,
    float* g_pair, float* g_sp_points, float* g_sp_t, float* g_sp_rot, float* g_sp_r, float* g_sp_s,
    float* g_log_radius, float* g_weight_logit, void* workspace, size_t workspace_bytes, void* stream) {
  FSGS_REQUIRE(N >= 0 && M > 0 && K > 0 && K <= 16 && S >= 0 && S <= 4, "lbs_blend_backward: bad sizes (K <= 16, S <= 4)");
  FSGS_REQUIRE(warp_mode >= 0 && warp_mode <= 2 && weight_mode >= 0 && weight_mode <= 3,
               "lbs_blend_backward: unknown mode");
  FSGS_REQUIRE(sp_points && sp_t && sp_r && g_sp_t && g_sp_r && (S == 0 || (sp_s && g_scale && g_sp_s)) && workspace,
               "lbs_blend_backward: null pointer");
  FSGS_REQUIRE((warp_mode == 0) == (sp_rot == nullptr) && (warp_mode == 0 || g_sp_rot),
               "lbs_blend_backward: sp_rot and g_sp_rot go with warp modes 1 and 2, and are absent in mode 0");
  FSGS_REQUIRE(weight_mode != 1 || (sp_log_radius && g_log_radius && (!g_weight_logit || sp_weight_logit)),
               "lbs_blend_backward: the kernel weights need sp_log_radius and g_log_radius");
  FSGS_REQUIRE(N == 0 || (points && pair_in && index && g_xyz && g_rot && g_pair), "lbs_blend_backward: null pointer");
  FSGS_REQUIRE((int64_t) M * (18 + S) < (1 << 30), "lbs_blend_backward: too many control points");
  FSGS_REQUIRE(weight_mode != 0 || temperature > 0, "lbs_blend_backward: temperature must be positive");
  const size_t need = fsgs_lbs_blend_backward_workspace_bytes(N, M, S);
  if (workspace_bytes < need)
    return fail(kWorkspaceSmall, "lbs_blend_backward: workspace %zu < %zu bytes", workspace_bytes, need);
  const LbsCols C = lbs_cols(warp_mode, weight_mode, S);
  const int cells = M * C.F;
  const TablePlan plan = plan_table(N, cells);
  float* xf      = (float*) workspace;
  float* acc     = (float*) ((char*) workspace + align_up((size_t) M * kXf * 4, 256));
  float* partial = (float*) ((char*) acc + align_up((size_t) M * (18 + S) * 4, 256));
  hipStream_t s = (hipStream_t) stream;
  hipLaunchKernelGGL(lbs_prepare_kernel, dim3(div_up(M, 256)), dim3(256), 0, s, M, warp_mode, sp_points, sp_t, sp_rot,
                     weight_mode == 1 ? sp_log_radius : nullptr, weight_mode == 1 ? sp_weight_logit : nullptr, xf);
  if (N == 0 || !plan.lds)
    hipLaunchKernelGGL(zero_floats_kernel, dim3(std::min(div_up(cells, 256), 1024)), dim3(256), 0, s, (size_t) cells,
                       acc);
  if (N > 0) {
    if (plan.lds) {
      const bool binned = cells <= kStageTable && M <= kAccThreads && K <= kBinK;
      auto kernel = binned ? lbs_backward_binned_kernel : lbs_backward_accumulate_kernel<1>;
      hipLaunchKernelGGL(kernel, dim3(plan.blocks), dim3(kAccThreads), 0, s, N, M, K, S, warp_mode, weight_mode,
                         (float) temperature, points, xf, sp_r, sp_s, pair_in, index, g_xyz, g_rot, g_scale, g_points,
                         g_pair, partial);
      hipLaunchKernelGGL(partial_sum_kernel, dim3(div_up(cells, kWave)), dim3(512), 0, s, cells, plan.blocks, partial,
                         acc);
    } else {
      hipLaunchKernelGGL(lbs_backward_accumulate_kernel<0>, dim3(plan.blocks), dim3(kAccThreads), 0, s, N, M, K, S,
                         warp_mode, weight_mode, (float) temperature, points, xf, sp_r, sp_s, pair_in, index, g_xyz,
                         g_rot, g_scale, g_points, g_pair, acc);
    }
  }
  hipLaunchKernelGGL(lbs_backward_finish_kernel, dim3(div_up(M, 256)), dim3(256), 0, s, M, S, warp_mode, weight_mode,
                     sp_points, xf, acc, g_sp_points, g_sp_t, g_sp_rot, g_sp_r, g_sp_s, g_log_radius, g_weight_logit);
  return check_launch("lbs_blend_backward");
}

FSGS_API size_t fsgs_knn_topk_backward_workspace_bytes(int N, int M, int D) {
  if (N < 0 || M <= 0 || D <= 0) return 0;
  return partial_bytes(N, M * D);
}

FSGS_API int fsgs_knn_topk_backward(int N, int M, int D, int K, const float* x, const float* y, const int64_t* index,
    const float* g_dist2, float* g_x, float* g_y, void* workspace, size_t workspace_bytes, void* stream) {
  FSGS_REQUIRE(N >= 0 && M > 0 && D > 0 && K > 0 && y && g_y && workspace, "knn_topk_backward: bad arguments");
  FSGS_REQUIRE(N == 0 || (x && index && g_dist2), "knn_topk_backward: null pointer");
  FSGS_REQUIRE((int64_t) M * D < (1 << 30), "knn_topk_backward: too many control points");
  const size_t need = fsgs_knn_topk_backward_workspace_bytes(N, M, D);
  if (workspace_bytes < need)
    return fail(kWorkspaceSmall, "knn_topk_backward: workspace %zu < %zu bytes", workspace_bytes, need);
  const int cells = M * D;
  const TablePlan plan = plan_table(N, cells);
  hipStream_t s = (hipStream_t) stream;
  // With an LDS table the per-block partials land in the workspace and g_y is written once by the ordered sum;
  // without one the atomics go straight into a zeroed g_y.
  float* partial = (float*) workspace;
  if (N == 0 || !plan.lds)
    hipLaunchKernelGGL(zero_floats_kernel, dim3(std::min(div_up(cells, 256), 1024)), dim3(256), 0, s, (size_t) cells,
                       g_y);
  if (N == 0) return check_launch("knn_topk_backward");
  if (plan.lds) {
    hipLaunchKernelGGL(knn_backward_accumulate_kernel<true>, dim3(plan.blocks), dim3(kAccThreads), 0, s, N, M, D, K, x,
                       y, index, g_dist2, g_x, partial);
    hipLaunchKernelGGL(partial_sum_kernel, dim3(div_up(cells, kWave)), dim3(512), 0, s, cells, plan.blocks, partial,
                       g_y);
  } else {
    hipLaunchKernelGGL(knn_backward_accumulate_kernel<false>, dim3(plan.blocks), dim3(kAccThreads), 0, s, N, M, D, K,
                       x, y, index, g_dist2, g_x, g_y);
  }
  return check_launch("knn_topk_backward");
}
