// Backward of the LBS blend and of the K-NN squared distances for gfx950.
//
// The reference differentiates fast_2d_gs/network.py:504 (pytorch3d.ops.knn_points), :517 (softmax weights) and :545-573
// (warp through lietorch.SE3) with torch autograd: ~30 elementwise / gather / scatter launches over [N,K,...] tensors and
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

namespace fsgs {
namespace {

constexpr int kTableFloats  = 36864;  // 144 KB of LDS for the per-block table
constexpr int kMaxAccBlocks = 256;    // partial tables per launch
constexpr int kAccThreads   = 1024;  // 16 wavefronts share one LDS table: the loop is bound by gather latency, not by the atomics

__global__ void __launch_bounds__(256) zero_floats_kernel(size_t n, float* __restrict__ p) {
  for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t) gridDim.x * blockDim.x)
    p[i] = 0.0f;
}

// Per control point: unit quaternion of r + (0,0,0,1), 1/|q| (0 when |q| <= 1e-12 so that the projection term drops),
// its rotation matrix and the effective translation. 20 floats: R[9] t[3] qhat[4] inv_norm degenerate pad pad.
constexpr int kXf = 20;
__global__ void __launch_bounds__(256) lbs_backward_prepare_kernel(int M, int centred,
    const float* __restrict__ sp_points, const float* __restrict__ sp_t, const float* __restrict__ sp_r,
    float* __restrict__ xf) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= M) return;
  const float q[4] = {sp_r[4 * j], sp_r[4 * j + 1], sp_r[4 * j + 2], sp_r[4 * j + 3] + 1.0f};
  const float nrm  = sqrtf(q[0] * q[0] + q[1] * q[1] + q[2] * q[2] + q[3] * q[3]);
  const float nq   = 1.0f / fmaxf(nrm, 1e-12f);
  const float x = q[0] * nq, y = q[1] * nq, z = q[2] * nq, w = q[3] * nq;
  float R[9];
  R[0] = 1 - 2 * (y * y + z * z), R[1] = 2 * (x * y - z * w), R[2] = 2 * (y * w + x * z);
  R[3] = 2 * (x * y + z * w), R[4] = 1 - 2 * (x * x + z * z), R[5] = 2 * (y * z - x * w);
  R[6] = 2 * (x * z - y * w), R[7] = 2 * (x * w + y * z), R[8] = 1 - 2 * (x * x + y * y);
  float t[3] = {sp_t[3 * j], sp_t[3 * j + 1], sp_t[3 * j + 2]};
  if (centred) {
    const float* c = sp_points + 3 * j;
#pragma unroll
    for (int a = 0; a < 3; ++a) t[a] = t[a] + c[a] - (R[a * 3] * c[0] + R[a * 3 + 1] * c[1] + R[a * 3 + 2] * c[2]);
  }
  float* o = xf + (size_t) kXf * j;
#pragma unroll
  for (int k = 0; k < 9; ++k) o[k] = R[k];
#pragma unroll
  for (int k = 0; k < 3; ++k) o[9 + k] = t[k];
  o[12] = x, o[13] = y, o[14] = z, o[15] = w, o[16] = nq, o[17] = nrm <= 1e-12f ? 1.0f : 0.0f, o[18] = 0, o[19] = 0;
}

// Table row of control point j: [0,9) dL/dR, [9,12) dL/dt_eff, [12,16) direct rotation-residual gradient,
// [16,16+S) scale-residual gradient.
// kMode 0: atomics into a zeroed accumulator in global memory. 1: block-private table in LDS, stored as one partial.
constexpr int kStageTable = 12288;  // table floats of the binned variant below (48 KB)
template <int kMode>
__global__ void __launch_bounds__(kAccThreads) lbs_backward_accumulate_kernel(int N, int M, int K, int S,
    float temperature, const float* __restrict__ points, const float* __restrict__ xf,
    const float* __restrict__ sp_r, const float* __restrict__ sp_s, const float* __restrict__ dist2,
    const int64_t* __restrict__ index, const float* __restrict__ g_xyz, const float* __restrict__ g_rot,
    const float* __restrict__ g_scale, float* __restrict__ g_points, float* __restrict__ g_dist2,
    float* __restrict__ out /* kMode > 0: partial[gridDim.x][M*F]; else accumulator[M*F], zeroed */) {
  constexpr bool kLds = kMode > 0;
  __shared__ float s_tab[kLds ? kTableFloats : 1];
  const int F = 16 + S, cells = M * F;
  float* tab = kLds ? s_tab : out;
  if (kLds) {
    for (int e = threadIdx.x; e < cells; e += kAccThreads) s_tab[e] = 0.0f;
    __syncthreads();
  }
  const float inv_t = 1.0f / temperature;
  for (int n = blockIdx.x * kAccThreads + threadIdx.x; n < N; n += gridDim.x * kAccThreads) {
    const float* d2   = dist2 + (size_t) n * K;
    const int64_t* id = index + (size_t) n * K;
    float mx = -__builtin_inff();
    for (int k = 0; k < K; ++k)
      if (id[k] >= 0 && id[k] < M) mx = fmaxf(mx, -d2[k] * inv_t);
    float den = 0.0f;
    for (int k = 0; k < K; ++k)
      if (id[k] >= 0 && id[k] < M) den += expf(-d2[k] * inv_t - mx);
    const float inv_den = den > 0.0f ? 1.0f / den : 0.0f;
    const float p[3]  = {points[3 * (size_t) n], points[3 * (size_t) n + 1], points[3 * (size_t) n + 2]};
    const float g[3]  = {g_xyz[3 * (size_t) n], g_xyz[3 * (size_t) n + 1], g_xyz[3 * (size_t) n + 2]};
    const float gr[4] = {g_rot[4 * (size_t) n], g_rot[4 * (size_t) n + 1], g_rot[4 * (size_t) n + 2],
                         g_rot[4 * (size_t) n + 3]};
    float gs[4] = {0, 0, 0, 0};
    for (int a = 0; a < S; ++a) gs[a] = g_scale[(size_t) S * n + a];
    float gp[3] = {-g[0], -g[1], -g[2]}, dot = 0.0f;
    for (int k = 0; k < K; ++k) {
      const int64_t j = id[k];
      if (j < 0 || j >= M) {
        g_dist2[(size_t) n * K + k] = 0.0f;
        continue;
      }
      const float w  = expf(-d2[k] * inv_t - mx) * inv_den;
      const float* X = xf + (size_t) kXf * j;
      float* row     = tab + (size_t) j * F;
      float v = 0.0f;
#pragma unroll
      for (int a = 0; a < 3; ++a) {
        v += g[a] * (X[a * 3] * p[0] + X[a * 3 + 1] * p[1] + X[a * 3 + 2] * p[2] + X[9 + a]);
        gp[a] += w * (X[a] * g[0] + X[3 + a] * g[1] + X[6 + a] * g[2]);
        const float wg = w * g[a];
        atomicAdd(&row[a * 3], wg * p[0]), atomicAdd(&row[a * 3 + 1], wg * p[1]), atomicAdd(&row[a * 3 + 2], wg * p[2]);
        atomicAdd(&row[9 + a], wg);
      }
#pragma unroll
      for (int a = 0; a < 4; ++a) v += gr[a] * sp_r[4 * j + a], atomicAdd(&row[12 + a], w * gr[a]);
      for (int a = 0; a < S; ++a) v += gs[a] * sp_s[(size_t) S * j + a], atomicAdd(&row[16 + a], w * gs[a]);
      g_dist2[(size_t) n * K + k] = v;  // parked until the weighted mean is known
      dot += w * v;
    }
    for (int k = 0; k < K; ++k) {
      const int64_t j = id[k];
      if (j < 0 || j >= M) continue;
      const float w = expf(-d2[k] * inv_t - mx) * inv_den;
      g_dist2[(size_t) n * K + k] = -(w * (g_dist2[(size_t) n * K + k] - dot)) * inv_t;
    }
    if (g_points) {
#pragma unroll
      for (int a = 0; a < 3; ++a) g_points[3 * (size_t) n + a] = gp[a];
    }
  }
  if (kLds) {
    __syncthreads();
    float* mine = out + (size_t) blockIdx.x * cells;
    for (int e = threadIdx.x; e < cells; e += kAccThreads) mine[e] = s_tab[e];
  }
}

// The same sums without float atomics, for tables of up to kStageTable cells and K <= kBinK neighbours: LDS float
// atomics retire about one lane every three cycles on this chip, and the 18 per neighbour above are what the kernel's
// time is made of. A block takes 1024 points at a time. Every lane does its point's own outputs and counts its
// neighbours per control point (integer LDS atomics), the counts are scanned, every (point, neighbour) pair is placed
// in its control point's bin (weight and the lane that owns the point), and then each table cell is summed by one lane
// over its control point's bin from the points' gradients parked in LDS. Partial tables go out as in mode 1.
constexpr int kBinK = 4;
constexpr int kBinFeat = 14;  // g[3] p[3] g_rot[4] g_scale[<= 4] per point
__global__ void __launch_bounds__(kAccThreads) lbs_backward_binned_kernel(int N, int M, int K, int S,
    float temperature, const float* __restrict__ points, const float* __restrict__ xf,
    const float* __restrict__ sp_r, const float* __restrict__ sp_s, const float* __restrict__ dist2,
    const int64_t* __restrict__ index, const float* __restrict__ g_xyz, const float* __restrict__ g_rot,
    const float* __restrict__ g_scale, float* __restrict__ g_points, float* __restrict__ g_dist2,
    float* __restrict__ out /* partial[gridDim.x][M*F] */) {
  __shared__ float s_tab[kStageTable];
  __shared__ float s_feat[kAccThreads][kBinFeat + 1];
  __shared__ float s_pw[kAccThreads * kBinK];
  __shared__ unsigned short s_pp[kAccThreads * kBinK];
  __shared__ int s_count[kAccThreads], s_off[kAccThreads + 1], s_cursor[kAccThreads], s_wsum[kAccThreads / kWave];
  const int F = 16 + S, cells = M * F;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int e = tid; e < cells; e += kAccThreads) s_tab[e] = 0.0f;
  const float inv_t = 1.0f / temperature;
  for (int n0 = blockIdx.x * kAccThreads; n0 < N; n0 += gridDim.x * kAccThreads) {
    const int n = n0 + tid;
    const bool live = n < N;
    s_count[tid] = 0;
    __syncthreads();
    float mx = -__builtin_inff(), inv_den = 0.0f;
    if (live) {
      const float* d2   = dist2 + (size_t) n * K;
      const int64_t* id = index + (size_t) n * K;
      for (int k = 0; k < K; ++k)
        if (id[k] >= 0 && id[k] < M) mx = fmaxf(mx, -d2[k] * inv_t);
      float den = 0.0f;
      for (int k = 0; k < K; ++k)
        if (id[k] >= 0 && id[k] < M) den += expf(-d2[k] * inv_t - mx);
      inv_den = den > 0.0f ? 1.0f / den : 0.0f;
      const float p[3]  = {points[3 * (size_t) n], points[3 * (size_t) n + 1], points[3 * (size_t) n + 2]};
      const float g[3]  = {g_xyz[3 * (size_t) n], g_xyz[3 * (size_t) n + 1], g_xyz[3 * (size_t) n + 2]};
      const float gr[4] = {g_rot[4 * (size_t) n], g_rot[4 * (size_t) n + 1], g_rot[4 * (size_t) n + 2],
                           g_rot[4 * (size_t) n + 3]};
      float gs[4] = {0, 0, 0, 0};
      for (int a = 0; a < S; ++a) gs[a] = g_scale[(size_t) S * n + a];
      float* ft = s_feat[tid];
#pragma unroll
      for (int a = 0; a < 3; ++a) ft[a] = g[a], ft[3 + a] = p[a];
#pragma unroll
      for (int a = 0; a < 4; ++a) ft[6 + a] = gr[a], ft[10 + a] = gs[a];
      float gp[3] = {-g[0], -g[1], -g[2]}, dot = 0.0f;
      for (int k = 0; k < K; ++k) {
        const int64_t j = id[k];
        if (j < 0 || j >= M) {
          g_dist2[(size_t) n * K + k] = 0.0f;
          continue;
        }
        atomicAdd(&s_count[j], 1);
        const float w  = expf(-d2[k] * inv_t - mx) * inv_den;
        const float* X = xf + (size_t) kXf * j;
        float v = 0.0f;
#pragma unroll
        for (int a = 0; a < 3; ++a) {
          v += g[a] * (X[a * 3] * p[0] + X[a * 3 + 1] * p[1] + X[a * 3 + 2] * p[2] + X[9 + a]);
          gp[a] += w * (X[a] * g[0] + X[3 + a] * g[1] + X[6 + a] * g[2]);
        }
#pragma unroll
        for (int a = 0; a < 4; ++a) v += gr[a] * sp_r[4 * j + a];
        for (int a = 0; a < S; ++a) v += gs[a] * sp_s[(size_t) S * j + a];
        g_dist2[(size_t) n * K + k] = v;  // parked until the weighted mean is known
        dot += w * v;
      }
      for (int k = 0; k < K; ++k) {
        const int64_t j = id[k];
        if (j < 0 || j >= M) continue;
        const float w = expf(-d2[k] * inv_t - mx) * inv_den;
        g_dist2[(size_t) n * K + k] = -(w * (g_dist2[(size_t) n * K + k] - dot)) * inv_t;
      }
      if (g_points) {
#pragma unroll
        for (int a = 0; a < 3; ++a) g_points[3 * (size_t) n + a] = gp[a];
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
      const float* d2   = dist2 + (size_t) n * K;
      const int64_t* id = index + (size_t) n * K;
      for (int k = 0; k < K; ++k) {
        const int64_t j = id[k];
        if (j < 0 || j >= M) continue;
        const int pos = atomicAdd(&s_cursor[j], 1);
        s_pw[pos] = expf(-d2[k] * inv_t - mx) * inv_den;
        s_pp[pos] = (unsigned short) tid;
      }
    }
    __syncthreads();
    // table row of control point j: [0,9) w g[a] p[b], [9,12) w g[a], [12,16) w g_rot[a], [16,16+S) w g_scale[a]
    for (int cell = tid; cell < cells; cell += kAccThreads) {
      const int j = cell / F, c = cell - j * F;
      const int fa = c < 9 ? c / 3 : (c < 12 ? c - 9 : c - 6), fb = c < 9 ? 3 + (c - 3 * (c / 3)) : -1;
      float sum = 0.0f;
      for (int q = s_off[j]; q < s_off[j + 1]; ++q) {
        const float* ft = s_feat[s_pp[q]];
        const float f   = fb >= 0 ? ft[fa] * ft[fb] : ft[fa];
        sum += s_pw[q] * f;
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

__global__ void __launch_bounds__(256) lbs_backward_finish_kernel(int M, int S, int centred,
    const float* __restrict__ sp_points, const float* __restrict__ xf, const float* __restrict__ acc,
    float* __restrict__ g_sp_points, float* __restrict__ g_sp_t, float* __restrict__ g_sp_r,
    float* __restrict__ g_sp_s) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= M) return;
  const int F     = 16 + S;
  const float* a  = acc + (size_t) j * F;
  const float* X  = xf + (size_t) kXf * j;
  float G[9];
#pragma unroll
  for (int k = 0; k < 9; ++k) G[k] = a[k];
  const float t[3] = {a[9], a[10], a[11]};
  float gc[3] = {0, 0, 0};
  if (centred) {
    const float* c = sp_points + 3 * j;
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      gc[r] = t[r] - (X[r] * t[0] + X[3 + r] * t[1] + X[6 + r] * t[2]);
#pragma unroll
      for (int b = 0; b < 3; ++b) G[r * 3 + b] -= t[r] * c[b];
    }
  }
  const float x = X[12], y = X[13], z = X[14], w = X[15], nq = X[16];
  float dq[4];
  dq[0] = 2 * (-2 * x * (G[4] + G[8]) + y * (G[1] + G[3]) + z * (G[2] + G[6]) + w * (G[7] - G[5]));
  dq[1] = 2 * (x * (G[1] + G[3]) - 2 * y * (G[0] + G[8]) + z * (G[5] + G[7]) + w * (G[2] - G[6]));
  dq[2] = 2 * (x * (G[2] + G[6]) + y * (G[5] + G[7]) - 2 * z * (G[0] + G[4]) + w * (G[3] - G[1]));
  dq[3] = 2 * (x * (G[7] - G[5]) + y * (G[2] - G[6]) + z * (G[3] - G[1]));
  const float along = X[17] != 0.0f ? 0.0f : x * dq[0] + y * dq[1] + z * dq[2] + w * dq[3];
  const float qh[4] = {x, y, z, w};
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    g_sp_t[3 * j + k] = t[k];
    if (g_sp_points) g_sp_points[3 * j + k] = gc[k];
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) g_sp_r[4 * j + k] = a[12 + k] + nq * (dq[k] - qh[k] * along);
  for (int k = 0; k < S; ++k) g_sp_s[(size_t) S * j + k] = a[16 + k];
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
  return align_up((size_t) M * kXf * 4, 256) + align_up((size_t) M * (16 + S) * 4, 256) + partial_bytes(N, M * (16 + S));
}

FSGS_API int fsgs_lbs_blend_backward(int N, int M, int K, int centred, double temperature, const float* points,
    const float* sp_points, const float* sp_t, const float* sp_r, const float* sp_s, int S, const float* dist2,
    const int64_t* index, const float* g_xyz, const float* g_rot, const float* g_scale, float* g_points,
    float* g_dist2, float* g_sp_points, float* g_sp_t, float* g_sp_r, float* g_sp_s, void* workspace,
    size_t workspace_bytes, void* stream) {
  FSGS_REQUIRE(N >= 0 && M > 0 && K > 0 && S >= 0 && S <= 4 && sp_points && sp_t && sp_r && g_sp_t && g_sp_r &&
                   (S == 0 || (sp_s && g_scale && g_sp_s)) && workspace,
               "lbs_blend_backward: bad arguments");
  FSGS_REQUIRE(N == 0 || (points && dist2 && index && g_xyz && g_rot && g_dist2), "lbs_blend_backward: null pointer");
  FSGS_REQUIRE((int64_t) M * (16 + S) < (1 << 30), "lbs_blend_backward: too many control points");
  FSGS_REQUIRE(temperature > 0, "lbs_blend_backward: temperature must be positive");
  const size_t need = fsgs_lbs_blend_backward_workspace_bytes(N, M, S);
  if (workspace_bytes < need)
    return fail(kWorkspaceSmall, "lbs_blend_backward: workspace %zu < %zu bytes", workspace_bytes, need);
  const int F = 16 + S, cells = M * F;
  const TablePlan plan = plan_table(N, cells);
  float* xf      = (float*) workspace;
  float* acc     = (float*) ((char*) workspace + align_up((size_t) M * kXf * 4, 256));
  float* partial = (float*) ((char*) acc + align_up((size_t) cells * 4, 256));
  hipStream_t s = (hipStream_t) stream;
  hipLaunchKernelGGL(lbs_backward_prepare_kernel, dim3(div_up(M, 256)), dim3(256), 0, s, M, centred, sp_points, sp_t,
                     sp_r, xf);
  if (N == 0 || !plan.lds)
    hipLaunchKernelGGL(zero_floats_kernel, dim3(std::min(div_up(cells, 256), 1024)), dim3(256), 0, s, (size_t) cells,
                       acc);
  if (N > 0) {
    if (plan.lds) {
      const bool binned = cells <= kStageTable && M <= kAccThreads && K <= kBinK;
      auto kernel = binned ? lbs_backward_binned_kernel : lbs_backward_accumulate_kernel<1>;
      hipLaunchKernelGGL(kernel, dim3(plan.blocks), dim3(kAccThreads), 0, s, N, M, K, S,
                         (float) temperature, points, xf, sp_r, sp_s, dist2, index, g_xyz, g_rot, g_scale, g_points,
                         g_dist2, partial);
      hipLaunchKernelGGL(partial_sum_kernel, dim3(div_up(cells, kWave)), dim3(512), 0, s, cells, plan.blocks, partial,
                         acc);
    } else {
      hipLaunchKernelGGL(lbs_backward_accumulate_kernel<0>, dim3(plan.blocks), dim3(kAccThreads), 0, s, N, M, K, S,
                         (float) temperature, points, xf, sp_r, sp_s, dist2, index, g_xyz, g_rot, g_scale, g_points,
                         g_dist2, acc);
    }
  }
  hipLaunchKernelGGL(lbs_backward_finish_kernel, dim3(div_up(M, 256)), dim3(256), 0, s, M, S, centred, sp_points, xf,
                     acc, g_sp_points, g_sp_t, g_sp_r, g_sp_s);
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
