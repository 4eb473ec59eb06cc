// Shared by the LBS blend forward and backward: the per-control-point table and the neighbour weights.
// Reference behaviour reproduced: fast_2d_gs/network.py:498-521 (calc_LBS_weight) and :545-573 (warp).
#pragma once
#include "common.hpp"

namespace fsgs {
namespace {

// Per control point (one lane each), kXf floats:
//   [0,9)  rotation matrix of qhat = normalize(sp_rot + (0,0,0,1)) (identity without sp_rot)
//   [9,12) translation (re-centred about the control point for warp mode 2: t + c - R c)
//   [12]   1 / (2 exp(log_radius)^2)     [13] sigmoid(weight_logit) (1 without one)
//   [14,18) qhat     [18] 1 / |q| (floored at 1e-12)     [19] 1 if |q| <= 1e-12 (the projection term of the
//   normalisation's derivative then drops), else 0.
constexpr int kXf = 20;
__global__ void __launch_bounds__(256) lbs_prepare_kernel(int M, int warp_mode, const float* __restrict__ sp_points,
    const float* __restrict__ sp_t, const float* __restrict__ sp_rot, const float* __restrict__ log_radius,
    const float* __restrict__ weight_logit, float* __restrict__ xf) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= M) return;
  float R[9] = {1, 0, 0, 0, 1, 0, 0, 0, 1};
  float t[3] = {sp_t[3 * j], sp_t[3 * j + 1], sp_t[3 * j + 2]};
  float qh[4] = {0, 0, 0, 1}, nq = 1.0f, degenerate = 0.0f;
  if (warp_mode != 0) {
    const float q[4] = {sp_rot[4 * j], sp_rot[4 * j + 1], sp_rot[4 * j + 2], sp_rot[4 * j + 3] + 1.0f};
    const float nrm  = sqrtf(q[0] * q[0] + q[1] * q[1] + q[2] * q[2] + q[3] * q[3]);
    nq               = 1.0f / fmaxf(nrm, 1e-12f);
    degenerate       = nrm <= 1e-12f ? 1.0f : 0.0f;
    const float x = q[0] * nq, y = q[1] * nq, z = q[2] * nq, w = q[3] * nq;
    qh[0] = x, qh[1] = y, qh[2] = z, qh[3] = w;
    R[0] = 1 - 2 * (y * y + z * z), R[1] = 2 * (x * y - z * w), R[2] = 2 * (y * w + x * z);
    R[3] = 2 * (x * y + z * w), R[4] = 1 - 2 * (x * x + z * z), R[5] = 2 * (y * z - x * w);
    R[6] = 2 * (x * z - y * w), R[7] = 2 * (x * w + y * z), R[8] = 1 - 2 * (x * x + y * y);
    if (warp_mode == 2) {
      const float* c = sp_points + 3 * j;
#pragma unroll
      for (int a = 0; a < 3; ++a) t[a] = t[a] + c[a] - (R[a * 3] * c[0] + R[a * 3 + 1] * c[1] + R[a * 3 + 2] * c[2]);
    }
  }
  float* o = xf + (size_t) kXf * j;
#pragma unroll
  for (int k = 0; k < 9; ++k) o[k] = R[k];
#pragma unroll
  for (int k = 0; k < 3; ++k) o[9 + k] = t[k];
  const float r = log_radius ? expf(log_radius[j]) : 1.0f;
  o[12] = 1.0f / (2.0f * r * r);
  o[13] = weight_logit ? 1.0f / (1.0f + expf(-weight_logit[j])) : 1.0f;
#pragma unroll
  for (int k = 0; k < 4; ++k) o[14 + k] = qh[k];
  o[18] = nq, o[19] = degenerate;
}

// Unnormalised weights u[k] of a point's K neighbour slots and the inverse of their sum.
//   weight_mode 0: softmax(-d2 / temperature)                                              (network.py:517)
//               1: exp(-d2 / (2 r^2)) * sigmoid(omega) + 1e-7, divided by the sum          (network.py:507-513)
//               2: softmax(logits), the caller having gathered sp_W[n, index[n, k]]        (network.py:514-515)
//               3: the caller's weights as they are (inv_den = 1)                          (warp() called on its own)
// Slots whose index is outside [0, M) (the -1 padding of a K-NN with K > M) get 0 and take no part in the sum.
// kMaxK bounds K at compile time so that the per-slot arrays stay in registers (every loop over slots is unrolled).
template <int kMaxK>
__device__ __forceinline__ void lbs_weights(int weight_mode, int K, int M, float inv_t, const float* __restrict__ in,
                                            const int64_t* __restrict__ id, const float* __restrict__ xf, float* u,
                                            float& inv_den) {
  float mx = -__builtin_inff();
  if (weight_mode == 0 || weight_mode == 2) {
#pragma unroll
    for (int k = 0; k < kMaxK; ++k)
      if (k < K && id[k] >= 0 && id[k] < M) mx = fmaxf(mx, weight_mode == 0 ? -in[k] * inv_t : in[k]);
  }
  float den = 0.0f;
#pragma unroll
  for (int k = 0; k < kMaxK; ++k) {
    const int64_t j = k < K ? id[k] : -1;
    float v = 0.0f;
    if (j >= 0 && j < M) {
      if (weight_mode == 0) v = expf(-in[k] * inv_t - mx);
      else if (weight_mode == 1) v = expf(-in[k] * xf[(size_t) kXf * j + 12]) * xf[(size_t) kXf * j + 13] + 1e-7f;
      else if (weight_mode == 2) v = expf(in[k] - mx);
      else v = in[k];
    }
    u[k] = v, den += v;
  }
  inv_den = weight_mode == 3 ? 1.0f : (den > 0.0f ? 1.0f / den : 0.0f);
}

}  // namespace
}  // namespace fsgs
