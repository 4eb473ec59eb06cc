// Per-surfel sums of per-(surfel, tile) gradient records in a fixed order, without atomics and without a zero fill of
// the outputs. The tile binning emits a surfel's instances at consecutive positions of the unsorted key list, starting at
// the surfel's prefix-scan offset; a backward block that has summed one instance over its tile's pixels writes the sums
// as one record at that position. Every instance's record is written by the blend kernel itself, zeros included (each
// block also clears the records of its tile's never-staged tail), so the buffer is never zero-filled. slot_sum_kernel
// then adds a surfel's records in position order and hands every component of every surfel to a scatter functor that
// knows the output tensors. (The fast path's key spans also hold positions that belong to no tile's list; its own sum
// kernel, in fast_blend.hip, repeats the binning's corner test and skips them.) The reference flushes these sums with
// one device-scope atomic per component, tile and surfel into caller-zeroed tensors (e.g. gaussian_render.cu:560-600,
// gs_2d_fast_redner.cu:520-560).
#pragma once
#include <algorithm>

#include "common.hpp"

namespace fsgs {

struct SlotWorkspace {
  float* records;  // [R][kFloats]
};

inline size_t slot_workspace_bytes(int64_t R, int floats) {
  return align_up((size_t) (R > 0 ? R : 0) * floats * 4 + 16, 256);
}
inline SlotWorkspace slot_workspace(void* base, int64_t, int) { return SlotWorkspace{(float*) base}; }

namespace {

// kFloats / 2 lanes per surfel, each owning one float2 of the record, so the lanes of a surfel read consecutive bytes
// and neighbouring surfels continue where the previous one ends. Eight records of a surfel are in flight together.
template <int kFloats, typename Scatter>
__global__ void __launch_bounds__(256) slot_sum_kernel(int P, const int64_t* __restrict__ point_offsets,
    const float* __restrict__ records, Scatter out) {
  static_assert(kFloats % 2 == 0 && kFloats <= 64, "records are whole float2s");
  constexpr int kLanes = kFloats / 2, kPerWave = 64 / kLanes, kDepth = 8;
  const int lane = threadIdx.x & 63;
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int sub = lane / kLanes, k = lane - sub * kLanes;
  const int i = wave * kPerWave + sub;
  if (sub >= kPerWave || i >= P) return;
  const int64_t e0 = i > 0 ? point_offsets[i - 1] : 0, e1 = point_offsets[i];
  const float2* src = (const float2*) records + k;
  float2 acc = make_float2(0.0f, 0.0f);
  for (int64_t base = e0; base < e1; base += kDepth) {
    float2 v[kDepth];
#pragma unroll
    for (int j = 0; j < kDepth; ++j) v[j] = src[(size_t) (base + j < e1 ? base + j : e1 - 1) * kLanes];
#pragma unroll
    for (int j = 0; j < kDepth; ++j) {
      const bool on = base + j < e1;
      acc.x += on ? v[j].x : 0.0f, acc.y += on ? v[j].y : 0.0f;
    }
  }
  out(i, 2 * k, acc.x);
  out(i, 2 * k + 1, acc.y);
}

template <int kFloats, typename Scatter>
inline void launch_slot_sum(int P, const int64_t* point_offsets, const SlotWorkspace& ws, Scatter out, hipStream_t s) {
  constexpr int kPerWave = 64 / (kFloats / 2);
  const int64_t waves = div_up(P, kPerWave);
  hipLaunchKernelGGL((slot_sum_kernel<kFloats, Scatter>), dim3((unsigned) div_up(waves * 64, 256)), dim3(256), 0, s, P,
                     point_offsets, ws.records, out);
}

}  // namespace
}  // namespace fsgs
