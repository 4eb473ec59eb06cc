// Mean squared distance of every point to its three nearest neighbours, for gfx950.
//
// Reference behaviour reproduced: fast_2d_gs/_C/src/other/knn.cu:180-205 (simple_knn -> knn) with kernels :57-178: the
// result for point i is (b0 + b1 + b2) / 3 where b0 <= b1 <= b2 are the three smallest squared distances
// dx*dx + dy*dy + dz*dz to the other points (a duplicate of the point counts with distance 0; with fewer than four
// points the missing entries stay FLT_MAX). The search is exact, so the output does not depend on how it is organised.
//
// The reference sorts the points along a 30-bit Morton curve, boxes them 1024 at a time and lets every point walk all
// boxes on its own, pruning with its own bound. Here the same ordering is used so that the 256 queries of a block are
// neighbours in space and can share their work: the block tests boxes (256 points each) against the widest bound of
// its queries, 256 boxes per step with one lane per box, stages the surviving boxes' points in LDS, and each lane scans
// a staged box only if it passes the lane's own bound. Bounds start from the three best of the six Morton neighbours,
// as in the reference, and tighten as boxes are consumed.
#include <cfloat>

#include "binning.hpp"

namespace fsgs {
namespace {

constexpr int kBox = 64;  // points per box == queries per block (one wavefront)

struct Bounds {
  float lo[3], hi[3];
};

// ---- bounding box of the cloud (the reference seeds both reductions with 0, so the origin is always inside) ----
__global__ void __launch_bounds__(256) bbox_partial_kernel(int P, const float* __restrict__ points,
                                                           float* __restrict__ partial /*[grid][6]*/) {
  __shared__ float s_red[6][256];
  float lo[3] = {0.0f, 0.0f, 0.0f}, hi[3] = {0.0f, 0.0f, 0.0f};
  for (int i = blockIdx.x * 256 + threadIdx.x; i < P; i += gridDim.x * 256)
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const float v = points[3 * (size_t) i + a];
      lo[a] = fminf(lo[a], v), hi[a] = fmaxf(hi[a], v);
    }
#pragma unroll
  for (int a = 0; a < 3; ++a) s_red[a][threadIdx.x] = lo[a], s_red[3 + a][threadIdx.x] = hi[a];
  __syncthreads();
  for (int off = 128; off >= 1; off >>= 1) {
    if ((int) threadIdx.x < off)
#pragma unroll
      for (int a = 0; a < 3; ++a) {
        s_red[a][threadIdx.x]     = fminf(s_red[a][threadIdx.x], s_red[a][threadIdx.x + off]);
        s_red[3 + a][threadIdx.x] = fmaxf(s_red[3 + a][threadIdx.x], s_red[3 + a][threadIdx.x + off]);
      }
    __syncthreads();
  }
  if (threadIdx.x < 6) partial[blockIdx.x * 6 + threadIdx.x] = s_red[threadIdx.x][0];
}

__global__ void __launch_bounds__(64) bbox_final_kernel(int n, const float* __restrict__ partial,
                                                        float* __restrict__ bbox /*[6]*/) {
  if (threadIdx.x >= 6) return;
  float v = 0.0f;
  for (int b = 0; b < n; ++b) v = threadIdx.x < 3 ? fminf(v, partial[b * 6 + threadIdx.x]) : fmaxf(v, partial[b * 6 + threadIdx.x]);
  bbox[threadIdx.x] = v;
}

// 10 bits spread to every third position (knn.cu:41-47).
__device__ __forceinline__ uint32_t spread3(uint32_t x) {
  x = (x | (x << 16)) & 0x030000FFu;
  x = (x | (x << 8)) & 0x0300F00Fu;
  x = (x | (x << 4)) & 0x030C30C3u;
  x = (x | (x << 2)) & 0x09249249u;
  return x;
}

__device__ __forceinline__ uint32_t quantise(float v, float lo, float hi) {
  const float t = ((v - lo) / (hi - lo)) * 1023.0f;  // degenerate extent: NaN / inf -> 0 / 1023 after the clamp
  return (uint32_t) min(max(f2i_sat(t), 0), 1023);
}

__global__ void __launch_bounds__(256) morton_kernel(int P, const float* __restrict__ points,
    const float* __restrict__ bbox, uint64_t* __restrict__ keys, int32_t* __restrict__ vals) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= P) return;
  const uint32_t x = spread3(quantise(points[3 * (size_t) i], bbox[0], bbox[3]));
  const uint32_t y = spread3(quantise(points[3 * (size_t) i + 1], bbox[1], bbox[4]));
  const uint32_t z = spread3(quantise(points[3 * (size_t) i + 2], bbox[2], bbox[5]));
  keys[i] = x | (y << 1) | (z << 2);
  vals[i] = i;
}

// Points in curve order (xyz + original index) and the bounds of every run of kBox of them.
__global__ void __launch_bounds__(kBox) gather_boxes_kernel(int P, const float* __restrict__ points,
    const int32_t* __restrict__ order, float4* __restrict__ sorted, Bounds* __restrict__ boxes) {
  __shared__ float s_red[6][kBox];
  const int i = blockIdx.x * kBox + threadIdx.x;
  float p[3] = {FLT_MAX, FLT_MAX, FLT_MAX}, q[3] = {-FLT_MAX, -FLT_MAX, -FLT_MAX};
  if (i < P) {
    const int id = order[i];
#pragma unroll
    for (int a = 0; a < 3; ++a) p[a] = q[a] = points[3 * (size_t) id + a];
    sorted[i] = make_float4(p[0], p[1], p[2], __int_as_float(id));
  }
#pragma unroll
  for (int a = 0; a < 3; ++a) s_red[a][threadIdx.x] = p[a], s_red[3 + a][threadIdx.x] = q[a];
  __syncthreads();
  for (int off = kBox / 2; off >= 1; off >>= 1) {
    if ((int) threadIdx.x < off)
#pragma unroll
      for (int a = 0; a < 3; ++a) {
        s_red[a][threadIdx.x]     = fminf(s_red[a][threadIdx.x], s_red[a][threadIdx.x + off]);
        s_red[3 + a][threadIdx.x] = fmaxf(s_red[3 + a][threadIdx.x], s_red[3 + a][threadIdx.x + off]);
      }
    __syncthreads();
  }
  if (threadIdx.x < 3) boxes[blockIdx.x].lo[threadIdx.x] = s_red[threadIdx.x][0];
  else if (threadIdx.x < 6) boxes[blockIdx.x].hi[threadIdx.x - 3] = s_red[threadIdx.x][0];
}

// Squared distance from a point to a box, component by component as knn.cu:103-109.
__device__ __forceinline__ float box_point_dist2(const Bounds& b, const float* p) {
#pragma clang fp contract(off)
  float d[3] = {0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int a = 0; a < 3; ++a)
    if (p[a] < b.lo[a] || p[a] > b.hi[a]) d[a] = fminf(fabsf(p[a] - b.lo[a]), fabsf(p[a] - b.hi[a]));
  return d[0] * d[0] + d[1] * d[1] + d[2] * d[2];
}

// Lower bound of the squared distance between two boxes (0 when they overlap).
__device__ __forceinline__ float box_box_dist2(const Bounds& a, const Bounds& b) {
#pragma clang fp contract(off)
  float s = 0.0f;
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    const float gap = fmaxf(fmaxf(a.lo[k] - b.hi[k], b.lo[k] - a.hi[k]), 0.0f);
    s += gap * gap;
  }
  return s;
}

__device__ __forceinline__ void update_best3(const float* ref, const float4 pt, float* best) {
#pragma clang fp contract(off)
  const float dx = pt.x - ref[0], dy = pt.y - ref[1], dz = pt.z - ref[2];
  float dist = dx * dx + dy * dy + dz * dz;
#pragma unroll
  for (int j = 0; j < 3; ++j)
    if (best[j] > dist) {
      const float t = best[j];
      best[j] = dist, dist = t;
    }
}

// Bounds of every run of 64 boxes (one wavefront per group): the first level of the candidate search.
__global__ void __launch_bounds__(kWave) group_boxes_kernel(int num_boxes, const Bounds* __restrict__ boxes,
                                                            Bounds* __restrict__ groups) {
  const int b = blockIdx.x * kWave + threadIdx.x;
  const Bounds mine = boxes[b < num_boxes ? b : num_boxes - 1];
#pragma unroll
  for (int a = 0; a < 3; ++a) {
    float lo = mine.lo[a], hi = mine.hi[a];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) lo = fminf(lo, __shfl_xor(lo, d, kWave)), hi = fmaxf(hi, __shfl_xor(hi, d, kWave));
    if (threadIdx.x == 0) groups[blockIdx.x].lo[a] = lo, groups[blockIdx.x].hi[a] = hi;
  }
}

// One wavefront = one box = 64 consecutive points of the curve, on its own: its pruning bound is the widest any of its
// 64 queries still has, its bounding box is tested against 64 candidates per ballot (one per lane) on two levels
// (groups of 64 boxes, then the boxes of a surviving group), and a surviving box's points are read with
// wavefront-uniform addresses, i.e. as scalar loads feeding the vector ALU directly: no LDS, no barriers. Boxes of 64
// points prune far better than longer runs of the curve, whose bounds overlap widely.
__global__ void __launch_bounds__(kBox) mean_dist_kernel(int P, int num_boxes, int num_groups,
    const float4* __restrict__ sorted, const Bounds* __restrict__ boxes, const Bounds* __restrict__ groups,
    float* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int idx  = blockIdx.x * kBox + threadIdx.x;
  const bool live = idx < P;
  float p[3] = {0.0f, 0.0f, 0.0f};
  int id = 0;
  if (live) {
    const float4 me = sorted[idx];
    p[0] = me.x, p[1] = me.y, p[2] = me.z, id = __float_as_int(me.w);
  }
  // pruning bound from the six neighbours along the curve (knn.cu:131-139)
  float best[3] = {FLT_MAX, FLT_MAX, FLT_MAX};
  if (live)
    for (int i = max(0, idx - 3); i <= min(P - 1, idx + 3); ++i)
      if (i != idx) update_best3(p, sorted[i], best);
  const float reject = best[2];
  best[0] = best[1] = best[2] = FLT_MAX;
  // bounds of this wavefront's points
  Bounds mine;
#pragma unroll
  for (int a = 0; a < 3; ++a) {
    float lo = live ? p[a] : FLT_MAX, hi = live ? p[a] : -FLT_MAX;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) lo = fminf(lo, __shfl_xor(lo, d, kWave)), hi = fmaxf(hi, __shfl_xor(hi, d, kWave));
    mine.lo[a] = lo, mine.hi[a] = hi;
  }
  if (__ballot(live) == 0ull) return;

  // the widest bound any query of the wavefront still has; its lane exchanges need all 64 lanes, so it is evaluated on
  // its own line, never on the right of a short-circuit inside a ballot
  auto wave_bound = [&]() {
    float bound = live ? fminf(reject, best[2]) : 0.0f;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) bound = fmaxf(bound, __shfl_xor(bound, d, kWave));
    return bound;
  };
  // two levels, 64 candidates per ballot: groups of 64 boxes, then the boxes of a group that can still matter
  for (int g0 = 0; g0 < num_groups; g0 += kWave) {
    const int g = g0 + lane;
    const float group_bound = wave_bound();
    unsigned long long mg =
        __ballot(g < num_groups && box_box_dist2(mine, groups[g < num_groups ? g : 0]) <= group_bound);
    while (mg) {
      const int b0 = (g0 + __builtin_ctzll(mg)) * kWave;  // the same group for every lane
      mg &= mg - 1;
      const int b = b0 + lane;
      const float box_bound = wave_bound();
      unsigned long long m =
          __ballot(b < num_boxes && box_box_dist2(mine, boxes[b < num_boxes ? b : 0]) <= box_bound);
      while (m) {
        const int cb = b0 + __builtin_ctzll(m);  // the same box for every lane
        m &= m - 1;
        const float dist = box_point_dist2(boxes[cb], p);
        const bool take  = live && !(dist > reject || dist > best[2]);  // knn.cu:149
        if (__ballot(take) == 0ull) continue;
        const int first = cb * kBox, count = min(kBox, P - first);
        if (take) {
          for (int i = 0; i < count; ++i)
            if (first + i != idx) update_best3(p, sorted[first + i], best);
        }
      }
    }
  }
  if (live) {
#pragma clang fp contract(off)
    out[id] = (best[0] + best[1] + best[2]) / 3.0f;
  }
}

struct KnnLayout {
  size_t sort, order, sorted, boxes, groups, partial, bbox, bytes;
  int num_boxes, num_groups, bbox_blocks;
};

KnnLayout knn_layout(int P) {
  KnnLayout L;
  const int n     = P > 0 ? P : 1;
  L.num_boxes   = div_up(n, kBox);
  L.num_groups  = div_up(L.num_boxes, kWave);
  L.bbox_blocks = std::min(div_up(n, 256), 512);
  size_t o = 0;
  L.sort = o, o = align_up(o + sort_workspace_bytes(n), 256);
  L.order = o, o = align_up(o + (size_t) n * 4, 256);
  L.sorted = o, o = align_up(o + (size_t) n * 16, 256);
  L.boxes = o, o = align_up(o + (size_t) L.num_boxes * sizeof(Bounds), 256);
  L.groups = o, o = align_up(o + (size_t) L.num_groups * sizeof(Bounds), 256);
  L.partial = o, o = align_up(o + (size_t) L.bbox_blocks * 6 * 4, 256);
  L.bbox = o, o = align_up(o + 6 * 4, 256);
  L.bytes = o;
  return L;
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API size_t fsgs_simple_knn_workspace_bytes(int P) { return P < 0 ? 0 : knn_layout(P).bytes; }

FSGS_API int fsgs_simple_knn(int P, const float* points, float* mean_dist2, void* workspace, size_t workspace_bytes,
                             void* stream) {
  FSGS_REQUIRE(P >= 0, "simple_knn: negative point count");
  if (P == 0) return kOk;
  FSGS_REQUIRE(points && mean_dist2 && workspace, "simple_knn: null pointer");
  const KnnLayout L = knn_layout(P);
  if (workspace_bytes < L.bytes)
    return fail(kWorkspaceSmall, "simple_knn: workspace %zu < %zu bytes", workspace_bytes, L.bytes);
  char* ws = (char*) workspace;
  hipStream_t s = (hipStream_t) stream;
  float* partial = (float*) (ws + L.partial);
  float* bbox    = (float*) (ws + L.bbox);
  int32_t* order = (int32_t*) (ws + L.order);
  float4* sorted = (float4*) (ws + L.sorted);
  Bounds* boxes  = (Bounds*) (ws + L.boxes);
  void* sort_ws  = ws + L.sort;
  hipLaunchKernelGGL(bbox_partial_kernel, dim3(L.bbox_blocks), dim3(256), 0, s, P, points, partial);
  hipLaunchKernelGGL(bbox_final_kernel, dim3(1), dim3(64), 0, s, L.bbox_blocks, partial, bbox);
  const int bits = 30;
  hipLaunchKernelGGL(morton_kernel, dim3(div_up(P, 256)), dim3(256), 0, s, P, points, bbox, sort_keys_in(P, sort_ws),
                     sort_vals_in(P, bits, sort_ws, order));
  const uint64_t* sorted_keys = nullptr;
  radix_sort_pairs(P, bits, sort_ws, order, &sorted_keys, s);
  hipLaunchKernelGGL(gather_boxes_kernel, dim3(L.num_boxes), dim3(kBox), 0, s, P, points, order, sorted, boxes);
  Bounds* groups = (Bounds*) (ws + L.groups);
  hipLaunchKernelGGL(group_boxes_kernel, dim3(L.num_groups), dim3(kWave), 0, s, L.num_boxes, boxes, groups);
  hipLaunchKernelGGL(mean_dist_kernel, dim3(L.num_boxes), dim3(kBox), 0, s, P, L.num_boxes, L.num_groups, sorted, boxes,
                     groups, mean_dist2);
  return check_launch("simple_knn");
}
