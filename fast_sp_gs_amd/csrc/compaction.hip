// Adaptive density control as stream compaction, for gfx950: ordered selection of rows by a mask, one fused row gather
// over all per-point tensors (parameters, both Adam moments, statistics), the clone / split / prune masks, the children
// of a split and the per-step densification statistics.
//
// Reference behaviour reproduced (host torch indexing there, one launch per tensor and per operation):
//   fast_2d_gs/gaussian_splatting.py:497-555 (change_optimizer: `t[mask]`, `torch.cat`), :557-568 (prune_points),
//   :570-579 (densification_postfix), :581-608 (densify_and_split), :610-621 (densify_and_clone), :623-628 (densify),
//   :630-637 (prune), :486-495 (add_densification_stats); fast_2d_gs/network.py:1156-1193 (split with the flat third
//   axis of a surfel), :1276-1282 (per-step statistics).
//
// A mask becomes an ascending index list (what `torch.nonzero` gives); every structural change of the point set is then
// ONE table `source_row[new_row]` (-1 = a row of zeros, used for the Adam moments of new points) applied to all tensors
// by one launch that reads only the rows it keeps and writes the new tensors front to back.
#include "common.hpp"

namespace fsgs {
namespace {

constexpr int kSelThreads = 1024;
constexpr int kSelItems   = 4;  // mask bytes per lane
constexpr int kSelChunk   = kSelThreads * kSelItems;

// Mask bytes of one lane (zero past the end); `invert` selects the zero bytes instead.
__device__ __forceinline__ unsigned lane_flags(int P, const uint8_t* __restrict__ mask, int invert, int base) {
  unsigned f = 0;
#pragma unroll
  for (int k = 0; k < kSelItems; ++k)
    if (base + k < P) f |= (unsigned) ((mask[base + k] != 0) != (invert != 0)) << k;
  return f;
}

// Exclusive prefix of one count per lane over a 1024-lane block; also the block total.
__device__ __forceinline__ int block_prefix(int v, int* s_wave /*[16]*/, int& total) {
  const int lane = __lane_id(), wave = threadIdx.x / kWave;
  int inc = v;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int o = __shfl_up(inc, d, kWave);
    if (lane >= d) inc += o;
  }
  if (lane == kWave - 1) s_wave[wave] = inc;
  __syncthreads();
  int base = 0;
  total    = 0;
#pragma unroll
  for (int w = 0; w < kSelThreads / kWave; ++w) {
    const int s = s_wave[w];
    if (w < wave) base += s;
    total += s;
  }
  __syncthreads();
  return base + inc - v;
}

__global__ void __launch_bounds__(kSelThreads) select_count_kernel(int P, const uint8_t* __restrict__ mask, int invert,
                                                                   int* __restrict__ block_counts) {
  __shared__ int s_wave[kSelThreads / kWave];
  const unsigned f = lane_flags(P, mask, invert, blockIdx.x * kSelChunk + threadIdx.x * kSelItems);
  int total;
  block_prefix(__popc(f), s_wave, total);
  if (threadIdx.x == 0) block_counts[blockIdx.x] = total;
}

__global__ void __launch_bounds__(kSelThreads) select_spine_kernel(int n, int* __restrict__ block_counts,
                                                                   int64_t* __restrict__ count_out) {
  __shared__ int s_wave[kSelThreads / kWave];
  int carry = 0;
  for (int start = 0; start < n; start += kSelThreads) {
    const int i = start + threadIdx.x;
    const int v = i < n ? block_counts[i] : 0;
    int total;
    const int ex = block_prefix(v, s_wave, total);
    if (i < n) block_counts[i] = carry + ex;
    carry += total;
  }
  if (threadIdx.x == 0) *count_out = carry;
}

__global__ void __launch_bounds__(kSelThreads) select_scatter_kernel(int P, const uint8_t* __restrict__ mask,
    int invert, const int* __restrict__ block_offsets, int32_t* __restrict__ indices) {
  __shared__ int s_wave[kSelThreads / kWave];
  const int base   = blockIdx.x * kSelChunk + threadIdx.x * kSelItems;
  const unsigned f = lane_flags(P, mask, invert, base);
  int total;
  int at = block_offsets[blockIdx.x] + block_prefix(__popc(f), s_wave, total);
#pragma unroll
  for (int k = 0; k < kSelItems; ++k)
    if (f >> k & 1u) indices[at++] = base + k;
}

// ---- one gather over many tensors ------------------------------------------------------------------------------------
constexpr int kMaxTensors    = 24;
constexpr int kRowsPerBlock  = 256;
constexpr int kGatherThreads = 256;

struct RowTable {
  const void* src[kMaxTensors];
  void* dst[kMaxTensors];
  int row_units[kMaxTensors];  // units per row
  int unit_log2[kMaxTensors];  // 0: bytes, 2: 32-bit words, 4: 16-byte vectors
};

template <typename U>
__device__ __forceinline__ void gather_units(const U* __restrict__ src, U* __restrict__ dst, int row_units, int64_t row0,
                                             int rows, const int* __restrict__ s_src_row) {
  const unsigned n = (unsigned) rows * (unsigned) row_units;
  for (unsigned u = threadIdx.x; u < n; u += kGatherThreads) {
    const unsigned r = u / (unsigned) row_units, c = u - r * (unsigned) row_units;
    const int from = s_src_row[r];
    U v{};
    if (from >= 0) v = src[(int64_t) from * row_units + c];
    dst[(row0 + r) * row_units + c] = v;
  }
}

// blockIdx.y = tensor, blockIdx.x = chunk of 256 destination rows.
__global__ void __launch_bounds__(kGatherThreads) gather_rows_kernel(RowTable table, int64_t n_rows,
                                                                     const int32_t* __restrict__ source_row) {
  __shared__ int s_src_row[kRowsPerBlock];
  const int t        = blockIdx.y;
  const int64_t row0 = (int64_t) blockIdx.x * kRowsPerBlock;
  const int rows     = (int) (n_rows - row0 < kRowsPerBlock ? n_rows - row0 : kRowsPerBlock);
  if (threadIdx.x < rows) s_src_row[threadIdx.x] = source_row[row0 + threadIdx.x];
  __syncthreads();
  const int units = table.row_units[t];
  switch (table.unit_log2[t]) {
    case 4: gather_units((const uint4*) table.src[t], (uint4*) table.dst[t], units, row0, rows, s_src_row); break;
    case 2: gather_units((const uint32_t*) table.src[t], (uint32_t*) table.dst[t], units, row0, rows, s_src_row); break;
    default: gather_units((const uint8_t*) table.src[t], (uint8_t*) table.dst[t], units, row0, rows, s_src_row); break;
  }
}

// ---- masks -----------------------------------------------------------------------------------------------------------
__device__ __forceinline__ float max_scale(const float* __restrict__ scaling, int S, int i) {
  float m = scaling[(size_t) i * S];
  for (int a = 1; a < S; ++a) m = fmaxf(m, scaling[(size_t) i * S + a]);
  return m;
}

__global__ void __launch_bounds__(256) densify_masks_kernel(int P, int S, const float* __restrict__ grad_accum,
    const float* __restrict__ denom, const float* __restrict__ scaling, float grad_threshold, float scale_threshold,
    uint8_t* __restrict__ clone_mask, uint8_t* __restrict__ split_mask) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= P) return;
  float g = grad_accum[i] / denom[i];
  if (g != g) g = 0.0f;
  const float m = max_scale(scaling, S, i);
  clone_mask[i] = fabsf(g) >= grad_threshold && m <= scale_threshold;
  split_mask[i] = g >= grad_threshold && m > scale_threshold;
}

__global__ void __launch_bounds__(256) prune_mask_kernel(int P, int S, const float* __restrict__ opacity,
    const float* __restrict__ max_radii2D, const float* __restrict__ scaling, float min_opacity, int use_size,
    float max_screen_size, float world_threshold, uint8_t* __restrict__ mask) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= P) return;
  bool m = opacity[i] < min_opacity;
  if (use_size) m = m || max_radii2D[i] > max_screen_size || max_scale(scaling, S, i) > world_threshold;
  mask[i] = m;
}

// ---- children of a split -----------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) split_children_kernel(int n_sel, int N, int S,
    const int32_t* __restrict__ selected, const float* __restrict__ xyz, const float* __restrict__ scaling,
    const float* __restrict__ rotations, const float* __restrict__ noise, float* __restrict__ out_xyz,
    float* __restrict__ out_scaling) {
#pragma clang fp contract(off)
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j >= n_sel * N) return;
  const int p = selected[j % n_sel];
  float s[3] = {0.0f, 0.0f, 0.0f};
  for (int a = 0; a < S; ++a) s[a] = scaling[(size_t) p * S + a];
  const float sx = noise[3 * (size_t) j] * s[0], sy = noise[3 * (size_t) j + 1] * s[1],
              sz = noise[3 * (size_t) j + 2] * s[2];
  float x = rotations[4 * (size_t) p], y = rotations[4 * (size_t) p + 1], z = rotations[4 * (size_t) p + 2],
        w     = rotations[4 * (size_t) p + 3];
  const float n = fmaxf(sqrtf(x * x + y * y + z * z + w * w), 1e-12f);
  x /= n, y /= n, z /= n, w /= n;
  const float r00 = 1 - 2 * y * y - 2 * z * z, r01 = 2 * x * y - 2 * w * z, r02 = 2 * w * y + 2 * x * z;
  const float r10 = 2 * x * y + 2 * w * z, r11 = 1 - 2 * x * x - 2 * z * z, r12 = 2 * y * z - 2 * w * x;
  const float r20 = 2 * x * z - 2 * w * y, r21 = 2 * w * x + 2 * y * z, r22 = 1 - 2 * x * x - 2 * y * y;
  out_xyz[3 * (size_t) j]     = r00 * sx + r01 * sy + r02 * sz + xyz[3 * (size_t) p];
  out_xyz[3 * (size_t) j + 1] = r10 * sx + r11 * sy + r12 * sz + xyz[3 * (size_t) p + 1];
  out_xyz[3 * (size_t) j + 2] = r20 * sx + r21 * sy + r22 * sz + xyz[3 * (size_t) p + 2];
  const float shrink = 0.8f * (float) N;
  for (int a = 0; a < S; ++a) out_scaling[(size_t) j * S + a] = logf(s[a] / shrink);
}

// ---- per-step statistics -----------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) densification_stats_kernel(int P, int grad_stride,
    const int32_t* __restrict__ radii, const float* __restrict__ grad, const float* __restrict__ factor,
    float* __restrict__ max_radii2D, float* __restrict__ grad_accum, float* __restrict__ denom,
    uint8_t* __restrict__ visible) {
#pragma clang fp contract(off)
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= P) return;
  const int r   = radii[i];
  const bool on = r > 0;
  if (visible) visible[i] = on;
  if (!on) return;
  max_radii2D[i] = fmaxf(max_radii2D[i], (float) r);
  const float gx = grad[(size_t) i * grad_stride], gy = grad[(size_t) i * grad_stride + 1];
  float n = sqrtf(gx * gx + gy * gy);
  if (factor) n = n * factor[i];
  grad_accum[i] = grad_accum[i] + n;
  denom[i]      = denom[i] + 1.0f;
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API size_t fsgs_select_indices_workspace_bytes(int P) {
  return align_up((size_t) div_up(P > 0 ? P : 1, kSelChunk) * sizeof(int), 256) + 256;
}

FSGS_API int fsgs_select_indices(int P, const uint8_t* mask, int invert, int32_t* indices, void* workspace,
                                 size_t workspace_bytes, int64_t* count_host, void* stream) {
  FSGS_REQUIRE(P >= 0 && count_host, "select_indices: bad arguments");
  *count_host = 0;
  if (P == 0) return kOk;
  FSGS_REQUIRE(mask && indices && workspace, "select_indices: null pointer");
  if (workspace_bytes < fsgs_select_indices_workspace_bytes(P))
    return fail(kWorkspaceSmall, "select_indices: workspace %zu < %zu bytes", workspace_bytes,
                fsgs_select_indices_workspace_bytes(P));
  hipStream_t s  = (hipStream_t) stream;
  const int nb   = div_up(P, kSelChunk);
  int* counts    = (int*) workspace;
  int64_t* total = (int64_t*) ((char*) workspace + align_up((size_t) nb * sizeof(int), 256));
  hipLaunchKernelGGL(select_count_kernel, dim3(nb), dim3(kSelThreads), 0, s, P, mask, invert, counts);
  hipLaunchKernelGGL(select_spine_kernel, dim3(1), dim3(kSelThreads), 0, s, nb, counts, total);
  hipLaunchKernelGGL(select_scatter_kernel, dim3(nb), dim3(kSelThreads), 0, s, P, mask, invert, counts, indices);
  if (int rc = check_launch("select_indices")) return rc;
  // the count sizes the caller's next allocations, so it has to reach the host here (torch's boolean indexing blocks
  // in the same place)
  FSGS_HIP(hipMemcpyAsync(count_host, total, sizeof(int64_t), hipMemcpyDeviceToHost, s));
  FSGS_HIP(hipStreamSynchronize(s));
  return kOk;
}

FSGS_API int fsgs_gather_rows_max_tensors(void) { return kMaxTensors; }

FSGS_API int fsgs_gather_rows(int n_tensors, const void* const* src_host, void* const* dst_host,
                              const int64_t* row_bytes_host, int64_t n_rows, const int32_t* source_row, void* stream) {
  FSGS_REQUIRE(n_tensors >= 0 && n_tensors <= kMaxTensors && n_rows >= 0, "gather_rows: bad arguments (at most %d tensors)",
               kMaxTensors);
  if (n_tensors == 0 || n_rows == 0) return kOk;
  FSGS_REQUIRE(src_host && dst_host && row_bytes_host && source_row, "gather_rows: null pointer");
  RowTable table{};
  for (int t = 0; t < n_tensors; ++t) {
    const int64_t rb = row_bytes_host[t];
    FSGS_REQUIRE(rb > 0 && rb <= (1 << 20), "gather_rows: tensor %d has a row of %lld bytes", t, (long long) rb);
    FSGS_REQUIRE(dst_host[t], "gather_rows: tensor %d has no destination", t);
    // a source may be absent only if every row is new (-1); the kernel never reads it then, but it cannot know:
    FSGS_REQUIRE(src_host[t], "gather_rows: tensor %d has no source", t);
    const uintptr_t both = (uintptr_t) src_host[t] | (uintptr_t) dst_host[t] | (uintptr_t) rb;
    const int lg         = both % 16 == 0 ? 4 : both % 4 == 0 ? 2 : 0;
    table.src[t] = src_host[t], table.dst[t] = dst_host[t];
    table.row_units[t] = (int) (rb >> lg), table.unit_log2[t] = lg;
  }
  const int64_t chunks = (n_rows + kRowsPerBlock - 1) / kRowsPerBlock;
  FSGS_REQUIRE(chunks < (int64_t) 0x7fffffff, "gather_rows: too many rows");
  hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned) chunks, n_tensors), dim3(kGatherThreads), 0,
                     (hipStream_t) stream, table, n_rows, source_row);
  return check_launch("gather_rows");
}

FSGS_API int fsgs_densify_masks(int P, int S, const float* grad_accum, const float* denom, const float* scaling,
                                float grad_threshold, float scale_threshold, uint8_t* clone_mask, uint8_t* split_mask,
                                void* stream) {
  FSGS_REQUIRE(P >= 0 && S >= 1 && S <= 3, "densify_masks: bad arguments");
  if (P == 0) return kOk;
  FSGS_REQUIRE(grad_accum && denom && scaling && clone_mask && split_mask, "densify_masks: null pointer");
  hipLaunchKernelGGL(densify_masks_kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P, S, grad_accum,
                     denom, scaling, grad_threshold, scale_threshold, clone_mask, split_mask);
  return check_launch("densify_masks");
}

FSGS_API int fsgs_prune_mask(int P, int S, const float* opacity, const float* max_radii2D, const float* scaling,
                             float min_opacity, int use_size, float max_screen_size, float world_threshold,
                             uint8_t* mask, void* stream) {
  FSGS_REQUIRE(P >= 0 && S >= 1 && S <= 3, "prune_mask: bad arguments");
  if (P == 0) return kOk;
  FSGS_REQUIRE(opacity && mask && (!use_size || (max_radii2D && scaling)), "prune_mask: null pointer");
  hipLaunchKernelGGL(prune_mask_kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P, S, opacity,
                     max_radii2D, scaling, min_opacity, use_size, max_screen_size, world_threshold, mask);
  return check_launch("prune_mask");
}

FSGS_API int fsgs_split_children(int P, int n_selected, int N, int S, const int32_t* selected, const float* xyz,
                                 const float* scaling, const float* rotations, const float* noise, float* out_xyz,
                                 float* out_scaling, void* stream) {
  FSGS_REQUIRE(P >= 0 && n_selected >= 0 && n_selected <= P && N >= 1 && S >= 2 && S <= 3,
               "split_children: bad arguments");
  FSGS_REQUIRE((int64_t) n_selected * N < (int64_t) 0x7fffffff, "split_children: too many children");
  if (n_selected == 0) return kOk;
  FSGS_REQUIRE(selected && xyz && scaling && rotations && noise && out_xyz && out_scaling,
               "split_children: null pointer");
  hipLaunchKernelGGL(split_children_kernel, dim3(div_up((int64_t) n_selected * N, 256)), dim3(256), 0,
                     (hipStream_t) stream, n_selected, N, S, selected, xyz, scaling, rotations, noise, out_xyz,
                     out_scaling);
  return check_launch("split_children");
}

FSGS_API int fsgs_densification_stats(int P, int grad_stride, const int32_t* radii, const float* grad,
                                      const float* factor, float* max_radii2D, float* grad_accum, float* denom,
                                      uint8_t* visible, void* stream) {
  FSGS_REQUIRE(P >= 0 && grad_stride >= 2, "densification_stats: bad arguments");
  if (P == 0) return kOk;
  FSGS_REQUIRE(radii && grad && max_radii2D && grad_accum && denom, "densification_stats: null pointer");
  hipLaunchKernelGGL(densification_stats_kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P,
                     grad_stride, radii, grad, factor, max_radii2D, grad_accum, denom, visible);
  return check_launch("densification_stats");
}
