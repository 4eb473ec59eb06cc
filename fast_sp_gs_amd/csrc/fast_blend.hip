// Per-tile alpha blend of the "fast" 2D-Gaussian-surfel path for gfx950: the ray-splat intersection is three dot
// products with the adjugate of the transform (p = adj(M) (x, y, 1), s = p.xy / p.z) instead of a cross product of two
// planes, 8 auxiliary maps, optional snapshots of the running state every 32 list entries, and two backward channel
// sets.
//
// Reference behaviour reproduced: fast_2d_gs/_C/src/gaussian_splatting/gs_2d_fast_redner.cu:22-271 (forward),
// :273-561 (backward, per-pixel form), :563-837 (backward, per-splat form), :839-1074 (host entries).
// The per-splat form of the reference re-walks 32-entry buckets from the forward snapshots with one warp per bucket;
// its result is the same derivative with a different set of live channels (no distortion gradient, M1/M2 maps as
// plain weighted sums with the M1 depth term overwritten, :751-757). Here both forms run the same tile-per-block
// back-to-front kernel by default and differ only in that channel set; the per-splat decomposition itself is
// fast_bucket_backward_kernel below, which consumes the forward's snapshots (slower on this chip). Optical flow (a second set of transforms, :247-255): the forward divides the weighted sum of
// displacements by the final opacity (:259-263); both backward forms take dL/dflow as the gradient of the UNDIVIDED sum
// (:366, :704), and the per-splat form subtracts the DIVIDED final flow from its partial sums (:706), which amounts to
// an opacity-map gradient lowered by (final flow . dL/dflow) -- reproduced here in that algebraic form.
//
// Layout as in the standard blend: one 256-lane block per tile, wavefront w owns an 8x8 quadrant, surfels staged in
// LDS (64-byte hot record with the adjugate, 32-byte cold record), per-quadrant work lists from a conservative bound;
// the backward queues its blended (pixel, entry) pairs and forms their gradient components 64 pairs at a time
// (pair_queue.hpp).
#include "binning.hpp"
#include "blend.hpp"
#include "ordered_sums.hpp"
#include "pair_queue.hpp"

namespace fsgs {
namespace {

struct __attribute__((aligned(16))) FastHot {
  float a[9];           // adjugate of the ray-splat transform
  float tw0, tw1, tw2;  // third row of the transform (depth along the ray)
  float cx, cy, opacity, pad;
};

struct FastSplat {
  FastHot hot;
  SplatCold cold;
  float m[6];  // first two rows of the transform, only used for the quadrant bound while staging
};

__device__ __forceinline__ FastSplat gather_fast(int id, const float2* __restrict__ means2D,
                                                 const float* __restrict__ colors,
                                                 const float4* __restrict__ normal_opacity,
                                                 const float* __restrict__ trans_mat,
                                                 const float* __restrict__ inverse_m) {
  FastSplat s;
  const float* A = inverse_m + 9 * (size_t) id;
  const float* M = trans_mat + 9 * (size_t) id;
#pragma unroll
  for (int k = 0; k < 9; ++k) s.hot.a[k] = A[k];
#pragma unroll
  for (int k = 0; k < 6; ++k) s.m[k] = M[k];
  s.hot.tw0 = M[6], s.hot.tw1 = M[7], s.hot.tw2 = M[8];
  const float2 c  = means2D[id];
  const float4 no = normal_opacity[id];
  s.hot.cx = c.x, s.hot.cy = c.y, s.hot.opacity = no.w, s.hot.pad = 0.0f;
  s.cold.nx = no.x, s.cold.ny = no.y, s.cold.nz = no.z;
  s.cold.r = colors[3 * (size_t) id], s.cold.g = colors[3 * (size_t) id + 1], s.cold.b = colors[3 * (size_t) id + 2];
  s.cold.id = id, s.cold.pad = 0;
  return s;
}

__device__ __forceinline__ unsigned fast_quadrant_mask(const FastSplat& s, int tile_px, int tile_py, int flags) {
  SplatHot h;
#pragma unroll
  for (int k = 0; k < 6; ++k) h.m[k] = s.m[k];
  h.m[6] = s.hot.tw0, h.m[7] = s.hot.tw1, h.m[8] = s.hot.tw2;
  h.cx = s.hot.cx, h.cy = s.hot.cy, h.opacity = s.hot.opacity;
  return quadrant_mask(h, tile_px, tile_py, flags);
}

struct FastHit {
  float pz, sx, sy, dx, dy, rho3d, rho2d, depth, G, alpha;
};

// gs_2d_fast_redner.cu:150-186. Returns false when the reference would `continue`.
// Written without early exits: every lane runs the whole sequence and the rejections (behind the camera plane, nearer
// than `near`, positive exponent, alpha < 1/255) are combined into one predicate at the end, so the callers have one
// divergent region instead of a nest of them on their per-entry critical path.
// `lanes`, if given: mask of the lanes that pass, from the four comparisons' own lane masks (scalar registers).
__device__ __forceinline__ bool fast_intersect_flat(const FastHot& h, float pxf, float pyf, float near_n, FastHit& o,
                                                    unsigned long long* lanes = nullptr) {
  // Every fused multiply-add is written out and contraction is off: the kernels inline this more than once (two copies
  // of a loop body that alternate their registers), and which copy evaluates an entry depends on the work list, so the
  // copies must round alike. Exponent in base 2 (one v_exp_f32, the factor folded into the scale of rho); the
  // reference's `power > 0` rejection cannot fire for a sum of squares and is not evaluated.
#pragma clang fp contract(off)
  const float p0 = fmaf(h.a[0], pxf, fmaf(h.a[1], pyf, h.a[2]));
  const float p1 = fmaf(h.a[3], pxf, fmaf(h.a[4], pyf, h.a[5]));
  o.pz           = fmaf(h.a[6], pxf, fmaf(h.a[7], pyf, h.a[8]));
  const float rz = __builtin_amdgcn_rcpf(o.pz);
  o.sx = p0 * rz, o.sy = p1 * rz;
  o.rho3d = fmaf(o.sx, o.sx, o.sy * o.sy);
  o.dx = h.cx - pxf, o.dy = h.cy - pyf;
  const float d2 = fmaf(o.dx, o.dx, o.dy * o.dy);
  o.rho2d = 2.0f * d2;
  o.depth = fmaf(o.sx, h.tw0, fmaf(o.sy, h.tw1, h.tw2));
  const float power2 = fmaxf(o.rho3d * -0.72134752044448170368f, d2 * -1.44269504088896340736f);
  o.G     = __builtin_amdgcn_exp2f(power2);
  o.alpha = fminf(0.99f, h.opacity * o.G);
  const bool c0 = o.pz != 0.0f, c1 = !(o.depth < near_n), c3 = !(o.alpha < (1.0f / 255.0f));
  if (lanes) *lanes = wave_ballot(c0) & wave_ballot(c1) & wave_ballot(c3);
  return c0 & c1 & c3;
}

// Sums 8 per-lane values over each 16-lane row at once: three merge steps inside aligned groups of 8 lanes, one rotate
// by 8 inside the row. On return lane l of every row holds that row's total of v[l & 7].
__device__ __forceinline__ float row_sum8_transposed(const float (&v)[8]) {
#pragma clang fp contract(off)  // an input that is a product must not be formed a second time inside a fused add
  const int lane = __lane_id();
  const bool b0 = lane & 1, b1 = lane & 2, b2 = lane & 4;
  float w[4], x[2];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float a = v[2 * i + 1] + dpp_shift_zero<0x111, 0xf, 0xf>(v[2 * i + 1]);  // row_shr:1
    const float b = v[2 * i] + dpp_shift_zero<0x101, 0xf, 0xf>(v[2 * i]);          // row_shl:1
    w[i] = b0 ? a : b;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const float a = w[2 * i + 1] + dpp_shift_zero<0x112, 0xf, 0xf>(w[2 * i + 1]);  // row_shr:2
    const float b = w[2 * i] + dpp_shift_zero<0x102, 0xf, 0xf>(w[2 * i]);          // row_shl:2
    x[i] = b1 ? a : b;
  }
  const float a = x[1] + dpp_shift_zero<0x114, 0xf, 0xf>(x[1]);  // row_shr:4
  const float b = x[0] + dpp_shift_zero<0x104, 0xf, 0xf>(x[0]);  // row_shl:4
  float z = b2 ? a : b;
  z += dpp_shift_zero<0x128, 0xf, 0xf>(z);  // row_ror:8
  return z;
}
// The same over the 64 lanes: every lane holds the wave total of v[lane & 7].
__device__ __forceinline__ float wave_sum8_transposed(const float (&v)[8]) { return cross_row_sum(row_sum8_transposed(v)); }

template <bool kAux, bool kSnap, bool kAccum, bool kFlow>
__global__ void __launch_bounds__(kBlendThreads) fast_blend_forward_kernel(
    int ordered, const int* __restrict__ tile_order, int W, int H, float near_n, float far_n, const int64_t* __restrict__ ranges, const int32_t* __restrict__ point_list,
    const float2* __restrict__ means2D, const float* __restrict__ colors, const float* __restrict__ trans_mat,
    const float* __restrict__ inverse_m, const float4* __restrict__ normal_opacity,
    const float* __restrict__ trans_mat_t2, const int64_t* __restrict__ bucket_offset, int32_t* __restrict__ n_contrib,
    float* __restrict__ out_color, float* __restrict__ out_opacity, float* __restrict__ out_extras,
    float2* __restrict__ out_flow, int32_t* __restrict__ max_contrib,
    int32_t* __restrict__ bucket_to_tile, float* __restrict__ sampled_T, float* __restrict__ sampled_acc,
    float* __restrict__ sampled_aux, int32_t* __restrict__ accum_max_count, float* __restrict__ accum_weights_p,
    int32_t* __restrict__ accum_weights_count) {
  __shared__ FastHot s_hot[kBatch];
  __shared__ SplatCold s_cold[kBatch];
  __shared__ float s_t2[kFlow ? kBatch * 9 : 1];  // second-time-step transforms of the staged surfels
  __shared__ unsigned char s_mask[kBatch];
  __shared__ int s_max_contrib;
  constexpr int kNum = kFlow ? 10 : 8;  // channels of a snapshot

  const int gx = (W + kTile - 1) / kTile;
  const int tile = scheduled_tile(ordered, tile_order), tile_x = tile % gx, tile_y = tile / gx;
  int px, py;
  lane_pixel(tile_x, tile_y, px, py);
  const bool inside = px < W && py < H;
  const size_t HW   = (size_t) H * W;
  const size_t pix  = (size_t) W * py + px;
  const float pxf = (float) px, pyf = (float) py;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rank = (py - tile_y * kTile) * kTile + (px - tile_x * kTile);  // row-major position inside the tile

  const int64_t r0 = ranges[2 * (size_t) tile], r1 = ranges[2 * (size_t) tile + 1];
  const int n_todo = (int) (r1 - r0);
  const int rounds = (n_todo + kBatch - 1) / kBatch;

  int64_t bucket0 = 0;
  if (kSnap) {
    bucket0 = tile == 0 ? 0 : bucket_offset[tile - 1];
    const int nb = (n_todo + 31) / 32;
    for (int k = threadIdx.x; k < nb; k += kBlendThreads) bucket_to_tile[bucket0 + k] = tile;
    if (threadIdx.x == 0) s_max_contrib = 0;
  }

  // blending state of the pixel (float: its test is one comparison) and of the wavefront (a lane mask in scalar
  // registers: "is anybody still blending" costs no vector instruction)
  float live = inside ? 1.0f : -1.0f;
  unsigned long long live_lanes = wave_ballot(inside);
  const float far_scale = far_n / (far_n - near_n);
  float T = 1.0f, C0 = 0, C1 = 0, C2 = 0;
  float N0 = 0, N1 = 0, N2 = 0, D = 0, M1 = 0, M2 = 0, dist = 0, median = 0, f0 = 0, f1 = 0;
  int last = 0, median_c = -1;
  ArgmaxRun argmax;

  FastSplat next;
  float next_t2[9];
  if ((int) threadIdx.x < n_todo) {
    const int id = point_list[r0 + threadIdx.x];
    next = gather_fast(id, means2D, colors, normal_opacity, trans_mat, inverse_m);
    if (kFlow) {
#pragma unroll
      for (int k = 0; k < 9; ++k) next_t2[k] = trans_mat_t2[9 * (size_t) id + k];
    }
  }

  for (int b = 0; b < rounds; ++b) {
    if (__syncthreads_count(live < 0.0f) == kBlendThreads) break;
    const int n_here = min(kBatch, n_todo - b * kBatch);
    if ((int) threadIdx.x < n_here) {
      s_hot[threadIdx.x]  = next.hot;
      s_cold[threadIdx.x] = next.cold;
      s_mask[threadIdx.x] = (unsigned char) fast_quadrant_mask(next, tile_x * kTile, tile_y * kTile, ordered);
      if (kFlow) {
#pragma unroll
        for (int k = 0; k < 9; ++k) s_t2[threadIdx.x * 9 + k] = next_t2[k];
      }
    }
    __syncthreads();
    const int nxt = (b + 1) * kBatch + (int) threadIdx.x;
    if (nxt < n_todo) {
      const int id = point_list[r0 + nxt];
      next = gather_fast(id, means2D, colors, normal_opacity, trans_mat, inverse_m);
      if (kFlow) {
#pragma unroll
        for (int k = 0; k < 9; ++k) next_t2[k] = trans_mat_t2[9 * (size_t) id + k];
      }
    }

    for (int c = 0; c < kBatch / kWave; ++c) {
      const int jj = c * kWave + lane;
      const unsigned long long todo_all = __ballot(jj < n_here && ((s_mask[jj] >> wave) & 1u));
      for (int half = 0; half < (kSnap ? 2 : 1); ++half) {
        unsigned long long todo = todo_all;
        if (kSnap) {
          const int base = c * kWave + half * 32;
          if (base >= n_here) break;
          if (live > 0.0f) {
            // state before list entry b * 256 + base, which starts a bucket of 32 (gs_2d_fast_redner.cu:126-147)
            const size_t bk = (size_t) (bucket0 + (b * kBatch + base) / 32);
            sampled_T[bk * 256 + rank]             = T;
            sampled_acc[(bk * 3 + 0) * 256 + rank] = C0;
            sampled_acc[(bk * 3 + 1) * 256 + rank] = C1;
            sampled_acc[(bk * 3 + 2) * 256 + rank] = C2;
            if (kAux) {
              sampled_aux[(bk * kNum + 0) * 256 + rank] = D;
              sampled_aux[(bk * kNum + 1) * 256 + rank] = N0;
              sampled_aux[(bk * kNum + 2) * 256 + rank] = N1;
              sampled_aux[(bk * kNum + 3) * 256 + rank] = N2;
              sampled_aux[(bk * kNum + 5) * 256 + rank] = dist;
              sampled_aux[(bk * kNum + 6) * 256 + rank] = M1;
              sampled_aux[(bk * kNum + 7) * 256 + rank] = M2;
              if (kFlow) {
                sampled_aux[(bk * kNum + 8) * 256 + rank] = f0;
                sampled_aux[(bk * kNum + 9) * 256 + rank] = f1;
              }
            }
          }
          todo &= half ? 0xffffffff00000000ull : 0x00000000ffffffffull;
        }
        // one entry of the wavefront's work list; its records were requested from LDS while the entry before it ran
        auto blend_entry = [&](const FastHot& hot, const SplatCold& cold, int j) {
#pragma clang fp contract(off)  // two copies of this body exist (alternating registers): both must round alike
          FastHit h;
          unsigned long long pass;
          const bool hit = fast_intersect_flat(hot, pxf, pyf, near_n, h, &pass) && live > 0.0f;
          pass &= live_lanes;
          if (pass == 0ull) return;
          const float test_T = T * (1.0f - h.alpha);
          const bool sat     = hit && test_T < 0.0001f;
          live               = sat ? -1.0f : live;
          live_lanes &= ~(pass & wave_ballot(test_T < 0.0001f));
          const float w         = h.alpha * T;
          if (kAccum && (accum_weights_p || accum_weights_count))
            wave_accumulate_weights(hit && !sat, w, cold.id, accum_weights_p, accum_weights_count);
          if (!hit || sat) return;
          const int contributor = b * kBatch + j + 1;
          if (kAux) {
            const float A = 1.0f - T;
            const float m = far_scale * (1.0f - near_n * __builtin_amdgcn_rcpf(h.depth));
            const float mm = m * m;
            dist = fmaf(fmaf(mm, A, fmaf(-2.0f * m, M1, M2)), w, dist);
            D    = fmaf(h.depth, w, D);
            M1   = fmaf(m, w, M1);
            M2   = fmaf(mm, w, M2);
            if (T > 0.5f) median = h.depth, median_c = contributor;
            N0 = fmaf(cold.nx, w, N0), N1 = fmaf(cold.ny, w, N1), N2 = fmaf(cold.nz, w, N2);
            if (kAccum) argmax_run_step(argmax, w, cold.id, accum_max_count);
            if (kFlow) {
              const float* Q = &s_t2[j * 9];
              const float u2 = fmaf(Q[0], h.sx, fmaf(Q[1], h.sy, Q[2]));
              const float v2 = fmaf(Q[3], h.sx, fmaf(Q[4], h.sy, Q[5]));
              float w2       = fmaf(Q[6], h.sx, fmaf(Q[7], h.sy, Q[8]));
              w2             = fabsf(w2) < 1e-5f ? 1e-5f : w2;
              f0 = fmaf(u2 / w2 - pxf, w, f0);
              f1 = fmaf(v2 / w2 - pyf, w, f1);
            }
          }
          C0 = fmaf(cold.r, w, C0), C1 = fmaf(cold.g, w, C1), C2 = fmaf(cold.b, w, C2);
          T    = test_T;
          last = contributor;
        };
        if (todo == 0ull) continue;
        auto pop = [&]() {
          const int j = c * kWave + __builtin_ctzll(todo);
          todo &= todo - 1;
          return j;
        };
        auto peek = [&]() { return c * kWave + (todo ? __builtin_ctzll(todo) : 0); };
        FastHot hot_a = s_hot[peek()], hot_b;
        while (todo) {
          if (live_lanes == 0ull) break;  // every pixel of this quadrant is saturated
          {
            const int j = pop();
            hot_b       = s_hot[peek()];
            const SplatCold cold = s_cold[j];  // used only if a pixel blends the surfel, but then without waiting
            __builtin_amdgcn_sched_barrier(0);
            blend_entry(hot_a, cold, j);
          }
          if (todo == 0ull || live_lanes == 0ull) break;
          {
            const int j = pop();
            hot_a       = s_hot[peek()];
            const SplatCold cold = s_cold[j];
            __builtin_amdgcn_sched_barrier(0);
            blend_entry(hot_b, cold, j);
          }
        }
      }
    }
  }

  if (kAccum) argmax_run_flush(argmax, accum_max_count);
  if (inside) {
    out_opacity[pix]        = 1.0f - T;
    n_contrib[pix]          = last;
    n_contrib[pix + HW]     = kAux ? median_c : 0;
    out_color[pix]          = C0;
    out_color[pix + HW]     = C1;
    out_color[pix + 2 * HW] = C2;
    if (kAux) {
      out_extras[pix + 0 * HW] = D;
      out_extras[pix + 1 * HW] = N0;
      out_extras[pix + 2 * HW] = N1;
      out_extras[pix + 3 * HW] = N2;
      out_extras[pix + 4 * HW] = median;
      out_extras[pix + 5 * HW] = dist;
      out_extras[pix + 6 * HW] = M1;
      out_extras[pix + 7 * HW] = M2;
      if (kFlow) {
        const float A = 1.0f - T;
        out_flow[pix] = A > 0.0f ? make_float2(f0 / A, f1 / A) : make_float2(0.0f, 0.0f);
      }
    }
  }
  if (kSnap) {
    int wave_max = last;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) wave_max = max(wave_max, __shfl_xor(wave_max, d, kWave));
    __syncthreads();  // s_max_contrib was cleared before the first barrier of the loop only if the loop ran
    if (lane == 0) atomicMax(&s_max_contrib, wave_max);
    __syncthreads();
    if (threadIdx.x == 0) max_contrib[tile] = s_max_contrib;
  }
}

// Per-surfel gradient slots: 0-2 colours | 3-11 adjugate | 12-14 normal | 15 opacity | 16-18 transform row 2 |
// 19-20 means2D.
constexpr int kFastGradSlots  = 21;
constexpr int kFastRecordSlots = 22;  // a record of the ordered-sum path: the 21 slots + one float of padding

// Where slot_sum_kernel puts component c of surfel i: 0-2 colours | 3-11 inverse transform | 12-15 normal, opacity |
// 16-18 third row of the transform (the other two rows get no gradient from the blend: zeros) | 19-20 means2D.
struct FastScatter {
  float *g_means2D, *g_normal_opacity, *g_colors, *g_trans, *g_inv;
  __device__ __forceinline__ void operator()(int i, int c, float v) const {
    if (c < 3) g_colors[3 * (size_t) i + c] = v;
    else if (c < 12) g_inv[9 * (size_t) i + (c - 3)] = v;
    else if (c < 16) g_normal_opacity[4 * (size_t) i + (c - 12)] = v;
    else if (c < 19) {
      g_trans[9 * (size_t) i + 6 + (c - 16)] = v;
      g_trans[9 * (size_t) i + 2 * (c - 16)] = 0.0f, g_trans[9 * (size_t) i + 2 * (c - 16) + 1] = 0.0f;
    } else if (c < 21) g_means2D[2 * (size_t) i + (c - 19)] = v;
  }
};

// Sum of a surfel's records on the fast path. Its key span holds one position per tile of its rectangle, x-major, but
// only the tiles that pass the binning's corner test are in a tile list, and only those positions were written by the
// blend (a list entry's record by the flush of its batch, or zeros by its tile's block if the entry lies behind the
// deepest contributor). The test is repeated here, with the binning's own arithmetic, so the other positions are
// neither cleared nor read. 11 lanes per surfel, each owning one float2 of the 88-byte record: a step covers 11
// positions of the span -- lane k tests position base + k, the 11 verdicts are shared through a ballot, and the
// records of the positions that passed are requested together.
// `keep_masks` (optional, what the preprocess kernel left): the verdicts for rectangles of at most 32 tiles, bit = position
// in the span; a wavefront none of whose surfels has a larger rectangle then reads neither the adjugates nor the opacity
// and does not set the test up.
__global__ void __launch_bounds__(256) fast_slot_sum_kernel(int P, int gx, int gy,
    const int64_t* __restrict__ point_offsets, const int32_t* __restrict__ radii, const float2* __restrict__ means2D,
    const float* __restrict__ inverse_m, const float4* __restrict__ normal_opacity,
    const uint32_t* __restrict__ keep_masks, const float* __restrict__ records, FastScatter out) {
  constexpr int kLanes = kFastRecordSlots / 2, kPerWave = 64 / kLanes;
  const int lane = threadIdx.x & 63;
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int sub = lane / kLanes, k = lane - sub * kLanes;
  const int i = wave * kPerWave + sub;
  const bool active = sub < kPerWave && i < P;
  const int radius = active ? radii[i] : 0;
  int count = 0, h = 1, x0 = 0, y0 = 0;
  float IM[9], opacity = 1.0f;
#pragma unroll
  for (int q = 0; q < 9; ++q) IM[q] = 0.0f;
  const float2* src = (const float2*) records;
  uint32_t mask = 0u;
  bool masked = false;  // this surfel's verdicts come from its mask
  if (radius > 0) {
    const float2 c   = means2D[i];
    const TileRect r = tile_rect(c.x, c.y, radius, gx, gy);
    h = max(r.y1 - r.y0, 1), count = max(r.x1 - r.x0, 0) * max(r.y1 - r.y0, 0), x0 = r.x0, y0 = r.y0;
    masked = keep_masks != nullptr && count <= 32;
    if (masked) mask = keep_masks[i];
    src += (size_t) (i > 0 ? point_offsets[i - 1] : 0) * kLanes + k;
  }
  const bool tested     = radius > 0 && !masked;
  const bool any_tested = wave_ballot(tested) != 0ull;  // wave-uniform
  if (tested) {
#pragma unroll
    for (int q = 0; q < 9; ++q) IM[q] = inverse_m[9 * (size_t) i + q];
    opacity = normal_opacity[i].w;
  }
  CornerTest ct;
  if (any_tested) ct = CornerTest(IM, opacity);
  float2 acc = make_float2(0.0f, 0.0f);
  // the wavefront's surfels step together (the ballot needs every lane): as many steps as its largest rectangle asks
  int steps = (count + kLanes - 1) / kLanes;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) steps = max(steps, __shfl_xor(steps, d, kWave));
  for (int st = 0; st < steps; ++st) {
    const int base = st * kLanes, p = base + k, x = p / h, y = p - x * h;  // x-major over the rectangle
    bool on = masked && p < count && ((mask >> (p & 31)) & 1u) != 0u;
    if (any_tested) on = on || (tested && p < count && ct.tile(x0 + x, y0 + y));
    const unsigned bits = (unsigned) (wave_ballot(on) >> (sub * kLanes)) & ((1u << kLanes) - 1u);
    float2 v[kLanes];
#pragma unroll
    for (int j = 0; j < kLanes; ++j)
      v[j] = ((bits >> j) & 1u) ? src[(size_t) (base + j) * kLanes] : make_float2(0.0f, 0.0f);
#pragma unroll
    for (int j = 0; j < kLanes; ++j) acc.x += v[j].x, acc.y += v[j].y;
  }
  if (!active) return;
  out(i, 2 * k, acc.x);
  out(i, 2 * k + 1, acc.y);
}

// kSlots: the per-surfel sums go through per-instance records (ordered_sums.hpp) instead of device-scope atomics.
template <bool kAux, bool kPerSplat, bool kFlow, bool kSlots>
// Four blocks per compute unit where the per-surfel sums go through records (the flush of the other form keeps more
// values live and would spill in the loop over the entries): the launch lasts little longer than the block with the
// longest list, and the more wavefronts share a SIMD with that block's, the sooner the other blocks are out of the way.
__global__ void __launch_bounds__(kBlendThreads)
    __attribute__((amdgpu_waves_per_eu(kSlots && !kFlow ? 4 : 1, kSlots && !kFlow ? 4 : 8))) fast_blend_backward_kernel(
    int ordered, const int* __restrict__ tile_order, int W, int H, float near_n, float far_n, const int64_t* __restrict__ ranges, const int32_t* __restrict__ point_list,
    const int32_t* __restrict__ n_contrib, const float2* __restrict__ means2D,
    const float4* __restrict__ normal_opacity, const float* __restrict__ colors, const float* __restrict__ trans_mat,
    const float* __restrict__ inverse_m, const float* __restrict__ trans_mat_t2, const float* __restrict__ out_opacity,
    const float* __restrict__ out_extras, const float2* __restrict__ out_flow,
    const float* __restrict__ dL_dpix, const float* __restrict__ dL_dextras, const float* __restrict__ dL_dopacity,
    const float2* __restrict__ dL_dflow,
    float* __restrict__ g_means2D, float* __restrict__ g_normal_opacity, float* __restrict__ g_colors,
    float* __restrict__ g_trans, float* __restrict__ g_inv, const int64_t* __restrict__ point_offsets,
    const int32_t* __restrict__ radii, float* __restrict__ slot_records) {
  constexpr int kB = 64;  // surfels staged per round
  static_assert(kB == kWave, "one ballot covers a round, and a queued pair names its entry in a byte");
  // Two passes (pair_queue.hpp): the order-bound recurrence queues the blending pairs, the components are formed and
  // summed 64 pairs at a time. Not with a second set of transforms, whose per-pair terms would double the item.
  constexpr bool kQueue = !kFlow;
  __shared__ float4 s_queue[kQueue ? 4 : 1][kQueue ? kQueueItems : 1];
  __shared__ FastHot s_hot[kB];
  __shared__ SplatCold s_cold[kB];
  __shared__ float s_t2[kFlow ? kB * 9 : 1];
  // each wavefront's sums per staged surfel, written once per entry with a plain store and added in wavefront order at
  // the flush (LDS float atomics cost about three cycles per lane)
  __shared__ float s_part[4][kB][kFastGradSlots];
  __shared__ int s_max_contrib;
  __shared__ unsigned char s_mask[kB];

  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const int tile = scheduled_tile(ordered, tile_order), tile_x = tile % gx, tile_y = tile / gx;
  int px, py;
  lane_pixel(tile_x, tile_y, px, py);
  const bool inside = px < W && py < H;
  const size_t HW   = (size_t) H * W;
  const size_t pix  = (size_t) W * py + px;
  const float pxf = (float) px, pyf = (float) py;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float qx0 = pxf - (float) (lane & 7), qy0 = pyf - (float) (lane >> 3);  // first pixel of the wavefront's quadrant
  PairQueue q;

  const int64_t r0 = ranges[2 * (size_t) tile], r1 = ranges[2 * (size_t) tile + 1];
  const int last_contrib   = inside ? n_contrib[pix] : 0;
  const int median_contrib = (kAux && inside) ? n_contrib[pix + HW] : 0;

  if (threadIdx.x == 0) s_max_contrib = 0;
  __syncthreads();
  int wave_max_contrib = last_contrib;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) wave_max_contrib = max(wave_max_contrib, __shfl_xor(wave_max_contrib, d, kWave));
  if (lane == 0) atomicMax(&s_max_contrib, wave_max_contrib);
  for (int e = threadIdx.x; e < 4 * kB * kFastGradSlots; e += kBlendThreads) (&s_part[0][0][0])[e] = 0.0f;
  __syncthreads();
  const int n_todo = min(s_max_contrib, (int) (r1 - r0));
  const int rounds = (n_todo + kB - 1) / kB;
  // No zero fill of the record buffer: every staged instance writes its record at the flush, zeros included, and the
  // instances behind the tile's deepest contributor, which are never staged, are cleared here.
  if (kSlots) {
    for (int e = n_todo + (int) threadIdx.x; e < (int) (r1 - r0); e += kBlendThreads) {
      const int id = point_list[r0 + e];
      const float2 c = means2D[id];
      const TileRect r = tile_rect(c.x, c.y, radii[id], gx, gy);
      const int64_t at = (id == 0 ? 0 : point_offsets[id - 1]) + (int64_t) (tile_x - r.x0) * (r.y1 - r.y0) + (tile_y - r.y0);
      float2* dst = (float2*) (slot_records + (size_t) at * kFastRecordSlots);
#pragma unroll
      for (int c2 = 0; c2 < kFastRecordSlots / 2; ++c2) dst[c2] = make_float2(0.0f, 0.0f);
    }
  }

  const float T_final = inside ? 1.0f - out_opacity[pix] : 0.0f;
  float T = T_final;
  float dLp0 = 0, dLp1 = 0, dLp2 = 0;
  float dL_dreg = 0, dL_ddepth = 0, dL_daccum = 0, dLn0 = 0, dLn1 = 0, dLn2 = 0, dL_dmedian = 0, dL_dM1 = 0, dL_dM2 = 0;
  float final_D = 0, final_D2 = 0, dLf0 = 0, dLf1 = 0;
  if (inside) {
    dLp0 = dL_dpix[pix], dLp1 = dL_dpix[pix + HW], dLp2 = dL_dpix[pix + 2 * HW];
    if (kAux) {
      dL_daccum  = dL_dopacity[pix];
      dL_ddepth  = dL_dextras[pix + 0 * HW];
      dLn0       = dL_dextras[pix + 1 * HW];
      dLn1       = dL_dextras[pix + 2 * HW];
      dLn2       = dL_dextras[pix + 3 * HW];
      dL_dmedian = dL_dextras[pix + 4 * HW];
      if (kPerSplat) dL_dM1 = dL_dextras[pix + 6 * HW], dL_dM2 = dL_dextras[pix + 7 * HW];
      else dL_dreg = dL_dextras[pix + 5 * HW];
      final_D  = out_extras[pix + 6 * HW];
      final_D2 = out_extras[pix + 7 * HW];
    } else if (kPerSplat) {
      dL_daccum = dL_dopacity[pix];
    }
    if (kFlow) {
      const float2 gf = dL_dflow[pix];
      dLf0 = gf.x, dLf1 = gf.y;
      if (kPerSplat) {
        // partial sum - DIVIDED final flow  ==  -(sum over later entries) - final flow * T_final: the second part acts
        // like the opacity map's gradient (both carry T_final / (1 - alpha) per entry)
        const float2 ff = out_flow[pix];
        dL_daccum -= ff.x * gf.x + ff.y * gf.y;
      }
    }
  }
  const float far_scale = far_n / (far_n - near_n), far_near = far_scale * near_n;
  // the distortion term's per-pixel constants, folded once: with m the normalised depth of a pair,
  //   dL/dweight = (D2 + m^2 A - 2 m D) dL/dreg = reg_D2 + m (m reg_A - reg_2D),  dL/dm = w (m reg_2A - reg_2D)
  const float reg_A = (1.0f - T_final) * dL_dreg, reg_2A = 2.0f * reg_A, reg_2D = 2.0f * final_D * dL_dreg,
              reg_D2 = final_D2 * dL_dreg;

  float acc_lin = 0;  // what the pairs behind the current one accumulated: alpha_j c_j weighted by the transmittance between

  FastSplat next;
  float next_t2[9];
  int next_radius = 0;
  int64_t next_off = 0;
  size_t slot = 0;  // record position of the entry this lane staged (the same lane flushes it)
  auto gather = [&](int at) {
    const int id = point_list[r0 + at];
    next = gather_fast(id, means2D, colors, normal_opacity, trans_mat, inverse_m);
    if (kFlow) {
#pragma unroll
      for (int k = 0; k < 9; ++k) next_t2[k] = trans_mat_t2[9 * (size_t) id + k];
    }
    if (kSlots) next_radius = radii[id], next_off = id == 0 ? 0 : point_offsets[id - 1];
  };
  if ((int) threadIdx.x < min(n_todo, kB)) gather(n_todo - 1 - (int) threadIdx.x);

  for (int b = 0; b < rounds; ++b) {
    const int n_here = min(kB, n_todo - b * kB);
    if ((int) threadIdx.x < n_here) {
      s_hot[threadIdx.x]  = next.hot;
      s_cold[threadIdx.x] = next.cold;
      s_mask[threadIdx.x] = (unsigned char) fast_quadrant_mask(next, tile_x * kTile, tile_y * kTile, ordered);
      if (kFlow) {
#pragma unroll
        for (int k = 0; k < 9; ++k) s_t2[threadIdx.x * 9 + k] = next_t2[k];
      }
      if (kSlots) {
        // The fused binning reserves one key position per tile of the surfel's rectangle, from its prefix-scan offset
        // on (the tiles that pass its corner test are packed to the front of that span, the rest is padding). Any
        // position of the span that no other tile of the surfel uses will do for the record: x-major over the rectangle.
        const TileRect r = tile_rect(next.hot.cx, next.hot.cy, next_radius, gx, gy);
        slot = (size_t) (next_off + (int64_t) (tile_x - r.x0) * (r.y1 - r.y0) + (tile_y - r.y0));
      }
    }
    __syncthreads();
    const int nxt = (b + 1) * kB + (int) threadIdx.x;
    if ((int) threadIdx.x < kB && nxt < n_todo) gather(n_todo - 1 - nxt);

    // The part of a pair that is bound to the list's order: advances the pixel's back-to-front state and leaves the
    // pair's weight, dL/dalpha (times the transmittance in front of the pair), dL/d(depth along the ray) and, with a
    // second set of transforms, dL/d(intersection) through it. Only entered by lanes whose pixel blends the entry.
    auto advance_pixel = [&](const SplatCold& cold, int j, int pos, const FastHit& h, float& w, float& dL_dalpha,
                             float& dL_dz, float& fsx, float& fsy) {
      T = T * __builtin_amdgcn_rcpf(1.0f - h.alpha);
      w = h.alpha * T;
      // one back-to-front recurrence for every channel that enters the image linearly: c = <upstream gradient,
      // channel values of this surfel> replaces the reference's per-channel accumulators
      float c_lin = cold.r * dLp0 + cold.g * dLp1 + cold.b * dLp2;
      if (kAux) {
        const float rd     = __builtin_amdgcn_rcpf(h.depth);
        const float m_d    = far_scale - far_near * rd;
        const float dmd_dd = far_near * rd * rd;
        if (pos == median_contrib - 1) dL_dz += dL_dmedian;
        if (!kPerSplat) {
          // dL/dweight of the distortion enters dL/dalpha as a linear channel does (its value minus what the pairs
          // behind it accumulated, with the same weights): it rides on the shared recurrence
          c_lin += reg_D2 + m_d * (m_d * reg_A - reg_2D);
          dL_dz += w * (m_d * reg_2A - reg_2D) * dmd_dd;
        } else {
          c_lin += m_d * dL_dM1 + (m_d * m_d) * dL_dM2;
          dL_dz += dmd_dd * (2.0f * m_d * w * dL_dM2);
        }
        c_lin += h.depth * dL_ddepth + cold.nx * dLn0 + cold.ny * dLn1 + cold.nz * dLn2;
        dL_dz += w * dL_ddepth;
      }
      if (kAux || kPerSplat) c_lin += dL_daccum;
      if (kFlow) {
        const float* Q = &s_t2[j * 9];
        const float u2 = Q[0] * h.sx + Q[1] * h.sy + Q[2];
        const float v2 = Q[3] * h.sx + Q[4] * h.sy + Q[5];
        float w2       = Q[6] * h.sx + Q[7] * h.sy + Q[8];
        w2             = fabsf(w2) < 1e-5f ? 1e-5f : w2;
        const float rw = 1.0f / w2;
        c_lin += (u2 * rw - pxf) * dLf0 + (v2 * rw - pyf) * dLf1;
        const float gu = w * rw * dLf0, gv = w * rw * dLf1;
        const float gw = -w * rw * rw * (u2 * dLf0 + v2 * dLf1);
        fsx = Q[0] * gu + Q[3] * gv + Q[6] * gw;
        fsy = Q[1] * gu + Q[4] * gv + Q[7] * gw;
      }
      dL_dalpha = c_lin - acc_lin;
      acc_lin   = fmaf(1.0f - h.alpha, acc_lin, h.alpha * c_lin);
      dL_dalpha *= T;
    };

    // ---- order-free part: 64 queued pairs at a time, four 16-lane rows, every row one entry ---------------------------
    // A lane rebuilds the intersection through its pair's pixel from the staged adjugate and forms the 16 + 5 components
    // as products of the three queued numbers with quantities that are finite in every lane (padding items carry zeros
    // and no flags, and the reciprocal of p_z is only taken under the pair's flags).
    auto drain = [&](int n_valid) {
      const unsigned jrows = queue_front_rows(q);
      const int j = (int) ((jrows >> ((lane >> 4) * 8)) & 255u);
      const float4 it = s_queue[wave][q.head + lane];
      const FastHot hot = s_hot[j];
      float* const acc  = &s_part[wave][j][lane & 15];
      const bool second = (lane & 15) < 5;  // lanes 0-4 of a row add the five other components
      float* const acc2 = &s_part[wave][j][16 + (second ? (lane & 15) : 0)];
      const float before = *acc;
      const float before2 = (kAux && second) ? *acc2 : 0.0f;
      const int bits = __float_as_int(it.w);
      const int qp = bits & 63;
      const bool blends = (bits & kItemHit) != 0, by_ray = (bits & kItemRay) != 0;
      // the upstream gradients of the pair's pixel sit in the registers of the lane that owns it
      auto from_owner = [&](float v) {
        return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(qp << 2, __builtin_bit_cast(int, v)));
      };
      const float up_x = from_owner(dLp0), up_y = from_owner(dLp1), up_z = from_owner(dLp2);
      const float fx = qx0 + (float) (qp & 7), fy = qy0 + (float) (qp >> 3);
      const float w = it.x, GdA = it.y, dL_dz = it.z;
      // the same fused forms as the per-pixel test: for a surfel seen edge-on p_z is a small difference of large terms
      const float p0 = fmaf(hot.a[0], fx, fmaf(hot.a[1], fy, hot.a[2]));
      const float p1 = fmaf(hot.a[3], fx, fmaf(hot.a[4], fy, hot.a[5]));
      const float pz = fmaf(hot.a[6], fx, fmaf(hot.a[7], fy, hot.a[8]));
      const float rz_s = blends ? __builtin_amdgcn_rcpf(pz) : 0.0f;  // s is used by both cases of a blending pair
      const float rz_p = by_ray ? rz_s : 0.0f;                        // d/dp only by the intersection case
      const float sx = p0 * rz_s, sy = p1 * rz_s;
      const float oG = hot.opacity * GdA;
      float dsx = -(oG * sx), dsy = -(oG * sy);
      if (kAux) dsx += dL_dz * hot.tw0, dsy += dL_dz * hot.tw1;
      const float s_ds = dsx * sx + dsy * sy;
      const float da = dsx * rz_p, db = dsy * rz_p, dc = -(s_ds * rz_p);
      float g[16];
      g[0] = w * up_x, g[1] = w * up_y, g[2] = w * up_z;
      g[3] = da * fx, g[4] = da * fy, g[5] = da;
      g[6] = db * fx, g[7] = db * fy, g[8] = db;
      g[9] = dc * fx, g[10] = dc * fy, g[11] = dc;
      if (kAux) {
        g[12] = w * from_owner(dLn0), g[13] = w * from_owner(dLn1), g[14] = w * from_owner(dLn2);
      } else {
        g[12] = g[13] = g[14] = 0.0f;
      }
      g[15] = GdA;
      queue_accumulate(acc, before, row_sum16_transposed(g), jrows, n_valid, true);
      const bool filtered = blends && !by_ray;
      const float to_centre = filtered ? -2.0f * oG : 0.0f;
      if (kAux) {
        float g8[8];
        g8[0] = dL_dz * sx, g8[1] = dL_dz * sy, g8[2] = dL_dz;
        g8[3] = to_centre * (hot.cx - fx), g8[4] = to_centre * (hot.cy - fy);
        g8[5] = g8[6] = g8[7] = 0.0f;
        queue_accumulate(acc2, before2, row_sum8_transposed(g8), jrows, n_valid, second);
      } else if (wave_ballot(filtered) != 0ull) {  // some pair met its surfel by the projected centre
        float cx = to_centre * (hot.cx - fx), cy = to_centre * (hot.cy - fy);  // totals of a row end up in its lane 15
        cx += dpp_shift_zero<0x111, 0xf, 0xf>(cx), cy += dpp_shift_zero<0x111, 0xf, 0xf>(cy);
        cx += dpp_shift_zero<0x112, 0xf, 0xf>(cx), cy += dpp_shift_zero<0x112, 0xf, 0xf>(cy);
        cx += dpp_shift_zero<0x114, 0xf, 0xf>(cx), cy += dpp_shift_zero<0x114, 0xf, 0xf>(cy);
        cx += dpp_shift_zero<0x118, 0xf, 0xf>(cx), cy += dpp_shift_zero<0x118, 0xf, 0xf>(cy);
        if ((lane >> 4) < ((n_valid + 15) >> 4) && (lane & 15) == 15)
          atomicAdd(&s_part[wave][j][19], cx), atomicAdd(&s_part[wave][j][20], cy);
      }
      queue_pop(q, n_valid);
    };

    // one entry of the wavefront's work list; its records were requested from LDS while the entry before it ran
    auto blend_entry = [&](const FastHot& hot, const SplatCold& cold, int j) {
        const int pos = n_todo - 1 - (b * kB + j);
        FastHit h;
        unsigned long long pass;
        const bool hit = fast_intersect_flat(hot, pxf, pyf, near_n, h, &pass) && (pos < last_contrib);
        pass &= wave_ballot(pos < last_contrib);
        if (pass == 0ull) return;
        float w = 0.0f, dL_dalpha = 0.0f, dL_dz = 0.0f, fsx = 0.0f, fsy = 0.0f;
        if (kQueue) {
          if (hit) {
            advance_pixel(cold, j, pos, h, w, dL_dalpha, dL_dz, fsx, fsy);
            dL_dalpha *= h.G;  // only G * dL/dalpha is ever used
          }
          const int flags = h.rho3d <= h.rho2d ? (kItemHit | kItemRay) : kItemHit;
          if (queue_append(s_queue[wave], q, j, hit, pass, w, dL_dalpha, dL_dz, flags)) drain(kWave);
          return;
        }

        // One pass per entry (second set of transforms: its per-pair terms would double the queue's item). The part
        // under `hit` leaves a few factors (zero in a lane whose pixel does not blend the entry); the components are
        // products of those factors with quantities that are finite in every lane, formed by all lanes alike: no
        // component needs a zero of its own, and the projected-centre case is the intersection case with a zero in
        // place of 1 / p_z.
        float g[16], g8[8];
        float dsx = 0.0f, dsy = 0.0f, s_ds = 0.0f, z_sx = 0.0f, z_sy = 0.0f;
        if (hit) {
          advance_pixel(cold, j, pos, h, w, dL_dalpha, dL_dz, fsx, fsy);
          // d/ds of the intersection case (times 1 / p_z below); s is not finite in a lane whose p_z is 0, and such a
          // lane never blends: every use of s sits on this side
          const float dL_dG = hot.opacity * dL_dalpha;
          dsx  = fsx + dL_dG * -h.G * h.sx + dL_dz * hot.tw0;
          dsy  = fsy + dL_dG * -h.G * h.sy + dL_dz * hot.tw1;
          s_ds = dsx * h.sx + dsy * h.sy;
          z_sx = dL_dz * h.sx, z_sy = dL_dz * h.sy;
        }
        const bool by_ray   = h.rho3d <= h.rho2d;
        const bool filtered = hit && !by_ray;
        const float rz = (hit && by_ray) ? __builtin_amdgcn_rcpf(h.pz) : 0.0f;
        const float da = dsx * rz, db = dsy * rz, dc = -(s_ds * rz);
        g[0] = w * dLp0, g[1] = w * dLp1, g[2] = w * dLp2;
        g[3] = da * pxf, g[4] = da * pyf, g[5] = da;
        g[6] = db * pxf, g[7] = db * pyf, g[8] = db;
        g[9] = dc * pxf, g[10] = dc * pyf, g[11] = dc;
        if (kAux) g[12] = w * dLn0, g[13] = w * dLn1, g[14] = w * dLn2;
        else      g[12] = g[13] = g[14] = 0.0f;
        g[15] = h.G * dL_dalpha;
        const float to_centre = filtered ? hot.opacity * dL_dalpha * (-2.0f * h.G) : 0.0f;
        g8[0] = z_sx, g8[1] = z_sy, g8[2] = dL_dz;
        g8[3] = to_centre * h.dx, g8[4] = to_centre * h.dy;
        g8[5] = g8[6] = g8[7] = 0.0f;
        const float tot = wave_sum16_transposed(g);
        if (lane < 16) s_part[wave][j][lane] = tot;
        if (kAux) {
          const float tot8 = wave_sum8_transposed(g8);
          if (lane < 5) s_part[wave][j][16 + lane] = tot8;
        } else if (wave_ballot(filtered) != 0ull) {
          const float sx = wave_sum_to_lane63(g8[3]), sy = wave_sum_to_lane63(g8[4]);
          if (lane == 63) s_part[wave][j][19] = sx, s_part[wave][j][20] = sy;
        }
    };
    unsigned long long todo = __ballot(lane < n_here && ((s_mask[lane] >> wave) & 1u) &&
                                       (n_todo - 1 - (b * kB + lane)) < wave_max_contrib);
    if (todo != 0ull) {
      auto pop = [&]() {
        const int j = __builtin_ctzll(todo);
        todo &= todo - 1;
        return j;
      };
      auto peek = [&]() { return todo ? (int) __builtin_ctzll(todo) : 0; };
      FastHot hot_a = s_hot[peek()], hot_b;
      while (todo) {
        {
          const int j = pop();
          hot_b       = s_hot[peek()];
          const SplatCold cold = s_cold[j];
          __builtin_amdgcn_sched_barrier(0);
          blend_entry(hot_a, cold, j);
        }
        if (todo == 0ull) break;
        {
          const int j = pop();
          hot_a       = s_hot[peek()];
          const SplatCold cold = s_cold[j];
          __builtin_amdgcn_sched_barrier(0);
          blend_entry(hot_b, cold, j);
        }
      }
      if (kQueue && q.count > 0) drain(q.count);  // the staged records are replaced after the next barrier
    }
    __syncthreads();
    if ((int) threadIdx.x < n_here) {
      const int id = s_cold[threadIdx.x].id;
      float a[kFastGradSlots];
#pragma unroll
      for (int c = 0; c < kFastGradSlots; ++c) {
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) sum += s_part[w][threadIdx.x][c], s_part[w][threadIdx.x][c] = 0.0f;
        a[c] = sum;
      }
      if (kSlots) {
        float2* dst = (float2*) (slot_records + slot * kFastRecordSlots);
#pragma unroll
        for (int c = 0; c < kFastRecordSlots / 2; ++c)
          dst[c] = make_float2(a[2 * c], 2 * c + 1 < kFastGradSlots ? a[2 * c + 1] : 0.0f);
      } else {
#pragma unroll
        for (int c = 0; c < 3; ++c)
          if (a[c] != 0.0f) atomicAdd(&g_colors[3 * (size_t) id + c], a[c]);
#pragma unroll
        for (int c = 0; c < 9; ++c)
          if (a[3 + c] != 0.0f) atomicAdd(&g_inv[9 * (size_t) id + c], a[3 + c]);
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (a[12 + c] != 0.0f) atomicAdd(&g_normal_opacity[4 * (size_t) id + c], a[12 + c]);
#pragma unroll
        for (int c = 0; c < 3; ++c)
          if (a[16 + c] != 0.0f) atomicAdd(&g_trans[9 * (size_t) id + 6 + c], a[16 + c]);
#pragma unroll
        for (int c = 0; c < 2; ++c)
          if (a[19 + c] != 0.0f) atomicAdd(&g_means2D[2 * (size_t) id + c], a[19 + c]);
      }
    }
  }
}


// The reference's second backward (gs_2d_fast_redner.cu:563-837), the per-splat decomposition itself: a lane owns ONE
// list entry of a tile and keeps that surfel's 21 gradient sums in registers, the tile's pixels pass through the lanes
// one lane per step, front to back, each carrying its blending state from the forward's snapshot in front of the
// bucket on. Where the reference hands 27 values from lane to lane (transmittance, three colour and eight auxiliary
// partial sums, the upstream gradients and counters of the pixel), here two travel: the transmittance T and
//   S = <dL/d(outputs), partial sums - final outputs> + T_final dL/dopacity,
// because dL/dalpha = T c + S / (1 - alpha) with c = <dL/d(outputs), this pair's channel values> only needs the partial
// sums through that one product (S += w c per blended pair); the per-pixel constants are staged in LDS once and read
// by pixel number. Laid out for a 64-lane wavefront as the 3D-Gaussian form of this decomposition: one wavefront takes
// 64 consecutive entries = two of the forward's 32-entry buckets (the wavefront of the odd bucket leaves at once), the
// state moves with one whole-wavefront DPP shift per value, and only the pixels that still blend at the group's first
// entry are fed in. Channel set of the reference's kernel: image, opacity, depth, normal, median depth, M1, M2 (no
// distortion; the depth gradient through M1 is dropped as there, :751-757).
template <bool kAux, bool kSlots>
__global__ void __launch_bounds__(64) fast_bucket_backward_kernel(int W, int H, float near_n, float far_n,
    const int64_t* __restrict__ ranges, const int32_t* __restrict__ point_list, const float2* __restrict__ means2D,
    const float4* __restrict__ normal_opacity, const float* __restrict__ colors, const float* __restrict__ trans_mat,
    const float* __restrict__ inverse_m, const float* __restrict__ images, const float* __restrict__ out_opacity,
    const float* __restrict__ out_extras, const int32_t* __restrict__ n_contrib,
    const int32_t* __restrict__ max_contrib, const int64_t* __restrict__ bucket_offset,
    const int32_t* __restrict__ bucket_to_tile, const float* __restrict__ sampled_T,
    const float* __restrict__ sampled_acc, const float* __restrict__ sampled_aux, const float* __restrict__ dL_dpix,
    const float* __restrict__ dL_dextras, const float* __restrict__ dL_dopacity, float* __restrict__ g_means2D,
    float* __restrict__ g_normal_opacity, float* __restrict__ g_colors, float* __restrict__ g_trans,
    float* __restrict__ g_inv, const int64_t* __restrict__ point_offsets, const int32_t* __restrict__ radii,
    float* __restrict__ slot_records) {
  __shared__ float4 s_up[256];                // dL/d(r, g, b) | dL/ddepth
  __shared__ float4 s_up2[kAux ? 256 : 1];    // dL/dnormal | dL/dM1
  __shared__ float4 s_up3[kAux ? 256 : 1];    // dL/dM2 | dL/d(median depth) | median contributor (int bits) | -
  __shared__ float4 s_pixel[256];             // x | y | last contributor (int bits) | -
  __shared__ float2 s_state[256];             // snapshot: T | S
  const int bucket = blockIdx.x, lane = threadIdx.x;
  const int tile = bucket_to_tile[bucket];
  const int in_tile = bucket - (int) (tile == 0 ? 0 : bucket_offset[tile - 1]);
  if (in_tile & 1) return;
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const int tile_x = tile % gx, tile_y = tile / gx;
  const int64_t r0 = ranges[2 * (size_t) tile], r1 = ranges[2 * (size_t) tile + 1];
  const int first = in_tile * 32, entry = first + lane;
  const bool valid = entry < (int) (r1 - r0);
  const size_t HW = (size_t) H * W;
  const float far_scale = far_n / (far_n - near_n), far_near = far_scale * near_n;

  FastHot hot{};
  SplatCold cold{};
  size_t slot = 0;
  if (valid) {
    const FastSplat g = gather_fast(point_list[r0 + entry], means2D, colors, normal_opacity, trans_mat, inverse_m);
    hot = g.hot, cold = g.cold;
    if (kSlots) {
      const TileRect r = tile_rect(hot.cx, hot.cy, radii[cold.id], gx, gy);
      slot = (size_t) ((cold.id == 0 ? 0 : point_offsets[cold.id - 1]) + (int64_t) (tile_x - r.x0) * (r.y1 - r.y0) +
                       (tile_y - r.y0));
    }
  }

  // the pixels that still blend at this group's first entry, in row-major order of the tile
  int n_live = 0;
  if (first < max_contrib[tile]) {
#pragma unroll
    for (int part = 0; part < 4; ++part) {
      const int rank = part * 64 + lane;
      const int px = tile_x * kTile + (rank & 15), py = tile_y * kTile + (rank >> 4);
      const bool inside = px < W && py < H;
      const size_t pix = (size_t) W * py + px;
      const int last = inside ? n_contrib[pix] : 0;
      const bool live = last > first;
      const unsigned long long live_lanes = wave_ballot(live);
      if (live) {
        const int at = n_live + __builtin_amdgcn_mbcnt_hi((unsigned) (live_lanes >> 32),
                                                          __builtin_amdgcn_mbcnt_lo((unsigned) live_lanes, 0u));
        const size_t snap = (size_t) bucket * 256 + rank;
        const float up0 = dL_dpix[pix], up1 = dL_dpix[HW + pix], up2 = dL_dpix[2 * HW + pix];
        float S = (1.0f - out_opacity[pix]) * dL_dopacity[pix];
        S += up0 * (sampled_acc[((size_t) bucket * 3 + 0) * 256 + rank] - images[pix]);
        S += up1 * (sampled_acc[((size_t) bucket * 3 + 1) * 256 + rank] - images[HW + pix]);
        S += up2 * (sampled_acc[((size_t) bucket * 3 + 2) * 256 + rank] - images[2 * HW + pix]);
        float up_depth = 0.0f;
        if (kAux) {
          auto behind = [&](int c) { return sampled_aux[((size_t) bucket * 8 + c) * 256 + rank] - out_extras[c * HW + pix]; };
          up_depth = dL_dextras[pix];
          const float n0 = dL_dextras[1 * HW + pix], n1 = dL_dextras[2 * HW + pix], n2 = dL_dextras[3 * HW + pix];
          const float m1 = dL_dextras[6 * HW + pix], m2 = dL_dextras[7 * HW + pix];
          S += up_depth * behind(0) + n0 * behind(1) + n1 * behind(2) + n2 * behind(3) + m1 * behind(6) + m2 * behind(7);
          s_up2[at] = make_float4(n0, n1, n2, m1);
          s_up3[at] = make_float4(m2, dL_dextras[4 * HW + pix], __int_as_float(n_contrib[HW + pix]), 0.0f);
        }
        s_up[at]    = make_float4(up0, up1, up2, up_depth);
        s_state[at] = make_float2(sampled_T[snap], S);
        s_pixel[at] = make_float4((float) px, (float) py, __int_as_float(last), 0.0f);
      }
      n_live += __builtin_popcountll(live_lanes);
    }
  }
  __syncthreads();

  float g[kFastGradSlots];
#pragma unroll
  for (int c = 0; c < kFastGradSlots; ++c) g[c] = 0.0f;
  float T = 0.0f, S = 0.0f;
  // whole-wavefront shift by one lane (DPP wave_shr:1); lane 0 keeps `fresh`
  auto pass_on = [](float fresh, float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, fresh),
                                                                 __builtin_bit_cast(int, v), 0x138, 0xf, 0xf, false));
  };
  const int steps = n_live > 0 ? n_live + 63 : 0;
  float2 next_state = s_state[0];
  for (int i = 0; i < steps; ++i) {
    const float2 fresh = next_state;
    next_state = s_state[min(i + 1, n_live - 1)];  // requested a step ahead of its use (nothing new once all have entered)
    T = pass_on(fresh.x, T);
    S = pass_on(fresh.y, S);
    const int q = i - lane;
    if (q < 0 || q >= n_live) continue;
    const float4 pixel = s_pixel[q];
    FastHit h;
    const bool hit = fast_intersect_flat(hot, pixel.x, pixel.y, near_n, h) && valid && entry < __float_as_int(pixel.z);
    if (!hit) continue;
    const float4 up = s_up[q];
    const float w = h.alpha * T, inv = __builtin_amdgcn_rcpf(1.0f - h.alpha);
    float c_lin = cold.r * up.x + cold.g * up.y + cold.b * up.z;
    float dL_dz = 0.0f;
    if (kAux) {
      const float4 upn = s_up2[q], upm = s_up3[q];
      const float rd     = __builtin_amdgcn_rcpf(h.depth);
      const float m_d    = far_scale - far_near * rd;
      const float dmd_dd = far_near * rd * rd;
      c_lin += h.depth * up.w + cold.nx * upn.x + cold.ny * upn.y + cold.nz * upn.z + m_d * upn.w + (m_d * m_d) * upm.x;
      dL_dz = w * up.w + dmd_dd * (2.0f * m_d * w * upm.x);
      if (entry == __float_as_int(upm.z) - 1) dL_dz += upm.y;
      g[12] += w * upn.x, g[13] += w * upn.y, g[14] += w * upn.z;
    }
    S += w * c_lin;  // the partial sums up to and including this pair, minus the final outputs
    const float dL_dalpha = T * c_lin + inv * S;
    T *= 1.0f - h.alpha;
    const float GdA = h.G * dL_dalpha, oG = hot.opacity * GdA;
    const bool by_ray = h.rho3d <= h.rho2d;
    const float rz = by_ray ? __builtin_amdgcn_rcpf(h.pz) : 0.0f;
    const float dsx = dL_dz * hot.tw0 - oG * h.sx, dsy = dL_dz * hot.tw1 - oG * h.sy;
    const float da = dsx * rz, db = dsy * rz, dc = -(da * h.sx + db * h.sy);
    g[0] += w * up.x, g[1] += w * up.y, g[2] += w * up.z;
    g[3] += da * pixel.x, g[4] += da * pixel.y, g[5] += da;
    g[6] += db * pixel.x, g[7] += db * pixel.y, g[8] += db;
    g[9] += dc * pixel.x, g[10] += dc * pixel.y, g[11] += dc;
    g[15] += GdA;
    g[16] += dL_dz * h.sx, g[17] += dL_dz * h.sy, g[18] += dL_dz;
    const float to_centre = by_ray ? 0.0f : -2.0f * oG;
    g[19] += to_centre * h.dx, g[20] += to_centre * h.dy;
  }
  if (!valid) return;
  if (kSlots) {  // every list entry has a lane in some wavefront of this launch: all records are written, zeros included
    float2* dst = (float2*) (slot_records + slot * kFastRecordSlots);
#pragma unroll
    for (int c = 0; c < kFastRecordSlots / 2; ++c)
      dst[c] = make_float2(g[2 * c], 2 * c + 1 < kFastGradSlots ? g[2 * c + 1] : 0.0f);
  } else {
    const int id = cold.id;
#pragma unroll
    for (int c = 0; c < 3; ++c)
      if (g[c] != 0.0f) atomicAdd(&g_colors[3 * (size_t) id + c], g[c]);
#pragma unroll
    for (int c = 0; c < 9; ++c)
      if (g[3 + c] != 0.0f) atomicAdd(&g_inv[9 * (size_t) id + c], g[3 + c]);
#pragma unroll
    for (int c = 0; c < 4; ++c)
      if (g[12 + c] != 0.0f) atomicAdd(&g_normal_opacity[4 * (size_t) id + c], g[12 + c]);
#pragma unroll
    for (int c = 0; c < 3; ++c)
      if (g[16 + c] != 0.0f) atomicAdd(&g_trans[9 * (size_t) id + 6 + c], g[16 + c]);
#pragma unroll
    for (int c = 0; c < 2; ++c)
      if (g[19 + c] != 0.0f) atomicAdd(&g_means2D[2 * (size_t) id + c], g[19 + c]);
  }
}

void launch_fast_slot_sum(int P, int gx, int gy, const int64_t* point_offsets, const int32_t* radii,
                          const float* means2D, const float* inverse_m, const float* normal_opacity,
                          const uint32_t* keep_masks, const SlotWorkspace& ws, FastScatter out, hipStream_t s) {
  constexpr int kPerWave = 64 / (kFastRecordSlots / 2);
  const int64_t waves = div_up(P, kPerWave);
  hipLaunchKernelGGL(fast_slot_sum_kernel, dim3((unsigned) div_up(waves * 64, 256)), dim3(256), 0, s, P, gx, gy,
                     point_offsets, radii, (const float2*) means2D, inverse_m, (const float4*) normal_opacity,
                     keep_masks, ws.records, out);
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API int fsgs_gs_2d_fast_render_forward(int P, int W, int H, double near_n, double far_n, int only_image,
    const float* means2D, const float* colors, const float* normal_opacity, const float* trans_mat,
    const float* inverse_m, const int32_t* point_list, const int64_t* ranges, const float* trans_mat_t2,
    int32_t* accum_max_count, float* accum_weights_p, int32_t* accum_weights_count, const int64_t* bucket_offset,
    float* out_color, float* out_opacity, float* out_extras, float* out_flow, int32_t* n_contrib,
    int32_t* max_contrib, int32_t* bucket_to_tile, float* sampled_T, float* sampled_acc, float* sampled_aux,
    void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0, "GS_2D_fast_render_forward: bad sizes");
  FSGS_REQUIRE(ranges && out_color && out_opacity && n_contrib, "GS_2D_fast_render_forward: null pointer");
  FSGS_REQUIRE(P == 0 || (means2D && colors && normal_opacity && trans_mat && inverse_m),
               "GS_2D_fast_render_forward: null surfel tensor");
  FSGS_REQUIRE(only_image || out_extras, "GS_2D_fast_render_forward: out_extras is required unless only_image");
  const bool aux   = !only_image;
  const bool snap  = aux && bucket_offset != nullptr;
  const bool accum = aux && (accum_max_count || accum_weights_p || accum_weights_count);
  const bool flow  = aux && trans_mat_t2 != nullptr;
  FSGS_REQUIRE(!flow || out_flow, "GS_2D_fast_render_forward: out_flow is required with trans_mat_t2");
  FSGS_REQUIRE(!snap || (max_contrib && bucket_to_tile && sampled_T && sampled_acc && sampled_aux),
               "GS_2D_fast_render_forward: snapshot outputs are required with per_tile_bucket_offset");
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const dim3 grid(gx * gy), block(kBlendThreads);
  hipStream_t s = (hipStream_t) stream;
  const int* tile_order = nullptr;
  const int ordered = launch_tile_order(gx, gy, ranges, s, &tile_order);
#define FSGS_LAUNCH_FWD(AUX, SNAP, ACC, FLOW)                                                                        \
  hipLaunchKernelGGL((fast_blend_forward_kernel<AUX, SNAP, ACC, FLOW>), grid, block, 0, s, ordered, tile_order, W, H,            \
                     (float) near_n, (float) far_n, ranges, point_list, (const float2*) means2D, colors, trans_mat,  \
                     inverse_m, (const float4*) normal_opacity, trans_mat_t2, bucket_offset, n_contrib, out_color,   \
                     out_opacity, out_extras, (float2*) out_flow, max_contrib, bucket_to_tile, sampled_T,            \
                     sampled_acc, sampled_aux, accum_max_count, accum_weights_p, accum_weights_count)
#define FSGS_LAUNCH_FWD_F(AUX, SNAP, ACC) \
  do { if (flow) FSGS_LAUNCH_FWD(AUX, SNAP, ACC, true); else FSGS_LAUNCH_FWD(AUX, SNAP, ACC, false); } while (0)
  if (!aux) FSGS_LAUNCH_FWD(false, false, false, false);
  else if (snap && accum) FSGS_LAUNCH_FWD_F(true, true, true);
  else if (snap) FSGS_LAUNCH_FWD_F(true, true, false);
  else if (accum) FSGS_LAUNCH_FWD_F(true, false, true);
  else FSGS_LAUNCH_FWD_F(true, false, false);
#undef FSGS_LAUNCH_FWD_F
#undef FSGS_LAUNCH_FWD
  return check_launch("GS_2D_fast_render_forward");
}

FSGS_API size_t fsgs_gs_2d_fast_render_backward_workspace_bytes(int64_t R) {
  return slot_workspace_bytes(R, kFastRecordSlots);
}

FSGS_API int fsgs_gs_2d_fast_render_backward(int P, int W, int H, double near_n, double far_n, int per_splat_form,
    const float* means2D, const float* normal_opacity, const float* colors, const float* trans_mat,
    const float* inverse_m, const float* trans_mat_t2, const float* out_opacity, const float* out_extras,
    const float* out_flow, const float* dL_dpix, const float* dL_dopacity, const float* dL_dextras,
    const float* dL_dflow, const int64_t* ranges, const int32_t* point_list, const int32_t* n_contrib,
    float* g_colors, float* g_means2D, float* g_trans, float* g_inv, float* g_normal_opacity, int64_t R,
    const int64_t* point_offsets, const int32_t* radii, void* workspace, size_t workspace_bytes,
    const uint32_t* keep_masks, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0, "GS_2D_fast_render_backward: bad sizes");
  if (P == 0) return kOk;
  FSGS_REQUIRE(means2D && normal_opacity && colors && trans_mat && inverse_m && out_opacity && dL_dpix && dL_dopacity &&
                   ranges && n_contrib && g_colors && g_means2D && g_trans && g_inv && g_normal_opacity,
               "GS_2D_fast_render_backward: null pointer");
  const bool aux  = out_extras && dL_dextras;
  const bool flow = dL_dflow != nullptr;
  FSGS_REQUIRE(!flow || (aux && trans_mat_t2 && out_flow),
               "GS_2D_fast_render_backward: flow gradients need trans_mat2, out_flows and the auxiliary maps");
  const bool slots = point_offsets != nullptr;
  SlotWorkspace ws{nullptr};
  if (slots) {
    FSGS_REQUIRE(radii && workspace && R >= 0 && R < (int64_t) 0x7fffffff,
                 "GS_2D_fast_render_backward: the ordered-sum path needs radii, a workspace and the instance count R");
    if (workspace_bytes < slot_workspace_bytes(R, kFastRecordSlots))
      return fail(kWorkspaceSmall, "GS_2D_fast_render_backward: workspace %zu < %zu bytes", workspace_bytes,
                  slot_workspace_bytes(R, kFastRecordSlots));
    FSGS_REQUIRE(((uintptr_t) workspace & 15) == 0, "GS_2D_fast_render_backward: workspace must be 16-byte aligned");
    ws = slot_workspace(workspace, R, kFastRecordSlots);
  }
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const dim3 grid(gx * gy), block(kBlendThreads);
  hipStream_t s = (hipStream_t) stream;
  const int* tile_order = nullptr;
  const int ordered = launch_tile_order(gx, gy, ranges, s, &tile_order);
#define FSGS_LAUNCH_BWD_S(AUX, SPLAT, FLOW, SL)                                                                      \
  hipLaunchKernelGGL((fast_blend_backward_kernel<AUX, SPLAT, FLOW, SL>), grid, block, 0, s, ordered, tile_order, W, H, \
                     (float) near_n, (float) far_n, ranges, point_list, n_contrib, (const float2*) means2D,          \
                     (const float4*) normal_opacity, colors, trans_mat, inverse_m, trans_mat_t2, out_opacity,        \
                     out_extras, (const float2*) out_flow, dL_dpix, dL_dextras, dL_dopacity,                         \
                     (const float2*) dL_dflow, g_means2D, g_normal_opacity, g_colors, g_trans, g_inv, point_offsets, \
                     radii, ws.records)
#define FSGS_LAUNCH_BWD(AUX, SPLAT, FLOW) \
  do { if (slots) FSGS_LAUNCH_BWD_S(AUX, SPLAT, FLOW, true); else FSGS_LAUNCH_BWD_S(AUX, SPLAT, FLOW, false); } while (0)
  if (aux && per_splat_form && flow) FSGS_LAUNCH_BWD(true, true, true);
  else if (aux && flow) FSGS_LAUNCH_BWD(true, false, true);
  else if (aux && per_splat_form) FSGS_LAUNCH_BWD(true, true, false);
  else if (aux) FSGS_LAUNCH_BWD(true, false, false);
  else if (per_splat_form) FSGS_LAUNCH_BWD(false, true, false);
  else FSGS_LAUNCH_BWD(false, false, false);
#undef FSGS_LAUNCH_BWD
#undef FSGS_LAUNCH_BWD_S
  if (slots)
    launch_fast_slot_sum(P, gx, gy, point_offsets, radii, means2D, inverse_m, normal_opacity, keep_masks, ws,
                         FastScatter{g_means2D, g_normal_opacity, g_colors, g_trans, g_inv}, s);
  return check_launch("GS_2D_fast_render_backward");
}

// The per-splat decomposition itself (fast_bucket_backward_kernel), for callers that want the reference's second
// algorithm rather than its result: B = the number of 32-entry buckets the forward announced (bucket_to_tile's length).
FSGS_API int fsgs_gs_2d_fast_render_bucket_backward(int P, int W, int H, double near_n, double far_n, int B,
    const float* means2D, const float* normal_opacity, const float* colors, const float* trans_mat,
    const float* inverse_m, const float* images, const float* out_opacity, const float* out_extras,
    const int32_t* n_contrib, const int32_t* max_contrib, const int64_t* bucket_offset,
    const int32_t* bucket_to_tile, const float* sampled_T, const float* sampled_acc, const float* sampled_aux,
    const float* dL_dpix, const float* dL_dopacity, const float* dL_dextras, const int64_t* ranges,
    const int32_t* point_list, float* g_colors, float* g_means2D, float* g_trans, float* g_inv,
    float* g_normal_opacity, int64_t R, const int64_t* point_offsets, const int32_t* radii, void* workspace,
    size_t workspace_bytes, const uint32_t* keep_masks, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0 && B >= 0, "GS_2D_fast_render_bucket_backward: bad sizes");
  if (P == 0) return kOk;
  FSGS_REQUIRE(means2D && normal_opacity && colors && trans_mat && inverse_m && images && out_opacity && n_contrib &&
                   max_contrib && bucket_offset && dL_dpix && dL_dopacity && ranges && g_colors && g_means2D &&
                   g_trans && g_inv && g_normal_opacity &&
                   (B == 0 || (bucket_to_tile && point_list && sampled_T && sampled_acc)),
               "GS_2D_fast_render_bucket_backward: null pointer");
  const bool aux = out_extras && dL_dextras;
  FSGS_REQUIRE(!aux || B == 0 || sampled_aux,
               "GS_2D_fast_render_bucket_backward: the auxiliary maps need their snapshots");
  const bool slots = point_offsets != nullptr;
  SlotWorkspace ws{nullptr};
  if (slots) {
    FSGS_REQUIRE(radii && workspace && R >= 0 && R < (int64_t) 0x7fffffff,
                 "GS_2D_fast_render_bucket_backward: the ordered-sum path needs radii, a workspace and the instance count R");
    if (workspace_bytes < slot_workspace_bytes(R, kFastRecordSlots))
      return fail(kWorkspaceSmall, "GS_2D_fast_render_bucket_backward: workspace %zu < %zu bytes", workspace_bytes,
                  slot_workspace_bytes(R, kFastRecordSlots));
    FSGS_REQUIRE(((uintptr_t) workspace & 15) == 0, "GS_2D_fast_render_bucket_backward: workspace must be 16-byte aligned");
    ws = slot_workspace(workspace, R, kFastRecordSlots);
  }
  hipStream_t s = (hipStream_t) stream;
#define FSGS_FAST_BKT(AUX, SL)                                                                                        \
  hipLaunchKernelGGL((fast_bucket_backward_kernel<AUX, SL>), dim3(B), dim3(64), 0, s, W, H, (float) near_n,           \
                     (float) far_n, ranges, point_list, (const float2*) means2D, (const float4*) normal_opacity,      \
                     colors, trans_mat, inverse_m, images, out_opacity, out_extras, n_contrib, max_contrib,           \
                     bucket_offset, bucket_to_tile, sampled_T, sampled_acc, sampled_aux, dL_dpix, dL_dextras,         \
                     dL_dopacity, g_means2D, g_normal_opacity, g_colors, g_trans, g_inv, point_offsets, radii,        \
                     ws.records)
  if (B > 0) {
    if (aux && slots) FSGS_FAST_BKT(true, true);
    else if (aux) FSGS_FAST_BKT(true, false);
    else if (slots) FSGS_FAST_BKT(false, true);
    else FSGS_FAST_BKT(false, false);
  }
#undef FSGS_FAST_BKT
  if (slots)
    launch_fast_slot_sum(P, (W + kTile - 1) / kTile, (H + kTile - 1) / kTile, point_offsets, radii, means2D, inverse_m,
                         normal_opacity, keep_masks, ws,
                         FastScatter{g_means2D, g_normal_opacity, g_colors, g_trans, g_inv}, s);
  return check_launch("GS_2D_fast_render_bucket_backward");
}
