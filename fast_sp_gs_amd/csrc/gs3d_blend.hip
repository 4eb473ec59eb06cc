// Per-tile alpha blend of 3D Gaussians (conic footprint) and its backward, for gfx950.
//
// Reference behaviour reproduced: fast_2d_gs/_C/src/gaussian_splatting/gaussian_render.cu:20-173 (forward kernel; host
// gaussian_rasterize_forward :212-293) and :296-444 (backward kernel; host gaussian_rasterize_backward :486-536):
// alpha = min(0.99, o * exp(-0.5 (a dx^2 + c dy^2) - b dx dy)) with d = mean - pixel, skipped when the exponent is
// positive or alpha < 1/255, front-to-back blending until T * (1 - alpha) < 1e-4; 3 colour channels plus up to 4 extra
// per-Gaussian feature channels; optional accum_max_count / accum_weights_p / accum_weights_count. The backward walks
// each tile's list back to front, rebuilding T by division, with the reference's accumulators
// (sum of c * alpha * T behind the current Gaussian) and without masking the 0.99 clamp.
//
// Same skeleton as the surfel blend: one block = one 16x16 tile = 4 wavefronts x 8x8 quadrant, a batch of Gaussians
// staged in LDS with the next batch's gather in flight, a conservative per-quadrant footprint test (bounding box of the
// alpha >= 1/255 ellipse) whose ballot is the wavefront's work list, longest lists scheduled first. Where the
// reference issues 9 + E global float atomics per (pixel, Gaussian) pair, the backward sums the 9 + E gradient
// components over the 64 pixels of a wavefront with one transposed DPP butterfly, stores each wavefront's partial in
// its own LDS row (LDS float atomics cost about three cycles per lane here), adds the four rows in wavefront order and
// flushes one global atomic per Gaussian, component and tile.
#include "blend.hpp"
#include "ordered_sums.hpp"

namespace fsgs {
namespace {

constexpr int kG3Batch = 128;   // Gaussians staged per round
constexpr int kMaxExtra = 4;    // the reference dispatches E = 0..4 (gaussian_render.cu:455-481)

struct __attribute__((aligned(16))) G3Hot {
  float x, y;       // screen-space mean
  float a, b, c;    // conic
  float opacity;
  int id;
  unsigned mask;    // 8x8 quadrants of the tile the alpha >= 1/255 ellipse can reach
};

struct G3Entry {
  G3Hot hot;
  float feat[3 + kMaxExtra];
};

template <int E>
__device__ __forceinline__ G3Entry gather_gaussian(int id, const float2* __restrict__ means2D,
    const float4* __restrict__ conic_opacity, const float* __restrict__ colors, const float* __restrict__ extras) {
  G3Entry g;
  const float2 m = means2D[id];
  const float4 co = conic_opacity[id];
  g.hot.x = m.x, g.hot.y = m.y, g.hot.a = co.x, g.hot.b = co.y, g.hot.c = co.z, g.hot.opacity = co.w;
  g.hot.id = id, g.hot.mask = 0xfu;
#pragma unroll
  for (int k = 0; k < 3; ++k) g.feat[k] = colors[3 * (size_t) id + k];
#pragma unroll
  for (int k = 0; k < E; ++k) g.feat[3 + k] = extras[(size_t) E * id + k];
  return g;
}

// alpha >= 1/255 needs 0.5 d^T Q d <= tau = ln(255 o) with Q = [[a, b], [b, c]]: for a positive definite Q that is an
// ellipse with half extents sqrt(2 tau c / det), sqrt(2 tau a / det). Anything else (o < 1/255: never; Q not positive
// definite: unbounded) is decided without a box.
__device__ __forceinline__ unsigned conic_quadrant_mask(const G3Hot& h, int tile_px, int tile_py, int flags) {
  if (flags & kFlagNoCull) return 0xfu;
  const float oa = 255.0f * h.opacity;
  if (!(oa >= 1.0f)) return 0u;
  const float det = h.a * h.c - h.b * h.b;
  if (!(det > 0.0f) || !(h.a > 0.0f)) return 0xfu;
  const float tau2 = 2.0f * (__logf(oa) * 1.0001f + 1e-3f);
  const float ex = sqrtf(tau2 * h.c / det), ey = sqrtf(tau2 * h.a / det);
  if (!(ex == ex) || !(ey == ey)) return 0xfu;
  const float padx = kCullPad + 0.01f * ex, pady = kCullPad + 0.01f * ey;
  const float x0 = h.x - ex - padx, x1 = h.x + ex + padx, y0 = h.y - ey - pady, y1 = h.y + ey + pady;
  unsigned m = 0u;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float qx = (float) (tile_px + (q & 1) * 8), qy = (float) (tile_py + (q >> 1) * 8);
    if (x1 >= qx && x0 <= qx + 7.0f && y1 >= qy && y0 <= qy + 7.0f) m |= 1u << q;
  }
  return m;
}

struct G3Hit {
  float dx, dy, G, alpha;
};

// Alpha of one Gaussian at one pixel (gaussian_render.cu:118-130); false where the reference would `continue`. No early
// exit, and every fused multiply-add is written out with contraction off: a kernel that inlines this twice gets the
// same rounding from both copies.
// `lanes`, if given: mask of the lanes that pass, from the two comparisons' own lane masks (scalar registers).
__device__ __forceinline__ bool conic_alpha_flat(const G3Hot& h, float pxf, float pyf, G3Hit& o,
                                                 unsigned long long* lanes = nullptr) {
#pragma clang fp contract(off)
  o.dx = h.x - pxf, o.dy = h.y - pyf;
  const float power = fmaf(-0.5f, fmaf(h.a * o.dx, o.dx, h.c * o.dy * o.dy), -(h.b * o.dx * o.dy));
  o.G     = __expf(power);
  o.alpha = fminf(0.99f, h.opacity * o.G);
  const bool c0 = !(power > 0.0f), c1 = !(o.alpha < (1.0f / 255.0f));
  if (lanes) *lanes = wave_ballot(c0) & wave_ballot(c1);
  return c0 & c1;
}

// kSnap (gaussian_render.cu:51-63, :100-106, :168-172): the state of every pixel still blending before each 32nd list
// entry -- sampled_T[B,256], sampled_ar[B,3+E,256] by row-major position inside the tile -- plus bucket_to_tile[B] and
// the tile's deepest contributor max_contrib[T], which the per-Gaussian backward of the reference consumes.
template <int E, bool kAccum, bool kSnap>
__global__ void __launch_bounds__(kBlendThreads) gs3d_forward_kernel(int flags, const int* __restrict__ tile_order, int W, int H,
    const int64_t* __restrict__ ranges, const int32_t* __restrict__ point_list, const float2* __restrict__ means2D,
    const float4* __restrict__ conic_opacity, const float* __restrict__ colors, const float* __restrict__ extras,
    float* __restrict__ out_color, float* __restrict__ out_opacity, float* __restrict__ out_extras,
    int32_t* __restrict__ n_contrib, int32_t* __restrict__ accum_max_count, float* __restrict__ accum_weights_p,
    int32_t* __restrict__ accum_weights_count, const int64_t* __restrict__ bucket_offset,
    int32_t* __restrict__ max_contrib, int32_t* __restrict__ bucket_to_tile, float* __restrict__ sampled_T,
    float* __restrict__ sampled_ar) {
  __shared__ G3Hot s_hot[kG3Batch];
  __shared__ float s_feat[kG3Batch][3 + kMaxExtra + 1];  // odd stride
  __shared__ int s_max_contrib;
  const int gx = (W + kTile - 1) / kTile;
  const int tile = scheduled_tile(flags, tile_order), tile_x = tile % gx, tile_y = tile / gx;
  int px, py;
  lane_pixel(tile_x, tile_y, px, py);
  const bool inside = px < W && py < H;
  const size_t HW = (size_t) H * W, pix = (size_t) W * py + px;
  const float pxf = (float) px, pyf = (float) py;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t r0 = ranges[2 * (size_t) tile], r1 = ranges[2 * (size_t) tile + 1];
  const int n_todo = (int) (r1 - r0);
  const int rounds = (n_todo + kG3Batch - 1) / kG3Batch;
  const int rank = (py - tile_y * kTile) * kTile + (px - tile_x * kTile);  // row-major position inside the tile
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
  float T = 1.0f, C[3 + (E > 0 ? E : 1)];
#pragma unroll
  for (int k = 0; k < 3 + E; ++k) C[k] = 0.0f;
  int last = 0, wmax_id = -1;
  float wmax = 0.0f;
  bool flag = false;

  G3Entry next;
  if ((int) threadIdx.x < min(n_todo, kG3Batch))
    next = gather_gaussian<E>(point_list[r0 + threadIdx.x], means2D, conic_opacity, colors, extras);
  for (int b = 0; b < rounds; ++b) {
    if (__syncthreads_count(live < 0.0f) == kBlendThreads) break;
    const int n_here = min(kG3Batch, n_todo - b * kG3Batch);
    if ((int) threadIdx.x < n_here) {
      next.hot.mask = conic_quadrant_mask(next.hot, tile_x * kTile, tile_y * kTile, flags);
      s_hot[threadIdx.x] = next.hot;
#pragma unroll
      for (int k = 0; k < 3 + E; ++k) s_feat[threadIdx.x][k] = next.feat[k];
    }
    __syncthreads();
    const int nxt = (b + 1) * kG3Batch + (int) threadIdx.x;
    if ((int) threadIdx.x < kG3Batch && nxt < n_todo)
      next = gather_gaussian<E>(point_list[r0 + nxt], means2D, conic_opacity, colors, extras);
    for (int c = 0; c < kG3Batch / kWave; ++c) {
      const int jj = c * kWave + lane;
      unsigned long long todo = __ballot(jj < n_here && ((s_hot[jj < kG3Batch ? jj : 0].mask >> wave) & 1u));
      if (!kSnap && todo == 0ull) continue;  // with snapshots the state is stored even where nothing blends
      // One list entry. A wavefront walks its list alone and the launch lasts as long as its longest tile, so the next
      // entry's record is requested before the current one is evaluated (alternating registers) and the blend is one
      // divergent region behind one predicate.
      auto blend_entry = [&](const G3Hot& hot, int j) {
#pragma clang fp contract(off)  // two copies of this body exist: both must round alike
        G3Hit h;
        unsigned long long pass;
        const bool hit = conic_alpha_flat(hot, pxf, pyf, h, &pass) && live > 0.0f;
        pass &= live_lanes;
        if (pass == 0ull) return;
        const float test_T = T * (1.0f - h.alpha);
        const bool sat     = hit && test_T < 0.0001f;
        live               = sat ? -1.0f : live;
        live_lanes &= ~(pass & wave_ballot(test_T < 0.0001f));
        const float w      = h.alpha * T;
        if (kAccum && (accum_weights_p || accum_weights_count))
          wave_accumulate_weights(hit && !sat, w, hot.id, accum_weights_p, accum_weights_count);
        if (hit && !sat) {
#pragma unroll
          for (int k = 0; k < 3 + E; ++k) C[k] = fmaf(s_feat[j][k], w, C[k]);
          if (kAccum) {
            if (wmax < w) wmax = w, wmax_id = hot.id, flag = true;
          }
          T    = test_T;
          last = b * kG3Batch + j + 1;
        }
      };
      if (kSnap) {
        // the chunk of 64 staged entries holds two buckets of 32: the state is stored in front of each
        for (int half = 0; half < 2; ++half) {
          const int base = c * kWave + half * 32;
          if (base >= n_here) break;
          if (live > 0.0f) {
            const size_t bk = (size_t) (bucket0 + (b * kG3Batch + base) / 32);
            sampled_T[bk * 256 + rank] = T;
#pragma unroll
            for (int k = 0; k < 3 + E; ++k) sampled_ar[(bk * (3 + E) + k) * 256 + rank] = C[k];
          }
          unsigned long long part = todo & (half ? 0xffffffff00000000ull : 0x00000000ffffffffull);
          while (part) {
            if (live_lanes == 0ull) break;
            const int j = c * kWave + __builtin_ctzll(part);
            part &= part - 1;
            blend_entry(s_hot[j], j);
          }
        }
        continue;
      }
      auto pop = [&]() {
        const int j = c * kWave + __builtin_ctzll(todo);
        todo &= todo - 1;
        return j;
      };
      auto peek = [&]() { return c * kWave + (todo ? __builtin_ctzll(todo) : 0); };
      G3Hot hot_a = s_hot[peek()], hot_b;
      while (todo) {
        if (live_lanes == 0ull) break;
        {
          const int j = pop();
          hot_b       = s_hot[peek()];
          __builtin_amdgcn_sched_barrier(0);
          blend_entry(hot_a, j);
        }
        if (todo == 0ull || live_lanes == 0ull) break;
        {
          const int j = pop();
          hot_a       = s_hot[peek()];
          __builtin_amdgcn_sched_barrier(0);
          blend_entry(hot_b, j);
        }
      }
    }
  }
  if (kAccum && flag && accum_max_count) atomicAdd(&accum_max_count[wmax_id], 1);
  if (inside) {
    out_opacity[pix] = 1.0f - T;
    n_contrib[pix]   = last;
#pragma unroll
    for (int k = 0; k < 3; ++k) out_color[k * HW + pix] = C[k];
#pragma unroll
    for (int k = 0; k < E; ++k) out_extras[k * HW + pix] = C[3 + k];
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

// Per-pixel top-k blend weights (gaussian_topk.cu:12-93): the forward traversal with the k slots in registers instead of
// the reference's read-modify-write of global memory per contributing pair. `w >= slot` takes a slot (a later Gaussian
// wins ties); indices start at -1, weights at 0.
template <int kK>
__global__ void __launch_bounds__(kBlendThreads) gs3d_topk_kernel(int flags, const int* __restrict__ tile_order, int W, int H, int topk,
    const int64_t* __restrict__ ranges, const int32_t* __restrict__ point_list, const float2* __restrict__ means2D,
    const float4* __restrict__ conic_opacity, int32_t* __restrict__ top_indices, float* __restrict__ top_weights) {
  __shared__ G3Hot s_hot[kG3Batch];
  const int gx = (W + kTile - 1) / kTile;
  const int tile = scheduled_tile(flags, tile_order), tile_x = tile % gx, tile_y = tile / gx;
  int px, py;
  lane_pixel(tile_x, tile_y, px, py);
  const bool inside = px < W && py < H;
  const size_t pix  = (size_t) W * py + px;
  const float pxf = (float) px, pyf = (float) py;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t r0 = ranges[2 * (size_t) tile], r1 = ranges[2 * (size_t) tile + 1];
  const int n_todo = (int) (r1 - r0);
  const int rounds = (n_todo + kG3Batch - 1) / kG3Batch;
  bool done = !inside;
  float T = 1.0f, tw[kK];
  int ti[kK];
#pragma unroll
  for (int k = 0; k < kK; ++k) tw[k] = 0.0f, ti[k] = -1;
  for (int b = 0; b < rounds; ++b) {
    if (__syncthreads_count(done) == kBlendThreads) break;
    const int n_here = min(kG3Batch, n_todo - b * kG3Batch);
    if ((int) threadIdx.x < n_here) {
      const int id    = point_list[r0 + b * kG3Batch + threadIdx.x];
      const float2 c  = means2D[id];
      const float4 co = conic_opacity[id];
      G3Hot h;
      h.x = c.x, h.y = c.y, h.a = co.x, h.b = co.y, h.c = co.z, h.opacity = co.w, h.id = id;
      h.mask = conic_quadrant_mask(h, tile_x * kTile, tile_y * kTile, flags);
      s_hot[threadIdx.x] = h;
    }
    __syncthreads();
    for (int c = 0; c < kG3Batch / kWave; ++c) {
      const int jj = c * kWave + lane;
      unsigned long long todo = __ballot(jj < n_here && ((s_hot[jj < kG3Batch ? jj : 0].mask >> wave) & 1u));
      while (todo) {
        if (__ballot(!done) == 0ull) break;
        const int j = c * kWave + __builtin_ctzll(todo);
        todo &= todo - 1;
        const G3Hot hot = s_hot[j];
        G3Hit h;
        const bool hit = conic_alpha_flat(hot, pxf, pyf, h) && !done;
        if (__ballot(hit) == 0ull) continue;
        const float test_T = T * (1.0f - h.alpha);
        const bool sat     = hit && test_T < 0.0001f;
        done               = done || sat;
        if (hit && !sat) {
          // sorted insertion: a slot's new weight is the offered one clamped between the slot and the slot above, its
          // id follows the comparisons against the old list
          const float w = h.alpha * T;
          const int idx = hot.id;
          bool ge[kK];
#pragma unroll
          for (int k = 0; k < kK; ++k) ge[k] = k < topk && w >= tw[k];
#pragma unroll
          for (int k = kK - 1; k >= 1; --k) {
            if (k < topk) {
              tw[k] = __builtin_amdgcn_fmed3f(tw[k - 1], w, tw[k]);
              ti[k] = ge[k - 1] ? ti[k - 1] : (ge[k] ? idx : ti[k]);
            }
          }
          tw[0] = fmaxf(tw[0], w);
          ti[0] = ge[0] ? idx : ti[0];
          T = test_T;
        }
      }
    }
  }
  if (inside) {
#pragma unroll
    for (int k = 0; k < kK; ++k)
      if (k < topk) {
        top_weights[pix * topk + k] = tw[k];
        top_indices[pix * topk + k] = ti[k];
      }
  }
}

// gradient slots of one Gaussian: 0-2 colour | 3-6 extras | 7-8 mean2D | 9-11 conic | 12 opacity | 13-15 unused
constexpr int kG3Slots = 16;

// Where slot_sum_kernel puts component c of Gaussian i.
template <int E>
struct G3Scatter {
  float *g_means2D, *g_conic_opacity, *g_colors, *g_extras;
  __device__ __forceinline__ void operator()(int i, int c, float v) const {
    if (c < 3) g_colors[3 * (size_t) i + c] = v;
    else if (c < 7) {
      if (c - 3 < E) g_extras[(size_t) E * i + (c - 3)] = v;
    } else if (c < 9) g_means2D[2 * (size_t) i + (c - 7)] = v;
    else if (c < 13) g_conic_opacity[4 * (size_t) i + (c - 9)] = v;
  }
};

// kSlots: the per-Gaussian sums go through per-instance records (ordered_sums.hpp) instead of device-scope atomics.
template <int E, bool kSlots>
__global__ void __launch_bounds__(kBlendThreads) gs3d_backward_kernel(int flags, const int* __restrict__ tile_order, int W, int H,
    const int64_t* __restrict__ ranges, const int32_t* __restrict__ point_list, const float2* __restrict__ means2D,
    const float4* __restrict__ conic_opacity, const float* __restrict__ colors, const float* __restrict__ extras,
    const float* __restrict__ out_opacity, const int32_t* __restrict__ n_contrib, const float* __restrict__ dL_dpix,
    const float* __restrict__ dL_dout_extras, const float* __restrict__ dL_dout_opacity,
    float* __restrict__ g_means2D, float* __restrict__ g_conic_opacity, float* __restrict__ g_colors,
    float* __restrict__ g_extras, const int64_t* __restrict__ point_offsets, const int32_t* __restrict__ radii,
    float* __restrict__ slot_records) {
  constexpr int kB = 64;
  __shared__ G3Hot s_hot[kB];
  __shared__ float s_feat[kB][3 + kMaxExtra + 1];
  __shared__ float s_part[4][kB][17];  // each wavefront's sums per staged Gaussian: plain stores, added in wavefront order
  __shared__ int s_max_contrib;
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const int tile = scheduled_tile(flags, tile_order), tile_x = tile % gx, tile_y = tile / gx;
  int px, py;
  lane_pixel(tile_x, tile_y, px, py);
  const bool inside = px < W && py < H;
  const size_t HW = (size_t) H * W, pix = (size_t) W * py + px;
  const float pxf = (float) px, pyf = (float) py;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t r0 = ranges[2 * (size_t) tile], r1 = ranges[2 * (size_t) tile + 1];
  const int last_contrib = inside ? n_contrib[pix] : 0;

  if (threadIdx.x == 0) s_max_contrib = 0;
  __syncthreads();
  int wave_max = last_contrib;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) wave_max = max(wave_max, __shfl_xor(wave_max, d, kWave));
  if (lane == 0) atomicMax(&s_max_contrib, wave_max);
  for (int e = threadIdx.x; e < 4 * kB * 17; e += kBlendThreads) (&s_part[0][0][0])[e] = 0.0f;
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
      const int64_t at = (id == 0 ? 0 : point_offsets[id - 1]) + (int64_t) (tile_y - r.y0) * (r.x1 - r.x0) + (tile_x - r.x0);
      float4* dst = (float4*) (slot_records + (size_t) at * kG3Slots);
#pragma unroll
      for (int c4 = 0; c4 < kG3Slots / 4; ++c4) dst[c4] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
  }

  const float T_final = inside ? 1.0f - out_opacity[pix] : 0.0f;
  float T = T_final;
  const float dL_dT = inside ? -dL_dout_opacity[pix] : 0.0f;
  float g_out[3 + (E > 0 ? E : 1)], accum[3 + (E > 0 ? E : 1)];
#pragma unroll
  for (int k = 0; k < 3 + E; ++k) {
    accum[k] = 0.0f;
    g_out[k] = !inside ? 0.0f : (k < 3 ? dL_dpix[k * HW + pix] : dL_dout_extras[(k - 3) * HW + pix]);
  }

  G3Entry next;
  int next_radius = 0;
  int64_t next_off = 0;
  size_t slot = 0;  // record position of the entry this lane staged (the same lane flushes it)
  auto gather = [&](int at) {
    next = gather_gaussian<E>(point_list[r0 + at], means2D, conic_opacity, colors, extras);
    if (kSlots) next_radius = radii[next.hot.id], next_off = next.hot.id == 0 ? 0 : point_offsets[next.hot.id - 1];
  };
  if ((int) threadIdx.x < min(n_todo, kB)) gather(n_todo - 1 - (int) threadIdx.x);
  for (int b = 0; b < rounds; ++b) {
    const int n_here = min(kB, n_todo - b * kB);
    if ((int) threadIdx.x < n_here) {
      next.hot.mask = conic_quadrant_mask(next.hot, tile_x * kTile, tile_y * kTile, flags);
      s_hot[threadIdx.x] = next.hot;
#pragma unroll
      for (int k = 0; k < 3 + E; ++k) s_feat[threadIdx.x][k] = next.feat[k];
      if (kSlots) {
        // the binning emits a Gaussian's tiles row-major over its rectangle, from its prefix-scan offset on
        const TileRect r = tile_rect(next.hot.x, next.hot.y, next_radius, gx, gy);
        slot = (size_t) (next_off + (int64_t) (tile_y - r.y0) * (r.x1 - r.x0) + (tile_x - r.x0));
      }
    }
    __syncthreads();
    const int nxt = (b + 1) * kB + (int) threadIdx.x;
    if ((int) threadIdx.x < kB && nxt < n_todo) gather(n_todo - 1 - nxt);

    unsigned long long todo = __ballot(lane < n_here && ((s_hot[lane].mask >> wave) & 1u) &&
                                       (n_todo - 1 - (b * kB + lane)) < wave_max);
    while (todo) {
      const int j = __builtin_ctzll(todo);
      todo &= todo - 1;
      const int pos = n_todo - 1 - (b * kB + j);  // 0-based position in the tile's list
      G3Hit h;
      unsigned long long pass;
      const bool hit = conic_alpha_flat(s_hot[j], pxf, pyf, h, &pass) && (pos < last_contrib);
      if ((pass & wave_ballot(pos < last_contrib)) == 0ull) continue;
      // Under `hit`: the pixel's back-to-front state and two factors (zero in a lane that does not blend the entry). The
      // components are their products with quantities that are finite in every lane, formed by all lanes alike, so none
      // needs a zero of its own.
      float g[16];
      const G3Hot& hot = s_hot[j];
      float dch = 0.0f, dL_dalpha = 0.0f;
      if (hit) {
        T   = T * __builtin_amdgcn_rcpf(1.0f - h.alpha);
        dch = h.alpha * T;
#pragma unroll
        for (int k = 0; k < 3 + E; ++k) {
          const float v = s_feat[j][k];
          dL_dalpha += (v * T * (1.0f - h.alpha) - accum[k]) * g_out[k];
          accum[k] += v * dch;
        }
        dL_dalpha = (dL_dalpha - T_final * dL_dT) * __builtin_amdgcn_rcpf(1.0f - h.alpha);
      }
#pragma unroll
      for (int c = 0; c < 16; ++c) g[c] = 0.0f;
#pragma unroll
      for (int k = 0; k < 3 + E; ++k) g[k < 3 ? k : 3 + (k - 3)] = dch * g_out[k];
      // G = exp(power) overflows in a lane whose conic gives a large positive power; such a lane never blends
      const float G     = hit ? h.G : 0.0f;
      const float dL_dG = -hot.opacity * G * dL_dalpha;
      g[7]  = dL_dG * (hot.a * h.dx + hot.b * h.dy);
      g[8]  = dL_dG * (hot.c * h.dy + hot.b * h.dx);
      g[9]  = 0.5f * h.dx * h.dx * dL_dG;
      g[10] = h.dx * h.dy * dL_dG;
      g[11] = 0.5f * h.dy * h.dy * dL_dG;
      g[12] = G * dL_dalpha;
      const float tot = wave_sum16_transposed(g);
      if (lane < 16) s_part[wave][j][lane] = tot;  // a wavefront meets an entry once per batch
    }
    __syncthreads();
    if ((int) threadIdx.x < n_here) {
      float a[16];
#pragma unroll
      for (int c = 0; c < 16; ++c) {
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) sum += s_part[w][threadIdx.x][c], s_part[w][threadIdx.x][c] = 0.0f;
        a[c] = sum;
      }
      if (kSlots) {
        float4* dst = (float4*) (slot_records + slot * kG3Slots);
#pragma unroll
        for (int c = 0; c < kG3Slots / 4; ++c) dst[c] = make_float4(a[4 * c], a[4 * c + 1], a[4 * c + 2], a[4 * c + 3]);
      } else {
        const int id = s_hot[threadIdx.x].id;
#pragma unroll
        for (int c = 0; c < 3; ++c)
          if (a[c] != 0.0f) atomicAdd(&g_colors[3 * (size_t) id + c], a[c]);
#pragma unroll
        for (int c = 0; c < E; ++c)
          if (a[3 + c] != 0.0f) atomicAdd(&g_extras[(size_t) E * id + c], a[3 + c]);
#pragma unroll
        for (int c = 0; c < 2; ++c)
          if (a[7 + c] != 0.0f) atomicAdd(&g_means2D[2 * (size_t) id + c], a[7 + c]);
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (a[9 + c] != 0.0f) atomicAdd(&g_conic_opacity[4 * (size_t) id + c], a[9 + c]);
      }
    }
    // a lane only touches its own rows of s_part and its staged entry between this flush and the barrier that follows
    // the next batch's LDS store
  }
}

// The reference's second backward (gaussian_render.cu:540-694), the per-Gaussian decomposition: a lane owns ONE list
// entry of a tile and keeps that Gaussian's gradient sums in registers, the tile's pixels pass through the lanes one
// lane per step, each carrying its blending state (transmittance and accumulated colour, front to back, started from
// the forward's snapshot in front of the bucket), so no sum ever crosses lanes and nothing is reduced.
// Laid out for a 64-lane wavefront: one wavefront takes 64 consecutive entries = two of the forward's 32-entry buckets
// (the wavefront of the odd bucket leaves at once), the state moves with one whole-wavefront DPP shift per value, the
// per-pixel constants (upstream gradients, final transmittance, last contributor, coordinates) are staged in LDS once
// and read by pixel number instead of travelling through the lanes, and only the pixels that still blend at the
// group's first entry (n_contrib beyond it) are fed in, so a deep group takes `live + 63` steps instead of 256 + 63.
// Per-Gaussian results: one record per lane (kSlots; entries the pipeline never reaches write zeros) or atomics.
template <int E, bool kSlots>
__global__ void __launch_bounds__(64) gs3d_bucket_backward_kernel(int W, int H, const int64_t* __restrict__ ranges,
    const int32_t* __restrict__ point_list, const float2* __restrict__ means2D,
    const float4* __restrict__ conic_opacity, const float* __restrict__ colors, const float* __restrict__ extras,
    const float* __restrict__ images, const float* __restrict__ out_extras, const float* __restrict__ out_opacity,
    const int32_t* __restrict__ n_contrib, const int32_t* __restrict__ max_contrib,
    const int64_t* __restrict__ bucket_offset, const int32_t* __restrict__ bucket_to_tile,
    const float* __restrict__ sampled_T, const float* __restrict__ sampled_ar, const float* __restrict__ dL_dpix,
    const float* __restrict__ dL_dout_extras, const float* __restrict__ dL_dout_opacity,
    float* __restrict__ g_means2D, float* __restrict__ g_conic_opacity, float* __restrict__ g_colors,
    float* __restrict__ g_extras, const int64_t* __restrict__ point_offsets, const int32_t* __restrict__ radii,
    float* __restrict__ slot_records) {
  constexpr int kC = 3 + E;
  __shared__ float4 s_grad[256];   // dL/d(r, g, b) of the pixel | T_final * dL/dopacity
  __shared__ float4 s_state[256];  // snapshot: T | accumulated colour minus the final colour
  __shared__ float4 s_pixel[256];  // x | y | last contributor (int bits) | -
  __shared__ float s_extra[E > 0 ? 256 : 1][2 * (E > 0 ? E : 1)];  // extras: upstream gradient | accumulated minus final
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

  G3Hot hot{};
  float feat[kC];
#pragma unroll
  for (int k = 0; k < kC; ++k) feat[k] = 0.0f;
  size_t slot = 0;
  if (valid) {
    const G3Entry g = gather_gaussian<E>(point_list[r0 + entry], means2D, conic_opacity, colors, extras);
    hot = g.hot;
#pragma unroll
    for (int k = 0; k < kC; ++k) feat[k] = g.feat[k];
    if (kSlots) {
      const TileRect r = tile_rect(hot.x, hot.y, radii[hot.id], gx, gy);
      slot = (size_t) ((hot.id == 0 ? 0 : point_offsets[hot.id - 1]) + (int64_t) (tile_y - r.y0) * (r.x1 - r.x0) +
                       (tile_x - r.x0));
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
        const float T_final = 1.0f - out_opacity[pix];
        s_grad[at]  = make_float4(dL_dpix[pix], dL_dpix[HW + pix], dL_dpix[2 * HW + pix], T_final * dL_dout_opacity[pix]);
        const size_t snap = (size_t) bucket * 256 + rank;
        s_state[at] = make_float4(sampled_T[snap], sampled_ar[((size_t) bucket * kC + 0) * 256 + rank] - images[pix],
                                  sampled_ar[((size_t) bucket * kC + 1) * 256 + rank] - images[HW + pix],
                                  sampled_ar[((size_t) bucket * kC + 2) * 256 + rank] - images[2 * HW + pix]);
        s_pixel[at] = make_float4((float) px, (float) py, __int_as_float(last), 0.0f);
#pragma unroll
        for (int k = 0; k < E; ++k) {
          s_extra[at][k]     = dL_dout_extras[k * HW + pix];
          s_extra[at][E + k] = sampled_ar[((size_t) bucket * kC + 3 + k) * 256 + rank] - out_extras[k * HW + pix];
        }
      }
      n_live += __builtin_popcountll(live_lanes);
    }
  }
  __syncthreads();

  float g[16];
#pragma unroll
  for (int c = 0; c < 16; ++c) g[c] = 0.0f;
  float T = 0.0f, ar[kC];
#pragma unroll
  for (int k = 0; k < kC; ++k) ar[k] = 0.0f;
  // whole-wavefront shift by one lane (DPP wave_shr:1); lane 0 keeps `fresh`
  auto pass_on = [](float fresh, float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, fresh),
                                                                 __builtin_bit_cast(int, v), 0x138, 0xf, 0xf, false));
  };
  const int steps = n_live > 0 ? n_live + 63 : 0;
  float4 next_state = s_state[0];
  for (int i = 0; i < steps; ++i) {
    const int head = min(i, n_live - 1);  // the pixel that enters at lane 0 (nothing new once all have entered)
    const float4 fresh = next_state;
    next_state = s_state[min(i + 1, n_live - 1)];  // requested a step ahead of its use
    T     = pass_on(fresh.x, T);
    ar[0] = pass_on(fresh.y, ar[0]);
    ar[1] = pass_on(fresh.z, ar[1]);
    ar[2] = pass_on(fresh.w, ar[2]);
#pragma unroll
    for (int k = 0; k < E; ++k) ar[3 + k] = pass_on(s_extra[head][E + k], ar[3 + k]);
    const int q = i - lane;
    if (q < 0 || q >= n_live) continue;
    const float4 pixel = s_pixel[q];
    G3Hit h;
    const bool hit = conic_alpha_flat(hot, pixel.x, pixel.y, h) && valid && entry < __float_as_int(pixel.z);
    if (!hit) continue;
    const float4 up = s_grad[q];
    float dL[kC];
    dL[0] = up.x, dL[1] = up.y, dL[2] = up.z;
#pragma unroll
    for (int k = 0; k < E; ++k) dL[3 + k] = s_extra[q][k];
    const float w = h.alpha * T, inv = __builtin_amdgcn_rcpf(1.0f - h.alpha);
    float dL_dalpha = 0.0f;
#pragma unroll
    for (int k = 0; k < kC; ++k) {
      ar[k] += w * feat[k];  // accumulated colour up to and including this Gaussian, minus the final colour
      g[k < 3 ? k : 3 + (k - 3)] += w * dL[k];
      dL_dalpha += (feat[k] * T + inv * ar[k]) * dL[k];
    }
    dL_dalpha += inv * up.w;  // through the final transmittance: dL/dT_final = -dL/dopacity, dT_final/dalpha = -T_final / (1 - alpha)
    T *= 1.0f - h.alpha;
    const float dL_dG = -hot.opacity * h.G * dL_dalpha;
    g[7]  += dL_dG * (hot.a * h.dx + hot.b * h.dy);
    g[8]  += dL_dG * (hot.c * h.dy + hot.b * h.dx);
    g[9]  += 0.5f * h.dx * h.dx * dL_dG;
    g[10] += h.dx * h.dy * dL_dG;
    g[11] += 0.5f * h.dy * h.dy * dL_dG;
    g[12] += h.G * dL_dalpha;
  }
  if (!valid) return;
  if (kSlots) {
    float4* dst = (float4*) (slot_records + slot * kG3Slots);
#pragma unroll
    for (int c = 0; c < kG3Slots / 4; ++c) dst[c] = make_float4(g[4 * c], g[4 * c + 1], g[4 * c + 2], g[4 * c + 3]);
  } else {
    const int id = hot.id;
#pragma unroll
    for (int c = 0; c < 3; ++c)
      if (g[c] != 0.0f) atomicAdd(&g_colors[3 * (size_t) id + c], g[c]);
#pragma unroll
    for (int c = 0; c < E; ++c)
      if (g[3 + c] != 0.0f) atomicAdd(&g_extras[(size_t) E * id + c], g[3 + c]);
#pragma unroll
    for (int c = 0; c < 2; ++c)
      if (g[7 + c] != 0.0f) atomicAdd(&g_means2D[2 * (size_t) id + c], g[7 + c]);
#pragma unroll
    for (int c = 0; c < 4; ++c)
      if (g[9 + c] != 0.0f) atomicAdd(&g_conic_opacity[4 * (size_t) id + c], g[9 + c]);
  }
}

// Largest n_contrib of the tile's 256 pixels: no pixel looks past that list position.
__device__ __forceinline__ int block_max_contrib(int last_contrib, int* s_max) {
  if (threadIdx.x == 0) *s_max = 0;
  __syncthreads();
  int wave_max = last_contrib;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) wave_max = max(wave_max, __shfl_xor(wave_max, d, kWave));
  if ((threadIdx.x & 63) == 0) atomicMax(s_max, wave_max);
  __syncthreads();
  return *s_max;
}

// Feature channels [e0, e0 + kC) of an arbitrary-width per-Gaussian table blended with the weights of the main forward
// pass (gaussian_rasterizer_extra.cu:12-101): the traversal stops at the pixel's n_contrib. blockIdx.y selects the group
// of channels, so groups run side by side where the reference walks the list once per group in sequence. Output is
// pixel-major [H, W, E].
template <int kC>
__global__ void __launch_bounds__(kBlendThreads) gs3d_extra_forward_kernel(int flags, const int* __restrict__ tile_order, int W, int H, int E,
    const int64_t* __restrict__ ranges, const int32_t* __restrict__ point_list, const float2* __restrict__ means2D,
    const float4* __restrict__ conic_opacity, const int32_t* __restrict__ n_contrib, const float* __restrict__ extras,
    float* __restrict__ out) {
  constexpr int kHalf = kC / 2;  // two threads gather one Gaussian's channels
  __shared__ G3Hot s_hot[kG3Batch];
  __shared__ float s_feat[kG3Batch][kC + 1];
  __shared__ int s_max_contrib;
  const int gx = (W + kTile - 1) / kTile;
  const int tile = scheduled_tile(flags, tile_order), tile_x = tile % gx, tile_y = tile / gx;
  int px, py;
  lane_pixel(tile_x, tile_y, px, py);
  const bool inside = px < W && py < H;
  const size_t pix  = (size_t) W * py + px;
  const float pxf = (float) px, pyf = (float) py;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int e0 = blockIdx.y * kC, n_ch = min(kC, E - e0);
  const int64_t r0 = ranges[2 * (size_t) tile], r1 = ranges[2 * (size_t) tile + 1];
  const int last_contrib = inside ? n_contrib[pix] : 0;
  const int n_todo = min(block_max_contrib(last_contrib, &s_max_contrib), (int) (r1 - r0));
  const int rounds = (n_todo + kG3Batch - 1) / kG3Batch;
  const int slot = threadIdx.x & (kG3Batch - 1), half = threadIdx.x / kG3Batch;

  bool done = last_contrib == 0;
  float T = 1.0f, C[kC];
#pragma unroll
  for (int k = 0; k < kC; ++k) C[k] = 0.0f;

  for (int b = 0; b < rounds; ++b) {
    if (__syncthreads_count(done) == kBlendThreads) break;
    const int n_here = min(kG3Batch, n_todo - b * kG3Batch);
    if (slot < n_here) {
      const int id = point_list[r0 + b * kG3Batch + slot];
      if (half == 0) {
        const float2 c  = means2D[id];
        const float4 co = conic_opacity[id];
        G3Hot h;
        h.x = c.x, h.y = c.y, h.a = co.x, h.b = co.y, h.c = co.z, h.opacity = co.w, h.id = id;
        h.mask = conic_quadrant_mask(h, tile_x * kTile, tile_y * kTile, flags);
        s_hot[slot] = h;
      }
#pragma unroll
      for (int k = half * kHalf; k < half * kHalf + kHalf; ++k)
        s_feat[slot][k] = k < n_ch ? extras[(size_t) E * id + e0 + k] : 0.0f;
    }
    __syncthreads();
    for (int c = 0; c < kG3Batch / kWave; ++c) {
      const int jj = c * kWave + lane;
      unsigned long long todo = __ballot(jj < n_here && ((s_hot[jj < kG3Batch ? jj : 0].mask >> wave) & 1u));
      while (todo) {
        if (__ballot(!done) == 0ull) break;
        const int j = c * kWave + __builtin_ctzll(todo);
        todo &= todo - 1;
        const int pos = b * kG3Batch + j;  // 0-based position in the tile's list
        done = done || pos >= last_contrib;
        G3Hit h;
        const bool hit = conic_alpha_flat(s_hot[j], pxf, pyf, h) && !done;
        if (__ballot(hit) == 0ull) continue;
        const float test_T = T * (1.0f - h.alpha);
        const bool sat     = hit && test_T < 0.0001f;
        done               = done || sat;
        if (hit && !sat) {
          const float w = h.alpha * T;
#pragma unroll
          for (int k = 0; k < kC; ++k) C[k] = fmaf(s_feat[j][k], w, C[k]);
          T = test_T;
        }
      }
    }
  }
  if (inside) {
    float* o = out + pix * E + e0;
    if ((E & 3) == 0) {
#pragma unroll
      for (int k = 0; k < kC; k += 4)
        if (k < n_ch) *reinterpret_cast<float4*>(o + k) = make_float4(C[k], C[k + 1], C[k + 2], C[k + 3]);
    } else {
#pragma unroll
      for (int k = 0; k < kC; ++k)
        if (k < n_ch) o[k] = C[k];
    }
  }
}

// Backward of the feature-channel blend (gaussian_rasterizer_extra.cu:103-209), 8 channels per block: back to front from
// T_final = 1 - out_opacity without the background and opacity terms of the main backward. Each block adds its group's
// share of the mean / conic / opacity gradients, as each of the reference's sequential groups does.
// gradient slots of one Gaussian: 0-7 channels | 8-9 mean2D | 10-12 conic | 13 opacity | 14-15 unused
__global__ void __launch_bounds__(kBlendThreads) gs3d_extra_backward_kernel(int flags, const int* __restrict__ tile_order, int W, int H, int E,
    const int64_t* __restrict__ ranges, const int32_t* __restrict__ point_list, const float2* __restrict__ means2D,
    const float4* __restrict__ conic_opacity, const float* __restrict__ out_opacity,
    const int32_t* __restrict__ n_contrib, const float* __restrict__ extras, const float* __restrict__ dL_dout,
    float* __restrict__ g_means2D, float* __restrict__ g_conic_opacity, float* __restrict__ g_extras) {
  constexpr int kB = 64, kC = 8, kPart = kC / 4;  // four threads gather one Gaussian's channels
  __shared__ G3Hot s_hot[kB];
  __shared__ float s_feat[kB][kC + 1];
  __shared__ float s_part[4][kB][17];  // each wavefront's sums per staged Gaussian: plain stores, added in wavefront order
  __shared__ int s_max_contrib;
  const int gx = (W + kTile - 1) / kTile;
  const int tile = scheduled_tile(flags, tile_order), tile_x = tile % gx, tile_y = tile / gx;
  int px, py;
  lane_pixel(tile_x, tile_y, px, py);
  const bool inside = px < W && py < H;
  const size_t pix  = (size_t) W * py + px;
  const float pxf = (float) px, pyf = (float) py;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int e0 = blockIdx.y * kC, n_ch = min(kC, E - e0);
  const int64_t r0 = ranges[2 * (size_t) tile], r1 = ranges[2 * (size_t) tile + 1];
  const int last_contrib = inside ? n_contrib[pix] : 0;
  for (int e = threadIdx.x; e < 4 * kB * 17; e += kBlendThreads) (&s_part[0][0][0])[e] = 0.0f;
  const int n_todo = min(block_max_contrib(last_contrib, &s_max_contrib), (int) (r1 - r0));
  const int rounds = (n_todo + kB - 1) / kB;
  int wave_max = last_contrib;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) wave_max = max(wave_max, __shfl_xor(wave_max, d, kWave));

  float T = inside ? 1.0f - out_opacity[pix] : 0.0f;
  float g_out[kC], accum[kC];
#pragma unroll
  for (int k = 0; k < kC; ++k) {
    accum[k] = 0.0f;
    g_out[k] = (inside && k < n_ch) ? dL_dout[pix * E + e0 + k] : 0.0f;
  }
  const int slot = threadIdx.x & (kB - 1), part = threadIdx.x / kB;

  for (int b = 0; b < rounds; ++b) {
    const int n_here = min(kB, n_todo - b * kB);
    if (slot < n_here) {
      const int id = point_list[r0 + (n_todo - 1 - (b * kB + slot))];
      if (part == 0) {
        const float2 c  = means2D[id];
        const float4 co = conic_opacity[id];
        G3Hot h;
        h.x = c.x, h.y = c.y, h.a = co.x, h.b = co.y, h.c = co.z, h.opacity = co.w, h.id = id;
        h.mask = conic_quadrant_mask(h, tile_x * kTile, tile_y * kTile, flags);
        s_hot[slot] = h;
      }
#pragma unroll
      for (int k = part * kPart; k < part * kPart + kPart; ++k)
        s_feat[slot][k] = k < n_ch ? extras[(size_t) E * id + e0 + k] : 0.0f;
    }
    __syncthreads();
    unsigned long long todo = __ballot(lane < n_here && ((s_hot[lane].mask >> wave) & 1u) &&
                                       (n_todo - 1 - (b * kB + lane)) < wave_max);
    while (todo) {
      const int j = __builtin_ctzll(todo);
      todo &= todo - 1;
      const int pos = n_todo - 1 - (b * kB + j);  // 0-based position in the tile's list
      G3Hit h;
      unsigned long long pass;
      const bool hit = conic_alpha_flat(s_hot[j], pxf, pyf, h, &pass) && (pos < last_contrib);
      if ((pass & wave_ballot(pos < last_contrib)) == 0ull) continue;
      float g[16];
#pragma unroll
      for (int c = 0; c < 16; ++c) g[c] = 0.0f;
      if (hit) {
        const G3Hot& hot = s_hot[j];
        T = T * __builtin_amdgcn_rcpf(1.0f - h.alpha);
        const float dch = h.alpha * T;
        float dL_dalpha = 0.0f;
#pragma unroll
        for (int k = 0; k < kC; ++k) {
          const float v = s_feat[j][k];
          dL_dalpha += (v * T * (1.0f - h.alpha) - accum[k]) * g_out[k];
          accum[k] += v * dch;
          g[k] = dch * g_out[k];
        }
        dL_dalpha = dL_dalpha * __builtin_amdgcn_rcpf(1.0f - h.alpha);
        const float dL_dG = -hot.opacity * h.G * dL_dalpha;
        g[8]  = dL_dG * (hot.a * h.dx + hot.b * h.dy);
        g[9]  = dL_dG * (hot.c * h.dy + hot.b * h.dx);
        g[10] = 0.5f * h.dx * h.dx * dL_dG;
        g[11] = h.dx * h.dy * dL_dG;
        g[12] = 0.5f * h.dy * h.dy * dL_dG;
        g[13] = h.G * dL_dalpha;
      }
      const float tot = wave_sum16_transposed(g);
      if (lane < 16) s_part[wave][j][lane] = tot;  // a wavefront meets an entry once per batch
    }
    __syncthreads();
    if ((int) threadIdx.x < n_here) {
      float a[16];
#pragma unroll
      for (int c = 0; c < 16; ++c) {
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) sum += s_part[w][threadIdx.x][c], s_part[w][threadIdx.x][c] = 0.0f;
        a[c] = sum;
      }
      const int id = s_hot[threadIdx.x].id;
      if (g_extras)
#pragma unroll
        for (int c = 0; c < kC; ++c)
          if (c < n_ch && a[c] != 0.0f) atomicAdd(&g_extras[(size_t) E * id + e0 + c], a[c]);
      if (g_means2D)
#pragma unroll
        for (int c = 0; c < 2; ++c)
          if (a[8 + c] != 0.0f) atomicAdd(&g_means2D[2 * (size_t) id + c], a[8 + c]);
      if (g_conic_opacity)
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (a[10 + c] != 0.0f) atomicAdd(&g_conic_opacity[4 * (size_t) id + c], a[10 + c]);
    }
    // between this flush and the barrier after the next batch's LDS store a lane touches its own rows of s_part and
    // its own s_hot entry only; s_feat was last read before the barrier above
  }
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API int fsgs_gaussian_rasterize_forward(int P, int W, int H, int E, const float* means2D,
    const float* conic_opacity, const float* colors, const float* extras, const int32_t* point_list,
    const int64_t* ranges, int32_t* accum_max_count, float* accum_weights_p, int32_t* accum_weights_count,
    const int64_t* bucket_offset, float* out_color, float* out_opacity, float* out_extras, int32_t* n_contrib,
    int32_t* max_contrib, int32_t* bucket_to_tile, float* sampled_T, float* sampled_ar, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0, "gaussian_rasterize_forward: bad sizes");
  const bool snap = bucket_offset != nullptr;
  FSGS_REQUIRE(!snap || (max_contrib && bucket_to_tile && sampled_T && sampled_ar),
               "gaussian_rasterize_forward: snapshot outputs are required with per_tile_bucket_offset");
  FSGS_REQUIRE(E >= 0 && E <= kMaxExtra, "gaussian_rasterize_forward: only 0..%d extra channels are supported", kMaxExtra);
  FSGS_REQUIRE(ranges && out_color && out_opacity && n_contrib && (E == 0 || (extras && out_extras)),
               "gaussian_rasterize_forward: null pointer");
  FSGS_REQUIRE(P == 0 || (means2D && conic_opacity && colors), "gaussian_rasterize_forward: null pointer");
  hipStream_t s = (hipStream_t) stream;
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const int* tile_order = nullptr;
  const int flags = launch_tile_order(gx, gy, ranges, s, &tile_order);
  const dim3 grid(gx * gy), block(kBlendThreads);
  const bool accum = accum_max_count || accum_weights_p || accum_weights_count;
#define FSGS_G3_FWD(EE, ACC, SNAP)                                                                                  \
  hipLaunchKernelGGL((gs3d_forward_kernel<EE, ACC, SNAP>), grid, block, 0, s, flags, tile_order, W, H, ranges,      \
                     point_list, (const float2*) means2D, (const float4*) conic_opacity, colors, extras, out_color, \
                     out_opacity, out_extras, n_contrib, accum_max_count, accum_weights_p, accum_weights_count,     \
                     bucket_offset, max_contrib, bucket_to_tile, sampled_T, sampled_ar)
#define FSGS_G3_FWD_E(EE)                                     \
  do {                                                        \
    if (accum && snap) FSGS_G3_FWD(EE, true, true);           \
    else if (accum) FSGS_G3_FWD(EE, true, false);             \
    else if (snap) FSGS_G3_FWD(EE, false, true);              \
    else FSGS_G3_FWD(EE, false, false);                       \
  } while (0)
  switch (E) {
    case 0: FSGS_G3_FWD_E(0); break;
    case 1: FSGS_G3_FWD_E(1); break;
    case 2: FSGS_G3_FWD_E(2); break;
    case 3: FSGS_G3_FWD_E(3); break;
    default: FSGS_G3_FWD_E(4); break;
  }
#undef FSGS_G3_FWD_E
#undef FSGS_G3_FWD
  return check_launch("gaussian_rasterize_forward");
}

FSGS_API size_t fsgs_gaussian_rasterize_backward_workspace_bytes(int64_t R) {
  return slot_workspace_bytes(R, kG3Slots);
}

// Tile lists built by the culled binning leave out the instances whose keep bit is clear; no block stages them, so no
// block writes (or clears) their records, and the ordered sum reads every position of a Gaussian's span. Four lanes
// per Gaussian zero those records, 16 bytes each.
__global__ void __launch_bounds__(256) clear_culled_records_kernel(int P, const int64_t* __restrict__ point_offsets,
    const uint32_t* __restrict__ keep_masks, float* __restrict__ records) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x, i = t >> 2, part = t & 3;
  if (i >= P) return;
  const int64_t e0 = i > 0 ? point_offsets[i - 1] : 0, e1 = point_offsets[i];
  const int64_t count = e1 - e0;
  if (count <= 0 || count > 32) return;  // rectangles above 32 tiles are kept whole
  uint32_t dropped = ~keep_masks[i] & (count == 32 ? 0xffffffffu : (1u << (int) count) - 1u);
  while (dropped) {
    const int j = __builtin_ctz(dropped);
    dropped &= dropped - 1u;
    ((float4*) (records + (size_t) (e0 + j) * kG3Slots))[part] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  }
}

FSGS_API int fsgs_gaussian_rasterize_clear_culled(int P, int64_t R, const int64_t* point_offsets,
    const uint32_t* keep_masks, void* workspace, size_t workspace_bytes, void* stream) {
  static_assert(kG3Slots == 16, "four lanes of 16 bytes per record");
  FSGS_REQUIRE(P >= 0 && R >= 0, "gaussian_rasterize_clear_culled: bad sizes");
  if (P == 0 || R == 0) return kOk;
  FSGS_REQUIRE(point_offsets && keep_masks && workspace, "gaussian_rasterize_clear_culled: null pointer");
  FSGS_REQUIRE(((uintptr_t) workspace & 15) == 0, "gaussian_rasterize_clear_culled: workspace must be 16-byte aligned");
  if (workspace_bytes < slot_workspace_bytes(R, kG3Slots))
    return fail(kWorkspaceSmall, "gaussian_rasterize_clear_culled: workspace %zu < %zu bytes", workspace_bytes,
                slot_workspace_bytes(R, kG3Slots));
  hipLaunchKernelGGL(clear_culled_records_kernel, dim3((unsigned) div_up(4 * (int64_t) P, 256)), dim3(256), 0,
                     (hipStream_t) stream, P, point_offsets, keep_masks, (float*) workspace);
  return check_launch("gaussian_rasterize_clear_culled");
}

FSGS_API int fsgs_gaussian_rasterize_backward(int P, int W, int H, int E, const float* means2D,
    const float* conic_opacity, const float* colors, const float* extras, const float* out_opacity,
    const int32_t* n_contrib, const float* dL_dpix, const float* dL_dout_extras, const float* dL_dout_opacity,
    const int32_t* point_list, const int64_t* ranges, float* g_means2D, float* g_conic_opacity, float* g_colors,
    float* g_extras, int64_t R, const int64_t* point_offsets, const int32_t* radii, void* workspace,
    size_t workspace_bytes, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0, "gaussian_rasterize_backward: bad sizes");
  FSGS_REQUIRE(E >= 0 && E <= kMaxExtra, "gaussian_rasterize_backward: only 0..%d extra channels are supported", kMaxExtra);
  if (P == 0) return kOk;
  FSGS_REQUIRE(means2D && conic_opacity && colors && out_opacity && n_contrib && dL_dpix && dL_dout_opacity && ranges &&
                   g_means2D && g_conic_opacity && g_colors && (E == 0 || (extras && dL_dout_extras && g_extras)),
               "gaussian_rasterize_backward: null pointer");
  const bool slots = point_offsets != nullptr;
  SlotWorkspace ws{nullptr};
  if (slots) {
    FSGS_REQUIRE(radii && workspace && R >= 0 && R < (int64_t) 0x7fffffff,
                 "gaussian_rasterize_backward: the ordered-sum path needs radii, a workspace and the instance count R");
    if (workspace_bytes < slot_workspace_bytes(R, kG3Slots))
      return fail(kWorkspaceSmall, "gaussian_rasterize_backward: workspace %zu < %zu bytes", workspace_bytes,
                  slot_workspace_bytes(R, kG3Slots));
    FSGS_REQUIRE(((uintptr_t) workspace & 15) == 0, "gaussian_rasterize_backward: workspace must be 16-byte aligned");
    ws = slot_workspace(workspace, R, kG3Slots);
  }
  hipStream_t s = (hipStream_t) stream;
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const int* tile_order = nullptr;
  const int flags = launch_tile_order(gx, gy, ranges, s, &tile_order);
  const dim3 grid(gx * gy), block(kBlendThreads);
#define FSGS_G3_BWD(EE, SL)                                                                                         \
  hipLaunchKernelGGL((gs3d_backward_kernel<EE, SL>), grid, block, 0, s, flags, tile_order, W, H, ranges, point_list, \
                     (const float2*) means2D, (const float4*) conic_opacity, colors, extras, out_opacity, n_contrib, \
                     dL_dpix, dL_dout_extras, dL_dout_opacity, g_means2D, g_conic_opacity, g_colors, g_extras,      \
                     point_offsets, radii, ws.records)
#define FSGS_G3_BWD_E(EE)                                                                                           \
  do {                                                                                                              \
    if (slots) {                                                                                                    \
      FSGS_G3_BWD(EE, true);                                                                                        \
      launch_slot_sum<kG3Slots>(P, point_offsets, ws, G3Scatter<EE>{g_means2D, g_conic_opacity, g_colors, g_extras}, s); \
    } else {                                                                                                        \
      FSGS_G3_BWD(EE, false);                                                                                       \
    }                                                                                                               \
  } while (0)
  switch (E) {
    case 0: FSGS_G3_BWD_E(0); break;
    case 1: FSGS_G3_BWD_E(1); break;
    case 2: FSGS_G3_BWD_E(2); break;
    case 3: FSGS_G3_BWD_E(3); break;
    default: FSGS_G3_BWD_E(4); break;
  }
#undef FSGS_G3_BWD_E
#undef FSGS_G3_BWD
  return check_launch("gaussian_rasterize_backward");
}

// The reference's second backward walks 32-entry buckets from the forward's snapshots, one warp per bucket
// (gaussian_render.cu:540-694). It evaluates the same derivative as the back-to-front kernel, which is the faster of
// the two on this chip; this name runs that kernel, and the snapshot arguments are accepted (and checked for presence)
// so that the binding is a drop-in. fsgs_gaussian_rasterize_bucket_backward below runs the per-Gaussian decomposition.
FSGS_API int fsgs_gaussian_rasterize_fast_backward(int P, int W, int H, int E, const float* means2D,
    const float* conic_opacity, const float* colors, const float* extras, const float* images,
    const float* out_extras, const float* out_opacity, const int32_t* n_contrib, const int32_t* max_contrib,
    const int64_t* bucket_offset, const int32_t* bucket_to_tile, const float* sampled_T, const float* sampled_ar,
    const float* dL_dpix, const float* dL_dout_extras, const float* dL_dout_opacity, const int32_t* point_list,
    const int64_t* ranges, float* g_means2D, float* g_conic_opacity, float* g_colors, float* g_extras, int64_t R,
    const int64_t* point_offsets, const int32_t* radii, void* workspace, size_t workspace_bytes, void* stream) {
  if (P == 0) return kOk;
  FSGS_REQUIRE(images && max_contrib && bucket_offset && bucket_to_tile && sampled_T && sampled_ar &&
                   (E == 0 || out_extras),
               "gaussian_rasterize_fast_backward: null pointer");
  return fsgs_gaussian_rasterize_backward(P, W, H, E, means2D, conic_opacity, colors, extras, out_opacity, n_contrib,
                                          dL_dpix, dL_dout_extras, dL_dout_opacity, point_list, ranges, g_means2D,
                                          g_conic_opacity, g_colors, g_extras, R, point_offsets, radii, workspace,
                                          workspace_bytes, stream);
}

// The per-Gaussian decomposition itself (gs3d_bucket_backward_kernel), for callers that want the reference's second
// algorithm rather than its result: B = the number of 32-entry buckets the forward announced (bucket_to_tile's length).
FSGS_API int fsgs_gaussian_rasterize_bucket_backward(int P, int W, int H, int E, int B, const float* means2D,
    const float* conic_opacity, const float* colors, const float* extras, const float* images,
    const float* out_extras, const float* out_opacity, const int32_t* n_contrib, const int32_t* max_contrib,
    const int64_t* bucket_offset, const int32_t* bucket_to_tile, const float* sampled_T, const float* sampled_ar,
    const float* dL_dpix, const float* dL_dout_extras, const float* dL_dout_opacity, const int32_t* point_list,
    const int64_t* ranges, float* g_means2D, float* g_conic_opacity, float* g_colors, float* g_extras, int64_t R,
    const int64_t* point_offsets, const int32_t* radii, void* workspace, size_t workspace_bytes, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0 && B >= 0, "gaussian_rasterize_bucket_backward: bad sizes");
  FSGS_REQUIRE(E >= 0 && E <= kMaxExtra, "gaussian_rasterize_bucket_backward: only 0..%d extra channels are supported",
               kMaxExtra);
  if (P == 0) return kOk;
  FSGS_REQUIRE(means2D && conic_opacity && colors && images && out_opacity && n_contrib && max_contrib &&
                   bucket_offset && sampled_T && sampled_ar && dL_dpix && dL_dout_opacity && ranges && g_means2D &&
                   g_conic_opacity && g_colors && (B == 0 || (bucket_to_tile && point_list)) &&
                   (E == 0 || (extras && out_extras && dL_dout_extras && g_extras)),
               "gaussian_rasterize_bucket_backward: null pointer");
  const bool slots = point_offsets != nullptr;
  SlotWorkspace ws{nullptr};
  if (slots) {
    FSGS_REQUIRE(radii && workspace && R >= 0 && R < (int64_t) 0x7fffffff,
                 "gaussian_rasterize_bucket_backward: the ordered-sum path needs radii, a workspace and the instance count R");
    if (workspace_bytes < slot_workspace_bytes(R, kG3Slots))
      return fail(kWorkspaceSmall, "gaussian_rasterize_bucket_backward: workspace %zu < %zu bytes", workspace_bytes,
                  slot_workspace_bytes(R, kG3Slots));
    FSGS_REQUIRE(((uintptr_t) workspace & 15) == 0, "gaussian_rasterize_bucket_backward: workspace must be 16-byte aligned");
    ws = slot_workspace(workspace, R, kG3Slots);
  }
  hipStream_t s = (hipStream_t) stream;
#define FSGS_G3_BKT(EE, SL)                                                                                          \
  hipLaunchKernelGGL((gs3d_bucket_backward_kernel<EE, SL>), dim3(B), dim3(64), 0, s, W, H, ranges, point_list,       \
                     (const float2*) means2D, (const float4*) conic_opacity, colors, extras, images, out_extras,     \
                     out_opacity, n_contrib, max_contrib, bucket_offset, bucket_to_tile, sampled_T, sampled_ar,      \
                     dL_dpix, dL_dout_extras, dL_dout_opacity, g_means2D, g_conic_opacity, g_colors, g_extras,       \
                     point_offsets, radii, ws.records)
#define FSGS_G3_BKT_E(EE)                                                                                            \
  do {                                                                                                               \
    if (slots) {                                                                                                     \
      if (B > 0) FSGS_G3_BKT(EE, true);                                                                              \
      launch_slot_sum<kG3Slots>(P, point_offsets, ws, G3Scatter<EE>{g_means2D, g_conic_opacity, g_colors, g_extras}, s); \
    } else if (B > 0) {                                                                                              \
      FSGS_G3_BKT(EE, false);                                                                                        \
    }                                                                                                                \
  } while (0)
  switch (E) {
    case 0: FSGS_G3_BKT_E(0); break;
    case 1: FSGS_G3_BKT_E(1); break;
    case 2: FSGS_G3_BKT_E(2); break;
    case 3: FSGS_G3_BKT_E(3); break;
    default: FSGS_G3_BKT_E(4); break;
  }
#undef FSGS_G3_BKT_E
#undef FSGS_G3_BKT
  return check_launch("gaussian_rasterize_bucket_backward");
}

FSGS_API int fsgs_gaussian_topk_weights(int topk, int P, int W, int H, const float* means2D,
    const float* conic_opacity, const int64_t* ranges, const int32_t* point_list, int32_t* top_indices,
    float* top_weights, void* stream) {
  FSGS_REQUIRE(topk > 0 && W > 0 && H > 0 && P >= 0 && ranges && top_indices && top_weights,
               "gaussian_topk_weights: bad arguments");
  FSGS_REQUIRE(topk <= 16, "gaussian_topk_weights: topk=%d exceeds the supported maximum of 16", topk);
  FSGS_REQUIRE(P == 0 || (means2D && conic_opacity && point_list), "gaussian_topk_weights: null pointer");
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const dim3 grid(gx * gy), block(kBlendThreads);
  hipStream_t s   = (hipStream_t) stream;
  const int* tile_order = nullptr;
  const int flags = launch_tile_order(gx, gy, ranges, s, &tile_order);
#define FSGS_TOPK3(KK)                                                                                          \
  hipLaunchKernelGGL((gs3d_topk_kernel<KK>), grid, block, 0, s, flags, tile_order, W, H, topk, ranges, point_list,          \
                     (const float2*) means2D, (const float4*) conic_opacity, top_indices, top_weights)
  if (topk <= 4) FSGS_TOPK3(4);
  else if (topk <= 8) FSGS_TOPK3(8);
  else FSGS_TOPK3(16);
#undef FSGS_TOPK3
  return check_launch("gaussian_topk_weights");
}

FSGS_API int fsgs_gaussian_rasterize_extra_forward(int P, int W, int H, int E, const float* extras,
    const float* means2D, const float* conic_opacity, const int64_t* ranges, const int32_t* point_list,
    const int32_t* n_contrib, float* out_pixels, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0 && E > 0, "gaussian_rasterize_extra_forward: bad sizes");
  FSGS_REQUIRE(ranges && n_contrib && out_pixels, "gaussian_rasterize_extra_forward: null pointer");
  FSGS_REQUIRE(P == 0 || (extras && means2D && conic_opacity && point_list),
               "gaussian_rasterize_extra_forward: null pointer");
  FSGS_REQUIRE((E & 3) != 0 || (reinterpret_cast<uintptr_t>(out_pixels) & 15) == 0,
               "gaussian_rasterize_extra_forward: out_pixels must be 16-byte aligned");
  hipStream_t s = (hipStream_t) stream;
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const int* tile_order = nullptr;
  const int flags = launch_tile_order(gx, gy, ranges, s, &tile_order);
  const dim3 block(kBlendThreads);
#define FSGS_G3_EXTRA(CC)                                                                                          \
  hipLaunchKernelGGL((gs3d_extra_forward_kernel<CC>), dim3(gx * gy, (E + CC - 1) / CC), block, 0, s, flags, tile_order, W, H,  \
                     E, ranges, point_list, (const float2*) means2D, (const float4*) conic_opacity, n_contrib,     \
                     extras, out_pixels)
  if (E <= 8) FSGS_G3_EXTRA(8);
  else FSGS_G3_EXTRA(16);
#undef FSGS_G3_EXTRA
  return check_launch("gaussian_rasterize_extra_forward");
}

FSGS_API int fsgs_gaussian_rasterize_extra_backward(int P, int W, int H, int E, const float* extras,
    const float* out_opacity, const float* grad_out, const float* means2D, const float* conic_opacity,
    const int64_t* ranges, const int32_t* point_list, const int32_t* n_contrib, float* grad_extras,
    float* grad_means2D, float* grad_conic_opacity, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0 && E > 0, "gaussian_rasterize_extra_backward: bad sizes");
  if (P == 0 || (!grad_extras && !grad_means2D && !grad_conic_opacity)) return kOk;
  FSGS_REQUIRE(extras && out_opacity && grad_out && means2D && conic_opacity && ranges && point_list && n_contrib,
               "gaussian_rasterize_extra_backward: null pointer");
  hipStream_t s = (hipStream_t) stream;
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const int* tile_order = nullptr;
  const int flags = launch_tile_order(gx, gy, ranges, s, &tile_order);
  hipLaunchKernelGGL(gs3d_extra_backward_kernel, dim3(gx * gy, (E + 7) / 8), dim3(kBlendThreads), 0, s, flags, tile_order, W, H, E,
                     ranges, point_list, (const float2*) means2D, (const float4*) conic_opacity, out_opacity,
                     n_contrib, extras, grad_out, grad_means2D, grad_conic_opacity, grad_extras);
  return check_launch("gaussian_rasterize_extra_backward");
}
