// Per-tile back-to-front backward pass of the 2D-Gaussian-surfel alpha blend for gfx950.
//
// Reference behaviour reproduced: fast_2d_gs/_C/src/gaussian_splatting/gs_2d_redner.cu:238-539 (kernel) and :631-717
// (host entry GS_2D_render_backward). The transmittance is rebuilt by division T <- T / (1 - alpha) while walking the
// tile's list backwards, gradient channels consumed are image, opacity, aux 0-5 (depth, normal, median depth,
// distortion) and optional flow; the 0.99 alpha clamp is not masked in the gradient, as in the reference.
//
// Where the reference issues 18-21 global float atomics per (pixel, surfel) pair, this kernel splits the work of a pair
// into the part that depends on the order of the pixel's list and the part that does not:
//   1. order-bound, one wavefront per 8x8 pixel quadrant, one list entry per pass: the ray-splat intersection and the
//      pixel's back-to-front recurrences. A pixel that blends the entry leaves three numbers (blend weight,
//      G * dL/dalpha, dL/ddepth) and its (pixel, entry) pair in the wavefront's queue in LDS. Few lanes of a pass blend
//      (a quarter on the benchmark scene), so this part is kept as short as the recurrences allow.
//   2. order-free, all 64 lanes busy: the wavefront takes 64 queued pairs at a time -- an entry's pairs padded to a
//      16-lane row -- recomputes the two planes through the pixel from the staged record, forms the 16 + 2 gradient
//      components and sums them over each row with DPP row shifts (no LDS traffic); each row adds its 16 totals to the
//      entry's row of the wavefront's accumulator in LDS.
//   3. per staged batch the four wavefronts' accumulators are added in wavefront order and every staged (surfel, tile)
//      instance writes one record at its position in surfel order; slot_reduce_kernel sums a surfel's records in a
//      fixed order. (Without scan offsets: one global atomic per surfel, component and tile, as the reference's sums.)
// Surfels behind the deepest contributor of the whole tile are never gathered. The optical-flow instantiation keeps
// parts 1 and 2 in one pass per entry (its extra per-pair terms would double the queue record).
#include <algorithm>

#include "blend.hpp"
#include "pair_queue.hpp"

namespace fsgs {
namespace {

// Per-surfel gradient slots: 0-2 colours | 3-11 trans_mat | 12-14 normal | 15 opacity | 16-17 means2D.
// The first 16 go through one transposed row reduction; the means2D pair is only non-zero for pixels where the
// screen-space low-pass filter wins (rho2d < rho3d) and is reduced separately when any lane took that branch.
constexpr int kGradSlots = 18;
#ifndef FSGS_BWD_BATCH
#define FSGS_BWD_BATCH 64
#endif
#ifndef FSGS_BWD_WAVES
#define FSGS_BWD_WAVES 4
#endif
constexpr int kBwdBatch = FSGS_BWD_BATCH;  // surfels staged per round
static_assert(kBwdBatch == kWave, "one wavefront stages a batch, another flushes it, and a queued pair names its entry in 6 bits");
// the two-pass form (queue of blended pairs per wavefront, pair_queue.hpp) can be switched off at build time
#ifndef FSGS_BWD_QUEUE
#define FSGS_BWD_QUEUE 1
#endif
constexpr bool kBwdQueue = FSGS_BWD_QUEUE != 0;

template <bool kAux, bool kFlow, bool kSlots>
__global__ void __launch_bounds__(kBlendThreads) __attribute__((amdgpu_waves_per_eu(FSGS_BWD_WAVES, FSGS_BWD_WAVES)))
blend_backward_kernel(
    int ordered, const int* __restrict__ tile_order, int W, int H, float near_n, float far_n, const int64_t* __restrict__ ranges, const int32_t* __restrict__ point_list,
    const int32_t* __restrict__ n_contrib, const float2* __restrict__ means2D,
    const float4* __restrict__ normal_opacity, const float* __restrict__ colors, const float* __restrict__ trans_mat,
    const float* __restrict__ trans_mat_t2, const float* __restrict__ out_opacity, const float* __restrict__ out_extras,
    const float2* __restrict__ out_flow, const float* __restrict__ dL_dpix, const float* __restrict__ dL_dextras,
    const float* __restrict__ dL_dopacity, const float2* __restrict__ dL_dflow, float* __restrict__ g_means2D,
    float* __restrict__ g_normal_opacity, float* __restrict__ g_colors, float* __restrict__ g_trans,
    const int64_t* __restrict__ point_offsets, const int32_t* __restrict__ radii, float* __restrict__ slot_grads,
    const float4* __restrict__ records) {
  constexpr bool kQueue = kBwdQueue && !kFlow;
  __shared__ SplatHot s_hot[kBwdBatch];
  __shared__ SplatCold s_cold[kBwdBatch];
  // Each wavefront's sums over its 64 pixels, one row per staged surfel; the flush adds the four rows in wavefront
  // order, so a tile's sums do not depend on timing. +1: the odd stride keeps the flush free of bank conflicts.
  __shared__ float s_part[4][kBwdBatch][kGradSlots + 1];
  // Where a staged (surfel, tile) instance's sums go: its position in surfel order (kSlots) or the surfel's id. Two
  // copies by batch parity: wavefront 1 stages batch b + 1 while wavefront 0 still flushes batch b.
  __shared__ int s_slot[2][kBwdBatch];
  __shared__ float s_t2[kFlow ? kBwdBatch * 9 : 1];
  __shared__ int s_max_contrib;
  __shared__ unsigned char s_mask[kBwdBatch];  // which 8x8 quadrants of the tile each staged surfel can reach
  // queued pairs
  __shared__ float4 s_queue[kQueue ? 4 : 1][kQueue ? kQueueItems : 1];

  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const int tile = scheduled_tile(ordered, tile_order), tile_x = tile % gx, tile_y = tile / gx;
  int px, py;
  lane_pixel(tile_x, tile_y, px, py);
  const bool inside = px < W && py < H;
  const size_t HW   = (size_t) H * W;
  const size_t pix  = (size_t) W * py + px;
  const float pxf = (float) px, pyf = (float) py;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

  const int64_t r0 = ranges[2 * (size_t) tile], r1 = ranges[2 * (size_t) tile + 1];
  const int last_contrib   = inside ? n_contrib[pix] : 0;
  const int median_contrib = (kAux && inside) ? n_contrib[pix + HW] : 0;

  // deepest list position any pixel of the tile blended: nothing behind it needs to be gathered
  if (threadIdx.x == 0) s_max_contrib = 0;
  __syncthreads();
  int wave_max_contrib = last_contrib;  // deepest position blended by this wavefront's quadrant
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) wave_max_contrib = max(wave_max_contrib, __shfl_xor(wave_max_contrib, d, kWave));
  if (lane == 0) atomicMax(&s_max_contrib, wave_max_contrib);
  for (int e = threadIdx.x; e < 4 * kBwdBatch * (kGradSlots + 1); e += kBlendThreads) (&s_part[0][0][0])[e] = 0.0f;
  __syncthreads();
  const int n_todo = min(s_max_contrib, (int) (r1 - r0));  // positions [0, n_todo) of the tile's list, walked from n_todo-1 down to 0
  const int rounds = (n_todo + kBwdBatch - 1) / kBwdBatch;
  // No zero fill of the records: the instances behind the tile's deepest contributor are never staged, their records
  // are cleared here; every staged instance writes its record at the flush, zeros included
  if (kSlots) {
    for (int e = n_todo + (int) threadIdx.x; e < (int) (r1 - r0); e += kBlendThreads) {
      const int id = point_list[r0 + e];
      float cx, cy;
      int rad;
      int64_t off;
      if (records) {
        const float4 q2 = records[5 * (size_t) id + 2], q4 = records[5 * (size_t) id + 4];
        cx = q2.y, cy = q2.z, rad = __float_as_int(q4.z), off = (int64_t) __float_as_int(q4.w);
        if (rad < 0) rad = radii[id];  // a record packed without radii / offsets holds -1 there
        if (off < 0) off = id == 0 ? 0 : point_offsets[id - 1];
      } else {
        const float2 c = means2D[id];
        cx = c.x, cy = c.y, rad = radii[id], off = id == 0 ? 0 : point_offsets[id - 1];
      }
      const TileRect r = tile_rect(cx, cy, rad, gx, gy);
      const int64_t slot = off + (int64_t) (tile_y - r.y0) * (r.x1 - r.x0) + (tile_x - r.x0);
      float2* dst = (float2*) (slot_grads + (size_t) slot * kGradSlots);
#pragma unroll
      for (int c = 0; c < kGradSlots / 2; ++c) dst[c] = make_float2(0.0f, 0.0f);
    }
  }

  const float T_final = inside ? 1.0f - out_opacity[pix] : 0.0f;
  float T = T_final;
  float dLp0 = 0, dLp1 = 0, dLp2 = 0;
  float dL_dreg = 0, dL_ddepth = 0, dL_daccum = 0, dLn0 = 0, dLn1 = 0, dLn2 = 0, dL_dmedian = 0;
  float final_D = 0, final_D2 = 0, sum_w = 0;
  if (inside) {
    dLp0 = dL_dpix[pix], dLp1 = dL_dpix[pix + HW], dLp2 = dL_dpix[pix + 2 * HW];
    if (kAux) {
      dL_daccum  = dL_dopacity[pix];
      dL_ddepth  = dL_dextras[pix + 0 * HW];
      dLn0       = dL_dextras[pix + 1 * HW];
      dLn1       = dL_dextras[pix + 2 * HW];
      dLn2       = dL_dextras[pix + 3 * HW];
      dL_dmedian = dL_dextras[pix + 4 * HW];
      dL_dreg    = dL_dextras[pix + 5 * HW];
      final_D    = out_extras[pix + 6 * HW];
      final_D2   = out_extras[pix + 7 * HW];
      sum_w      = out_extras[pix + 8 * HW];
    }
  }
  const float far_scale = far_n / (far_n - near_n), far_near = far_scale * near_n;
  // The distortion term's per-pixel constants, folded once: with m the normalised depth of a pair,
  //   dL/dweight = (D2 + m^2 A - 2 m D) dL/dreg = D2 dL/dreg + m (m reg_A - reg_2D),
  //   dL/dm      = 2 w (m A - D) dL/dreg        = w (m reg_2A - reg_2D).
  const float reg_A = (1.0f - T_final) * dL_dreg, reg_2A = 2.0f * reg_A, reg_2D = 2.0f * final_D * dL_dreg,
              lin_const = final_D2 * dL_dreg + dL_daccum;  // dL/dweight's constant and the opacity map's gradient
  float dLf0 = 0, dLf1 = 0, dL_dsum_w = 0;
  if (kFlow && inside) {
    const float2 g = dL_dflow[pix], o = out_flow[pix];
    dL_dsum_w = -(g.x * o.x + g.y * o.y) / (sum_w * sum_w);
    dLf0 = g.x / sum_w, dLf1 = g.y / sum_w;
  }

  float acc_lin = 0;
  float last_alpha = 0, acc_w = 0;
  float acc_f0 = 0, acc_f1 = 0, last_f0 = 0, last_f1 = 0;
  PairQueue q;                                 // the wavefront's queue of blended pairs
  const int row_shift = (lane >> 4) * 8;       // this lane's byte of the four rows of a pass
  const float qx0 = (float) (tile_x * kTile + (wave & 1) * 8), qy0 = (float) (tile_y * kTile + (wave >> 1) * 8);

  Splat next;
  float next_t2[9];
  int next_radius = 0;
  int64_t next_off = 0;
  // Gathering and staging are wavefront 1's job, the flush of a finished batch wavefront 0's: both sit between the same
  // two barriers, where the other wavefronts wait, and so run side by side instead of one after the other.
  const int st = (int) threadIdx.x - kWave;  // staging slot of this lane (wavefront 1: 0 .. 63)
  if (st >= 0 && st < min(n_todo, kBwdBatch)) {
    SplatExtra ex;
    next = gather_splat(point_list[r0 + (n_todo - 1 - st)], means2D, colors, normal_opacity, trans_mat,
                        records, &ex);
    if (kFlow)
#pragma unroll
      for (int k = 0; k < 9; ++k) next_t2[k] = trans_mat_t2[9 * (size_t) next.cold.id + k];
    if (kSlots) {
      // a record carries the surfel's radius (-1 if it was packed without radii) and, once the binning's scan has
      // stored it, its offset (-1 until then)
      next_radius = records && ex.radius >= 0 ? ex.radius : radii[next.cold.id];
      next_off    = records && ex.offset >= 0 ? ex.offset : (next.cold.id == 0 ? 0 : point_offsets[next.cold.id - 1]);
    }
  }

  for (int b = 0; b < rounds; ++b) {
    const int n_here = min(kBwdBatch, n_todo - b * kBwdBatch);
    if (st >= 0 && st < n_here) {
      s_hot[st]  = next.hot;
      s_cold[st] = next.cold;
      s_mask[st] = (unsigned char) quadrant_mask(next.hot, tile_x * kTile, tile_y * kTile, ordered);
      if (kFlow)
#pragma unroll
        for (int k = 0; k < 9; ++k) s_t2[st * 9 + k] = next_t2[k];
      if (kSlots) {
        // position of this instance in the surfel-ordered key list: the binning emits a surfel's tiles row-major
        // over its rectangle, starting at the surfel's prefix-scan offset (gaussian_prepare.cu:47-83)
        const TileRect r = tile_rect(next.hot.cx, next.hot.cy, next_radius, gx, gy);
        s_slot[b & 1][st] = (int) (next_off + (int64_t) (tile_y - r.y0) * (r.x1 - r.x0) + (tile_x - r.x0));
      } else {
        s_slot[b & 1][st] = next.cold.id;
      }
    }
    __syncthreads();
    const int nxt = (b + 1) * kBwdBatch + st;
    if (st >= 0 && st < kBwdBatch && nxt < n_todo) {
      SplatExtra ex;
      next = gather_splat(point_list[r0 + (n_todo - 1 - nxt)], means2D, colors, normal_opacity, trans_mat, records,
                          &ex);
      if (kFlow)
#pragma unroll
        for (int k = 0; k < 9; ++k) next_t2[k] = trans_mat_t2[9 * (size_t) next.cold.id + k];
      if (kSlots) {
        next_radius = records && ex.radius >= 0 ? ex.radius : radii[next.cold.id];
        next_off    = records && ex.offset >= 0 ? ex.offset : (next.cold.id == 0 ? 0 : point_offsets[next.cold.id - 1]);
      }
    }

    // Work list of this wavefront for the staged surfels: those that can reach its quadrant and are not behind its
    // deepest contributor; consumed bit by bit with scalar instructions.
    unsigned long long todo = __ballot(lane < n_here && ((s_mask[lane] >> wave) & 1u) &&
                                       (n_todo - 1 - (b * kBwdBatch + lane)) < wave_max_contrib);
    // ---- order-bound part of one (pixel, entry) pair: advances the pixel's back-to-front state -------------------------
    // All channels that enter the image linearly (colour, depth, opacity, normal) share one recurrence: with
    // c = <upstream gradient, channel values of this surfel>, the reference's per-channel accumulators
    // acc_x = last_alpha * last_x + (1 - last_alpha) * acc_x contract to a single scalar, updated at the end of the
    // pair that supplies alpha and x. Leaves the blend weight w, dL/dalpha and dL/ddepth of the pair; call under `hit`
    // only.
    auto advance_pixel = [&](const SplatCold& cold, int pos, const Hit& h, float& w, float& dL_dalpha, float& dL_dz) {
      const float keep = 1.0f - h.alpha;
      T = T * __builtin_amdgcn_rcpf(keep);
      w = h.alpha * T;
      // one chain of fused multiply-adds; the per-pixel constant of the distortion term sits in lin_const
      float c_lin;
      if (kAux) {
        const float rd     = __builtin_amdgcn_rcpf(h.depth);
        const float m_d    = fmaf(-far_near, rd, far_scale);
        const float dmd_dd = far_near * rd * rd;
        // dL/dweight of the distortion enters dL/dalpha exactly as a linear channel does (its own value minus what the
        // pairs behind it accumulated, with the same weights), so it rides on the shared recurrence
        c_lin = fmaf(h.depth, dL_ddepth, lin_const);
        c_lin = fmaf(m_d, fmaf(m_d, reg_A, -reg_2D), c_lin);
        c_lin = fmaf(cold.nx, dLn0, fmaf(cold.ny, dLn1, fmaf(cold.nz, dLn2, c_lin)));
        // dL/ddepth: through the distortion's normalised depth, the depth map, and the median depth
        const float per_w = fmaf(fmaf(m_d, reg_2A, -reg_2D), dmd_dd, dL_ddepth);
        dL_dz = fmaf(w, per_w, pos == median_contrib - 1 ? dL_dmedian : 0.0f);
      } else {
        c_lin = 0.0f;
      }
      c_lin = fmaf(cold.r, dLp0, fmaf(cold.g, dLp1, fmaf(cold.b, dLp2, c_lin)));
      // acc_lin: what the pairs behind this one accumulated, alpha_j c_j weighted by the transmittance between
      dL_dalpha = c_lin - acc_lin;
      acc_lin   = fmaf(keep, acc_lin, h.alpha * c_lin);
    };
    if (kQueue) {
      // ---- order-free part: 64 queued pairs at a time, four 16-lane rows, every row one entry ---------------------------
      // A lane rebuilds the two planes through its pair's pixel from the staged record and forms the 16 + 2 components
      // as products of the three queued numbers with quantities that are finite in every lane (padding items carry
      // zeros and no flags, and the reciprocal of p_z is only taken under the pair's flags), so no component needs a
      // zero of its own; the projected-centre case is the intersection case with a zero in place of 1 / p_z.
      auto drain = [&](int n_valid) {
        // the entries of the four rows come from the wavefront's scalar bookkeeping, so the queued item, the staged
        // record and the accumulator row are requested together (one LDS round trip instead of three in a chain)
        const unsigned jrows = queue_front_rows(q);  // byte r = entry of row r
        const int j = (int) ((jrows >> row_shift) & 63u);
        const float4 it = s_queue[wave][q.head + lane];
        const SplatHot hot = s_hot[j];
        float* const acc = &s_part[wave][j][lane & 15];
        const float before = *acc;
        const int bits = __float_as_int(it.w);
        const int qp = bits & 63;
        const bool blends = (bits & kItemHit) != 0, by_ray = (bits & kItemRay) != 0;
        // the upstream gradients of the pair's pixel sit in the registers of the lane that owns it (lane qp of this
        // wavefront): fetched with lane permutes, no LDS copy of them is kept
        auto from_owner = [&](float v) {
          return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(qp << 2, __builtin_bit_cast(int, v)));
        };
        const float up_x = from_owner(dLp0), up_y = from_owner(dLp1), up_z = from_owner(dLp2);
        const float fx = qx0 + (float) (qp & 7), fy = qy0 + (float) (qp >> 3);
        const float w = it.x, GdA = it.y, dL_dz = it.z;
        const float kx = fx * hot.m[6] - hot.m[0], ky = fx * hot.m[7] - hot.m[1], kz = fx * hot.m[8] - hot.m[2];
        const float lx = fy * hot.m[6] - hot.m[3], ly = fy * hot.m[7] - hot.m[4], lz = fy * hot.m[8] - hot.m[5];
        const float p_x = ky * lz - kz * ly, p_y = kz * lx - kx * lz, p_z = kx * ly - ky * lx;
        const float rz_s = blends ? __builtin_amdgcn_rcpf(p_z) : 0.0f;  // s is used by both cases of a blending pair
        const float rz_p = by_ray ? rz_s : 0.0f;                         // d/dp only by the intersection case
        const float sx = p_x * rz_s, sy = p_y * rz_s;
        const float oG = hot.opacity * GdA;
        float dsx = -(oG * sx), dsy = -(oG * sy);
        if (kAux) dsx += dL_dz * hot.m[6], dsy += dL_dz * hot.m[7];
        const float s_ds = dsx * sx + dsy * sy;
        // d/dp of the homogeneous intersection point p = k x l, negated (the components below are minus the plane
        // gradients): p_xy = s p_z, so dp_xy = ds / p_z and dp_z = -<ds, s> / p_z
        const float npx = -(dsx * rz_p), npy = -(dsy * rz_p), npz = s_ds * rz_p;
        float g[16];
        g[0] = w * up_x, g[1] = w * up_y, g[2] = w * up_z;
        g[3] = ly * npz - lz * npy, g[4] = lz * npx - lx * npz, g[5] = lx * npy - ly * npx;
        g[6] = npy * kz - npz * ky, g[7] = npz * kx - npx * kz, g[8] = npx * ky - npy * kx;
        g[9]  = dL_dz * sx - (fx * g[3] + fy * g[6]);
        g[10] = dL_dz * sy - (fx * g[4] + fy * g[7]);
        g[11] = dL_dz - (fx * g[5] + fy * g[8]);
        if (kAux) {
          g[12] = w * from_owner(dLn0), g[13] = w * from_owner(dLn1), g[14] = w * from_owner(dLn2);
        } else {
          g[12] = g[13] = g[14] = 0.0f;
        }
        g[15] = GdA;
        // lane (row, c) holds the row's total of component c
        queue_accumulate(acc, before, row_sum16_transposed(g), jrows, n_valid, true);
        const bool filtered = blends && !by_ray;
        if (wave_ballot(filtered) != 0ull) {  // some pair met its surfel by the projected centre
          const float to_centre = filtered ? -2.0f * oG : 0.0f;
          float cx = to_centre * (hot.cx - fx), cy = to_centre * (hot.cy - fy);  // totals of a row end up in its lane 15
          cx += dpp_shift_zero<0x111, 0xf, 0xf>(cx), cy += dpp_shift_zero<0x111, 0xf, 0xf>(cy);
          cx += dpp_shift_zero<0x112, 0xf, 0xf>(cx), cy += dpp_shift_zero<0x112, 0xf, 0xf>(cy);
          cx += dpp_shift_zero<0x114, 0xf, 0xf>(cx), cy += dpp_shift_zero<0x114, 0xf, 0xf>(cy);
          cx += dpp_shift_zero<0x118, 0xf, 0xf>(cx), cy += dpp_shift_zero<0x118, 0xf, 0xf>(cy);
          if ((lane >> 4) < ((n_valid + 15) >> 4) && (lane & 15) == 15)
            atomicAdd(&s_part[wave][j][16], cx), atomicAdd(&s_part[wave][j][17], cy);
        }
        queue_pop(q, n_valid);
      };
      // ---- order-bound part of one entry, and the append of its blending pixels to the queue -----------------------------
      auto queue_entry = [&](const SplatHot& hot, const SplatCold& cold, int j) {
        const int pos = n_todo - 1 - (b * kBwdBatch + j);  // 0-based position in the tile's list
        Hit h;
        unsigned long long pass;
        const bool hit = intersect_flat(hot, pxf, pyf, near_n, h, &pass) && (pos < last_contrib);
        pass &= wave_ballot(pos < last_contrib);
        if (pass == 0ull) return;  // wave-uniform: nobody in this quadrant blends the surfel
        float w = 0.0f, dL_dalpha = 0.0f, dL_dz = 0.0f;
        if (hit) {
          advance_pixel(cold, pos, h, w, dL_dalpha, dL_dz);
          dL_dalpha *= T * h.G;  // only G * dL/dalpha is ever used
        }
        const int flags = h.rho3d <= h.rho2d ? (kItemHit | kItemRay) : kItemHit;
        if (queue_append(s_queue[wave], q, j, hit, pass, w, dL_dalpha, dL_dz, flags)) drain(kWave);
      };
      if (todo != 0ull) {
        auto pop = [&]() {
          const int j = __builtin_ctzll(todo);
          todo &= todo - 1;
          return j;
        };
        auto peek = [&]() { return todo ? (int) __builtin_ctzll(todo) : 0; };
        SplatHot hot_a = s_hot[peek()], hot_b;
        while (todo) {
          {
            const int j = pop();
            hot_b       = s_hot[peek()];
            const SplatCold cold = s_cold[j];
            __builtin_amdgcn_sched_barrier(0);
            queue_entry(hot_a, cold, j);
          }
          if (todo == 0ull) break;
          {
            const int j = pop();
            hot_a       = s_hot[peek()];
            const SplatCold cold = s_cold[j];
            __builtin_amdgcn_sched_barrier(0);
            queue_entry(hot_b, cold, j);
          }
        }
        if (q.count > 0) drain(q.count);  // the staged records are replaced after the next barrier
      }
    } else {
     // Gradient terms of one (pixel, entry) pair, formed in the pass that advances the pixel. The part under `hit` leaves
     // a few factors (zero for a lane whose pixel does not blend the entry); the 16 + 2 per-surfel components are
     // products of those factors with quantities that are finite in every lane, formed by all lanes alike, so no
     // component needs a zero of its own and the two ways a surfel is met (ray-splat intersection / projected centre)
     // share one instruction stream.
     auto pair_gradients = [&](const SplatHot& hot, const SplatCold& cold, int j, int pos, const Hit& h, bool hit,
                               float (&g)[16], float& g2x, float& g2y, unsigned long long& ray_lanes) {
       float w = 0.0f, dL_dalpha = 0.0f, dL_dz = 0.0f, dsx = 0.0f, dsy = 0.0f, s_ds = 0.0f, z_sx = 0.0f, z_sy = 0.0f;
       if (hit) {
         advance_pixel(cold, pos, h, w, dL_dalpha, dL_dz);
         if (kAux) dsx = dL_dz * hot.m[6], dsy = dL_dz * hot.m[7];
         if (kFlow) {
           const float* Q = &s_t2[j * 9];
           const float u2 = Q[0] * h.sx + Q[1] * h.sy + Q[2];
           const float v2 = Q[3] * h.sx + Q[4] * h.sy + Q[5];
           float w2       = Q[6] * h.sx + Q[7] * h.sy + Q[8];
           w2             = fabsf(w2) < 1e-5f ? 1e-5f : w2;
           acc_f0 = last_alpha * last_f0 + (1.0f - last_alpha) * acc_f0;
           acc_f1 = last_alpha * last_f1 + (1.0f - last_alpha) * acc_f1;
           last_f0 = u2 / w2 - pxf, last_f1 = v2 / w2 - pyf;
           dL_dalpha += (last_f0 - acc_f0) * dLf0 + (last_f1 - acc_f1) * dLf1;
           const float gu = w / w2 * dLf0, gv = w / w2 * dLf1;
           const float gw = -w / (w2 * w2) * (u2 * dLf0 + v2 * dLf1);
           dsx += Q[0] * gu + Q[3] * gv + Q[6] * gw;
           dsy += Q[1] * gu + Q[4] * gv + Q[7] * gw;
           acc_w = last_alpha + (1.0f - last_alpha) * acc_w;
           dL_dalpha += (1.0f - acc_w) * dL_dsum_w;
         }
         dL_dalpha *= T;
         last_alpha = h.alpha;
         // the Gaussian's own part of d/ds: only the intersection case uses it (times 1 / p_z below)
         const float dL_dG = hot.opacity * dL_dalpha;
         dsx += dL_dG * -h.G * h.sx;
         dsy += dL_dG * -h.G * h.sy;
         // s is not finite in a lane whose plane pair degenerates (p_z == 0), and such a lane never blends: every use
         // of s sits on this side
         s_ds = dsx * h.sx + dsy * h.sy;
         z_sx = dL_dz * h.sx, z_sy = dL_dz * h.sy;
       }
       const bool by_ray   = h.rho3d <= h.rho2d;
       const bool filtered = hit && !by_ray;
       ray_lanes           = wave_ballot(by_ray);  // taken where the comparison is made: its own lane mask, no instruction
       // d/dp of the homogeneous intersection point p = k x l, negated (the components below are minus the plane
       // gradients): p_xy = s p_z, so dp_xy = ds / p_z and dp_z = -<ds, s> / p_z
       const float rz  = (hit && by_ray) ? __builtin_amdgcn_rcpf(h.pz) : 0.0f;
       const float npx = -(dsx * rz), npy = -(dsy * rz), npz = s_ds * rz;
       const float nkx = h.ly * npz - h.lz * npy, nky = h.lz * npx - h.lx * npz, nkz = h.lx * npy - h.ly * npx;
       const float nlx = npy * h.kz - npz * h.ky, nly = npz * h.kx - npx * h.kz, nlz = npx * h.ky - npy * h.kx;
       g[0] = w * dLp0, g[1] = w * dLp1, g[2] = w * dLp2;
       g[3] = nkx, g[4] = nky, g[5] = nkz;
       g[6] = nlx, g[7] = nly, g[8] = nlz;
       g[9]  = z_sx - (pxf * nkx + pyf * nlx);
       g[10] = z_sy - (pxf * nky + pyf * nly);
       g[11] = dL_dz - (pxf * nkz + pyf * nlz);
       if (kAux) g[12] = w * dLn0, g[13] = w * dLn1, g[14] = w * dLn2;
       else      g[12] = g[13] = g[14] = 0.0f;
       g[15] = h.G * dL_dalpha;
       const float to_centre = filtered ? hot.opacity * dL_dalpha * (-2.0f * h.G) : 0.0f;
       g2x = to_centre * h.dx, g2y = to_centre * h.dy;
     };
     auto backward_entry = [&](const SplatHot& hot, const SplatCold& cold, int j) {
      const int pos = n_todo - 1 - (b * kBwdBatch + j);  // 0-based position in the tile's list
      Hit h;
      unsigned long long pass;
      const bool hit = intersect_flat(hot, pxf, pyf, near_n, h, &pass) && (pos < last_contrib);
      pass &= wave_ballot(pos < last_contrib);
      if (pass == 0ull) return;  // wave-uniform: nobody in this quadrant blends the surfel

      float g[16], g2x, g2y;
      unsigned long long ray_lanes;
      pair_gradients(hot, cold, j, pos, h, hit, g, g2x, g2y, ray_lanes);
      const float tot = wave_sum16_transposed(g);
      if (lane < 16) s_part[wave][j][lane] = tot;  // a wavefront meets an entry once per batch: a plain store
      if ((pass & ~ray_lanes) != 0ull) {  // some lane met the surfel by its projected centre
        const float sx = wave_sum_to_lane63(g2x), sy = wave_sum_to_lane63(g2y);
        if (lane == 63) s_part[wave][j][16] = sx, s_part[wave][j][17] = sy;
      }
     };
     // The record of the next entry is requested before the current one is evaluated (alternating registers): a
     // wavefront walks its list alone, so an exposed LDS round trip per entry sits on the tile's critical path.
     if (todo != 0ull) {
      auto pop = [&]() {
        const int j = __builtin_ctzll(todo);
        todo &= todo - 1;
        return j;
      };
      auto peek = [&]() { return todo ? (int) __builtin_ctzll(todo) : 0; };
      SplatHot hot_a = s_hot[peek()], hot_b;
      while (todo) {
        {
          const int j = pop();
          hot_b       = s_hot[peek()];
          const SplatCold cold = s_cold[j];
          __builtin_amdgcn_sched_barrier(0);
          backward_entry(hot_a, cold, j);
        }
        if (todo == 0ull) break;
        {
          const int j = pop();
          hot_a       = s_hot[peek()];
          const SplatCold cold = s_cold[j];
          __builtin_amdgcn_sched_barrier(0);
          backward_entry(hot_b, cold, j);
        }
      }
     }
    }
    __syncthreads();
    // flush the batch (wavefront 0: lane = staged surfel), adding the four wavefronts' rows in wavefront order
    if ((int) threadIdx.x < n_here) {
      float a[kGradSlots];
#pragma unroll
      for (int c = 0; c < kGradSlots; ++c) {
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) sum += s_part[w][threadIdx.x][c], s_part[w][threadIdx.x][c] = 0.0f;
        a[c] = sum;
      }
      if (kSlots) {
        // One 72-byte record per (surfel, tile) instance at the instance's position in surfel order; the per-surfel
        // sums are taken afterwards by slot_reduce_kernel. Every staged instance writes its record, zeros included (the
        // instances that are never staged were cleared at the start), so nobody has to clear the buffer beforehand. A
        // streaming zero fill of all records in front of this kernel took 13 us; the extra stores here move about as
        // many bytes (partial lines are written back more than once) but ride on memory pipes this kernel leaves
        // idle: operator 0.442 -> 0.434 ms. (Also measured, and slower than the fill: a "written" byte per instance
        // with the sum skipping unwritten records, 0.505 ms against 0.488 ms for the operator.)
        {
          float2* dst = (float2*) (slot_grads + (size_t) s_slot[b & 1][threadIdx.x] * kGradSlots);
#pragma unroll
          for (int c = 0; c < kGradSlots / 2; ++c) dst[c] = make_float2(a[2 * c], a[2 * c + 1]);
        }
      } else {
        // one global atomic per surfel and component for this tile
        const int id = s_slot[b & 1][threadIdx.x];
#pragma unroll
        for (int c = 0; c < 3; ++c)
          if (a[c] != 0.0f) atomicAdd(&g_colors[3 * (size_t) id + c], a[c]);
#pragma unroll
        for (int c = 0; c < 9; ++c)
          if (a[3 + c] != 0.0f) atomicAdd(&g_trans[9 * (size_t) id + c], a[3 + c]);
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (a[12 + c] != 0.0f) atomicAdd(&g_normal_opacity[4 * (size_t) id + c], a[12 + c]);
#pragma unroll
        for (int c = 0; c < 2; ++c)
          if (a[16 + c] != 0.0f) atomicAdd(&g_means2D[2 * (size_t) id + c], a[16 + c]);
      }
    }
    // No barrier needed here: between this flush and the barrier that follows the next batch's LDS store, wavefront 0
    // touches its lanes' rows of s_part and this batch's copy of s_slot, wavefront 1 the staging arrays and the other
    // copy of s_slot.
  }
}

// Per-surfel sums of the instance records. Nine lanes per surfel, each owning one float2 of the 18-float record, so
// the lanes of a surfel read 72 contiguous bytes per record and neighbouring surfels continue where the previous one
// ends. A surfel's records are fetched eight at a time (past its last record the last one is read again and not added),
// so most surfels need one round trip to memory; the sum itself runs in instance order. Every row of the four outputs
// is written (zeros for surfels without instances): no initialisation, no atomics, and the sum order is fixed.
__global__ void __launch_bounds__(256) slot_reduce_kernel(int P, const int64_t* __restrict__ point_offsets,
    const float* __restrict__ slot_grads, float* __restrict__ g_colors, float* __restrict__ g_means2D,
    float* __restrict__ g_trans, float* __restrict__ g_normal_opacity) {
  constexpr int kPerWave = 7, kLanes = 9;  // 63 of 64 lanes busy
  constexpr int kDepth   = 8;              // records of one surfel in flight together
  const int lane = threadIdx.x & 63;
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int sub = lane / kLanes, k = lane - sub * kLanes;
  const int i = wave * kPerWave + sub;
  if (sub >= kPerWave || i >= P) return;
  // A surfel without instances (not rendered) has equal scan offsets, so the visibility need not be read.
  const int64_t e0 = i > 0 ? point_offsets[i - 1] : 0, e1 = point_offsets[i];
  const float2* src = (const float2*) slot_grads + k;
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
  // record layout: 0-2 colours | 3-11 trans_mat | 12-14 normal | 15 opacity | 16-17 means2D
  const float vals[2] = {acc.x, acc.y};
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int c = 2 * k + h;
    if (c < 3) g_colors[3 * (size_t) i + c] = vals[h];
    else if (c < 12) g_trans[9 * (size_t) i + (c - 3)] = vals[h];
    else if (c < 16) g_normal_opacity[4 * (size_t) i + (c - 12)] = vals[h];
    else g_means2D[2 * (size_t) i + (c - 16)] = vals[h];
  }
}

// The same sum over lists built by the culled binning (fsgs_gs_prepare_*_culled): the positions of a surfel's span
// whose bit is clear in its keep mask belong to no list, were never written and are not read. Nine positions of the
// span per step, row-major over the surfel's rectangle, the records of the kept ones requested together.
__global__ void __launch_bounds__(256) slot_reduce_culled_kernel(int P, const int64_t* __restrict__ point_offsets,
    const uint32_t* __restrict__ masks, const float* __restrict__ slot_grads, float* __restrict__ g_colors,
    float* __restrict__ g_means2D, float* __restrict__ g_trans, float* __restrict__ g_normal_opacity) {
  constexpr int kPerWave = 7, kLanes = 9;
  const int lane = threadIdx.x & 63;
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int sub = lane / kLanes, k = lane - sub * kLanes;
  const int i = wave * kPerWave + sub;
  if (sub >= kPerWave || i >= P) return;
  const int64_t e0 = i > 0 ? point_offsets[i - 1] : 0, e1 = point_offsets[i];
  const int count = (int) (e1 - e0);
  // rectangles above kCullMaskTiles tiles are kept whole
  const uint32_t mask = count > kCullMaskTiles ? 0xffffffffu : masks[i];
  const float2* src = (const float2*) slot_grads + (size_t) e0 * kLanes + k;
  float2 acc = make_float2(0.0f, 0.0f);
  for (int base = 0; base < count; base += kLanes) {
    const uint32_t bits = count > kCullMaskTiles ? 0xffffffffu : (mask >> base);
    float2 v[kLanes];
#pragma unroll
    for (int j = 0; j < kLanes; ++j)
      v[j] = (base + j < count && ((bits >> j) & 1u)) ? src[(size_t) (base + j) * kLanes] : make_float2(0.0f, 0.0f);
#pragma unroll
    for (int j = 0; j < kLanes; ++j) acc.x += v[j].x, acc.y += v[j].y;
  }
  const float vals[2] = {acc.x, acc.y};
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int c = 2 * k + h;
    if (c < 3) g_colors[3 * (size_t) i + c] = vals[h];
    else if (c < 12) g_trans[9 * (size_t) i + (c - 3)] = vals[h];
    else if (c < 16) g_normal_opacity[4 * (size_t) i + (c - 12)] = vals[h];
    else g_means2D[2 * (size_t) i + (c - 16)] = vals[h];
  }
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API size_t fsgs_gs_2d_render_backward_workspace_bytes(int64_t R) {
  return align_up((size_t) (R > 0 ? R : 0) * kGradSlots * 4 + 16, 256);
}

namespace {
// keep_masks: the lists come from fsgs_gs_prepare_*_culled, so the record sum has to skip the positions the binning left out
int render_backward(int P, int W, int H, double near_n, double far_n, const float* means2D,
    const float* normal_opacity, const float* colors, const float* trans_mat, const float* trans_mat_t2,
    const float* out_opacity, const float* out_extras, const float* out_flow, const float* dL_dpix,
    const float* dL_dopacity, const float* dL_dextras, const float* dL_dflow, const int64_t* ranges,
    const int32_t* point_list, const int32_t* n_contrib, float* g_colors, float* g_means2D, float* g_trans,
    float* g_normal_opacity, int64_t R, const int64_t* point_offsets, const int32_t* radii, void* workspace,
    size_t workspace_bytes, const float* records, const uint32_t* keep_masks, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0, "GS_2D_render_backward: bad sizes");
  if (P == 0) return kOk;
  FSGS_REQUIRE(means2D && normal_opacity && colors && trans_mat && out_opacity && dL_dpix && dL_dopacity && ranges &&
                   n_contrib && g_colors && g_means2D && g_trans && g_normal_opacity,
               "GS_2D_render_backward: null pointer");
  const bool aux  = out_extras && dL_dextras;
  const bool flow = dL_dflow != nullptr;
  FSGS_REQUIRE(!flow || (trans_mat_t2 && out_flow && aux),
               "GS_2D_render_backward: flow gradients need trans_mat_t2, out_flow and the auxiliary maps");
  FSGS_REQUIRE(((uintptr_t) records & 15) == 0, "GS_2D_render_backward: records must be 16-byte aligned");
  const bool slots = point_offsets != nullptr;
  if (slots) {
    FSGS_REQUIRE(radii && workspace && R >= 0 && R < (int64_t) 0x7fffffff,
                 "GS_2D_render_backward: the ordered-sum path needs radii, a workspace and the instance count R");
    if (workspace_bytes < fsgs_gs_2d_render_backward_workspace_bytes(R))
      return fail(kWorkspaceSmall, "GS_2D_render_backward: workspace %zu < %zu bytes", workspace_bytes,
                  fsgs_gs_2d_render_backward_workspace_bytes(R));
  }
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const dim3 grid(gx * gy), block(kBlendThreads);
  hipStream_t s = (hipStream_t) stream;
  float* slot_grads = slots ? (float*) workspace : nullptr;
  const int* tile_order = nullptr;
  const int ordered = launch_tile_order(gx, gy, ranges, s, &tile_order);
#define FSGS_LAUNCH_BWD(AUX, FLOW, SLOTS)                                                                            \
  hipLaunchKernelGGL((blend_backward_kernel<AUX, FLOW, SLOTS>), grid, block, 0, s, ordered, tile_order, W, H, (float) near_n,    \
                     (float) far_n, ranges, point_list, n_contrib, (const float2*) means2D,                          \
                     (const float4*) normal_opacity, colors, trans_mat, trans_mat_t2, out_opacity, out_extras,       \
                     (const float2*) out_flow, dL_dpix, dL_dextras, dL_dopacity, (const float2*) dL_dflow,           \
                     g_means2D, g_normal_opacity, g_colors, g_trans, point_offsets, radii, slot_grads,               \
                     (const float4*) records)
  if (slots) {
    if (aux && flow) FSGS_LAUNCH_BWD(true, true, true);
    else if (aux) FSGS_LAUNCH_BWD(true, false, true);
    else FSGS_LAUNCH_BWD(false, false, true);
    const int waves = div_up(P, 7);  // kPerWave surfels per wavefront
    if (keep_masks && culling_enabled())
      hipLaunchKernelGGL(slot_reduce_culled_kernel, dim3(div_up((int64_t) waves * 64, 256)), dim3(256), 0, s, P,
                         point_offsets, keep_masks, slot_grads, g_colors, g_means2D, g_trans, g_normal_opacity);
    else
      hipLaunchKernelGGL(slot_reduce_kernel, dim3(div_up((int64_t) waves * 64, 256)), dim3(256), 0, s, P, point_offsets,
                         slot_grads, g_colors, g_means2D, g_trans, g_normal_opacity);
  } else {
    if (aux && flow) FSGS_LAUNCH_BWD(true, true, false);
    else if (aux) FSGS_LAUNCH_BWD(true, false, false);
    else FSGS_LAUNCH_BWD(false, false, false);
  }
#undef FSGS_LAUNCH_BWD
  return check_launch("GS_2D_render_backward");
}
}  // namespace

FSGS_API int fsgs_gs_2d_render_backward(int P, int W, int H, double near_n, double far_n, const float* means2D,
    const float* normal_opacity, const float* colors, const float* trans_mat, const float* trans_mat_t2,
    const float* out_opacity, const float* out_extras, const float* out_flow, const float* dL_dpix,
    const float* dL_dopacity, const float* dL_dextras, const float* dL_dflow, const int64_t* ranges,
    const int32_t* point_list, const int32_t* n_contrib, float* g_colors, float* g_means2D, float* g_trans,
    float* g_normal_opacity, int64_t R, const int64_t* point_offsets, const int32_t* radii, void* workspace,
    size_t workspace_bytes, const float* records, void* stream) {
  return render_backward(P, W, H, near_n, far_n, means2D, normal_opacity, colors, trans_mat, trans_mat_t2, out_opacity,
                         out_extras, out_flow, dL_dpix, dL_dopacity, dL_dextras, dL_dflow, ranges, point_list, n_contrib,
                         g_colors, g_means2D, g_trans, g_normal_opacity, R, point_offsets, radii, workspace,
                         workspace_bytes, records, nullptr, stream);
}

FSGS_API int fsgs_gs_2d_render_backward_culled(int P, int W, int H, double near_n, double far_n, const float* means2D,
    const float* normal_opacity, const float* colors, const float* trans_mat, const float* trans_mat_t2,
    const float* out_opacity, const float* out_extras, const float* out_flow, const float* dL_dpix,
    const float* dL_dopacity, const float* dL_dextras, const float* dL_dflow, const int64_t* ranges,
    const int32_t* point_list, const int32_t* n_contrib, float* g_colors, float* g_means2D, float* g_trans,
    float* g_normal_opacity, int64_t R, const int64_t* point_offsets, const int32_t* radii, void* workspace,
    size_t workspace_bytes, const float* records, const uint32_t* keep_masks, void* stream) {
  FSGS_REQUIRE(P == 0 || !point_offsets || keep_masks,
               "GS_2D_render_backward_culled: the ordered-sum path over culled lists needs the keep masks");
  return render_backward(P, W, H, near_n, far_n, means2D, normal_opacity, colors, trans_mat, trans_mat_t2, out_opacity,
                         out_extras, out_flow, dL_dpix, dL_dopacity, dL_dextras, dL_dflow, ranges, point_list, n_contrib,
                         g_colors, g_means2D, g_trans, g_normal_opacity, R, point_offsets, radii, workspace,
                         workspace_bytes, records, keep_masks, stream);
}
