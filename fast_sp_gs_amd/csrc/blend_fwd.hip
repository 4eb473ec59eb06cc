// Per-tile front-to-back alpha blend of 2D Gaussian surfels for gfx950.
//
// Reference behaviour reproduced: fast_2d_gs/_C/src/gaussian_splatting/gs_2d_redner.cu:28-236 (kernel) and :541-629
// (host entry GS_2D_render_forward): colour, opacity, the 9 auxiliary maps (depth, normal xyz, median depth,
// distortion, M1, M2, weight sum), optional flow, n_contrib = (last contributor, median contributor), and the optional
// accum_max_count / accum_weights_p / accum_weights_count side outputs with their quirks (the arg-max flag is never
// reset once set, :180-197). The side outputs are sums over (pixel, surfel) pairs; the kernel forms them per wavefront
// or per pixel first and issues few atomics (see ArgmaxRun and the weight staging below) instead of up to three per
// pair.
//
// Layout: one 256-lane block per 16x16 tile; wavefront w owns an 8x8 pixel quadrant. Surfels of the tile's sorted
// range are gathered 128 at a time (one per lane of the first two wavefronts, colours included so the blend never goes back to HBM) into LDS as
// 48-byte "hot" + 32-byte "cold" records; the next batch's gather is issued before the current batch is blended so its
// HBM latency overlaps the arithmetic. All lanes of a wavefront read the same LDS record (broadcast, conflict free).
#include "blend.hpp"

namespace fsgs {
namespace {

#ifndef FSGS_FWD_BATCH
#define FSGS_FWD_BATCH 128
#endif
constexpr int kFwdBatch = FSGS_FWD_BATCH;  // surfels staged per round (<= block size)

// kAccum: 0 = no side outputs, 1 = accum_max_count only (what the reference's training loop passes on every step),
// 2 = accum_weights_p and / or accum_weights_count as well.
constexpr int kAccSlots  = 16;  // entries whose per-pixel weights a wavefront stages before it sums them
constexpr int kAccStride = 68;  // floats per staged entry: 64 lanes + 4, so that the 16 readers of a row hit 16 x 4 banks

template <bool kAux, bool kFlow, int kAccum>
__global__ void __launch_bounds__(kBlendThreads) blend_forward_kernel(
    int ordered, const int* __restrict__ tile_order, int W, int H, float near_n, float far_n, const int64_t* __restrict__ ranges, const int32_t* __restrict__ point_list,
    const float2* __restrict__ means2D, const float* __restrict__ colors, const float* __restrict__ trans_mat,
    const float4* __restrict__ normal_opacity, const float4* __restrict__ records,
    const float* __restrict__ trans_mat_t2, int32_t* __restrict__ n_contrib,
    float* __restrict__ out_color, float* __restrict__ out_opacity, float* __restrict__ out_extras,
    float2* __restrict__ out_flow, int32_t* __restrict__ accum_max_count, float* __restrict__ accum_weights_p,
    int32_t* __restrict__ accum_weights_count) {
  __shared__ SplatHot s_hot[kFwdBatch];
  __shared__ SplatCold s_cold[kFwdBatch];
  __shared__ float s_t2[kFlow ? kFwdBatch * 9 : 1];
  __shared__ unsigned char s_mask[kFwdBatch];  // which 8x8 quadrants of the tile each staged surfel can reach
  // accum_weights_*: every lane of a wavefront blends the same entry, so an entry's per-pixel weights all go to one
  // address. Each wavefront parks them in its own LDS rows (one plain store per entry), and after kAccSlots entries sums
  // all rows at once -- lane l adds 16 lanes' worth of entry l & 15, two row / half swaps finish the sum -- and lanes
  // 0..15 issue one atomic per entry and output.
  __shared__ __attribute__((aligned(16))) float s_accw[kAccum == 2 ? 4 * kAccSlots * kAccStride : 4];
  __shared__ int s_accid[kAccum == 2 ? 4 * kAccSlots : 1], s_accn[kAccum == 2 ? 4 * kAccSlots : 1];

  const int gx = (W + kTile - 1) / kTile;
  const int tile = scheduled_tile(ordered, tile_order), tile_x = tile % gx, tile_y = tile / gx;
  int px, py;
  lane_pixel(tile_x, tile_y, px, py);
  const bool inside = px < W && py < H;
  const size_t HW   = (size_t) H * W;
  const size_t pix  = (size_t) W * py + px;
  const float pxf = (float) px, pyf = (float) py;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

  const int64_t r0 = ranges[2 * (size_t) tile], r1 = ranges[2 * (size_t) tile + 1];
  const int n_todo = (int) (r1 - r0);
  const int rounds = (n_todo + kFwdBatch - 1) / kFwdBatch;

  // A pixel stops blending once its transmittance would fall below 1e-4. The state is a float, not a bool: the test
  // is then one comparison whose lane mask feeds the branches directly (a bool carried round the loop lives in a
  // register as 0 / 1 and is turned into a mask again at every use).
  float live = inside ? 1.0f : -1.0f;
  // the same for the wavefront, as a lane mask in scalar registers: "is anybody still blending" costs no vector work
  unsigned long long live_lanes = wave_ballot(inside);
  const float far_scale = far_n / (far_n - near_n), far_near = far_scale * near_n;
  float T = 1.0f, C0 = 0, C1 = 0, C2 = 0;
  float N0 = 0, N1 = 0, N2 = 0, D = 0, M1 = 0, M2 = 0, dist = 0, median = 0, wsum = 0, f0 = 0, f1 = 0;
  int last = 0, median_c = -1;
  ArgmaxRun argmax;
  int acc_slot = 0;  // staged entries of this wavefront (wave-uniform)
  auto flush_weights = [&]() {
    if (acc_slot == 0) return;
    const float4* src = (const float4*) &s_accw[(wave * kAccSlots + (lane & 15)) * kAccStride + (lane >> 4) * 16];
    const float4 a = src[0], b = src[1], c = src[2], d = src[3];
    float t = (((a.x + a.y) + (a.z + a.w)) + ((b.x + b.y) + (b.z + b.w))) +
              (((c.x + c.y) + (c.z + c.w)) + ((d.x + d.y) + (d.z + d.w)));
    t = cross_row_sum(t);
    if (lane < acc_slot) {
      const int id = s_accid[wave * kAccSlots + lane];
      if (accum_weights_p) atomicAdd(&accum_weights_p[id], t);
      if (accum_weights_count) atomicAdd(&accum_weights_count[id], s_accn[wave * kAccSlots + lane]);
    }
    acc_slot = 0;
  };

  Splat next;
  float next_t2[9];
  if ((int) threadIdx.x < min(n_todo, kFwdBatch)) {
    next = gather_splat(point_list[r0 + threadIdx.x], means2D, colors, normal_opacity, trans_mat, records);
    if (kFlow)
#pragma unroll
      for (int k = 0; k < 9; ++k) next_t2[k] = trans_mat_t2[9 * (size_t) next.cold.id + k];
  }

  for (int b = 0; b < rounds; ++b) {
    // everyone has finished reading the previous batch; leave as soon as no pixel of the tile is still blending
    if (__syncthreads_count(live < 0.0f) == kBlendThreads) break;
    const int n_here = min(kFwdBatch, n_todo - b * kFwdBatch);
    if ((int) threadIdx.x < n_here) {
      s_hot[threadIdx.x]  = next.hot;
      s_cold[threadIdx.x] = next.cold;
      s_mask[threadIdx.x] = (unsigned char) quadrant_mask(next.hot, tile_x * kTile, tile_y * kTile, ordered);
      if (kFlow)
#pragma unroll
        for (int k = 0; k < 9; ++k) s_t2[threadIdx.x * 9 + k] = next_t2[k];
    }
    __syncthreads();
    const int nxt = (b + 1) * kFwdBatch + threadIdx.x;
    if ((int) threadIdx.x < kFwdBatch && nxt < n_todo) {
      next = gather_splat(point_list[r0 + nxt], means2D, colors, normal_opacity, trans_mat, records);
      if (kFlow)
#pragma unroll
        for (int k = 0; k < 9; ++k) next_t2[k] = trans_mat_t2[9 * (size_t) next.cold.id + k];
    }

    // Each wavefront walks only the surfels that can reach its quadrant: the ballot of the mask bit over 64 staged
    // surfels is the (depth-ordered) work list, consumed bit by bit with scalar instructions.
    for (int c = 0; c < kFwdBatch / kWave; ++c) {
      const int jj = c * kWave + lane;
      unsigned long long todo = __ballot(jj < n_here && ((s_mask[jj] >> wave) & 1u));
      if (todo == 0ull) continue;
      // One list entry: `hot` was requested an entry earlier. A wavefront walks its list alone, so everything that
      // waits -- the LDS round trip for a surfel's record, chains of nested divergent branches -- is paid once per
      // entry on the tile's critical path (the launch lasts as long as its longest tile). Hence: the NEXT entry's record
      // is requested before the current one is evaluated, into alternating registers; the intersection runs without
      // early exits and yields one predicate; the blend is one divergent region.
      auto blend_entry = [&](const SplatHot& hot, const SplatCold& cold, int j) {
#pragma clang fp contract(off)  // two copies of this body exist (alternating registers): both must round alike
        Hit h;
        unsigned long long pass;
        const bool hit = intersect_flat(hot, pxf, pyf, near_n, h, &pass) && live > 0.0f;
        pass &= live_lanes;
        if (pass == 0ull) return;
        const float test_T = T * (1.0f - h.alpha);
        const bool sat     = hit && test_T < 0.0001f;
        live               = sat ? -1.0f : live;
        live_lanes &= ~(pass & wave_ballot(test_T < 0.0001f));
        const float w      = h.alpha * T;
        if (kAccum == 2) {
          const unsigned long long who = wave_ballot(hit && !sat);
          if (who != 0ull) {
            s_accw[(wave * kAccSlots + acc_slot) * kAccStride + lane] = hit && !sat ? w : 0.0f;
            if (lane == 0) s_accid[wave * kAccSlots + acc_slot] = cold.id, s_accn[wave * kAccSlots + acc_slot] = (int) __popcll(who);
            if (++acc_slot == kAccSlots) flush_weights();
          }
        }
        if (hit && !sat) {
          const int contributor = b * kFwdBatch + j + 1;
          if (kAux) {
            const float A  = 1.0f - T;
            const float m  = fmaf(-far_near, __builtin_amdgcn_rcpf(h.depth), far_scale);
            const float mm = m * m;
            dist = fmaf(fmaf(-2.0f * m, M1, fmaf(mm, A, M2)), w, dist);
            D    = fmaf(h.depth, w, D);
            M1   = fmaf(m, w, M1);
            M2   = fmaf(mm, w, M2);
            if (T > 0.5f) median = h.depth, median_c = contributor;
            N0 = fmaf(cold.nx, w, N0), N1 = fmaf(cold.ny, w, N1), N2 = fmaf(cold.nz, w, N2);
            if (kAccum != 0) argmax_run_step(argmax, w, cold.id, accum_max_count);
            if (kFlow) {
              const float* Q = &s_t2[j * 9];
              const float u2 = fmaf(Q[0], h.sx, fmaf(Q[1], h.sy, Q[2]));
              const float v2 = fmaf(Q[3], h.sx, fmaf(Q[4], h.sy, Q[5]));
              float w2       = fmaf(Q[6], h.sx, fmaf(Q[7], h.sy, Q[8]));
              w2             = fabsf(w2) < 1e-5f ? 1e-5f : w2;
              f0 = fmaf(u2 / w2 - pxf, w, f0);
              f1 = fmaf(v2 / w2 - pyf, w, f1);
            }
            wsum += w;
          }
          C0 = fmaf(cold.r, w, C0), C1 = fmaf(cold.g, w, C1), C2 = fmaf(cold.b, w, C2);
          T    = test_T;
          last = contributor;
        }
      };
      auto pop = [&]() {
        const int j = c * kWave + __builtin_ctzll(todo);
        todo &= todo - 1;
        return j;
      };
      auto peek = [&]() { return c * kWave + (todo ? __builtin_ctzll(todo) : 0); };
      SplatHot hot_a = s_hot[peek()], hot_b;
      while (todo) {
        if (live_lanes == 0ull) break;  // every pixel of this quadrant is saturated
        {
          const int j = pop();
          hot_b       = s_hot[peek()];
          const SplatCold cold = s_cold[j];  // read only if a pixel blends the surfel, but then without waiting
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

  if (kAccum != 0) argmax_run_flush(argmax, accum_max_count);
  if (kAccum == 2) flush_weights();
  if (inside) {
    out_opacity[pix]      = 1.0f - T;
    n_contrib[pix]        = last;
    n_contrib[pix + HW]   = kAux ? median_c : 0;
    out_color[pix]        = C0;
    out_color[pix + HW]   = C1;
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
      out_extras[pix + 8 * HW] = wsum;
      if (kFlow) {
        const float ws = wsum == 0.0f ? 1e-7f : wsum;
        out_flow[pix]  = make_float2(f0 / ws, f1 / ws);
      }
    }
  }
}

__global__ void __launch_bounds__(256) pack_records_kernel(int P, const float2* __restrict__ means2D,
    const float* __restrict__ colors, const float4* __restrict__ normal_opacity, const float* __restrict__ trans_mat,
    const int32_t* __restrict__ radii, const int64_t* __restrict__ point_offsets, float4* __restrict__ records) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= P) return;
  const float* M  = trans_mat + 9 * (size_t) i;
  const float2 c  = means2D[i];
  const float4 no = normal_opacity[i];
  const float* rgb = colors + 3 * (size_t) i;
  const int radius  = radii ? radii[i] : -1;  // -1: not known, the backward then reads its radii argument
  const int offset  = point_offsets ? (i == 0 ? 0 : (int) point_offsets[i - 1]) : -1;  // -1: not known
  float4* r = records + 5 * (size_t) i;
  r[0] = make_float4(M[0], M[1], M[2], M[3]);
  r[1] = make_float4(M[4], M[5], M[6], M[7]);
  r[2] = make_float4(M[8], c.x, c.y, no.w);
  r[3] = make_float4(no.x, no.y, no.z, rgb[0]);
  r[4] = make_float4(rgb[1], rgb[2], __int_as_float(radius), __int_as_float(offset));
}

}  // namespace
}  // namespace fsgs

using namespace fsgs;

FSGS_API int fsgs_gs_2d_pack_records(int P, const float* means2D, const float* colors, const float* normal_opacity,
    const float* trans_mat, const int32_t* radii, const int64_t* point_offsets, float* records, void* stream) {
  FSGS_REQUIRE(P >= 0, "gs_2d_pack_records: bad size");
  if (P == 0) return kOk;
  FSGS_REQUIRE(means2D && colors && normal_opacity && trans_mat && records && ((uintptr_t) records & 15) == 0,
               "gs_2d_pack_records: null or misaligned pointer");
  hipLaunchKernelGGL(pack_records_kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P,
                     (const float2*) means2D, colors, (const float4*) normal_opacity, trans_mat, radii, point_offsets,
                     (float4*) records);
  return check_launch("gs_2d_pack_records");
}

FSGS_API int fsgs_gs_2d_render_forward(int P, int W, int H, double near_n, double far_n, int only_image,
    const float* means2D, const float* colors, const float* normal_opacity, const float* trans_mat,
    const int32_t* point_list, const int64_t* ranges, const float* trans_mat_t2, int32_t* accum_max_count,
    float* accum_weights_p, int32_t* accum_weights_count, float* out_color, float* out_opacity, float* out_extras,
    float* out_flow, int32_t* n_contrib, const float* records, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0, "GS_2D_render_forward: bad sizes");
  FSGS_REQUIRE(ranges && out_color && out_opacity && n_contrib, "GS_2D_render_forward: null pointer");
  FSGS_REQUIRE(P == 0 || records || (means2D && colors && normal_opacity && trans_mat),
               "GS_2D_render_forward: null surfel tensor");
  FSGS_REQUIRE(((uintptr_t) records & 15) == 0, "GS_2D_render_forward: records must be 16-byte aligned");
  FSGS_REQUIRE(only_image || out_extras, "GS_2D_render_forward: out_extras is required unless only_image");
  const bool aux   = !only_image;
  const bool flow  = aux && trans_mat_t2 != nullptr;
  const int accum = !aux ? 0 : (accum_weights_p || accum_weights_count) ? 2 : accum_max_count ? 1 : 0;
  FSGS_REQUIRE(!flow || out_flow, "GS_2D_render_forward: out_flow is required with trans_mat_t2");
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const dim3 grid(gx * gy), block(kBlendThreads);
  hipStream_t s = (hipStream_t) stream;
  const int* tile_order = nullptr;
  const int ordered = launch_tile_order(gx, gy, ranges, s, &tile_order);
#define FSGS_LAUNCH_FWD(AUX, FLOW, ACC)                                                                              \
  hipLaunchKernelGGL((blend_forward_kernel<AUX, FLOW, ACC>), grid, block, 0, s, ordered, tile_order, W, H, (float) near_n, (float) far_n, \
                     ranges, point_list, (const float2*) means2D, colors, trans_mat, (const float4*) normal_opacity, \
                     (const float4*) records, trans_mat_t2, n_contrib, out_color, out_opacity, out_extras, (float2*) out_flow,                \
                     accum_max_count, accum_weights_p, accum_weights_count)
  if (!aux) FSGS_LAUNCH_FWD(false, false, 0);
  else if (flow && accum == 2) FSGS_LAUNCH_FWD(true, true, 2);
  else if (flow && accum == 1) FSGS_LAUNCH_FWD(true, true, 1);
  else if (flow) FSGS_LAUNCH_FWD(true, true, 0);
  else if (accum == 2) FSGS_LAUNCH_FWD(true, false, 2);
  else if (accum == 1) FSGS_LAUNCH_FWD(true, false, 1);
  else FSGS_LAUNCH_FWD(true, false, 0);
#undef FSGS_LAUNCH_FWD
  return check_launch("GS_2D_render_forward");
}

FSGS_API int fsgs_debug_tile_order(int gx, int gy, const int64_t* ranges, int32_t* table, void* stream) {
  using namespace fsgs;
  FSGS_REQUIRE(gx > 0 && gy > 0 && (int64_t) gx * gy <= kMaxOrderedTiles && ranges && table,
               "debug_tile_order: bad arguments (at most %d tiles)", kMaxOrderedTiles);
  hipLaunchKernelGGL(tile_order_kernel, dim3(1), dim3(1024), 0, (hipStream_t) stream, gx, gy, ranges, table);
  return check_launch("debug_tile_order");
}

