// Shared pieces of the per-tile alpha-blend kernels: the LDS surfel record, the cooperative gather of a batch of
// surfels, the ray-splat intersection, and wave64 cross-lane reductions.
#pragma once
#include "common.hpp"
#include "cull_bound.hpp"

namespace fsgs {

// Launch flags of the blend kernels (see launch_tile_order).
constexpr int kFlagOrdered = 1, kFlagNoCull = 2;
bool culling_enabled();  // host-side switch, on by default

constexpr int kBlendThreads = 256;  // one 16x16 tile per block = 4 wavefronts, each owning an 8x8 pixel quadrant
constexpr int kBatch        = 256;  // surfels staged in LDS per round

// Hot part of a staged surfel (what every pixel needs to decide whether the surfel touches it), 48 bytes.
struct __attribute__((aligned(16))) SplatHot {
  float m[9];      // ray-splat matrix rows Tu, Tv, Tw
  float cx, cy;    // screen-space centre (low-pass filter)
  float opacity;
};
// Cold part, only read once a pixel in the wavefront actually blends the surfel, 32 bytes.
struct __attribute__((aligned(16))) SplatCold {
  float nx, ny, nz;
  float r, g, b;
  int id;
  int pad;
};

struct Splat {
  SplatHot hot;
  SplatCold cold;
};

// Optional packed copy of everything the blend kernels gather per surfel: one 80-byte, 16-byte-aligned record
// (five float4) instead of four tensors, i.e. one or two 128-byte lines per list entry instead of four to six.
//   q0 = M0 M1 M2 M3 | q1 = M4 M5 M6 M7 | q2 = M8 cx cy opacity | q3 = nx ny nz r | q4 = g b radius(int) offset(int)
// radius / offset (prefix scan of tiles_touched before this surfel) are only meaningful when the packer was given them.
constexpr int kRecordFloats = 20;

struct SplatExtra {
  int radius;
  int64_t offset;  // exclusive prefix-scan offset of the surfel's instances; -1 until the binning's scan has stored it
};

__device__ __forceinline__ Splat gather_splat(int id, const float2* __restrict__ means2D,
                                              const float* __restrict__ colors,
                                              const float4* __restrict__ normal_opacity,
                                              const float* __restrict__ trans_mat,
                                              const float4* __restrict__ records, SplatExtra* extra = nullptr) {
  Splat s;
  if (records != nullptr) {
    const float4* r = records + 5 * (size_t) id;
    const float4 q0 = r[0], q1 = r[1], q2 = r[2], q3 = r[3], q4 = r[4];
    s.hot.m[0] = q0.x, s.hot.m[1] = q0.y, s.hot.m[2] = q0.z, s.hot.m[3] = q0.w;
    s.hot.m[4] = q1.x, s.hot.m[5] = q1.y, s.hot.m[6] = q1.z, s.hot.m[7] = q1.w;
    s.hot.m[8] = q2.x, s.hot.cx = q2.y, s.hot.cy = q2.z, s.hot.opacity = q2.w;
    s.cold.nx = q3.x, s.cold.ny = q3.y, s.cold.nz = q3.z, s.cold.r = q3.w;
    s.cold.g = q4.x, s.cold.b = q4.y;
    s.cold.id = id, s.cold.pad = 0;
    if (extra) extra->radius = __float_as_int(q4.z), extra->offset = (int64_t) __float_as_int(q4.w);
    return s;
  }
  const float* M = trans_mat + 9 * (size_t) id;
#pragma unroll
  for (int k = 0; k < 9; ++k) s.hot.m[k] = M[k];
  const float2 c = means2D[id];
  const float4 no = normal_opacity[id];
  s.hot.cx = c.x, s.hot.cy = c.y, s.hot.opacity = no.w;
  s.cold.nx = no.x, s.cold.ny = no.y, s.cold.nz = no.z;
  s.cold.r = colors[3 * (size_t) id], s.cold.g = colors[3 * (size_t) id + 1], s.cold.b = colors[3 * (size_t) id + 2];
  s.cold.id = id, s.cold.pad = 0;
  return s;
}

// Pixel owned by a lane: wavefront w covers the 8x8 quadrant (w & 1, w >> 1) of the 16x16 tile.
__device__ __forceinline__ void lane_pixel(int tile_x, int tile_y, int& px, int& py) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  px = tile_x * kTile + (wave & 1) * 8 + (lane & 7);
  py = tile_y * kTile + (wave >> 1) * 8 + (lane >> 3);
}

// The same quadrant with every 16-lane DPP row on a 4x4 pixel block: row r = lane >> 4 is block (r & 1, r >> 1) of the
// quadrant, lane & 15 runs row-major inside the block.
__device__ __forceinline__ void lane_pixel_blocks(int tile_x, int tile_y, int& px, int& py) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int row = lane >> 4, in = lane & 15;
  px = tile_x * kTile + (wave & 1) * 8 + (row & 1) * 4 + (in & 3);
  py = tile_y * kTile + (wave >> 1) * 8 + (row >> 1) * 4 + (in >> 2);
}

struct Hit {
  float kx, ky, kz, lx, ly, lz;  // the two homogeneous planes through the pixel
  float pz;                      // z of their cross product
  float sx, sy;                  // intersection in the surfel's tangent frame
  float dx, dy;                  // centre - pixel
  float rho3d, rho2d;
  float depth;
  float G;                       // exp(-rho/2)
  float alpha;
};

// Ray-splat intersection and alpha of one surfel at one pixel (gs_2d_redner.cu:122-155); false where the reference
// would `continue`. No early exits: every lane runs the whole sequence and the rejections are combined at the end, so the
// caller gets one predicate instead of nested divergent regions. Contraction is switched off and every fused
// multiply-add is written out, so that each inlined copy rounds alike (a kernel that instantiates it twice must not
// depend on which copy evaluated a surfel). The exponent is formed in base 2 (-rho / 2 * log2(e) =
// max(-log2(e) / 2 * rho3d, -log2(e) * |d|^2), one v_exp_f32). rho is a sum of squares, so the reference's `power > 0`
// rejection can only differ from `true` for a NaN, which passes it there as here.
// The intersection point is formed the reference's way, as the cross product of the two planes k = x Tw - Tu and
// l = y Tw - Tv. (It is also linear in the pixel, p = p(c) - (c_x - x) Tv x Tw - (c_y - y) Tw x Tu, which takes six
// instructions less per test once the two cross products are staged per surfel; for surfels seen edge-on, where p_z
// nearly vanishes over the footprint, that form lands three times farther from the exact value than this one does --
// measured on the 300k-surfel scene against the float64 evaluation -- so it is not used.)
// `lanes`, if given, receives the mask of the lanes that pass, as the AND of the comparisons' own lane masks: a
// wave-uniform "does any lane pass" then stays in scalar registers (the ballot of a combined predicate is rebuilt by
// the compiler from a 0 / 1 register, two vector instructions and their latency on the entry's critical path).
// Forward and backward of the standard path decide a pair with this function, so they agree on every pair.
__device__ __forceinline__ bool intersect_flat(const SplatHot& h, float pxf, float pyf, float near_n, Hit& o,
                                               unsigned long long* lanes = nullptr) {
#pragma clang fp contract(off)
  o.kx = fmaf(pxf, h.m[6], -h.m[0]), o.ky = fmaf(pxf, h.m[7], -h.m[1]), o.kz = fmaf(pxf, h.m[8], -h.m[2]);
  o.lx = fmaf(pyf, h.m[6], -h.m[3]), o.ly = fmaf(pyf, h.m[7], -h.m[4]), o.lz = fmaf(pyf, h.m[8], -h.m[5]);
  const float p_x = fmaf(o.ky, o.lz, -(o.kz * o.ly));
  const float p_y = fmaf(o.kz, o.lx, -(o.kx * o.lz));
  o.pz            = fmaf(o.kx, o.ly, -(o.ky * o.lx));
  const float rz = __builtin_amdgcn_rcpf(o.pz);
  o.sx = p_x * rz, o.sy = p_y * rz;
  o.rho3d = fmaf(o.sx, o.sx, o.sy * o.sy);
  o.dx = h.cx - pxf, o.dy = h.cy - pyf;
  const float d2 = fmaf(o.dx, o.dx, o.dy * o.dy);
  o.rho2d = 2.0f * d2;
  o.depth = fmaf(o.sx, h.m[6], fmaf(o.sy, h.m[7], h.m[8]));
  const float power2 = fmaxf(o.rho3d * -0.72134752044448170368f, d2 * -1.44269504088896340736f);
  o.G     = __builtin_amdgcn_exp2f(power2);
  o.alpha = fminf(0.99f, h.opacity * o.G);
  const bool c0 = o.pz != 0.0f, c1 = !(o.depth < near_n), c3 = !(o.alpha < (1.0f / 255.0f));
  if (lanes) *lanes = wave_ballot(c0) & wave_ballot(c1) & wave_ballot(c3);
  return c0 & c1 & c3;
}

// ---- conservative per-quadrant culling ------------------------------------------------------------------------------
// A surfel can only be blended at a pixel if alpha = min(0.99, o * exp(-rho / 2)) >= 1/255, i.e. rho <= tau with
// tau = 2 ln(255 o), where rho = min(rho3d, rho2d). The pixels with rho3d <= tau are the perspective image of the
// ellipse u^2 + v^2 <= tau in the surfel's tangent plane; its exact screen-space bounding box follows from the same
// homogeneous form the preprocess uses for its 3-sigma bound (gs_2d_preprocess.cu:125-156) with cutoff^2 = tau. The
// pixels with rho2d <= tau are a disc of radius sqrt(tau / 2) around the screen-space centre. The union of both boxes,
// padded by 1/8 pixel + 0.5 % of its extent against rounding, is tested against the four 8x8 quadrants of the tile; a
// clear bit means no pixel of that quadrant can pass the reference's alpha test, so skipping it changes nothing.
// Surfels whose tau-ellipse reaches the camera plane (no finite box) keep all bits set.

__device__ __forceinline__ unsigned quadrant_mask(const SplatHot& h, int tile_px, int tile_py, int flags) {
  if (flags & kFlagNoCull) return 0xfu;
  const float oa = 255.0f * h.opacity;
  if (!(oa >= 1.0f)) return 0u;  // alpha can never reach 1/255
  const float tau = 2.0f * __logf(oa) * 1.0001f + 1e-3f;
  // Work in coordinates relative to the screen-space centre: the box centre and half extents are differences of
  // squares (c^2 - ...), which cancel catastrophically at pixel coordinates in the thousands but not near the origin.
  const float ox = h.cx, oy = h.cy;
  float x0, x1, y0, y1;
  const float r2 = sqrtf(0.5f * tau);
  x0 = -r2, x1 = r2, y0 = -r2, y1 = r2;
  const float* M = h.m;
  const float u0 = M[0] - ox * M[6], u1 = M[1] - ox * M[7], u2 = M[2] - ox * M[8];
  const float v0 = M[3] - oy * M[6], v1 = M[4] - oy * M[7], v2 = M[5] - oy * M[8];
  const float d  = tau * (M[6] * M[6] + M[7] * M[7]) - M[8] * M[8];
  bool finite_box = (M[8] > 0.0f) && (d < -1e-6f * M[8] * M[8]);
  if (finite_box) {
    const float inv = 1.0f / d;
    const float f0 = tau * inv, f2 = -inv;
    const float cx = f0 * (u0 * M[6] + u1 * M[7]) + f2 * (u2 * M[8]);
    const float cy = f0 * (v0 * M[6] + v1 * M[7]) + f2 * (v2 * M[8]);
    const float hx = cx * cx - (f0 * (u0 * u0 + u1 * u1) + f2 * (u2 * u2));
    const float hy = cy * cy - (f0 * (v0 * v0 + v1 * v1) + f2 * (v2 * v2));
    const float ex = sqrtf(fmaxf(hx, 0.0f)), ey = sqrtf(fmaxf(hy, 0.0f));
    finite_box = (ex == ex) && (ey == ey) && (cx == cx) && (cy == cy);
    x0 = fminf(x0, cx - ex), x1 = fmaxf(x1, cx + ex);
    y0 = fminf(y0, cy - ey), y1 = fmaxf(y1, cy + ey);
  }
  if (!finite_box) return 0xfu;
  const float padx = kCullPad + 0.005f * (x1 - x0), pady = kCullPad + 0.005f * (y1 - y0);
  x0 -= padx, x1 += padx, y0 -= pady, y1 += pady;
  // The same bound along the two diagonals (the extents of x + y and of x - y over the footprint, from the same
  // homogeneous form with the rows added / subtracted) cuts the corners off the box: an 8x8 quadrant that only meets a
  // corner of the box of a round or diagonally stretched footprint is not met by the footprint itself.
  float a0 = -1e30f, a1 = 1e30f, b0 = -1e30f, b1 = 1e30f;
  {
    const float d  = tau * (M[6] * M[6] + M[7] * M[7]) - M[8] * M[8];
    const float inv = 1.0f / d, f0 = tau * inv, f2 = -inv;
    const float p0 = u0 + v0, p1 = u1 + v1, p2 = u2 + v2, q0 = u0 - v0, q1 = u1 - v1, q2 = u2 - v2;
    const float ca = f0 * (p0 * M[6] + p1 * M[7]) + f2 * (p2 * M[8]);
    const float cb = f0 * (q0 * M[6] + q1 * M[7]) + f2 * (q2 * M[8]);
    const float ha = ca * ca - (f0 * (p0 * p0 + p1 * p1) + f2 * (p2 * p2));
    const float hb = cb * cb - (f0 * (q0 * q0 + q1 * q1) + f2 * (q2 * q2));
    const float ea = sqrtf(fmaxf(ha, 0.0f)), eb = sqrtf(fmaxf(hb, 0.0f));
    if ((ea == ea) && (eb == eb) && (ca == ca) && (cb == cb)) {
      const float rd = 1.41421357f * r2;  // the low-pass disc along a diagonal
      const float la = fminf(ca - ea, -rd), ua = fmaxf(ca + ea, rd), lb = fminf(cb - eb, -rd), ub = fmaxf(cb + eb, rd);
      const float pa = 1.5f * kCullPad + 0.005f * (ua - la), pb = 1.5f * kCullPad + 0.005f * (ub - lb);
      a0 = la - pa, a1 = ua + pa, b0 = lb - pb, b1 = ub + pb;
    }
  }
  unsigned m = 0u;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    // the quadrant's pixel centres relative to the surfel's centre
    const float qx0 = (float) (tile_px + (q & 1) * 8) - ox, qy0 = (float) (tile_py + (q >> 1) * 8) - oy;
    const float qx1 = qx0 + 7.0f, qy1 = qy0 + 7.0f;
    const bool box  = x1 >= qx0 && x0 <= qx1 && y1 >= qy0 && y0 <= qy1;
    const bool diag = a1 >= qx0 + qy0 && a0 <= qx1 + qy1 && b1 >= qx0 - qy1 && b0 <= qx1 - qy0;
    if (box && diag) m |= 1u << q;
  }
  return m;
}

// ---- tile schedule: longest lists first, neighbouring tiles on the same XCD, equal work per CU ------------------------
// Blocks are handed out in blockIdx order, consecutive blocks go to consecutive XCDs (8 of them, each with its own L2,
// 32 CUs behind each), and a tile's cost is proportional to the length of its list. The blend kernels therefore map
// blockIdx -> tile through a table built once per frame: small square groups of tiles are dealt to 8 regions, region r
// owns the table positions p with p % 8 == r (as long as it has tiles left), and inside a region tiles are listed by
// descending list length (sixteen buckets per octave, arbitrary order inside a bucket). Long lists start first and short ones
// fill the tail of the launch; a surfel that overlaps several neighbouring tiles is gathered by blocks that share an L2.
// An XCD places the first blocks it receives on its CUs in turn, and as many rounds of 32 as blocks fit on a CU stay
// there together for most of the launch: CU c works on the region's tiles number c, 32 + c, 64 + c, ... In plain
// descending order CU 0 would get the longest tile of every round and CU 31 the shortest (15 % above the mean for the
// chord-length profile of a ball of surfels), and the launch lasts as long as its busiest CU. Inside each of the first
// rounds the tiles are therefore dealt by load: the CU with the least work so far gets the round's longest tile.
// Later rounds go wherever a slot frees up; for them descending order is what balances.
// The table is kMaxOrderedTiles ints in a file-scope device array of the library (no allocation), one slot per
// (device, stream) that bins or blends: calls on one stream are ordered by the stream, calls on different streams use
// different tables, and a stream that finds every slot taken runs without a table.
#ifndef FSGS_ORDER_FRAC_BITS
#define FSGS_ORDER_FRAC_BITS 4
#endif
#ifndef FSGS_ORDER_BALANCE_ROUNDS
#define FSGS_ORDER_BALANCE_ROUNDS 4
#endif
constexpr int kMaxOrderedTiles = 1 << 16;
constexpr int kOrderFracBits   = FSGS_ORDER_FRAC_BITS;  // buckets per octave of list length = 2^this
constexpr int kOrderFrac       = 1 << kOrderFracBits;
constexpr int kOrderBuckets    = 32 * kOrderFrac;
constexpr int kOrderRegions    = 8;
constexpr int kCusPerXcd       = 32;  // compute units behind one region's table positions
// rounds of a region's list whose tiles are dealt by CU load: the blocks of the blend backward that fit on a CU (4,
// bounded by its 128 registers per lane); measured best among 3, 4, 5, 6, 8, 16
constexpr int kBalanceRounds   = FSGS_ORDER_BALANCE_ROUNDS;

// (tile_order_table, tile_order_invalidate and tile_order_release are declared in common.hpp.)

namespace {

__device__ __forceinline__ int length_bucket(int64_t len64) {
  const unsigned len = len64 > 0x7fffffff ? 0x7fffffffu : (unsigned) (len64 < 0 ? 0 : len64);
  if (len == 0) return 0;
  const int m    = 31 - __clz(len);
  const int frac = m >= kOrderFracBits ? (int) ((len >> (m - kOrderFracBits)) & (kOrderFrac - 1))
                                       : (int) ((len << (kOrderFracBits - m)) & (kOrderFrac - 1));
  return 1 + m * kOrderFrac + frac;  // <= 31 * kOrderFrac
}

#ifndef FSGS_TILE_GROUP
#define FSGS_TILE_GROUP 2
#endif
// Groups of FSGS_TILE_GROUP x FSGS_TILE_GROUP tiles are dealt to the 8 regions in a skewed pattern, so every region is a
// fine-grained sample of the whole image (equal load whatever the scene's layout) while direct neighbours mostly share
// a region.
__device__ __forceinline__ int tile_region(int t, int gx, int gy) {
  const int tx = t % gx, ty = t / gx;
  (void) gy;
  return ((tx / FSGS_TILE_GROUP) + 3 * (ty / FSGS_TILE_GROUP)) & (kOrderRegions - 1);
}

// LDS of one block that builds a table (24.6 KB)
struct TileOrderLds {
  int count[kOrderRegions][kOrderBuckets];
  int total[kOrderRegions];
  int tile[kOrderRegions][kBalanceRounds * kCusPerXcd], len[kOrderRegions][kBalanceRounds * kCusPerXcd];
};

// The work of one whole block (any size that is a multiple of 64 with at least 8 wavefronts): either a launch of its
// own (tile_order_kernel) or one extra block of a kernel that has nothing to do with it but runs at the right time --
// the binning's scatter, whose other blocks keep the chip busy while this one orders 2 500 numbers (a single-block
// launch of its own holds up the stream for 10 us).
__device__ __forceinline__ void build_tile_order(int gx, int gy, const int64_t* __restrict__ ranges,
                                                 int* __restrict__ tile_order, TileOrderLds& lds) {
  auto& s_count = lds.count;
  auto& s_total = lds.total;
  auto& s_tile  = lds.tile;
  auto& s_len   = lds.len;
  const int T = gx * gy;
  for (int b = threadIdx.x; b < kOrderRegions * kOrderBuckets; b += blockDim.x) (&s_count[0][0])[b] = 0;
  __syncthreads();
  for (int t = threadIdx.x; t < T; t += blockDim.x)
    atomicAdd(&s_count[tile_region(t, gx, gy)][length_bucket(ranges[2 * (size_t) t + 1] - ranges[2 * (size_t) t])], 1);
  __syncthreads();
  {  // exclusive prefix from the longest bucket down, one wavefront per region
    const int lane = threadIdx.x & 63, r = threadIdx.x >> 6;
    constexpr int kPer = kOrderBuckets / 64;
    if (r < kOrderRegions) {
      int c[kPer], sum = 0;
#pragma unroll
      for (int i = 0; i < kPer; ++i) c[i] = s_count[r][kOrderBuckets - 1 - (lane * kPer + i)], sum += c[i];
      int inc = sum;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(inc, d, 64);
        if (lane >= d) inc += up;
      }
      int run = inc - sum;
#pragma unroll
      for (int i = 0; i < kPer; ++i) s_count[r][kOrderBuckets - 1 - (lane * kPer + i)] = run, run += c[i];
      if (lane == 63) s_total[r] = inc;
    }
  }
  __syncthreads();
  // position of the k-th tile of region r when the regions are dealt round-robin, skipping exhausted ones
  auto position = [&](int r, int k) {
    int pos = 0;
#pragma unroll
    for (int q = 0; q < kOrderRegions; ++q) pos += min(s_total[q], k) + ((q < r && s_total[q] > k) ? 1 : 0);
    return pos;
  };
  for (int t = threadIdx.x; t < T; t += blockDim.x) {
    const int r       = tile_region(t, gx, gy);
    const int64_t len = ranges[2 * (size_t) t + 1] - ranges[2 * (size_t) t];
    const int k       = atomicAdd(&s_count[r][length_bucket(len)], 1);
    if (k < kBalanceRounds * kCusPerXcd) {
      s_tile[r][k] = t;
      s_len[r][k]  = (int) (len > 0x7fffffff ? 0x7fffffff : len);
    } else {
      tile_order[position(r, k)] = t;
    }
  }
  __syncthreads();
  // The first rounds of a region, one wavefront per region, lane c = the c-th longest tile of the round: the CUs are
  // sorted by the work they hold so far (bitonic network over the lanes) and the c-th longest tile goes to the CU with
  // the c-th smallest load. Round 0 keeps its order, round 1 comes out reversed, later rounds even out what is left.
  {
    const int lane = threadIdx.x & 63, r = threadIdx.x >> 6;
    if (r < kOrderRegions && lane < kCusPerXcd) {
      unsigned long long key = (unsigned long long) lane;  // (load << 8) | cu
      const int n = s_total[r];
      for (int j = 0; j < kBalanceRounds && j * kCusPerXcd < n; ++j) {
        const int k = j * kCusPerXcd + lane;
        if ((j + 1) * kCusPerXcd > n) {  // a partial last round keeps its order
          if (k < n) tile_order[position(r, k)] = s_tile[r][k];
          break;
        }
#pragma unroll
        for (int size = 2; size <= kCusPerXcd; size <<= 1)
#pragma unroll
          for (int d = size >> 1; d > 0; d >>= 1) {
            const unsigned long long other = __shfl_xor(key, d, kCusPerXcd);
            const bool up = (lane & size) == 0, low = (lane & d) == 0;
            key = (low == up) ? (key < other ? key : other) : (key < other ? other : key);
          }
        const int cu = (int) (key & 0xffull);
        tile_order[position(r, j * kCusPerXcd + cu)] = s_tile[r][k];
        key += (unsigned long long) (unsigned) s_len[r][k] << 8;
      }
    }
  }
}

__global__ void __launch_bounds__(1024) tile_order_kernel(int gx, int gy, const int64_t* __restrict__ ranges,
                                                          int* __restrict__ tile_order) {
  __shared__ TileOrderLds lds;
  build_tile_order(gx, gy, ranges, tile_order, lds);
}

// Launch flags of the blend kernels: bit 0 = the tile table was built for this launch (T small enough; otherwise blocks
// map to tiles directly), bit 1 = per-quadrant culling switched off (verification aid, see fsgs_debug_set_culling).
inline int launch_tile_order(int gx, int gy, const int64_t* ranges, hipStream_t s, const int** table) {
  int flags = culling_enabled() ? 0 : kFlagNoCull;
  *table    = nullptr;
  if ((int64_t) gx * gy > kMaxOrderedTiles) return flags;
  bool rebuild = false;
  int* t = tile_order_table(s, ranges, gx, gy, &rebuild);
  if (!t) return flags;
  if (rebuild) hipLaunchKernelGGL(tile_order_kernel, dim3(1), dim3(1024), 0, s, gx, gy, ranges, t);
  *table = t;
  return flags | kFlagOrdered;
}

// The same, with the build left to a kernel the caller is about to launch on the stream anyway: *build receives the
// table to fill (build_tile_order in one extra block), or stays nullptr when the table is up to date or there is none.
inline int defer_tile_order(int gx, int gy, const int64_t* ranges, hipStream_t s, const int** table, int** build) {
  int flags = culling_enabled() ? 0 : kFlagNoCull;
  *table = nullptr, *build = nullptr;
  if ((int64_t) gx * gy > kMaxOrderedTiles) return flags;
  bool rebuild = false;
  int* t = tile_order_table(s, ranges, gx, gy, &rebuild);
  if (!t) return flags;
  if (rebuild) *build = t;
  *table = t;
  return flags | kFlagOrdered;
}

__device__ __forceinline__ int scheduled_tile(int flags, const int* __restrict__ tile_order) {
  return (flags & kFlagOrdered) ? tile_order[blockIdx.x] : (int) blockIdx.x;
}

}  // namespace

// ---- wave64 reductions through DPP --------------------------------------------------------------------------------
template <int kCtrl, int kRowMask, int kBankMask>
__device__ __forceinline__ float dpp_shift_zero(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, kRowMask, kBankMask, true));
}

// Sum over the 64 lanes; the total is valid in lane 63 only.
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
#pragma clang fp contract(off)  // as in row_sum16_transposed: an input product must not be formed a second time
  v += dpp_shift_zero<0x111, 0xf, 0xf>(v);  // row_shr:1
  v += dpp_shift_zero<0x112, 0xf, 0xf>(v);  // row_shr:2
  v += dpp_shift_zero<0x114, 0xf, 0xf>(v);  // row_shr:4
  v += dpp_shift_zero<0x118, 0xf, 0xf>(v);  // row_shr:8  -> lane 15 of every row holds the row total
  v += dpp_shift_zero<0x142, 0xa, 0xf>(v);  // row_bcast:15 into rows 1 and 3
  v += dpp_shift_zero<0x143, 0xc, 0xf>(v);  // row_bcast:31 into rows 2 and 3 -> lane 63 holds the wave total
  return v;
}

// ---- per-surfel side sums of the forward blends ---------------------------------------------------------------------
// accum_weights_p / accum_weights_count: a wavefront blends one list entry at a time, so the up to 64 per-pixel adds of
// an entry go to one address. They are summed in the wavefront first (one DPP reduction, one population count) and lane 63
// issues one atomic per output. Must be reached by all 64 lanes; `id` and the two pointers are wave-uniform.
__device__ __forceinline__ void wave_accumulate_weights(bool blended, float w, int id, float* __restrict__ weights_p,
                                                        int32_t* __restrict__ weights_count) {
  const unsigned long long who = __ballot(blended);
  if (who == 0ull) return;
  const float total = wave_sum_to_lane63(blended ? w : 0.0f);
  if ((threadIdx.x & 63) == 63) {
    if (weights_p) atomicAdd(&weights_p[id], total);
    if (weights_count) atomicAdd(&weights_count[id], (int) __popcll(who));
  }
}

// accum_max_count in the surfel paths: the reference adds 1 to the count of the pixel's current arg-max surfel at EVERY
// blended entry from the first one on (its flag is never reset). A pixel's arg-max changes a few times at most, so the
// adds are kept as a run length and issued when the arg-max moves and once after the last entry: the same integer
// totals with a few atomics per pixel instead of one per blended entry.
struct ArgmaxRun {
  float wmax = 0.0f;
  int id     = -1;
  int run    = 0;
};
__device__ __forceinline__ void argmax_run_flush(ArgmaxRun& a, int32_t* __restrict__ max_count) {
  if (a.run > 0 && max_count) atomicAdd(&max_count[a.id], a.run);
  a.run = 0;
}
__device__ __forceinline__ void argmax_run_step(ArgmaxRun& a, float w, int id, int32_t* __restrict__ max_count) {
  if (a.wmax < w) {
    argmax_run_flush(a, max_count);
    a.wmax = w, a.id = id;
  }
  ++a.run;
}

// Adds the values held by the same lane position of the four 16-lane rows; every lane gets the total.
// gfx950's row/half swaps do it in the VALU (no LDS round trip as with a bpermute): after swapping the odd rows of one
// copy with the even rows of another, copy A holds rows (0,0,2,2) and copy B rows (1,1,3,3); the 32-lane swap does the
// same for the halves. Written as inline assembly because the compiler's builtin for these instructions returns the
// first result twice; the s_nop cover the VALU-write -> swap-read wait states the compiler would insert itself.
__device__ __forceinline__ float cross_row_sum(float z) {
#ifdef FSGS_NO_PERMLANE_SWAP
  z += __shfl_xor(z, 16, kWave);
  z += __shfl_xor(z, 32, kWave);
  return z;
#else
  float a = z, b = z;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32_e32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  z = a + b;
  a = z, b = z;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32_e32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return a + b;
#endif
}

// Sums 16 per-lane values over the 64 lanes at once ("transposed" butterfly): each step halves the number of live
// registers while doubling the lanes a partial covers, so 16 wave-wide sums cost 15 merge steps (2 DPP adds + 1 select
// each) plus two cross-row exchanges, instead of 16 x 6 dependent DPP adds. On return every lane holds the wave total of
// v[lane & 15].
// On return lane l of every 16-lane row holds that ROW's total of v[l & 15].
__device__ __forceinline__ float row_sum16_transposed(const float (&v)[16]) {
  // no contraction: an input that is a product would otherwise be formed twice, as a multiply for the shifted operand
  // and again inside a fused multiply-add for the lane's own, in place of one multiply and one DPP add
#pragma clang fp contract(off)
  const int lane = __lane_id();
  const bool b0 = lane & 1, b1 = lane & 2, b2 = lane & 4, b3 = lane & 8;
  float w[8], x[4], y[2];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float a = v[2 * i + 1] + dpp_shift_zero<0x111, 0xf, 0xf>(v[2 * i + 1]);  // row_shr:1, kept by odd lanes
    const float b = v[2 * i] + dpp_shift_zero<0x101, 0xf, 0xf>(v[2 * i]);          // row_shl:1, kept by even lanes
    w[i] = b0 ? a : b;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float a = w[2 * i + 1] + dpp_shift_zero<0x112, 0xf, 0xf>(w[2 * i + 1]);  // row_shr:2
    const float b = w[2 * i] + dpp_shift_zero<0x102, 0xf, 0xf>(w[2 * i]);          // row_shl:2
    x[i] = b1 ? a : b;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const float a = x[2 * i + 1] + dpp_shift_zero<0x114, 0xf, 0xf>(x[2 * i + 1]);  // row_shr:4
    const float b = x[2 * i] + dpp_shift_zero<0x104, 0xf, 0xf>(x[2 * i]);          // row_shl:4
    y[i] = b2 ? a : b;
  }
  const float a = y[1] + dpp_shift_zero<0x118, 0xf, 0xf>(y[1]);  // row_shr:8
  const float b = y[0] + dpp_shift_zero<0x108, 0xf, 0xf>(y[0]);  // row_shl:8
  return b3 ? a : b;
}
__device__ __forceinline__ float wave_sum16_transposed(const float (&v)[16]) {
  return cross_row_sum(row_sum16_transposed(v));
}

}  // namespace fsgs
