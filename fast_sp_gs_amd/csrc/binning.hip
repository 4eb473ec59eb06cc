// Tile binning for gfx950: prefix sum of per-surfel tile counts, then the (tile, depth) ordering of all (surfel, tile)
// instances and the per-tile ranges.
//
// Reference behaviour reproduced bit for bit: fast_2d_gs/_C/src/gaussian_splatting/gaussian_prepare.cu:32-83
// (getHigherMsb, duplicateWithKeys), :192-220 (identifyTileRanges), :222-308 (prepare / GS_prepare, which uses
// cub::DeviceScan::InclusiveSum and cub::DeviceRadixSort::SortPairs on bits [0, 32 + msb(T))).
//
// Wave64 design notes
//  * scan: 2048 counts per 256-lane block, lane-local sums + wave prefix by cross-lane shifts + LDS across the 4 waves.
//  * standard path: bucket the instances by tile (count -> scan -> scatter) and sort every tile's segment on its own
//    (see "binning by tile buckets" below); rectangles above 32 tiles are walked cooperatively by the whole wavefront
//    so one huge surfel cannot serialise a wave.
//  * device-wide radix sort (used by the fused corner-test binning of the fast path, whose padding entries and sort width
//    follow the reference): 8-bit digits. Per pass: block histograms -> per-digit scan over blocks -> scatter. The
//    scatter ranks keys with 64-bit ballot match masks (8 ballots per round, popcount of the mask below the lane),
//    which is stable by construction: within a wave lower rounds and lower lanes come first, waves are ordered by an
//    LDS prefix, blocks by the scanned histogram.
#include <algorithm>

#include "binning.hpp"
#include "blend.hpp"

namespace fsgs {
namespace {

constexpr int kScanThreads = 256;
constexpr int kScanItems   = 8;
constexpr int kScanChunk   = kScanThreads * kScanItems;

constexpr int kSortThreads = 256;
constexpr int kSortWaves   = kSortThreads / kWave;
constexpr int kSortItems   = 8;                          // keys per lane
constexpr int kSortChunk   = kSortThreads * kSortItems;  // keys per block
constexpr int kRadixBits   = 8;
constexpr int kRadix       = 1 << kRadixBits;

__device__ __forceinline__ unsigned long long lanemask_lt() {
  const unsigned lane = __lane_id();
  return lane == 0 ? 0ull : (~0ull >> (64 - lane));
}

template <typename T>
__device__ __forceinline__ T wave_inclusive_scan(T v) {
  const int lane = __lane_id();
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const T o = __shfl_up(v, d, kWave);
    if (lane >= d) v += o;
  }
  return v;
}

// Block-wide exclusive prefix of one value per thread (256 threads); also returns the block total.
template <typename T>
__device__ __forceinline__ T block_exclusive_scan(T v, T* s_wave /*[4]*/, T& total) {
  const int lane = __lane_id(), wave = threadIdx.x / kWave;
  const T inc = wave_inclusive_scan(v);
  if (lane == kWave - 1) s_wave[wave] = inc;
  __syncthreads();
  T base = 0;
  total  = 0;
#pragma unroll
  for (int w = 0; w < kScanThreads / kWave; ++w) {
    const T s = s_wave[w];
    if (w < wave) base += s;
    total += s;
  }
  __syncthreads();
  return base + inc - v;
}

// ---- inclusive scan of tiles_touched (int32) into int64 offsets ----------------------------------------------------
__global__ void __launch_bounds__(kScanThreads) scan_block_sums_kernel(int P, const int32_t* __restrict__ in,
                                                                       int64_t* __restrict__ block_sums) {
  __shared__ int64_t s_wave[kScanThreads / kWave];
  const int base = blockIdx.x * kScanChunk + threadIdx.x * kScanItems;
  int64_t sum = 0;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k)
    if (base + k < P) sum += in[base + k];
  int64_t total;
  block_exclusive_scan<int64_t>(sum, s_wave, total);
  if (threadIdx.x == 0) block_sums[blockIdx.x] = total;
}

// records (optional): the blend kernels' packed per-surfel records ([P][20] floats); the surfel's exclusive offset goes
// into the last word of its record, so the blend backward finds it in the record it gathers anyway.
__global__ void __launch_bounds__(kScanThreads) scan_apply_kernel(int P, const int32_t* __restrict__ in,
                                                                  const int64_t* __restrict__ block_sums,
                                                                  int64_t* __restrict__ out,
                                                                  float* __restrict__ records) {
  __shared__ int64_t s_wave[kScanThreads / kWave];
  const int base = blockIdx.x * kScanChunk + threadIdx.x * kScanItems;
  int32_t v[kScanItems];
  int64_t sum = 0;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) {
    v[k] = base + k < P ? in[base + k] : 0;
    sum += v[k];
  }
  // The sum of the chunks in front of this one is formed here, by every block for itself (a few hundred values at most),
  // instead of by a one-block kernel between the two passes: one launch less in front of the host's wait for the count.
  int64_t before = 0;
  for (int i = threadIdx.x; i < (int) blockIdx.x; i += kScanThreads) before += block_sums[i];
  int64_t total;
  block_exclusive_scan<int64_t>(before, s_wave, total);
  const int64_t chunk_start = total;
  int64_t run = chunk_start + block_exclusive_scan<int64_t>(sum, s_wave, total);
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) {
    if (records && base + k < P) records[20 * (size_t) (base + k) + 19] = __int_as_float((int) run);
    run += v[k];
    if (base + k < P) out[base + k] = run;
  }
}

constexpr int kCoopThreshold = 32;  // rectangles with more tiles are walked by the whole wavefront
static_assert(kCoopThreshold == kCullMaskTiles, "a lane's serial walk covers exactly the rectangles that have a keep mask");

// ---- binning by tile buckets -----------------------------------------------------------------------------------------
// The reference sorts all (tile << 32 | depth bits) keys with one device-wide radix sort (6 passes of 8 bits for 2500
// tiles). The same final order -- tiles ascending, inside a tile depth bits ascending, equal depths by surfel index,
// which is what the stable radix sort leaves from the emission order -- is produced here in four steps that touch the
// instances twice instead of twelve times:
//   1. count the instances of every tile: blocks of 1024 lanes walk a slice of the surfels each and count in LDS; a
//      block's counts become one row of a (block x tile) matrix,
//   2. prefix of every matrix column over the blocks and exclusive scan of the column totals over the tiles:
//      ranges[t] = (start, end), final from here on,
//   3. the same walk again scatters (depth bits << 32 | surfel) into the tile's segment; a block's cursor of a tile
//      starts at the tile's start plus its column prefix, so neither step 1 nor step 3 issues a global atomic,
//   4. one block per tile sorts its segment (unique 64-bit keys, so the arbitrary order inside a block's run does not
//      matter): bitonic network in LDS for segments up to 16384 entries, in global memory beyond that.
// Empty tiles get (0, 0) as the reference's zero-initialised ranges have. Tile grids above kMaxLdsTiles tiles (no room
// for one LDS counter per tile) count and scatter with 64-bit global atomics on ranges[t].y instead (tile_emit_kernel).

// Visits every (surfel, tile) pair; kScatter = false counts, true scatters. `masks` (optional): a surfel's keep mask,
// the cleared bits of a rectangle of at most kCoopThreshold tiles are passed over.
template <bool kScatter>
__global__ void __launch_bounds__(256) tile_emit_kernel(int P, int gx, int gy, int64_t R,
    const float2* __restrict__ means2D, const float* __restrict__ depths, const int32_t* __restrict__ radii,
    const uint32_t* __restrict__ masks, unsigned long long* __restrict__ ranges, uint64_t* __restrict__ entries) {
  const int i    = blockIdx.x * blockDim.x + threadIdx.x;
  const int lane = __lane_id();
  int x0 = 0, y0 = 0, w = 0, h = 0;
  uint32_t dbits = 0;
  if (i < P && radii[i] > 0) {
    const float2 c   = means2D[i];
    const TileRect r = tile_rect(c.x, c.y, radii[i], gx, gy);
    x0 = r.x0, y0 = r.y0, w = max(r.x1 - r.x0, 0), h = max(r.y1 - r.y0, 0);
    if (kScatter) dbits = __float_as_uint(depths[i]);
  }
  auto visit = [&](int tile, uint32_t bits, int id) {
    unsigned long long* slot = ranges + 2 * (size_t) tile + 1;
    if (kScatter) {
      const unsigned long long pos = atomicAdd(slot, 1ull);
      if ((int64_t) pos < R) entries[pos] = ((uint64_t) bits << 32) | (uint32_t) id;
    } else {
      atomicAdd(slot, 1ull);
    }
  };
  const int count = w * h;
  if (count > 0 && count <= kCoopThreshold) {
    uint32_t keep = masks ? masks[i] : 0xffffffffu;
    for (int y = 0; y < h; ++y)
      for (int x = 0; x < w; ++x, keep >>= 1)
        if (keep & 1u) visit((y0 + y) * gx + (x0 + x), dbits, i);
  }
  unsigned long long big = __ballot(count > kCoopThreshold);
  while (big) {
    const int src = __ffsll((long long) big) - 1;
    big &= big - 1;
    const int sx0 = __shfl(x0, src, kWave), sy0 = __shfl(y0, src, kWave), sw = __shfl(w, src, kWave);
    const int scount = __shfl(count, src, kWave), sid = __shfl(i, src, kWave);
    const uint32_t sbits = __shfl(dbits, src, kWave);
    for (int e = lane; e < scount; e += kWave) {
      const int y = e / sw, x = e - y * sw;
      visit((sy0 + y) * gx + (sx0 + x), sbits, sid);
    }
  }
}

// The same traversal with the counters in LDS, one per tile (tile grids up to kMaxLdsTiles tiles): blocks of 1024 lanes
// walk a slice of the surfels each; what they do with an instance is up to the caller (tile_hist_kernel,
// tile_scatter_kernel).
constexpr int kMaxLdsTiles = 16384;

// Which tiles of a surfel's rectangle are visited: all of them (the reference's lists), those that pass the fast path's
// corner test (CornerTest, from the surfel's adjugate and opacity), or those whose bit is set in the surfel's keep mask
// (cull_mask_kernel: the tiles some pixel of which can blend the surfel; rectangles above 32 tiles are kept whole).
// kWalkCornerMask is the corner test with its verdicts for rectangles of at most 32 tiles taken from a mask the
// preprocess kernel left (bit x * h + y: x-major, the order of the fast path's key span), so that the test's set-up (a
// double-precision logarithm among it) runs once per surfel and view instead of once per walk; larger rectangles are
// tested here.
enum WalkMode { kWalkAll = 0, kWalkCorner = 1, kWalkMask = 2, kWalkCornerMask = 3 };

// What a mode reads beside centres and radii: kWalkCorner the adjugates and opacities, kWalkMask the keep masks,
// kWalkCornerMask all three.
struct WalkInputs {
  const float* inverse_m;
  const float* opacities;
  const uint32_t* keep_masks;
};

template <int kMode, typename Visit>
__device__ __forceinline__ void for_each_instance(int i, int P, int gx, int gy, const float2* __restrict__ means2D,
                                                  const int32_t* __restrict__ radii, const WalkInputs& in,
                                                  Visit visit) {
  constexpr bool kCorner = kMode == kWalkCorner || kMode == kWalkCornerMask;  // large rectangles are corner-tested
  const int lane = __lane_id();
  int x0 = 0, y0 = 0, w = 0, h = 0;
  float IM[kCorner ? 9 : 1], opacity = 1.0f;
#pragma unroll
  for (int k = 0; k < (kCorner ? 9 : 1); ++k) IM[k] = 0.0f;
  uint32_t keep_mask = 0xffffffffu;
  if (i < P && radii[i] > 0) {
    const float2 c   = means2D[i];
    const TileRect r = tile_rect(c.x, c.y, radii[i], gx, gy);
    x0 = r.x0, y0 = r.y0, w = max(r.x1 - r.x0, 0), h = max(r.y1 - r.y0, 0);
    if (kMode == kWalkCorner || (kMode == kWalkCornerMask && w * h > kCoopThreshold)) {
      opacity = in.opacities[i];
#pragma unroll
      for (int k = 0; k < 9; ++k) IM[k] = in.inverse_m[9 * (size_t) i + k];
    }
    if (kMode == kWalkMask || kMode == kWalkCornerMask) keep_mask = in.keep_masks[i];
  }
  const int count = w * h;
  if (count > 0 && count <= kCoopThreshold) {
    if (kMode == kWalkCorner) {
      const CornerTest ct(IM, opacity);
      for (int y = 0; y < h; ++y)
        for (int x = 0; x < w; ++x)
          if (ct.tile(x0 + x, y0 + y)) visit((y0 + y) * gx + (x0 + x), i);
    } else {
      int e = 0;
      for (int y = 0; y < h; ++y)
        for (int x = 0; x < w; ++x, ++e) {
          const int bit   = kMode == kWalkCornerMask ? x * h + y : e;
          const bool keep = kMode == kWalkAll || ((keep_mask >> bit) & 1u) != 0u;
          if (keep) visit((y0 + y) * gx + (x0 + x), i);
        }
    }
  }
  unsigned long long big = __ballot(count > kCoopThreshold);
  while (big) {
    const int src = __ffsll((long long) big) - 1;
    big &= big - 1;
    const int sx0 = __shfl(x0, src, kWave), sy0 = __shfl(y0, src, kWave), sw = __shfl(w, src, kWave);
    const int scount = __shfl(count, src, kWave), sid = __shfl(i, src, kWave);
    float sIM[kCorner ? 9 : 1];
#pragma unroll
    for (int k = 0; k < (kCorner ? 9 : 1); ++k) sIM[k] = kCorner ? __shfl(IM[k], src, kWave) : 0.0f;
    const CornerTest ct(sIM, kCorner ? __shfl(opacity, src, kWave) : 1.0f);
    for (int e = lane; e < scount; e += kWave) {
      const int y = e / sw, x = e - y * sw;
      if (!kCorner || ct.tile(sx0 + x, sy0 + y)) visit((sy0 + y) * gx + (sx0 + x), sid);
    }
  }
}

// One lane per 3D Gaussian: the keep mask of its rectangle from its projected mean, conic and opacity.
__global__ void __launch_bounds__(256) conic_cull_mask_kernel(int P, int gx, int gy, const float2* __restrict__ means2D,
    const float4* __restrict__ conic_opacity, const int32_t* __restrict__ radii, uint32_t* __restrict__ masks) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= P) return;
  uint32_t m = 0xffffffffu;
  const int radius = radii[i];
  if (radius > 0) {
    const float2 c    = means2D[i];
    const TileRect r  = tile_rect(c.x, c.y, radius, gx, gy);
    const int w = max(r.x1 - r.x0, 0), h = max(r.y1 - r.y0, 0);
    if (w * h <= kCullMaskTiles) {
      const float4 co     = conic_opacity[i];
      const CullBounds cb = conic_cull_bounds(co.x, co.y, co.z, co.w);
      m = 0u;
      int e = 0;
      for (int y = 0; y < h; ++y)
        for (int x = 0; x < w; ++x, ++e)
          if (cull_keeps_tile(cb, c.x, c.y, r.x0 + x, r.y0 + y)) m |= 1u << e;
    }
  }
  masks[i] = m;
}

// One lane per surfel: the keep mask of its rectangle (see kCullMaskTiles) from its packed record.
__global__ void __launch_bounds__(256) cull_mask_kernel(int P, int gx, int gy, const float4* __restrict__ records,
                                                        const int32_t* __restrict__ radii, uint32_t* __restrict__ masks) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= P) return;
  uint32_t m = 0xffffffffu;
  const int radius = radii[i];
  if (radius > 0) {
    const float4* rec = records + 5 * (size_t) i;
    const float4 q0 = rec[0], q1 = rec[1], q2 = rec[2];
    const float M[9] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w, q2.x};
    const float ox = q2.y, oy = q2.z;
    const TileRect r = tile_rect(ox, oy, radius, gx, gy);
    const int w = max(r.x1 - r.x0, 0), h = max(r.y1 - r.y0, 0);
    if (w * h <= kCullMaskTiles) {
      const CullBounds cb = cull_bounds(M, ox, oy, q2.w);
      m = 0u;
      int e = 0;
      for (int y = 0; y < h; ++y)
        for (int x = 0; x < w; ++x, ++e)
          if (cull_keeps_tile(cb, ox, oy, r.x0 + x, r.y0 + y)) m |= 1u << e;
    }
  }
  masks[i] = m;
}

// Layout of the `bins` buffer of the bucket binning: the queue length of the long segments in front of the B x T matrix
// of per-(walk block, tile) instance counts.
constexpr size_t kBinsHeader = 256;
constexpr int kPrefixTiles = 64, kPrefixWaves = 16, kPrefixChunk = 32;  // walk blocks <= kPrefixWaves * kPrefixChunk
struct BinsLayout {
  int blocks;      // walk blocks B (0: the tile grid is too large for LDS counters, the global-atomic path is used)
  int per_block;   // surfels per walk block
  size_t bytes;
};
inline BinsLayout bins_layout(int P, int T) {
  BinsLayout l{0, 0, kBinsHeader};
  if (T > kMaxLdsTiles || P <= 0) return l;
  // one 1024-lane block per 1024 surfels while that keeps every block resident at once (two fit on a compute unit),
  // beyond that the blocks grow
  l.per_block = 1024 * std::max(1, div_up(P, 1024 * kPrefixWaves * kPrefixChunk));
  l.blocks    = div_up(P, l.per_block);
  l.bytes     = kBinsHeader + align_up((size_t) l.blocks * T * sizeof(uint32_t), 256);
  return l;
}

// Step 1: every block counts the instances of its surfels per tile in LDS and writes its row of the matrix with plain
// stores (zeros included, so the matrix needs no clearing). No global atomics: device-scope atomics on one address are
// served one after the other at fabric latency, and with surfels in no spatial order every block touches nearly
// every tile.
template <int kMode>
__global__ void __launch_bounds__(1024) tile_hist_kernel(int P, int per_block, int gx, int gy,
    const float2* __restrict__ means2D, const int32_t* __restrict__ radii, WalkInputs in,
    uint32_t* __restrict__ hist) {
  __shared__ unsigned s_count[kMaxLdsTiles];
  const int T = gx * gy;
  for (int t = threadIdx.x; t < T; t += blockDim.x) s_count[t] = 0u;
  __syncthreads();
  const int first = blockIdx.x * per_block, last = min(P, first + per_block);
  // whole wavefronts stay in the loop together: the traversal uses ballots and shuffles
  const int rounds = (last - first + (int) blockDim.x - 1) / (int) blockDim.x;
  for (int r = 0; r < rounds; ++r) {
    const int i = first + r * blockDim.x + threadIdx.x;
    for_each_instance<kMode>(i < last ? i : P, P, gx, gy, means2D, radii, in,
                             [&](int tile, int) { atomicAdd(&s_count[tile], 1u); });
  }
  __syncthreads();
  uint32_t* row = hist + (size_t) blockIdx.x * T;
  for (int t = threadIdx.x; t < T; t += blockDim.x) row[t] = s_count[t];
}

// Step 2: per tile, the exclusive prefix of its column over the walk blocks (in place) and the column total, which goes
// to ranges[t].y for tile_scan_kernel. 64 tiles per block, lane = tile, the 16 wavefronts share the walk blocks in
// contiguous chunks so that a wavefront's loads are all in flight at once.
__global__ void __launch_bounds__(kPrefixTiles * kPrefixWaves) tile_prefix_kernel(int T, int B,
    uint32_t* __restrict__ hist, unsigned long long* __restrict__ ranges) {
  __shared__ uint32_t s_sum[kPrefixWaves][kPrefixTiles];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t = blockIdx.x * kPrefixTiles + lane;
  const int chunk = (B + kPrefixWaves - 1) / kPrefixWaves, b0 = wave * chunk;
  // a wavefront's whole chunk of the column is loaded before anything is written back (B <= 512: at most 32 values per
  // lane), so the loads are in flight together; a load placed behind a store to the same array would wait for it
  uint32_t c[kPrefixChunk], sum = 0;
#pragma unroll
  for (int i = 0; i < kPrefixChunk; ++i) {
    const int b = b0 + i;
    c[i] = (t < T && i < chunk && b < B) ? hist[(size_t) b * T + t] : 0u;
    sum += c[i];
  }
  s_sum[wave][lane] = sum;
  __syncthreads();
  uint32_t run = 0, total = 0;
#pragma unroll
  for (int w = 0; w < kPrefixWaves; ++w) {
    const uint32_t v = s_sum[w][lane];
    if (w < wave) run += v;
    total += v;
  }
  if (t < T) {
#pragma unroll
    for (int i = 0; i < kPrefixChunk; ++i) {
      const int b = b0 + i;
      if (i < chunk && b < B) hist[(size_t) b * T + t] = run;
      run += c[i];
    }
    if (wave == 0) ranges[2 * (size_t) t + 1] = total;
  }
}

// Step 3: the walk of step 1 again; a block's cursor of a tile starts at the tile's start plus the instances of the
// blocks in front of it, so the placement needs no global atomics either.
template <int kMode>
__global__ void __launch_bounds__(1024) tile_scatter_kernel(int P, int per_block, int gx, int gy, int64_t R,
    const float2* __restrict__ means2D, const float* __restrict__ depths, const int32_t* __restrict__ radii,
    WalkInputs in, const uint32_t* __restrict__ hist, const unsigned long long* __restrict__ ranges,
    uint64_t* __restrict__ entries, int* __restrict__ order_table) {
  __shared__ unsigned s_cursor[kMaxLdsTiles];
  // One block more than the walk needs, when the frame's blockIdx -> tile schedule is still to be built: the ranges are
  // final, nothing in this kernel reads the table, and the per-tile sorts and the blend kernels that follow do.
  if (order_table && blockIdx.x == gridDim.x - 1) {
    static_assert(sizeof(TileOrderLds) <= sizeof(s_cursor), "the schedule's LDS fits the cursor array");
    build_tile_order(gx, gy, (const int64_t*) ranges, order_table, *reinterpret_cast<TileOrderLds*>(s_cursor));
    return;
  }
  const int T = gx * gy;
  const uint32_t* row = hist + (size_t) blockIdx.x * T;
  for (int t = threadIdx.x; t < T; t += blockDim.x) s_cursor[t] = (unsigned) ranges[2 * (size_t) t] + row[t];
  __syncthreads();
  const int first = blockIdx.x * per_block, last = min(P, first + per_block);
  const int rounds = (last - first + (int) blockDim.x - 1) / (int) blockDim.x;
  for (int r = 0; r < rounds; ++r) {
    const int i = first + r * blockDim.x + threadIdx.x;
    for_each_instance<kMode>(i < last ? i : P, P, gx, gy, means2D, radii, in, [&](int tile, int id) {
      const unsigned pos = atomicAdd(&s_cursor[tile], 1u);
      if ((int64_t) pos < R) entries[pos] = ((uint64_t) __float_as_uint(depths[id]) << 32) | (uint32_t) id;
    });
  }
}

// One block: exclusive scan of the per-tile counts, 4 tiles per lane and step.
// ends = false: ranges[t] = (start, start), for a scatter that advances ranges[t].y; ends = true: (start, end).
__global__ void __launch_bounds__(1024) tile_scan_kernel(int T, unsigned long long* __restrict__ ranges,
                                                         int* __restrict__ large_count, bool ends) {
  __shared__ unsigned long long s_wave[16];
  const int lane = __lane_id(), wave = threadIdx.x / kWave;
  unsigned long long carry = 0;
  for (int start = 0; start < T; start += 4096) {
    const int t0 = start + threadIdx.x * 4;
    unsigned long long c[4], sum = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) c[k] = t0 + k < T ? ranges[2 * (size_t) (t0 + k) + 1] : 0ull, sum += c[k];
    const unsigned long long inc = wave_inclusive_scan(sum);
    if (lane == kWave - 1) s_wave[wave] = inc;
    __syncthreads();
    unsigned long long base = 0, total = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const unsigned long long v = s_wave[w];
      if (w < wave) base += v;
      total += v;
    }
    __syncthreads();
    unsigned long long run = carry + base + inc - sum;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (t0 + k < T) ranges[2 * (size_t) (t0 + k)] = run, ranges[2 * (size_t) (t0 + k) + 1] = ends ? run + c[k] : run;
      run += c[k];
    }
    carry += total;
  }
  if (threadIdx.x == 0) large_count[0] = 0, large_count[1] = (int) carry;  // queue length | instances in all tiles
}

// Where element i of a segment sits in LDS. With kPad one slot in five stays empty: the rounds of the sorting network
// whose lanes each own four consecutive elements, or four elements 4 apart, then spread a wavefront's 8-byte accesses
// over all banks instead of piling them sixteen deep on a quarter of them.
template <bool kPad>
__device__ __forceinline__ int lds_slot(int i) { return kPad ? i + (i >> 2) : i; }

template <bool kPad>
__device__ __forceinline__ void tile_sort_output(int tile, int64_t start, int n, const uint64_t* sorted_local,
                                                 int32_t* __restrict__ point_list, int64_t* __restrict__ keys_out) {
  for (int k = threadIdx.x; k < n; k += blockDim.x) {
    const uint64_t e = sorted_local[lds_slot<kPad>(k)];
    point_list[start + k] = (int32_t) (uint32_t) e;
    if (keys_out) keys_out[start + k] = (int64_t) (((uint64_t) (uint32_t) tile << 32) | (e >> 32));
  }
}

// Bitonic sorting network for any length n (all compare-exchanges ascending: the first step of every merge pairs an
// element with its mirror image inside the block, the following steps are plain half-cleaners). Pairs whose upper
// element lies beyond n are skipped, which is the same as padding with +infinity. `sync` separates the steps.
template <typename Index, typename Sync>
__device__ __forceinline__ void bitonic_sort(uint64_t* e, Index n, int threads, Sync sync) {
  Index m = 2;
  while (m < n) m <<= 1;
  int log_half = 0;
  for (Index size = 2; size <= m; size <<= 1, ++log_half) {
    const Index half = size >> 1;
    for (Index k = threadIdx.x; k < (m >> 1); k += threads) {
      const Index blk = k >> log_half, off = k & (half - 1);
      const Index lo = blk * size + off, hi = blk * size + size - 1 - off;
      if (hi < n) {
        const uint64_t a = e[lo], b = e[hi];
        if (a > b) e[lo] = b, e[hi] = a;
      }
    }
    sync();
    for (Index stride = half >> 1; stride > 0; stride >>= 1) {
      for (Index k = threadIdx.x; k < (m >> 1); k += threads) {
        const Index lo = ((k & ~(stride - 1)) << 1) | (k & (stride - 1));  // index with the `stride` bit clear
        const Index hi = lo | stride;
        if (hi < n) {
          const uint64_t a = e[lo], b = e[hi];
          if (a > b) e[lo] = b, e[hi] = a;
        }
      }
      sync();
    }
  }
}

// The same network for a segment held in LDS, two network steps per barrier: a lane loads four elements that are closed
// under two consecutive steps (mirror + first half-cleaner, or two half-cleaners), exchanges them in registers and
// stores them back.
__device__ __forceinline__ void cx(uint64_t& a, uint64_t& b) {
  const uint64_t lo = a < b ? a : b, hi = a < b ? b : a;
  a = lo, b = hi;
}

// A lane's four elements of a round lie inside an aligned span of the array (the merge size for a mirror round, twice
// the larger stride for a pair of half-cleaners), and with quads dealt to lanes in order a wavefront's 64 quads of one
// loop iteration cover one aligned 256-element chunk. Rounds whose span fits such a chunk therefore exchange data only
// between lanes of the same wavefront, which needs no block-wide barrier (a wavefront's LDS operations complete in
// order): of the 33 rounds that sort 2048 entries only 7 end in a barrier.
constexpr int kWaveSpan = 4 * kWave;

__device__ __forceinline__ void end_round(int span, int next_span) {
  if (span <= kWaveSpan && next_span <= kWaveSpan) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  } else {
    __syncthreads();
  }
}

// Power of two that a segment of n entries is padded to (with +infinity keys) before bitonic_sort_lds.
__device__ __forceinline__ int padded_length(int n) {
  int m = 2;
  while (m < n) m <<= 1;
  return m;
}

// Sorts m = 2^k >= 2 entries; every one of the m slots holds a key (the caller pads with ~0), so no access is
// conditional: bounds checks around the loads and stores made the compiler serialise them, one LDS round trip each.
template <bool kPad>
__device__ __forceinline__ void bitonic_sort_lds(uint64_t* e, int m, int threads) {
  auto ld = [&](int i) { return e[lds_slot<kPad>(i)]; };
  auto st = [&](int i, uint64_t v) { e[lds_slot<kPad>(i)] = v; };
  // one network step on pairs (two pairs per lane and iteration, so that the quads-in-order property above holds)
  auto single = [&](int size, int log_half, int stride) {  // stride == 0: the mirror step of `size`
    for (int q = threadIdx.x; q < (m >> 2); q += threads) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int k = 2 * q + h;
        int lo, hi;
        if (stride == 0) {
          const int blk = k >> log_half, off = k & ((size >> 1) - 1);
          lo = blk * size + off, hi = blk * size + size - 1 - off;
        } else {
          lo = ((k & ~(stride - 1)) << 1) | (k & (stride - 1)), hi = lo | stride;
        }
        uint64_t a = ld(lo), b = ld(hi);
        cx(a, b);
        st(lo, a), st(hi, b);
      }
    }
  };
  int log_half = 0;
  for (int size = 2; size <= m; size <<= 1, ++log_half) {
    const int next_size_span = size < m ? 2 * size : 0;
    if (size == 2) {
      if (m == 2) {
        if (threadIdx.x == 0) {
          uint64_t a = ld(0), b = ld(1);
          cx(a, b);
          st(0, a), st(1, b);
        }
        __syncthreads();
        return;
      }
      single(2, 0, 0);
      end_round(2, next_size_span);
      continue;
    }
    const int quarter = size >> 2;
    for (int q = threadIdx.x; q < (m >> 2); q += threads) {  // mirror step + half-cleaner of stride size / 4
      const int blk = q >> (log_half - 1), off = q & (quarter - 1);
      const int base = blk * size;
      const int ia = base + off, ib = ia + quarter, ja = base + size - 1 - off, jb = ja - quarter;
      uint64_t a = ld(ia), b = ld(ib), bm = ld(jb), am = ld(ja);
      cx(a, am), cx(b, bm);
      cx(a, b), cx(bm, am);
      st(ia, a), st(ib, b), st(jb, bm), st(ja, am);
    }
    int stride = quarter >> 1;
    end_round(size, stride >= 2 ? 2 * stride : (stride == 1 ? 2 : next_size_span));
    for (; stride >= 2; stride >>= 2) {  // half-cleaners of strides `stride` and `stride / 2`
      const int lo_s = stride >> 1;
      for (int q = threadIdx.x; q < (m >> 2); q += threads) {
        const int base = ((q & ~(lo_s - 1)) << 2) | (q & (lo_s - 1));
        const int i0 = base, i1 = base | lo_s, i2 = base | stride, i3 = base | stride | lo_s;
        uint64_t v0 = ld(i0), v1 = ld(i1), v2 = ld(i2), v3 = ld(i3);
        cx(v0, v2), cx(v1, v3);
        cx(v0, v1), cx(v2, v3);
        st(i0, v0), st(i1, v1), st(i2, v2), st(i3, v3);
      }
      const int next = stride >> 2;
      end_round(2 * stride, next >= 2 ? 2 * next : (next == 1 ? 2 : next_size_span));
    }
    if (stride == 1) {
      single(size, log_half, 1);
      end_round(2, next_size_span);
    }
  }
  __syncthreads();
}

constexpr int kSmallSegment = 2048;   // entries sorted by a 256-lane block in 20 KB of LDS (1024 measured: this kernel
                                      // 29.6 -> 19.7 us, and 43 us for the queued segments in the 1024-lane kernel)
                                      // (512 lanes per block instead of 256: 27.5 against 29.6 us)
constexpr int kLargeSegment = 16384;  // entries sorted by a 1024-lane block in 128 KB of LDS

// One block per tile: segments up to kSmallSegment entries are sorted in LDS, longer ones are queued for
// tile_sort_large_kernel; empty tiles get the (0, 0) range the reference's zero-initialised output has.
// `order` (optional): the blend kernels' blockIdx -> tile table, longest lists first, so that the long segments start
// sorting at once instead of wherever the image puts them in tile order (the launch ends with its slowest block).
__global__ void __launch_bounds__(256) tile_sort_small_kernel(int64_t* __restrict__ ranges,
    const uint64_t* __restrict__ entries, int32_t* __restrict__ point_list, int64_t* __restrict__ keys_out,
    int* __restrict__ large_count, int* __restrict__ large_list, const int* __restrict__ order, int n_tiles,
    int64_t R, const int* __restrict__ kept, uint64_t pad_key) {
  __shared__ uint64_t s_e[kSmallSegment + kSmallSegment / 4];
  // Blocks past the tile grid (the fast path launches some): that path reserves one list position per tile of a
  // surfel's rectangle, and the positions behind the instances that passed the corner test hold the reference's padding
  // entries (key = T << 32, value = -1), which its sort leaves at the tail of the list. Written here, beside the sorts,
  // rather than by a launch of its own behind them.
  if ((int) blockIdx.x >= n_tiles) {
    const int64_t stride = (int64_t) (gridDim.x - n_tiles) * blockDim.x;
    for (int64_t o = (int64_t) *kept + (int64_t) (blockIdx.x - n_tiles) * blockDim.x + threadIdx.x; o < R; o += stride) {
      point_list[o] = -1;
      if (keys_out) keys_out[o] = (int64_t) pad_key;
    }
    return;
  }
  const int tile = order ? order[blockIdx.x] : (int) blockIdx.x;
  const int64_t start = ranges[2 * (size_t) tile];
  const int64_t len   = ranges[2 * (size_t) tile + 1] - start;
  if (len == 0) {
    if (threadIdx.x == 0) ranges[2 * (size_t) tile] = 0, ranges[2 * (size_t) tile + 1] = 0;
    return;
  }
  if (len > kSmallSegment) {
    if (threadIdx.x == 0) large_list[atomicAdd(large_count, 1)] = tile;
    return;
  }
  const int n = (int) len;
  const int m = padded_length(n);
  for (int k = threadIdx.x; k < m; k += 256) s_e[lds_slot<true>(k)] = k < n ? entries[start + k] : ~0ull;
  __syncthreads();
  bitonic_sort_lds<true>(s_e, m, 256);
  tile_sort_output<true>(tile, start, n, s_e, point_list, keys_out);
}

// A few blocks walk the queue of long segments: up to kLargeSegment entries in LDS, beyond that the same network on the
// global array (slow, but such a segment means tens of thousands of surfels over one 16x16 tile).
__global__ void __launch_bounds__(1024) tile_sort_large_kernel(const int64_t* __restrict__ ranges,
    uint64_t* __restrict__ entries, int32_t* __restrict__ point_list, int64_t* __restrict__ keys_out,
    const int* __restrict__ large_count, const int* __restrict__ large_list) {
  __shared__ uint64_t s_e[kLargeSegment];
  const int n_large = *large_count;
  for (int q = blockIdx.x; q < n_large; q += gridDim.x) {
    const int tile = large_list[q];
    const int64_t start = ranges[2 * (size_t) tile];
    const int64_t len   = ranges[2 * (size_t) tile + 1] - start;
    if (len <= kLargeSegment) {
      const int n = (int) len;
      const int m = padded_length(n);
      for (int k = threadIdx.x; k < m; k += 1024) s_e[k] = k < n ? entries[start + k] : ~0ull;
      __syncthreads();
      bitonic_sort_lds<false>(s_e, m, 1024);
      tile_sort_output<false>(tile, start, n, s_e, point_list, keys_out);
      __syncthreads();
    } else {
      uint64_t* e = entries + start;
      bitonic_sort<int64_t>(e, len, 1024, [] {
        __threadfence_block();
        __syncthreads();
      });
      tile_sort_output<false>(tile, start, (int) len, e, point_list, keys_out);
    }
  }
}

// ---- radix sort passes ----------------------------------------------------------------------------------------------
// hist[digit * nblocks + block] = number of keys of `block` whose current digit is `digit`
__global__ void __launch_bounds__(kSortThreads) sort_histogram_kernel(int64_t R, int shift, int nblocks,
    const uint64_t* __restrict__ keys, uint32_t* __restrict__ hist) {
  __shared__ uint32_t s_hist[kRadix];
  s_hist[threadIdx.x] = 0;
  __syncthreads();
  const int64_t base = (int64_t) blockIdx.x * kSortChunk;
#pragma unroll
  for (int k = 0; k < kSortItems; ++k) {
    const int64_t idx = base + k * kSortThreads + threadIdx.x;
    if (idx < R) atomicAdd(&s_hist[(keys[idx] >> shift) & (kRadix - 1)], 1u);
  }
  __syncthreads();
  hist[(size_t) threadIdx.x * nblocks + blockIdx.x] = s_hist[threadIdx.x];
}

// One block per digit: exclusive scan of that digit's row over blocks (in place) and the digit total.
__global__ void __launch_bounds__(kScanThreads) sort_scan_rows_kernel(int nblocks, uint32_t* __restrict__ hist,
                                                                      uint32_t* __restrict__ digit_totals) {
  __shared__ uint32_t s_wave[kScanThreads / kWave];
  uint32_t* row  = hist + (size_t) blockIdx.x * nblocks;
  uint32_t carry = 0;
  for (int start = 0; start < nblocks; start += kScanThreads) {
    const int i = start + threadIdx.x;
    const uint32_t v = i < nblocks ? row[i] : 0;
    uint32_t total;
    const uint32_t ex = block_exclusive_scan<uint32_t>(v, s_wave, total);
    if (i < nblocks) row[i] = carry + ex;
    carry += total;
  }
  if (threadIdx.x == 0) digit_totals[blockIdx.x] = carry;
}

__global__ void __launch_bounds__(kSortThreads) sort_scatter_kernel(int64_t R, int shift, int nblocks,
    const uint64_t* __restrict__ keys_in, const int32_t* __restrict__ vals_in, const uint32_t* __restrict__ hist,
    const uint32_t* __restrict__ digit_totals, uint64_t* __restrict__ keys_out, int32_t* __restrict__ vals_out) {
  __shared__ uint32_t s_cnt[kSortWaves][kRadix];  // per-wave running digit counts, then per-wave global bases
  __shared__ uint32_t s_wave[kScanThreads / kWave];
  const int lane = __lane_id(), wave = threadIdx.x / kWave;
#pragma unroll
  for (int w = 0; w < kSortWaves; ++w) s_cnt[w][threadIdx.x] = 0;
  // digit base = exclusive scan of digit totals (256 values, one per thread) + this block's offset inside the digit
  uint32_t total_unused;
  const uint32_t digit_base = block_exclusive_scan<uint32_t>(digit_totals[threadIdx.x], s_wave, total_unused) +
                              hist[(size_t) threadIdx.x * nblocks + blockIdx.x];
  // block_exclusive_scan ends with a barrier, so s_cnt is zeroed for everyone here.

  const int64_t wave_base = (int64_t) blockIdx.x * kSortChunk + (int64_t) wave * (kSortItems * kWave);
  uint64_t key[kSortItems];
  int32_t val[kSortItems];
  uint32_t pos[kSortItems];
  const unsigned long long lt = lanemask_lt();
#pragma unroll
  for (int r = 0; r < kSortItems; ++r) {
    const int64_t idx = wave_base + r * kWave + lane;
    const bool valid  = idx < R;
    key[r] = valid ? keys_in[idx] : 0;
    val[r] = valid ? vals_in[idx] : 0;
    const uint32_t d = (uint32_t) (key[r] >> shift) & (kRadix - 1);
    unsigned long long peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < kRadixBits; ++b) {
      const unsigned long long m = __ballot((d >> b) & 1u);
      peers &= ((d >> b) & 1u) ? m : ~m;
    }
    const uint32_t rank  = __popcll(peers & lt);
    const uint32_t count = __popcll(peers);
    const int leader     = __ffsll((long long) peers) - 1;
    uint32_t old = 0;
    if (valid && lane == leader) {
      old = s_cnt[wave][d];
      s_cnt[wave][d] = old + count;
    }
    old    = __shfl(old, leader < 0 ? 0 : leader, kWave);
    pos[r] = old + rank;
  }
  __syncthreads();
  {  // turn per-wave counts into per-wave global bases for digit == threadIdx.x
    uint32_t run = digit_base;
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w) {
      const uint32_t c = s_cnt[w][threadIdx.x];
      s_cnt[w][threadIdx.x] = run;
      run += c;
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < kSortItems; ++r) {
    const int64_t idx = wave_base + r * kWave + lane;
    if (idx < R) {
      const uint32_t d   = (uint32_t) (key[r] >> shift) & (kRadix - 1);
      const uint32_t dst = s_cnt[wave][d] + pos[r];
      keys_out[dst] = key[r];
      vals_out[dst] = val[r];
    }
  }
}

// ---- ranges -----------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) fill_zero_i64_kernel(int64_t n, int64_t* __restrict__ p) {
  const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

__global__ void __launch_bounds__(256) tile_ranges_kernel(int64_t R, int num_tiles, const uint64_t* __restrict__ keys,
                                                          int64_t* __restrict__ ranges) {
  const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= R) return;
  const uint32_t cur = (uint32_t) (keys[i] >> 32);
  const bool cur_ok  = cur < (uint32_t) num_tiles;
  if (i == 0) {
    if (cur_ok) ranges[2 * (size_t) cur] = 0;
  } else {
    const uint32_t prev = (uint32_t) (keys[i - 1] >> 32);
    if (cur != prev) {
      if (prev < (uint32_t) num_tiles) ranges[2 * (size_t) prev + 1] = i;
      if (cur_ok) ranges[2 * (size_t) cur] = i;
    }
  }
  if (i == R - 1 && cur_ok) ranges[2 * (size_t) cur + 1] = R;
}

}  // namespace

uint32_t higher_msb(uint32_t n) {  // number of bits needed for the tile id, as gaussian_prepare.cu:32-44 computes it
  uint32_t msb = sizeof(n) * 4, step = msb;
  while (step > 1) {
    step /= 2;
    if (n >> msb) msb += step;
    else msb -= step;
  }
  if (n >> msb) msb++;
  return msb;
}

struct SortLayout {
  int nblocks;
  size_t keys0, keys1, vals_alt, hist, totals, bytes;
};

SortLayout sort_layout(int64_t R) {
  SortLayout L;
  L.nblocks = div_up(R > 0 ? R : 1, kSortChunk);
  size_t o  = 0;
  L.keys0 = o, o = align_up(o + (size_t) R * 8, 256);
  L.keys1 = o, o = align_up(o + (size_t) R * 8, 256);
  L.vals_alt = o, o = align_up(o + (size_t) R * 4, 256);
  L.hist = o, o = align_up(o + (size_t) kRadix * L.nblocks * 4, 256);
  L.totals = o, o = align_up(o + (size_t) kRadix * 4, 256);
  L.bytes = o;
  return L;
}


// Stable LSD radix sort of (key, value) pairs on key bits [0, bits). `vals_in` holds the unsorted payload (it is one of
// the two ping-pong buffers); on return the sorted payload is in `vals_out` and *sorted_keys points at the sorted keys
// (inside the workspace). The caller picks vals_in so that the last pass lands in vals_out: see sort_vals_in().
int radix_sort_pairs(int64_t R, int bits, void* workspace, int32_t* vals_out, const uint64_t** sorted_keys,
                     hipStream_t s) {
  const SortLayout L = sort_layout(R);
  char* ws          = (char*) workspace;
  uint64_t* kbuf[2] = {(uint64_t*) (ws + L.keys0), (uint64_t*) (ws + L.keys1)};
  uint32_t* hist    = (uint32_t*) (ws + L.hist);
  uint32_t* totals  = (uint32_t*) (ws + L.totals);
  const int passes  = (bits + kRadixBits - 1) / kRadixBits;
  int32_t* vbuf[2];
  vbuf[passes & 1]       = vals_out;
  vbuf[(passes & 1) ^ 1] = (int32_t*) (ws + L.vals_alt);
  for (int p = 0; p < passes; ++p) {
    const int shift = p * kRadixBits;
    const int a = p & 1, b = a ^ 1;
    hipLaunchKernelGGL(sort_histogram_kernel, dim3(L.nblocks), dim3(kSortThreads), 0, s, R, shift, L.nblocks, kbuf[a],
                       hist);
    hipLaunchKernelGGL(sort_scan_rows_kernel, dim3(kRadix), dim3(kScanThreads), 0, s, L.nblocks, hist, totals);
    hipLaunchKernelGGL(sort_scatter_kernel, dim3(L.nblocks), dim3(kSortThreads), 0, s, R, shift, L.nblocks, kbuf[a],
                       vbuf[a], hist, totals, kbuf[b], vbuf[b]);
  }
  *sorted_keys = kbuf[passes & 1];
  return passes;
}

// Where the unsorted keys / payload must be written before radix_sort_pairs(R, bits, workspace, vals_out, ...).
uint64_t* sort_keys_in(int64_t R, void* workspace) { return (uint64_t*) ((char*) workspace + sort_layout(R).keys0); }
int32_t* sort_vals_in(int64_t R, int bits, void* workspace, int32_t* vals_out) {
  const int passes = (bits + kRadixBits - 1) / kRadixBits;
  return (passes & 1) ? (int32_t*) ((char*) workspace + sort_layout(R).vals_alt) : vals_out;
}
size_t sort_workspace_bytes(int64_t R) { return sort_layout(R).bytes; }

void launch_zero_ranges(int num_tiles, int64_t* ranges, hipStream_t s) {
  hipLaunchKernelGGL(fill_zero_i64_kernel, dim3(div_up(2 * (int64_t) num_tiles, 256)), dim3(256), 0, s,
                     2 * (int64_t) num_tiles, ranges);
}
void launch_tile_ranges(int64_t R, int num_tiles, const uint64_t* sorted_keys, int64_t* ranges, hipStream_t s) {
  hipLaunchKernelGGL(tile_ranges_kernel, dim3(div_up(R, 256)), dim3(256), 0, s, R, num_tiles, sorted_keys, ranges);
}

size_t fast_bucket_bins_bytes(int P, int W, int H) {
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const BinsLayout bl = bins_layout(P, gx * gy);
  return bl.blocks > 0 ? bl.bytes : 0;
}

int fast_bucket_fill(int P, int W, int H, const float* means2D, const float* inverse_m, const float* depths,
                     const float* opacities, const int32_t* radii, const uint32_t* keep_masks, int64_t R,
                     int64_t* ranges, int32_t* point_list, int64_t* sorted_keys_out, void* workspace, void* bins,
                     hipStream_t s) {
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const int T  = gx * gy;
  const BinsLayout bl = bins_layout(P, T);
  unsigned long long* rng = (unsigned long long*) ranges;
  int* header      = (int*) bins;  // [0] length of the long-segment queue, [1] instances kept by the corner test
  uint32_t* hist   = (uint32_t*) ((char*) bins + kBinsHeader);
  uint64_t* entries = sort_keys_in(R, workspace);
  int* large_list   = (int*) ((char*) workspace + sort_layout(R).keys1);
  const WalkInputs in{inverse_m, opacities, keep_masks};
  if (keep_masks)
    hipLaunchKernelGGL(tile_hist_kernel<kWalkCornerMask>, dim3(bl.blocks), dim3(1024), 0, s, P, bl.per_block, gx, gy,
                       (const float2*) means2D, radii, in, hist);
  else
    hipLaunchKernelGGL(tile_hist_kernel<kWalkCorner>, dim3(bl.blocks), dim3(1024), 0, s, P, bl.per_block, gx, gy,
                       (const float2*) means2D, radii, in, hist);
  hipLaunchKernelGGL(tile_prefix_kernel, dim3(div_up(T, kPrefixTiles)), dim3(kPrefixTiles * kPrefixWaves), 0, s, T,
                     bl.blocks, hist, rng);
  hipLaunchKernelGGL(tile_scan_kernel, dim3(1), dim3(1024), 0, s, T, rng, header, true);
  // the schedule the blend kernels of this view find under `ranges`, built by an extra block of the scatter
  const int* order = nullptr;
  int* build       = nullptr;
  (void) defer_tile_order(gx, gy, ranges, s, &order, &build);
  if (keep_masks)
    hipLaunchKernelGGL(tile_scatter_kernel<kWalkCornerMask>, dim3(bl.blocks + (build ? 1 : 0)), dim3(1024), 0, s, P,
                       bl.per_block, gx, gy, R, (const float2*) means2D, depths, radii, in, (const uint32_t*) hist, rng,
                       entries, build);
  else
    hipLaunchKernelGGL(tile_scatter_kernel<kWalkCorner>, dim3(bl.blocks + (build ? 1 : 0)), dim3(1024), 0, s, P,
                       bl.per_block, gx, gy, R, (const float2*) means2D, depths, radii, in, (const uint32_t*) hist, rng,
                       entries, build);
  // 256 blocks more than tiles: they write the padding entries behind the kept instances
  hipLaunchKernelGGL(tile_sort_small_kernel, dim3(T + 256), dim3(256), 0, s, ranges, entries, point_list,
                     sorted_keys_out, header, large_list, order, T, R, (const int*) (header + 1),
                     (uint64_t) (uint32_t) T << 32);
  hipLaunchKernelGGL(tile_sort_large_kernel, dim3(256), dim3(1024), 0, s, ranges, entries, point_list, sorted_keys_out,
                     header, large_list);
  return check_launch("gs_2d_fast_prepare_fill");
}

}  // namespace fsgs

using namespace fsgs;

FSGS_API size_t fsgs_gs_prepare_scan_workspace_bytes(int P) {
  return align_up((size_t) div_up(P > 0 ? P : 1, kScanChunk) * 8, 256);
}

namespace {
// One event per host thread marks "the instance count has been copied": waiting on it instead of on the stream lets the
// caller queue work that does not depend on the count behind the copy.
hipEvent_t count_event() {
  static thread_local hipEvent_t ev = nullptr;
  if (!ev && hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) ev = nullptr;
  return ev;
}
thread_local bool t_count_pending = false;  // a scan_begin of this thread has queued a copy nobody has waited for
}  // namespace

FSGS_API int fsgs_gs_prepare_scan_begin(int P, const int32_t* tiles_touched, int64_t* point_offsets, void* workspace,
                                        size_t workspace_bytes, int64_t* num_rendered_host, float* records,
                                        void* stream) {
  FSGS_REQUIRE(P >= 0 && num_rendered_host, "gs_prepare_scan: bad arguments");
  *num_rendered_host = 0;
  t_count_pending    = false;
  if (P == 0) return kOk;  // nothing is queued, nothing to wait for
  hipStream_t s = (hipStream_t) stream;
  hipEvent_t ev = count_event();
  FSGS_REQUIRE(ev != nullptr, "gs_prepare_scan: cannot create an event");
  {
    FSGS_REQUIRE(tiles_touched && point_offsets && workspace, "gs_prepare_scan: null pointer");
    if (workspace_bytes < fsgs_gs_prepare_scan_workspace_bytes(P))
      return fail(kWorkspaceSmall, "gs_prepare_scan: workspace %zu < %zu bytes", workspace_bytes,
                  fsgs_gs_prepare_scan_workspace_bytes(P));
    const int nb      = div_up(P, kScanChunk);
    int64_t* blk_sums = (int64_t*) workspace;
    hipLaunchKernelGGL(scan_block_sums_kernel, dim3(nb), dim3(kScanThreads), 0, s, P, tiles_touched, blk_sums);
    hipLaunchKernelGGL(scan_apply_kernel, dim3(nb), dim3(kScanThreads), 0, s, P, tiles_touched, blk_sums,
                       point_offsets, records);
    if (int rc = check_launch("gs_prepare_scan")) return rc;
    // The number of (surfel, tile) instances sizes the caller's output, so it has to reach the host
    // (the reference blocks for it, gaussian_prepare.cu:238-239).
    FSGS_HIP(hipMemcpyAsync(num_rendered_host, point_offsets + (P - 1), sizeof(int64_t), hipMemcpyDeviceToHost, s));
  }
  FSGS_HIP(hipEventRecord(ev, s));
  t_count_pending = true;
  return kOk;
}

FSGS_API int fsgs_gs_prepare_scan_end(void) {
  if (!t_count_pending) return kOk;
  t_count_pending = false;
  hipEvent_t ev   = count_event();
  FSGS_REQUIRE(ev != nullptr, "gs_prepare_scan: cannot create an event");
  FSGS_HIP(hipEventSynchronize(ev));
  return kOk;
}

FSGS_API int fsgs_gs_prepare_scan(int P, const int32_t* tiles_touched, int64_t* point_offsets, void* workspace,
                                  size_t workspace_bytes, int64_t* num_rendered_host, void* stream) {
  if (int rc = fsgs_gs_prepare_scan_begin(P, tiles_touched, point_offsets, workspace, workspace_bytes,
                                          num_rendered_host, nullptr, stream))
    return rc;
  return fsgs_gs_prepare_scan_end();
}

FSGS_API size_t fsgs_gs_prepare_fill_workspace_bytes(int64_t R) { return sort_layout(R).bytes; }

FSGS_API int fsgs_gs_prepare_sort_bits(int W, int H) {
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  return 32 + (int) higher_msb((uint32_t) (gx * gy));
}

namespace {
// First part of the bucket binning, independent of the instance count: per-tile instance counts and the tile ranges
// (start, end); the long-segment queue's counter (first word of `bins`) is reset.
// keep_masks (optional): the per-surfel keep masks of cull_mask_kernel; with them an instance is only counted (and
// later scattered) when its bit is set.
int fill_count(int P, int W, int H, const float* means2D, const int32_t* radii, const uint32_t* keep_masks,
               int64_t* ranges, void* bins, hipStream_t s) {
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const int T  = gx * gy;
  unsigned long long* rng = (unsigned long long*) ranges;
  int* header = (int*) bins;
  const BinsLayout bl = bins_layout(P, T);
  if (bl.blocks > 0) {
    uint32_t* hist = (uint32_t*) ((char*) bins + kBinsHeader);
    if (keep_masks)
      hipLaunchKernelGGL(tile_hist_kernel<kWalkMask>, dim3(bl.blocks), dim3(1024), 0, s, P, bl.per_block, gx, gy,
                         (const float2*) means2D, radii, WalkInputs{nullptr, nullptr, keep_masks}, hist);
    else
      hipLaunchKernelGGL(tile_hist_kernel<kWalkAll>, dim3(bl.blocks), dim3(1024), 0, s, P, bl.per_block, gx, gy,
                         (const float2*) means2D, radii, WalkInputs{nullptr, nullptr, nullptr}, hist);
    hipLaunchKernelGGL(tile_prefix_kernel, dim3(div_up(T, kPrefixTiles)), dim3(kPrefixTiles * kPrefixWaves), 0, s, T,
                       bl.blocks, hist, rng);
    hipLaunchKernelGGL(tile_scan_kernel, dim3(1), dim3(1024), 0, s, T, rng, header, true);
    // The ranges are final here; the schedule table the blend kernels of this frame are going to use (and the per-tile
    // sorts) is built from them by an extra block of the scatter, in the second part.
  } else {
    // no room for one LDS counter per tile (or no surfels): count straight into ranges[t].y, then scan to (start, start)
    hipLaunchKernelGGL(fill_zero_i64_kernel, dim3(div_up(2 * (int64_t) T, 256)), dim3(256), 0, s, 2 * (int64_t) T,
                       ranges);
    if (P > 0)
      hipLaunchKernelGGL(tile_emit_kernel<false>, dim3(div_up(P, 256)), dim3(256), 0, s, P, gx, gy, (int64_t) 0,
                         (const float2*) means2D, (const float*) nullptr, radii, keep_masks, rng, (uint64_t*) nullptr);
    hipLaunchKernelGGL(tile_scan_kernel, dim3(1), dim3(1024), 0, s, T, rng, header, false);
  }
  return check_launch("gs_prepare_count");
}

// Second part: scatter (depth bits << 32 | surfel) into the tile segments and sort every segment.
int fill_sort(int P, int W, int H, const float* means2D, const float* depths, const int32_t* radii,
              const uint32_t* keep_masks, int64_t R, int64_t* ranges, int32_t* point_list, int64_t* sorted_keys_out,
              void* workspace, void* bins, hipStream_t s) {
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  const int T  = gx * gy;
  unsigned long long* rng = (unsigned long long*) ranges;
  uint64_t* entries       = sort_keys_in(R, workspace);
  int* large_count        = (int*) bins;
  // queue of long segments: at most R / kSmallSegment tiles, kept behind the entries in the workspace
  int* large_list = (int*) ((char*) workspace + sort_layout(R).keys1);
  const BinsLayout bl = bins_layout(P, T);
  // The schedule table: built by one extra block of the scatter (the ranges are final since the counting part), or by a
  // launch of its own on the global-atomic path, whose ranges only become final with the scatter.
  const int* order = nullptr;
  int* build       = nullptr;
  if (bl.blocks > 0) (void) defer_tile_order(gx, gy, ranges, s, &order, &build);
  const dim3 scatter_grid(bl.blocks + (build ? 1 : 0));
  if (bl.blocks > 0 && keep_masks)
    hipLaunchKernelGGL(tile_scatter_kernel<kWalkMask>, scatter_grid, dim3(1024), 0, s, P, bl.per_block, gx, gy, R,
                       (const float2*) means2D, depths, radii, WalkInputs{nullptr, nullptr, keep_masks},
                       (const uint32_t*) ((const char*) bins + kBinsHeader), rng, entries, build);
  else if (bl.blocks > 0)
    hipLaunchKernelGGL(tile_scatter_kernel<kWalkAll>, scatter_grid, dim3(1024), 0, s, P, bl.per_block, gx, gy, R,
                       (const float2*) means2D, depths, radii, WalkInputs{nullptr, nullptr, nullptr},
                       (const uint32_t*) ((const char*) bins + kBinsHeader), rng, entries, build);
  else {
    hipLaunchKernelGGL(tile_emit_kernel<true>, dim3(div_up(P, 256)), dim3(256), 0, s, P, gx, gy, R,
                       (const float2*) means2D, depths, radii, keep_masks, rng, entries);
    (void) launch_tile_order(gx, gy, ranges, s, &order);
  }
  hipLaunchKernelGGL(tile_sort_small_kernel, dim3(T), dim3(256), 0, s, ranges, entries, point_list, sorted_keys_out,
                     large_count, large_list, order, T, (int64_t) 0, (const int*) nullptr, (uint64_t) 0);
  hipLaunchKernelGGL(tile_sort_large_kernel, dim3(256), dim3(1024), 0, s, ranges, entries, point_list, sorted_keys_out,
                     large_count, large_list);
  return check_launch("gs_prepare_fill");
}
}  // namespace

FSGS_API size_t fsgs_gs_prepare_bins_bytes(int P, int W, int H) {
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  return bins_layout(P, gx * gy).bytes;
}

FSGS_API int fsgs_gs_prepare_count(int P, int W, int H, const float* means2D, const int32_t* radii, int64_t* ranges,
                                   void* bins, size_t bins_bytes, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0 && ranges && bins, "gs_prepare_count: bad arguments");
  FSGS_REQUIRE(P == 0 || (means2D && radii), "gs_prepare_count: null pointer");
  if (bins_bytes < fsgs_gs_prepare_bins_bytes(P, W, H))
    return fail(kWorkspaceSmall, "gs_prepare_count: bins %zu < %zu bytes", bins_bytes,
                fsgs_gs_prepare_bins_bytes(P, W, H));
  tile_order_invalidate((hipStream_t) stream);  // the ranges are rewritten: the blend schedule of this stream is stale
  return fill_count(P, W, H, means2D, radii, nullptr, ranges, bins, (hipStream_t) stream);
}

FSGS_API int fsgs_gs_prepare_fill_counted(int P, int W, int H, const float* means2D, const float* depths,
                                          const int32_t* radii, int64_t R, int64_t* ranges, int32_t* point_list,
                                          int64_t* sorted_keys_out, void* bins, size_t bins_bytes, void* workspace,
                                          size_t workspace_bytes, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0 && R >= 0 && ranges && bins, "gs_prepare_fill: bad arguments");
  FSGS_REQUIRE(R < (int64_t) 0x7fffffff, "gs_prepare_fill: %lld instances exceed the 2^31-1 limit", (long long) R);
  if (R == 0 || P == 0) return kOk;  // the counting part left every range empty
  FSGS_REQUIRE(means2D && depths && radii && point_list && workspace, "gs_prepare_fill: null pointer");
  if (workspace_bytes < sort_workspace_bytes(R))
    return fail(kWorkspaceSmall, "gs_prepare_fill: workspace %zu < %zu bytes", workspace_bytes,
                sort_workspace_bytes(R));
  if (bins_bytes < fsgs_gs_prepare_bins_bytes(P, W, H))
    return fail(kWorkspaceSmall, "gs_prepare_fill: bins %zu < %zu bytes", bins_bytes,
                fsgs_gs_prepare_bins_bytes(P, W, H));
  return fill_sort(P, W, H, means2D, depths, radii, nullptr, R, ranges, point_list, sorted_keys_out, workspace, bins,
                   (hipStream_t) stream);
}

// Keep masks for the culled binning: a bit per tile of a surfel's rectangle (row-major, rectangles of at most 32 tiles;
// larger ones are kept whole), set when some pixel of the tile can blend the surfel by the blend kernels' own bound.
FSGS_API int fsgs_gs_2d_cull_masks(int P, int W, int H, const float* records, const int32_t* radii, uint32_t* masks,
                                   void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0, "gs_2d_cull_masks: bad sizes");
  if (P == 0) return kOk;
  FSGS_REQUIRE(records && radii && masks, "gs_2d_cull_masks: null pointer");
  FSGS_REQUIRE(((uintptr_t) records & 15) == 0, "gs_2d_cull_masks: records must be 16-byte aligned");
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  hipLaunchKernelGGL(cull_mask_kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P, gx, gy,
                     (const float4*) records, radii, masks);
  return check_launch("gs_2d_cull_masks");
}

// The same for 3D Gaussians, from the tensors their preprocess leaves (gaussian_rasterize's alpha test in place of the
// surfel's).
FSGS_API int fsgs_gs_cull_masks(int P, int W, int H, const float* means2D, const float* conic_opacity,
                                const int32_t* radii, uint32_t* masks, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0, "gs_cull_masks: bad sizes");
  if (P == 0) return kOk;
  FSGS_REQUIRE(means2D && conic_opacity && radii && masks, "gs_cull_masks: null pointer");
  FSGS_REQUIRE(((uintptr_t) conic_opacity & 15) == 0 && ((uintptr_t) means2D & 7) == 0,
               "gs_cull_masks: means2D / conic_opacity must be 8 / 16-byte aligned");
  const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
  hipLaunchKernelGGL(conic_cull_mask_kernel, dim3(div_up(P, 256)), dim3(256), 0, (hipStream_t) stream, P, gx, gy,
                     (const float2*) means2D, (const float4*) conic_opacity, radii, masks);
  return check_launch("gs_cull_masks");
}

// The two phases of the binning over the kept tiles only (masks: fsgs_gs_2d_cull_masks). A process with the culling
// switched off for debugging gets the full lists.
FSGS_API int fsgs_gs_prepare_count_culled(int P, int W, int H, const float* means2D, const int32_t* radii,
                                          const uint32_t* masks, int64_t* ranges, void* bins, size_t bins_bytes,
                                          void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0 && ranges && bins, "gs_prepare_count_culled: bad arguments");
  FSGS_REQUIRE(P == 0 || (means2D && radii && masks), "gs_prepare_count_culled: null pointer");
  if (bins_bytes < fsgs_gs_prepare_bins_bytes(P, W, H))
    return fail(kWorkspaceSmall, "gs_prepare_count_culled: bins %zu < %zu bytes", bins_bytes,
                fsgs_gs_prepare_bins_bytes(P, W, H));
  tile_order_invalidate((hipStream_t) stream);
  return fill_count(P, W, H, means2D, radii, culling_enabled() ? masks : nullptr, ranges, bins,
                    (hipStream_t) stream);
}

FSGS_API int fsgs_gs_prepare_fill_counted_culled(int P, int W, int H, const float* means2D, const float* depths,
                                                 const int32_t* radii, const uint32_t* masks, int64_t R,
                                                 int64_t* ranges, int32_t* point_list, int64_t* sorted_keys_out,
                                                 void* bins, size_t bins_bytes, void* workspace,
                                                 size_t workspace_bytes, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0 && R >= 0 && ranges && bins, "gs_prepare_fill_culled: bad arguments");
  FSGS_REQUIRE(R < (int64_t) 0x7fffffff, "gs_prepare_fill_culled: %lld instances exceed the 2^31-1 limit", (long long) R);
  if (R == 0 || P == 0) return kOk;
  FSGS_REQUIRE(means2D && depths && radii && masks && point_list && workspace, "gs_prepare_fill_culled: null pointer");
  if (workspace_bytes < sort_workspace_bytes(R))
    return fail(kWorkspaceSmall, "gs_prepare_fill_culled: workspace %zu < %zu bytes", workspace_bytes,
                sort_workspace_bytes(R));
  if (bins_bytes < fsgs_gs_prepare_bins_bytes(P, W, H))
    return fail(kWorkspaceSmall, "gs_prepare_fill_culled: bins %zu < %zu bytes", bins_bytes,
                fsgs_gs_prepare_bins_bytes(P, W, H));
  return fill_sort(P, W, H, means2D, depths, radii, culling_enabled() ? masks : nullptr, R, ranges,
                   point_list, sorted_keys_out, workspace, bins, (hipStream_t) stream);
}

FSGS_API int fsgs_gs_prepare_fill(int P, int W, int H, const float* means2D, const float* depths,
                                  const int32_t* radii, const int64_t* point_offsets, int64_t R, int64_t* ranges,
                                  int32_t* point_list, int64_t* sorted_keys_out, void* bins, size_t bins_bytes,
                                  void* workspace, size_t workspace_bytes, void* stream) {
  FSGS_REQUIRE(P >= 0 && W > 0 && H > 0 && R >= 0 && ranges, "gs_prepare_fill: bad arguments");
  FSGS_REQUIRE(R < (int64_t) 0x7fffffff, "gs_prepare_fill: %lld instances exceed the 2^31-1 limit", (long long) R);
  hipStream_t s = (hipStream_t) stream;
  tile_order_invalidate(s);  // the ranges are rewritten: the blend schedule of this stream is stale
  if (R == 0 || P == 0) {
    const int gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
    hipLaunchKernelGGL(fill_zero_i64_kernel, dim3(div_up(2 * (int64_t) gx * gy, 256)), dim3(256), 0, s,
                       2 * (int64_t) gx * gy, ranges);
    return check_launch("gs_prepare_fill(zero)");
  }
  FSGS_REQUIRE(means2D && depths && radii && point_offsets && point_list && workspace && bins,
               "gs_prepare_fill: null pointer");
  if (workspace_bytes < sort_workspace_bytes(R))
    return fail(kWorkspaceSmall, "gs_prepare_fill: workspace %zu < %zu bytes", workspace_bytes,
                sort_workspace_bytes(R));
  if (bins_bytes < fsgs_gs_prepare_bins_bytes(P, W, H))
    return fail(kWorkspaceSmall, "gs_prepare_fill: bins %zu < %zu bytes", bins_bytes,
                fsgs_gs_prepare_bins_bytes(P, W, H));
  if (int rc = fill_count(P, W, H, means2D, radii, nullptr, ranges, bins, s)) return rc;
  return fill_sort(P, W, H, means2D, depths, radii, nullptr, R, ranges, point_list, sorted_keys_out, workspace, bins, s);
}
