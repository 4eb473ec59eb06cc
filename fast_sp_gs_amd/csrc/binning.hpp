// Internal interface of the binning building blocks (prefix scan is reached through its C-ABI entry point), shared by
// the standard and the fused "fast" binning.
#pragma once
#include "common.hpp"

namespace fsgs {

uint32_t higher_msb(uint32_t n);
size_t sort_workspace_bytes(int64_t R);
uint64_t* sort_keys_in(int64_t R, void* workspace);
int32_t* sort_vals_in(int64_t R, int bits, void* workspace, int32_t* vals_out);
int radix_sort_pairs(int64_t R, int bits, void* workspace, int32_t* vals_out, const uint64_t** sorted_keys,
                     hipStream_t s);
void launch_zero_ranges(int num_tiles, int64_t* ranges, hipStream_t s);
void launch_tile_ranges(int64_t R, int num_tiles, const uint64_t* sorted_keys, int64_t* ranges, hipStream_t s);

// The per-tile (bucket) binning with the fast path's corner test: only the tiles of a surfel's rectangle that pass
// CornerTest are counted, scattered and sorted; point_list / sorted_keys_out beyond the kept instances are filled with
// the reference's padding entries (-1 / T << 32) up to R. `bins`: fast_bucket_bins_bytes(P, W, H) bytes (0: the tile
// grid is too large for this scheme and the caller sorts device-wide instead); `workspace`: sort_workspace_bytes(R).
size_t fast_bucket_bins_bytes(int P, int W, int H);
// `keep_masks` (optional): the verdicts of the test for rectangles of at most 32 tiles, bit x * h + y of a surfel's word
// (fast_preprocess_forward_kernel writes them); the walks then test only the larger rectangles themselves.
int fast_bucket_fill(int P, int W, int H, const float* means2D, const float* inverse_m, const float* depths,
                     const float* opacities, const int32_t* radii, const uint32_t* keep_masks, int64_t R,
                     int64_t* ranges, int32_t* point_list, int64_t* sorted_keys_out, void* workspace, void* bins,
                     hipStream_t s);

// Implicit conic of the alpha >= 1/255 region, evaluated at tile corners in tile units (gs_2d_fast_preprocess.cu:277-304).
// Contraction off, the reference's operation order: which tiles a surfel keeps must not depend on the compiler's choice
// of fused multiply-adds (the lists are compared bit for bit with a plain IEEE evaluation).
struct CornerTest {
  float Wxx, Wyy, Wxy, Wx_, Wy_, W__;
  __device__ __forceinline__ CornerTest() : Wxx(0), Wyy(0), Wxy(0), Wx_(0), Wy_(0), W__(1) {}  // passes nowhere
  __device__ __forceinline__ CornerTest(const float* IM, float opacity) {
#pragma clang fp contract(off)
    const float d = -2.0f * 0.69314718055f * (7.9886846867721655f + (float) log2((double) opacity));
    Wxx = IM[0] * IM[0] + IM[3] * IM[3] + d * IM[6] * IM[6];
    Wyy = IM[1] * IM[1] + IM[4] * IM[4] + d * IM[7] * IM[7];
    W__ = IM[2] * IM[2] + IM[5] * IM[5] + d * IM[8] * IM[8];
    Wxy = 2 * (IM[0] * IM[1] + IM[3] * IM[4] + d * IM[6] * IM[7]);
    Wx_ = 2 * (IM[0] * IM[2] + IM[3] * IM[5] + d * IM[6] * IM[8]);
    Wy_ = 2 * (IM[1] * IM[2] + IM[4] * IM[5] + d * IM[7] * IM[8]);
    Wxx = Wxx * 16 * 16, Wyy = Wyy * 16 * 16, Wxy = Wxy * 16 * 16, Wx_ = Wx_ * 16, Wy_ = Wy_ * 16;
  }
  __device__ __forceinline__ bool at(float u, float v) const {
#pragma clang fp contract(off)
    return Wxx * u * u + Wyy * v * v + Wxy * u * v + Wx_ * u + Wy_ * v + W__ <= 0;
  }
  __device__ __forceinline__ bool tile(int x, int y) const {
    return at((float) x, (float) y) || at((float) (x + 1), (float) y) || at((float) x, (float) (y + 1)) ||
           at((float) (x + 1), (float) (y + 1));
  }
};

}  // namespace fsgs
