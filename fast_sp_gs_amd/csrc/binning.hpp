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

}  // namespace fsgs
