/* fsgs_debug.h -- measurement and verification aids of libfsgs_hip.so. None of them has a counterpart in the reference
 * and none is part of the drop-in operator boundary (include/fsgs.h); tests and the benchmark use them.
 * Same conventions as fsgs.h: extern "C", plain pointers and sizes, 0 on success, fsgs_last_error() for the message. */
#ifndef FSGS_DEBUG_H
#define FSGS_DEBUG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Copies nbytes (multiple of 16, 16-byte aligned) from src to dst with a plain streaming kernel; benchmarks use it as
 * the achievable-bandwidth yardstick and counter calibration. */
int fsgs_copy_probe(const void* src, void* dst, size_t nbytes, void* stream);

/* The blend kernels skip, per 8x8 pixel quadrant, surfels whose alpha >= 1/255 footprint cannot reach it. enabled = 0
 * turns that skip off process-wide (every staged surfel is then evaluated at every pixel, as the reference does), so
 * tests can show that results do not depend on it. Default: on. Process-global: not for use next to concurrent renders. */
int fsgs_debug_set_culling(int enabled);

/* Writes the blockIdx -> tile table the blend kernels would use for a gx x gy tile grid whose lists are ranges[t] =
 * (start, end) into table[gx * gy] (device memory; gx * gy <= 65536): a permutation of the tile numbers, longest lists
 * first inside each of the 8 interleaved position classes. For tests of the schedule itself. */
int fsgs_debug_tile_order(int gx, int gy, const int64_t* ranges, int32_t* table, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* FSGS_DEBUG_H */
