// Shared host-side plumbing for the C-ABI library: error reporting, launch checks, small device helpers.
// gfx950 (CDNA4) only: 64-wide wavefronts are assumed throughout.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#define FSGS_API extern "C" __attribute__((visibility("default")))

namespace fsgs {

constexpr int kWave = 64;
constexpr int kTile = 16;  // tile edge in pixels (BLOCK_X == BLOCK_Y == 16 in the reference, gaussian_render.h:28-29)

enum Status : int {
  kOk              = 0,
  kInvalidArgument = 1,
  kLaunchFailure   = 2,
  kWorkspaceSmall  = 3,
  kUnsupported     = 4,
};

char* last_error_buffer();
int fail(int code, const char* fmt, ...);

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(kLaunchFailure, "%s: %s", what, hipGetErrorString(e));
  return kOk;
}

#define FSGS_REQUIRE(cond, ...)                                  \
  do {                                                           \
    if (!(cond)) return ::fsgs::fail(::fsgs::kInvalidArgument, __VA_ARGS__); \
  } while (0)

#define FSGS_HIP(call)                                                                         \
  do {                                                                                         \
    hipError_t e_ = (call);                                                                    \
    if (e_ != hipSuccess) return ::fsgs::fail(::fsgs::kLaunchFailure, "%s: %s", #call, hipGetErrorString(e_)); \
  } while (0)

inline int div_up(int64_t a, int64_t b) { return (int) ((a + b - 1) / b); }

// Block barrier that orders LDS traffic only. __syncthreads() also waits for every global load and store the
// wavefront has in flight (s_waitcnt vmcnt(0)), which puts the latency of loads issued ahead of time, and of stores
// nobody in the block reads back, on the critical path of each round; this one waits for LDS alone.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Mask of the lanes where `b` holds, straight from the comparison's lane mask: HIP's __ballot takes an int, which makes
// the compiler materialise the predicate in a register and compare it again.
__device__ __forceinline__ unsigned long long wave_ballot(bool b) { return __builtin_amdgcn_ballot_w64(b); }

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// float -> int with saturation and NaN -> 0 (what v_cvt_i32_f32 does; spelled out so the result does not depend on
// how the compiler lowers an out-of-range cast).
__device__ __forceinline__ int f2i_sat(float v) {
  if (!(v == v)) return 0;
  if (v >= 2147483647.0f) return 2147483647;
  if (v <= -2147483648.0f) return (-2147483647 - 1);
  return (int) v;
}

struct TileRect {
  int x0, y0, x1, y1;
};

// Tile rectangle covered by a disc of integer radius r around p; mirrors getRect (gaussian_render.h:33-39) including
// its evaluation order ((p + r) + 16) - 1.
__device__ __forceinline__ TileRect tile_rect(float px, float py, int r, int gx, int gy) {
#pragma clang fp contract(off)
  TileRect q;
  const float rf = (float) r;
  q.x0 = min(gx, max(0, f2i_sat((px - rf) / 16.0f)));
  q.y0 = min(gy, max(0, f2i_sat((py - rf) / 16.0f)));
  q.x1 = min(gx, max(0, f2i_sat((((px + rf) + 16.0f) - 1.0f) / 16.0f)));
  q.y1 = min(gy, max(0, f2i_sat((((py + rf) + 16.0f) - 1.0f) / 16.0f)));
  return q;
}

// ---- blockIdx -> tile schedule of the blend kernels (built by tile_order_kernel in blend.hpp) ------------------------
// Each (device, stream) that bins or blends owns one of a few tables held in a file-scope device array (api.hip), keyed
// on the tile ranges it was built from (address and grid size). tile_order_table returns the stream's table, or nullptr
// when the device's tables are all taken (then blocks map to tiles directly), and sets *rebuild when the key changed: the
// caller then launches tile_order_kernel on that stream. The binning entry points forget the key of their stream when
// they rewrite a ranges buffer, so a frame builds the table once and the frame's blend launches (forward, backward,
// top-k, extra channels) reuse it. A ranges buffer rewritten behind the library's back (or binned on another stream)
// keeps an older frame's order: still a permutation of the same tile grid, so every tile is processed exactly once --
// only the longest-first order is stale. All three functions take the same lock.
int* tile_order_table(hipStream_t stream, const int64_t* ranges, int gx, int gy, bool* rebuild);
void tile_order_invalidate(hipStream_t stream);
void tile_order_release(hipStream_t stream);

}  // namespace fsgs
