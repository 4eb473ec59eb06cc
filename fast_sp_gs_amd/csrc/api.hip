// Library-level entry points of the C-ABI: error text, version, device check.
#include "common.hpp"

#include <cstring>
#include <map>
#include <mutex>
#include <utility>

namespace fsgs {

char* last_error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

// One blockIdx -> tile table (65536 ints, see blend.hpp) per (device, stream) that a blend entry point was called on,
// with the tile ranges it was built from.
TileOrderState* tile_order_state(hipStream_t stream) {
  static std::mutex mu;
  static std::map<std::pair<int, hipStream_t>, TileOrderState> tables;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  auto it = tables.find({dev, stream});
  if (it != tables.end()) return it->second.table ? &it->second : nullptr;
  int* p = nullptr;
  if (hipMalloc((void**) &p, sizeof(int) * (1 << 16)) != hipSuccess) {
    (void) hipGetLastError();
    p = nullptr;
  }
  TileOrderState& st = tables[{dev, stream}];
  st = TileOrderState{p, nullptr, 0, 0};
  return p ? &st : nullptr;
}

void tile_order_invalidate(hipStream_t stream) {
  if (TileOrderState* st = tile_order_state(stream)) st->ranges = nullptr;
}

static bool g_culling_enabled = true;
bool culling_enabled() { return g_culling_enabled; }

namespace {
// Plain streaming copy, 16 bytes per lane and grid-stride: the yardstick for achievable HBM bandwidth and the known-size
// kernel against which hardware byte counters are calibrated.
__global__ void __launch_bounds__(256) copy_probe_kernel(const float4* __restrict__ src, float4* __restrict__ dst,
                                                         size_t n) {
  for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t) gridDim.x * blockDim.x)
    dst[i] = src[i];
}
}  // namespace

}  // namespace fsgs

FSGS_API int fsgs_copy_probe(const void* src, void* dst, size_t nbytes, void* stream) {
  FSGS_REQUIRE(src && dst && nbytes % 16 == 0 && (((uintptr_t) src | (uintptr_t) dst) & 15) == 0,
               "copy_probe: buffers must be 16-byte aligned and a multiple of 16 bytes long");
  const size_t n = nbytes / 16;
  if (n == 0) return fsgs::kOk;
  const size_t blocks = (n + 255) / 256;
  hipLaunchKernelGGL(fsgs::copy_probe_kernel, dim3((unsigned) (blocks < 16384 ? blocks : 16384)), dim3(256), 0,
                     (hipStream_t) stream, (const float4*) src, (float4*) dst, n);
  return fsgs::check_launch("copy_probe");
}

FSGS_API int fsgs_debug_set_culling(int enabled) {
  fsgs::g_culling_enabled = enabled != 0;
  return fsgs::kOk;
}

FSGS_API const char* fsgs_last_error() { return fsgs::last_error_buffer(); }

FSGS_API int fsgs_version() { return 100; }

// Returns 0 when the current device can run this library's code objects (gfx950), else a non-zero status with text.
FSGS_API int fsgs_check_device() {
  int dev = 0;
  FSGS_HIP(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  FSGS_HIP(hipGetDeviceProperties(&prop, dev));
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fsgs::fail(fsgs::kUnsupported, "device %d is %s; this library is built for gfx950 only", dev,
                      prop.gcnArchName);
  return fsgs::kOk;
}
