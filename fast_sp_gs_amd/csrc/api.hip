// Library-level entry points of the C-ABI: error text, version, device check.
#include "common.hpp"

#include <cstring>
#include <mutex>

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

// blockIdx -> tile tables of the blend kernels (see blend.hpp): kTableSlots tables of kMaxOrderedTiles ints each in a
// file-scope device array, so the library never calls hipMalloc. A (device, stream) pair takes a free slot on its first
// binning or blend call and keeps it until fsgs_stream_release or the end of the process; when every slot of a device
// is taken, further streams get no table and their blocks map to tiles directly (same results, no longest-first order).
// Slots are never taken away from a stream behind its back: a kernel of that stream may still be reading the table.
constexpr int kTableSlots   = 8;
constexpr int kTableInts    = 1 << 16;  // == kMaxOrderedTiles
constexpr int kMaxDevices   = 64;
static __device__ __align__(256) int g_tile_order_tables[kTableSlots][kTableInts];

namespace {
struct TableSlot {
  bool used = false;
  hipStream_t stream = nullptr;
  const int64_t* ranges = nullptr;  // what the table was built from (nullptr: nothing)
  int gx = 0, gy = 0;
};
struct DeviceTables {
  int* base = nullptr;  // device address of g_tile_order_tables on this device (each device holds its own copy)
  bool resolved = false;
  TableSlot slot[kTableSlots];
};
std::mutex g_table_mu;
DeviceTables g_tables[kMaxDevices];

// Caller holds g_table_mu. Returns the slot of (current device, stream), taking a free one if `take`; -1 if none.
int find_slot(hipStream_t stream, bool take, DeviceTables** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return -1;
  DeviceTables& d = g_tables[dev];
  *out = &d;
  if (!d.resolved) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_tile_order_tables)) != hipSuccess) {
      (void) hipGetLastError();
      p = nullptr;
    }
    d.base = (int*) p, d.resolved = true;
  }
  if (!d.base) return -1;
  int free_slot = -1;
  for (int i = 0; i < kTableSlots; ++i) {
    if (d.slot[i].used && d.slot[i].stream == stream) return i;
    if (!d.slot[i].used && free_slot < 0) free_slot = i;
  }
  if (!take || free_slot < 0) return -1;
  d.slot[free_slot] = TableSlot{true, stream, nullptr, 0, 0};
  return free_slot;
}
}  // namespace

int* tile_order_table(hipStream_t stream, const int64_t* ranges, int gx, int gy, bool* rebuild) {
  std::lock_guard<std::mutex> lock(g_table_mu);
  *rebuild = false;
  DeviceTables* d = nullptr;
  const int i = find_slot(stream, true, &d);
  if (i < 0) return nullptr;
  TableSlot& t = d->slot[i];
  if (t.ranges != ranges || t.gx != gx || t.gy != gy) {
    t.ranges = ranges, t.gx = gx, t.gy = gy;
    *rebuild = true;
  }
  return d->base + (size_t) i * kTableInts;
}

void tile_order_invalidate(hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_table_mu);
  DeviceTables* d = nullptr;
  const int i = find_slot(stream, false, &d);
  if (i >= 0) d->slot[i].ranges = nullptr;
}

void tile_order_release(hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_table_mu);
  DeviceTables* d = nullptr;
  const int i = find_slot(stream, false, &d);
  if (i >= 0) d->slot[i] = TableSlot{};
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

FSGS_API int fsgs_stream_release(void* stream) {
  fsgs::tile_order_release((hipStream_t) stream);
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
