// Library-level entry points of the C-ABI: error text, version, device check.
#include "common.hpp"

#include <cstring>

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

}  // namespace fsgs

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
