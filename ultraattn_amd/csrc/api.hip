// Version, error strings and the device check shared by the entry points.
#include <atomic>
#include <cstring>
#include "ua_common.h"

namespace ua {

int check_device() {
  // Cache per device ordinal: 0 unknown, 1 gfx950, 2 something else.
  static std::atomic<int> cache[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return UA_ERR_DEVICE;
  if (dev < 0 || dev >= 64) return UA_ERR_DEVICE;
  int st = cache[dev].load(std::memory_order_relaxed);
  if (st == 0) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return UA_ERR_DEVICE;
    st = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 2;
    cache[dev].store(st, std::memory_order_relaxed);
  }
  return st == 1 ? UA_OK : UA_ERR_DEVICE;
}

}  // namespace ua

extern "C" int ua_version(void) { return UA_VERSION; }

extern "C" const char* ua_strerror(int rc) {
  switch (rc) {
    case UA_OK: return "ok";
    case UA_ERR_NULL: return "a required pointer is NULL";
    case UA_ERR_SHAPE: return "non-positive or inconsistent sizes";
    case UA_ERR_UNSUPPORTED: return "unsupported configuration (head_dim must be 128, softmax_scale > 0, 1..16 partials)";
    case UA_ERR_ALIGN: return "pointer not 16-byte aligned or stride not a multiple of 8 elements";
    case UA_ERR_MASK: return "block mask holds a value other than 0 (EMPTY), 1 (FULL), 2 (CAUSAL)";
    case UA_ERR_LAUNCH: return "HIP kernel launch failed";
    case UA_ERR_DEVICE: return "current device is not a gfx950 (MI355X) GPU";
    case UA_ERR_TOO_LARGE: return "input exceeds the fixed scratch of the no-allocation entry point";
    default: return "unknown error code";
  }
}
