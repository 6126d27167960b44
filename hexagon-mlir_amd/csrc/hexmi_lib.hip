// Library-level entry points: version, status text, device query.
#include "hexmi_common.h"

extern "C" const char* hexmi_version(void) { return "hexmi 0.3 gfx950"; }

extern "C" const char* hexmi_strerror(int status) {
  switch (status) {
    case HEXMI_OK: return "ok";
    case HEXMI_EINVAL: return "invalid argument (null pointer, negative size, bad leading dimension or alignment)";
    case HEXMI_ENOTSUP: return "unsupported dtype or shape";
    case HEXMI_ELAUNCH: return "HIP launch failed";
    case HEXMI_ETOOBIG: return "size exceeds the fixed capacity of this entry point";
    default: return "unknown status";
  }
}

extern "C" int hexmi_num_cus(void) {
  // launchers ask on every call: the attribute is looked up once per device (a racing first call stores the same
  // value twice)
  constexpr int kMaxDevices = 64;
  static int cached[kMaxDevices];
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < kMaxDevices && cached[dev] > 0) return cached[dev];
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < kMaxDevices) cached[dev] = cus;
  return cus;
}
