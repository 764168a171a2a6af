// Library-level entry points: ABI version, error strings, device check.
#include <string.h>

#include "common.h"

extern "C" int dsx_abi_version(void) { return DSX_ABI_VERSION; }

extern "C" const char* dsx_strerror(int code) {
  switch (code) {
    case DSX_OK: return "ok";
    case DSX_EBADSHAPE: return "unsupported shape, size or stride";
    case DSX_EALIGN: return "pointer, stride or leading dimension is not suitably aligned";
    case DSX_EARCH: return "current device is not gfx950 (MI355X)";
    case DSX_ELAUNCH: return "kernel launch failed";
    case DSX_ENULL: return "required pointer is NULL";
    case DSX_EWORKSPACE: return "scratch memory missing or too small for this call";
    default: return "unknown dsx error code";
  }
}

extern "C" int dsx_check_device(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return DSX_EARCH;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return DSX_EARCH;
  return strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? DSX_OK : DSX_EARCH;
}
