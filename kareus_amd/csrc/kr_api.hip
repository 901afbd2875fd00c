#include "kr_common.h"

extern "C" int kr_version(void) { return 100; }

extern "C" int kr_device_clock_mhz(void) {
  int dev = 0, khz = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&khz, hipDeviceAttributeClockRate, dev) != hipSuccess) return 0;
  return khz / 1000;
}

extern "C" const char* kr_error_string(int code) {
  switch (code) {
    case KR_OK: return "ok";
    case KR_EINVAL: return "invalid argument (null/misaligned pointer, bad size or stride)";
    case KR_EUNSUPPORTED: return "shape not supported by the gfx950 kernels";
    case KR_ELAUNCH: return "HIP runtime rejected the kernel launch";
    default: return "unknown error code";
  }
}
