// lib.hip — library-level entry points and host helpers of libtriton_int_hip.so.
#include <stdarg.h>
#include <string.h>

#include "ti_common.h"

namespace ti {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// The kernels are written for gfx950 only (MFMA shapes, 160 KB LDS, buffer loads into LDS); on
// any other device the launch would fail or fault, so refuse early with a clear message.
int check_device() {
  static int checked[64];  // 0 unknown, 1 ok, -1 wrong arch
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return fail((int)err, "hipGetDevice: %s", hipGetErrorString(err));
  if (dev < 0 || dev >= 64) return TI_OK;
  if (checked[dev] == 0) {
    hipDeviceProp_t prop;
    err = hipGetDeviceProperties(&prop, dev);
    if (err != hipSuccess) return fail((int)err, "hipGetDeviceProperties: %s", hipGetErrorString(err));
    checked[dev] = strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : -1;
    if (checked[dev] < 0) set_error("device %d is %s; this library only runs on gfx950", dev, prop.gcnArchName);
  }
  if (checked[dev] < 0) {
    set_error("device %d is not gfx950", dev);
    return TI_E_DEVICE;
  }
  return TI_OK;
}

int launch_status(const char* what) {
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return fail((int)err, "launch of %s failed: %s", what, hipGetErrorString(err));
  return TI_OK;
}

}  // namespace ti

extern "C" {

int ti_version(void) { return 1; }

const char* ti_last_error(void) { return ti::g_err; }

}  // extern "C"
