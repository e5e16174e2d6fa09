// The calling thread's last refusal or fault, and the device's size.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"
#include "llmp_hip.h"

namespace llmp_hip {
namespace {
thread_local char g_error[512] = "";
}

void SetError(const char* format, ...) {
  va_list args;
  va_start(args, format);
  vsnprintf(g_error, sizeof(g_error), format, args);
  va_end(args);
}

int Refuse(int code, const char* format, ...) {
  va_list args;
  va_start(args, format);
  vsnprintf(g_error, sizeof(g_error), format, args);
  va_end(args);
  return code;
}

int LaunchStatus(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return 0;
  SetError("%s: %s", what, hipGetErrorString(e));
  return -static_cast<int>(e);
}

}  // namespace llmp_hip

extern "C" const char* llmp_hip_last_error(void) { return llmp_hip::g_error; }

extern "C" int llmp_hip_compute_units(void) {
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  int units = 0;
  if (e == hipSuccess) e = hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device);
  if (e != hipSuccess) {
    llmp_hip::SetError("compute units: %s", hipGetErrorString(e));
    return -static_cast<int>(e);
  }
  return units;
}
