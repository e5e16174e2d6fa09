// The calling thread's last refusal or fault, and the device's size.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"
#include "llmp_hip.h"

namespace llmp_hip {
namespace {
thread_local char g_error[512] = "";
// A failure met while preparing a launch (the kernel's LDS allowance), reported by the next LaunchStatus.
thread_local int g_pending = 0;
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

void BeginLaunches() {
  g_pending = 0;
  (void)hipGetLastError();  // an error an earlier, unrelated call left on this thread is not this call's
}

bool AllowLds(const void* kernel, int bytes, bool* sized) {
  if (*sized) return true;
  const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    SetError("allowing a kernel %d bytes of LDS: %s", bytes, hipGetErrorString(e));
    g_pending = -static_cast<int>(e);
    return false;  // asked again by the next call: the flag stays clear
  }
  *sized = true;
  return true;
}

int LaunchStatus(const char* what) {
  if (g_pending != 0) {
    const int code = g_pending;
    g_pending = 0;
    return code;
  }
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
