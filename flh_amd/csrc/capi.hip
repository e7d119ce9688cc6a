// Error reporting and set-up entry points of libflh_hip.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "common.h"

namespace flh {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(FLH_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
  return FLH_OK;
}

int current_device(int* dev, const char* what) {
  if (hipGetDevice(dev) != hipSuccess) return fail(FLH_EDEVICE, "%s: no current HIP device", what);
  if (*dev < 0 || *dev >= kMaxDevices)
    return fail(FLH_EDEVICE, "%s: device index %d is beyond the %d this library keeps set-up for", what, *dev, kMaxDevices);
  return FLH_OK;
}

int reserve_lds(const void* kernel, size_t bytes, LdsGrant& grant, const char* what) {
  int dev = 0;
  if (int rc = current_device(&dev, what)) return rc;
  if (bytes <= grant.bytes[dev].load(std::memory_order_acquire)) return FLH_OK;
  static std::mutex growing;                           // two sizes at once must not leave the smaller one in force
  std::lock_guard<std::mutex> lock(growing);
  if (bytes <= grant.bytes[dev].load(std::memory_order_relaxed)) return FLH_OK;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess)
    return fail(FLH_ELAUNCH, "%s: cannot reserve %zu bytes of LDS", what, bytes);
  grant.bytes[dev].store(bytes, std::memory_order_release);
  return FLH_OK;
}

int rotate_quant_mfma_init();  // fwht_mfma.hip

}  // namespace flh

extern "C" int flh_abi_version(void) { return 1; }

extern "C" const char* flh_last_error(void) { return flh::g_err; }

extern "C" int flh_init(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return flh::fail(FLH_EDEVICE, "no HIP device");
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return flh::fail(FLH_EDEVICE, "cannot query device %d", dev);
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return flh::fail(FLH_EDEVICE, "device %d is %s; this library is built for gfx950 only", dev, prop.gcnArchName);
  return flh::rotate_quant_mfma_init();   // constant tables, so that no later call has to wait for them
}
