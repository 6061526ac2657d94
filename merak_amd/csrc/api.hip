// Error string, version and device identification of the C ABI.
#include "mtp_common.h"
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

namespace {
thread_local char g_err[512] = "";
}

void mtp_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" int mtp_abi_version(void) { return MTP_ABI_VERSION; }

extern "C" const char* mtp_last_error(void) { return g_err; }

extern "C" int mtp_device_arch(char* buf, int len) {
  MTP_REQUIRE(buf && len > 0, MTP_EINVAL, "device_arch: bad buffer");
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    mtp_set_error("device_arch: hipGetDevice: %s", hipGetErrorString(e));
    return MTP_EDEVICE;
  }
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) {
    mtp_set_error("device_arch: hipGetDeviceProperties: %s", hipGetErrorString(e));
    return MTP_EDEVICE;
  }
  // gcnArchName looks like "gfx950:sramecc+:xnack-"
  const char* colon = strchr(prop.gcnArchName, ':');
  size_t n = colon ? (size_t)(colon - prop.gcnArchName) : strlen(prop.gcnArchName);
  if (n >= (size_t)len) n = (size_t)len - 1;
  memcpy(buf, prop.gcnArchName, n);
  buf[n] = 0;
  return MTP_OK;
}
