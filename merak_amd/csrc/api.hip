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

// ---- tuning variables: read once, re-read on request ----------------------------------------------------
#include <atomic>
#include <mutex>
#include <stdlib.h>
namespace {
std::mutex g_tune_mu;
MtpTune* g_tune_head = nullptr;
void tune_read(MtpTune* t) {
  const char* e = getenv(t->name);
  if (e && *e) {
    t->value = atoi(e);
    __atomic_store_n(&t->state, 2, __ATOMIC_RELEASE);
  } else {
    __atomic_store_n(&t->state, 1, __ATOMIC_RELEASE);
  }
}
}  // namespace

MtpTune::MtpTune(const char* n) : name(n), value(0), state(0), next(nullptr) {
  std::lock_guard<std::mutex> lk(g_tune_mu);
  next = g_tune_head;
  g_tune_head = this;
}
bool MtpTune::is_set() {
  int st = __atomic_load_n(&state, __ATOMIC_ACQUIRE);
  if (st == 0) {
    std::lock_guard<std::mutex> lk(g_tune_mu);
    if (state == 0) tune_read(this);
    st = state;
  }
  return st == 2;
}
int MtpTune::get(int dflt) { return is_set() ? value : dflt; }

extern "C" void mtp_reload_tuning(void) {
  std::lock_guard<std::mutex> lk(g_tune_mu);
  for (MtpTune* t = g_tune_head; t; t = t->next) tune_read(t);
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
